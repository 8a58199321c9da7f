// layer.h -- the element-wise steps of a full-attention layer that sit either side of the
// page kernels, with the reference's names, parameter order and meaning
// (src/machina/layer.h:77-79, 124-140) and HIP vocabulary types.  Elements are of type
// ModelConfig::IO_DTYPE (fp16 by default, as in the reference); `__half*` then just
// means "16-bit element".  Launchers return void, are asynchronous on `stream` and log a
// failure.  The fused forms of these steps are in paged_attention.h.
#pragma once

#include "model.h"
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

namespace deusridet {

// Sigmoid gate: out = x * sigmoid(gate) over n elements (n a multiple of 8)
void sigmoid_gate(const __half* x, const __half* gate, __half* out, int n, hipStream_t stream = 0);

// Partial RoPE, half-half pairing (i, i + rotary_dim/2), one token at position *d_pos:
// q [num_heads, head_dim], k [num_kv_heads, head_dim], in place.
void apply_rope(__half* q, __half* k, int num_heads, int num_kv_heads, int head_dim, int rotary_dim, const int* d_pos,
                float theta, hipStream_t stream = 0);

// Per-head RMSNorm: x, out [num_heads, head_dim], weight [head_dim]
void head_norm(const __half* x, const __half* weight, __half* out, int num_heads, int head_dim, float eps,
               hipStream_t stream = 0);

} // namespace deusridet
