// layer.cpp -- see layer.h.  Forwarders to the C ABI.
#include "layer.h"
#include "../communis/log.h"
#include "drk_kv.h"

namespace deusridet {

void sigmoid_gate(const __half* x, const __half* gate, __half* out, int n, hipStream_t stream)
{
    if (n <= 0) return;
    // any row length that divides n works for an element-wise step; the reference moves
    // 8 elements per thread and ignores a remainder (layer.cu:410, 434)
    if (drk_sigmoid_gate(x, gate, out, (size_t)n / 8, 8, 8, ModelConfig::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "sigmoid_gate: %s", drk_last_error());
}

void apply_rope(__half* q, __half* k, int num_heads, int num_kv_heads, int head_dim, int rotary_dim, const int* d_pos,
                float theta, hipStream_t stream)
{
    if (drk_apply_rope(q, k, 1, num_heads, num_kv_heads, head_dim, rotary_dim, d_pos, 0, theta, nullptr, 0,
                       ModelConfig::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "apply_rope: %s", drk_last_error());
}

void head_norm(const __half* x, const __half* weight, __half* out, int num_heads, int head_dim, float eps,
               hipStream_t stream)
{
    if (drk_head_norm(x, weight, out, num_heads, head_dim, eps, ModelConfig::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "head_norm: %s", drk_last_error());
}

} // namespace deusridet
