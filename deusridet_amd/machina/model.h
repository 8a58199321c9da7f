// model.h -- the part of the reference's ModelConfig that the paged-KV path
// reads (src/machina/model.h:30-73): runtime statics for the attention geometry.
// The reference fills them from a model's config.json (src/machina/model.cpp:
// 127-221); here set_attention_geometry() does it, because this build ships the
// KV-cache path only, not the model loader.
#pragma once

#include "drk_kv.h"
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

namespace deusridet {

// The members of the reference's weight and state structs that the two layer wrappers
// full_attention_forward_paged[_prefill] read (src/machina/model.h:89-93, 132-146, 232-293);
// same names, same meaning.  A build inside the reference's tree uses its own model.h instead.
struct Linear {                      // model.h:89-93
    __half* weight = nullptr;        // [out_features, in_features] row-major
    int in_features  = 0;
    int out_features = 0;
};

struct FullAttentionWeights {        // model.h:132-146
    Linear fp16_q;                   // hidden -> NUM_ATTN_HEADS * HEAD_DIM * 2 (Q | gate, interleaved per head)
    Linear fp16_k;                   // hidden -> NUM_KV_HEADS * HEAD_DIM
    Linear fp16_v;
    Linear fp16_o;                   // NUM_ATTN_HEADS * HEAD_DIM -> hidden
    __half* q_norm = nullptr;        // [HEAD_DIM]
    __half* k_norm = nullptr;        // [HEAD_DIM]
};

struct InferenceState {              // model.h:232-293, the buffers this path touches
    __half* norm_out = nullptr;      // [max_seq, hidden]            O projection lands here
    __half* attn_out = nullptr;      // [max_seq, NUM_ATTN_HEADS * HEAD_DIM]
    __half* q_buf    = nullptr;      // [max_seq, NUM_ATTN_HEADS * HEAD_DIM * 2]   Q | gate projection
    __half* kv_buf   = nullptr;      // [max_seq, NUM_KV_HEADS * HEAD_DIM]         K projection (prefill)
    __half* mlp_gate = nullptr;      // scratch the reference parks the gate in; not written here
    __half* dn_qkv   = nullptr;      // [max_seq, >= NUM_ATTN_HEADS * HEAD_DIM]    rope(norm(q))
    __half* dn_z     = nullptr;      // [max_seq, >= 2 * NUM_KV_HEADS * HEAD_DIM]  K, V projections (decode), V (prefill)
    int*    d_pos    = nullptr;      // [1] device: current sequence position
    hipStream_t compute_stream = nullptr;
};

struct ModelConfig {
    static int NUM_ATTN_HEADS;   // model.h:39
    static int NUM_KV_HEADS;     // model.h:40
    static int HEAD_DIM;         // model.h:41
    static int NUM_KV_GROUPS;    // model.h:42, ATTN_HEADS / KV_HEADS
    static int NUM_FA_LAYERS;    // model.h:73
    static float RMS_EPS;        // model.h:36 (default 1e-6)
    static float ROPE_THETA;     // model.h:49 (default 1e7)
    static int ROTARY_DIM;       // model.h:51, HEAD_DIM * partial_rotary_factor (default HEAD_DIM / 4)
    // Not in the reference (its cache is fp16 only): storage type of the pool and
    // element type of Q / out / append sources, DRK_* from drk_kv.h.
    static int KV_DTYPE;         // DRK_F16 (default), DRK_BF16, DRK_INT8, DRK_FP8_E4M3
    static int IO_DTYPE;         // DRK_F16 (default) or DRK_BF16

    // Returns false (and changes nothing) when the numbers are inconsistent.
    static bool set_attention_geometry(int num_fa_layers, int num_attn_heads, int num_kv_heads, int head_dim,
                                       int kv_dtype = DRK_F16, int io_dtype = -1);

    // rotary_dim must be 16 * 2^k and at most HEAD_DIM; false (nothing changed) otherwise.
    static bool set_rope(int rotary_dim, float theta, float rms_eps);

    // The C-ABI layout for a pool of max_phys_blocks blocks of block_size tokens.
    static drk_kv_layout layout(int max_phys_blocks, int block_size);
};

} // namespace deusridet
