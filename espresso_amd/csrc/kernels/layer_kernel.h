// One launch for the whole decoder trunk of a batch-1 decode step (kernels/layer_kernel.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace esp {

struct TrunkLayer {
    const uint8_t *wqkv, *wo, *w13, *w2;   // Q4_K super-blocks, row-major
    const float *rms_att, *rms_ffn;
    void *k_cache, *v_cache;               // [seq][max_seq][kvDim]
};

constexpr int kTrunkSyncWords = 2048;      // barrier state, cleared before every launch

struct TrunkArgs {
    const TrunkLayer *layers;   // device array
    int n_layer;
    float *hidden;              // [d] in: embedding row, out: trunk output
    float *q;                   // [attnDim]
    uint16_t *ctx;              // [attnDim] fp16
    uint16_t *act;              // [hidden] fp16
    float *attn_scratch;        // [kvHeads][splits][group][head_dim + 2]
    const float *rope_cos, *rope_sin;
    const int *pos, *seq;       // row 0
    int n_head, n_kv_head, max_seq, kv_f16;
    int splits;                 // slices of the prefix per KV head (1..32)
    size_t cache_seq_stride;
    float norm_eps;
    unsigned *sync;             // kTrunkSyncWords words
};

// True when the fused kernel has an instantiation for this architecture (Q4_K everywhere).
bool trunk_kernel_supports(int d_model, int hidden_dim, int head_dim, int n_head, int n_kv_head);
// Clears the barrier state and runs the trunk.  The grid is sized so that every workgroup is resident.
hipError_t launch_trunk_kernel(const TrunkArgs &args, int d_model, int hidden_dim, hipStream_t stream);
// Barrier time-outs recorded by launches so far (0 in a healthy run); reading it synchronises the stream.
hipError_t trunk_kernel_timeouts(const unsigned *sync, hipStream_t stream, unsigned *out);

}  // namespace esp
