#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace esp {
hipError_t launch_gather_columns(const uint16_t *surface, int channels, int spatial, int lanes, uint16_t *out16, float *out32, hipStream_t s);
hipError_t launch_scatter_columns(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s);
// the same with rows of `in` `in_stride` floats apart (a slice of a wider row)
hipError_t launch_scatter_columns_strided(const float *in, int in_stride, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s);
// Half-split RoPE in place on lane 0 of the q and k surfaces (MetalAttentionKernel.swift:1756-1795, rope_decode).
hipError_t launch_surface_rope(uint16_t *q, uint16_t *k, int n_heads, int n_kv_heads, int head_dim, int position, float theta, int lane_stride, hipStream_t s);
// Lane 0 of the k / v surfaces into column `token_index` of the channel-first caches (MetalAttentionKernel.swift:1805-1820, kv_cache_scatter).
hipError_t launch_surface_kv_scatter(const uint16_t *k_src, const uint16_t *v_src, uint16_t *k_cache, uint16_t *v_cache, int kv_dim, int token_index,
                                     int cache_stride, int lane_stride, hipStream_t s);
// Single-query attention over channel-first fp16 caches [kvDim, cacheStride] into lane 0 of the context surface
// (MetalAttentionKernel.swift:1824-1886, fused_decode_sdpa; CPU twin DecodeForwardPass.swift:683-756).
hipError_t launch_surface_sdpa(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *context, int heads, int kv_heads, int head_dim,
                               int visible_tokens, int token_base, int cache_stride, int lane_stride, hipStream_t s);
// Factored output head: expansion of the projected surface [bottleneck, spatial] (lanes 0 .. lanes - 1) by w [vocab][bottleneck / groups] fused with the
// arg-max (surface_io.c:1438-1700 with fp16 sums, MetalExpansionArgmax.swift:966-1186 with fp32 sums); `blocks` candidates per lane go through cand_v / cand_i.
hipError_t launch_expansion_argmax(const uint16_t *proj, int spatial, int lanes, const uint16_t *w, int bottleneck, int groups, int vocab, bool fp32_sums,
                                   int blocks, float *cand_v, int *cand_i, int *out_i, float *out_v, hipStream_t s);
hipError_t launch_row_max(const float *in, int channels, int spatial, int lanes, uint16_t *surface, hipStream_t s);
}  // namespace esp
