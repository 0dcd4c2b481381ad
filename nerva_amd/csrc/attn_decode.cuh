// Launch interface of the fused decode-attention kernels (attn_decode.hip).
#pragma once

#include "nv_common.cuh"

namespace nv {

constexpr uint32_t kKvBlockTokens = 16;   // tokens per paged KV block (types.cuh:64)
constexpr uint32_t kAttnMaxSplits = 64;   // split-KV partials per kv head

// KV cache layout (library-owned): [layer][physical block][kv_head][16 tokens][head_dim]
// 16-bit, K and V in separate arrays. One (block, kv_head) tile is contiguous
// (4 KiB at head_dim 128), so a wave streams it with four 1 KiB load instructions.
__host__ __device__ __forceinline__ uint64_t kv_tile_offset(uint32_t block_count, uint32_t kv_heads,
                                                            uint32_t head_dim, uint32_t layer,
                                                            uint32_t physical_block, uint32_t kv_head) {
  return ((static_cast<uint64_t>(layer) * block_count + physical_block) * kv_heads + kv_head) *
         kKvBlockTokens * head_dim;
}

struct AttnParams {
  const float *qkv;            // [heads*hd | kv_heads*hd | kv_heads*hd] raw f32 projections
  const uint16_t *q_norm, *k_norm;           // optional [hd]
  const uint16_t *q_bias, *k_bias, *v_bias;  // optional
  uint16_t *k_cache, *v_cache;
  const uint32_t *table;       // [block_count]
  const float *rope_freq;      // [hd/2]: powf(theta, 2i/hd), or null = no RoPE
  const float *rope_cs;        // optional [hd]: cos | sin of pos / rope_freq[i], precomputed for this step
  float *part_acc;             // [heads][splits][hd]  un-normalised partial outputs
  float *part_m, *part_l;      // [heads][splits]
  uint32_t *counters;          // [kv_heads] arrival counters, zero between launches
  float *out_f32;              // optional [heads*hd]
  uint16_t *out16;             // [heads*hd]
  uint32_t heads, kv_heads, head_dim, layer, block_count, splits;
  float eps;
  const uint32_t *cursor;      // device position, or null -> `position`
  uint32_t position, max_steps, append;
};

uint64_t attn_workspace_bytes(uint32_t heads, uint32_t head_dim);
// Carves part_acc/part_m/part_l/counters out of a workspace of attn_workspace_bytes().
void attn_bind_workspace(AttnParams &p, void *workspace);
hipError_t launch_attn_decode(uint32_t dtype, const AttnParams &p, hipStream_t stream);

}  // namespace nv
