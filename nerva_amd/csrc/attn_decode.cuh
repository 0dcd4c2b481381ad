// Launch interface of the fused decode-attention kernels (attn_decode.hip).
#pragma once

#include "nv_common.cuh"

namespace nv {

constexpr uint32_t kKvBlockTokens = 16;   // tokens per paged KV block (types.cuh:64)
constexpr uint32_t kAttnMaxSplits = 64;   // split-KV partials per kv head

// KV cache layout (library-owned): [layer][physical block][kv_head][tile of 16 tokens x head_dim]
// 16-bit, K and V in separate arrays. One (block, kv_head) tile is contiguous
// (4 KiB at head_dim 128), so a wave streams it with four 1 KiB load instructions.
// Inside a tile, head_dim 128 is stored in matrix-core operand order (kv_k_elem, kv_v_elem);
// every other head_dim is row-major [token][dim].
__host__ __device__ __forceinline__ uint64_t kv_tile_offset(uint32_t block_count, uint32_t kv_heads,
                                                            uint32_t head_dim, uint32_t layer,
                                                            uint32_t physical_block, uint32_t kv_head) {
  return ((static_cast<uint64_t>(layer) * block_count + physical_block) * kv_heads + kv_head) *
         kKvBlockTokens * head_dim;
}

// Element offset of (token row, dim d) inside a K tile. head_dim 128: load j of lane
// l = (d%32/8)*16 + row holds dims 32j + 8*(l/16) .. +7 of token l%16, the A operand of a
// 16x16x32 matrix-core product over dims.
__host__ __device__ __forceinline__ uint32_t kv_k_elem(uint32_t head_dim, uint32_t row, uint32_t d) {
  if (head_dim != 128) return row * head_dim + d;
  return (d / 32) * 512 + (((d % 32) / 8) * 16 + row) * 8 + d % 8;
}
// Same for a V tile. head_dim 128: load j of lane l = (row/4)*16 + d%16 holds tokens
// 4*(l/16) .. +3 of dim 32j + l%16, then of dim 32j + 16 + l%16: the A operands of two
// 16x16x16 products over tokens (V transposed).
__host__ __device__ __forceinline__ uint32_t kv_v_elem(uint32_t head_dim, uint32_t row, uint32_t d) {
  if (head_dim != 128) return row * head_dim + d;
  const uint32_t slab = d / 16, n = d % 16;
  return (slab / 2) * 512 + ((row / 4) * 16 + n) * 8 + (slab % 2) * 4 + row % 4;
}

// One sequence of a batch launch: the cache a token row belongs to and its position there.
struct AttnSeq {
  uint16_t *k_cache, *v_cache;
  const uint32_t *table;
  uint32_t block_count, position;
};

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
  // Decode step kernel: the splits' partials as (f32 value, tag) 8-byte words, [heads][splits][head_dim + 2]
  // (accumulators, then m and l), all tags zero between launches (attn_step_workspace_bytes)
  uint64_t *part_tagged;
  float *out_f32;              // optional [heads*hd]
  uint16_t *out16;             // [heads*hd]
  uint32_t heads, kv_heads, head_dim, layer, block_count, splits;
  float eps;
  const uint32_t *cursor;      // device position, or null -> `position`
  uint32_t position, max_steps, append;
  uint64_t *trace;             // tuning aid: [32] device timestamps of selected workgroups' stages, or null
  // A block of `tokens` consecutive positions in one launch (grid z; 0 or 1 = a single token).
  // Token z works at position + z (the cursor is not used then) with its own q/k/v, output, rotation
  // table and split workspace: the strides below are added z times.
  uint32_t tokens;
  uint32_t qkv_token_stride;   // f32 elements between tokens' q|k|v
  // Batches of sequences only: qkv_slices = 2..4 says that `qkv` holds that many partial sums of every value,
  // qkv_slice_stride f32 elements apart (the K slices of the projection, as its kernel leaves them), and the launch
  // adds them in slice order as it reads them - what the projection's own slice-adding launch would have written.
  uint32_t qkv_slices, qkv_slice_stride;
  uint32_t out_token_stride;   // elements between tokens' outputs (out16 and out_f32)
  uint32_t rope_token_stride;  // f32 elements between tokens' cos|sin tables
  uint64_t ws_token_stride;    // bytes between tokens' split workspaces (attn_workspace_bytes)
  // A batch of sequences instead of consecutive positions of one: token z belongs to seqs[z] (device
  // memory, `tokens` entries), which replaces k_cache, v_cache, table, block_count and the position.
  // Applies to z = 0 as well, and to a block of one token. With append = 1 every sequence's new row
  // is written to its cache by the launch itself.
  const AttnSeq *seqs;
  // Block launches only: != 0 writes out16 in the multi-row GEMM's operand order (gemm_x_packed_index)
  // with this many token tiles, instead of [token][heads * head_dim] rows.
  uint32_t out_packed_tiles;
  // Decode step only, optional: this step's split plan (attn_plan_fill), written once per step for
  // all layers - position, split geometry and every wave's first physical blocks - so that a launch
  // reaches its tile requests through one scalar read instead of position -> block table -> tiles.
  // Valid for launches with `splits` = the plan's split factor and 8 waves per workgroup.
  const uint32_t *plan;
  // Decode step only: up to this many blocks in use, one split takes them all (attn_split_geometry). 0: never.
  uint32_t single_split_blocks;
  // Decode step only, the splits' merge. A partial is valid for the launch whose tag it carries: the tag is made
  // of the launch's sequence number on this workspace - the plan's step number, or `launch_seq` without a plan -
  // and the layer, so a word that a late or earlier launch left behind can never be taken for this launch's.
  uint32_t launch_seq;
  // A merge gives up after this many polls of the words it waits for (0 = kAttnMergeSpinLimit), sets *fault
  // (optional device word, never cleared by a kernel) and leaves NaN in the outputs it feeds.
  uint32_t merge_spin_limit;
  uint32_t *fault;
  // Test hook: 1 + the index of a split that keeps its partial to itself (0 = none), so that the bounded wait of
  // the merges that need it can be seen to end; every kernel still exits normally.
  uint32_t withhold_split;
};
constexpr uint32_t kAttnMergeSpinLimit = 1u << 20;
// Tag of the partials of launch `seq` (never 0, the cleared state): distinct for 2^23 consecutive steps of up
// to 256 layers; the words are cleared after every merge and when a sequence starts as well.
__host__ __device__ __forceinline__ uint32_t attn_launch_tag(uint32_t seq, uint32_t layer) {
  return ((seq * 256u + (layer & 255u)) << 1) | 1u;
}
// The step kernel's merges need every active split of a kv head on the machine at once (a merging workgroup
// holds its CU while it polls), one 8-wave workgroup per CU: the largest split factor a launch may use there.
uint32_t attn_resident_splits(uint32_t kv_heads);

// ---- per-step split plan of the decode attention ---------------------------------------------
// words [0..7]: position, blocks, blocks per split, active splits, step number (the caller's), 3 spare;
// then one 8-word entry per (split, wave): tiles of the wave, its first block, the physical blocks
// of its first four tiles (clamped), 2 spare.
constexpr uint32_t kAttnPlanHeader = 8, kAttnPlanEntry = 8, kAttnPlanWaves = 8;
__host__ __device__ __forceinline__ uint64_t attn_plan_bytes(uint32_t splits) {
  return (kAttnPlanHeader + static_cast<uint64_t>(splits) * kAttnPlanWaves * kAttnPlanEntry) * sizeof(uint32_t);
}
// Split geometry shared by the kernel and the plan: a split takes ceil(blocks / splits) blocks - or all of
// them while the context is short (single_blocks, 0 = never): the exchange between splits costs about 3 us
// whatever the context, and up to some 300 keys one workgroup per kv head has read its keys before that
// (measured on the Qwen3-8B head shape: 64 keys 4.8 us against 12.7, 256 keys 6.5 against 8.2, 512 keys 10.0
// against 8.0).
constexpr uint32_t kAttnSingleSplitBlocks = 20;
__host__ __device__ __forceinline__ void attn_split_geometry(uint32_t pos, uint32_t splits, uint32_t single_blocks,
                                                             uint32_t &nblk, uint32_t &bps, uint32_t &active) {
  nblk = (pos + 1 + kKvBlockTokens - 1) / kKvBlockTokens;
  bps = nblk <= single_blocks ? nblk : (nblk + splits - 1) / splits;
  active = (nblk + bps - 1) / bps;
}
// One thread per (split, wave) entry (`entry` < splits * 8); entry 0 also writes the header.
__device__ __forceinline__ void attn_plan_fill(uint32_t *plan, const uint32_t *table, uint32_t pos, uint32_t splits,
                                               uint32_t single_blocks, uint32_t entry, uint32_t step_number) {
  uint32_t nblk, bps, active;
  attn_split_geometry(pos, splits, single_blocks, nblk, bps, active);
  if (entry == 0) {
    plan[0] = pos;
    plan[1] = nblk;
    plan[2] = bps;
    plan[3] = active;
    plan[4] = step_number;
  }
  const uint32_t split = entry / kAttnPlanWaves, wave = entry % kAttnPlanWaves;
  const uint32_t b0 = split * bps, b1 = min(nblk, b0 + bps), first = b0 + wave;
  uint32_t *e = plan + kAttnPlanHeader + entry * kAttnPlanEntry;
  e[0] = first < b1 ? (b1 - first + kAttnPlanWaves - 1) / kAttnPlanWaves : 0u;
  e[1] = first;
  for (uint32_t f = 0; f < 4; ++f) e[2 + f] = table[min(first + f * kAttnPlanWaves, nblk - 1)];
}

// Index of output element e (= head * head_dim + dim) behind a token's out16 base.
__host__ __device__ __forceinline__ uint32_t attn_out_elem(const AttnParams &p, uint32_t e) {
  return p.out_packed_tiles != 0 ? (e / 32u) * p.out_packed_tiles * 512u + ((e % 32u) / 8u) * 128u + e % 8u : e;
}
// Offset of token z's out16 base.
__host__ __device__ __forceinline__ uint64_t attn_out_token(const AttnParams &p, uint32_t z) {
  return p.out_packed_tiles != 0 ? static_cast<uint64_t>(z / 16u) * 512u + (z % 16u) * 8u
                                 : static_cast<uint64_t>(z) * p.out_token_stride;
}

// Split-KV factor. The matrix-core kernel keeps one 8-wave workgroup per CU, so kv_heads x splits
// stays within the 256 CUs (a second round of workgroups costs more than the shorter tile loops
// save); within that, more splits mean fewer 16-token tiles per wave in a row.
inline uint32_t attn_default_splits(uint32_t kv_heads, uint32_t block_count) {
  uint32_t splits = attn_resident_splits(kv_heads);
  if (splits > kAttnMaxSplits) splits = kAttnMaxSplits;
  if (splits > block_count) splits = block_count;
  return splits == 0 ? 1 : splits;
}
uint64_t attn_workspace_bytes(uint32_t heads, uint32_t head_dim);
// Bytes of AttnParams::part_tagged (head_dim 128), zero-initialised once.
uint64_t attn_step_workspace_bytes(uint32_t heads);
// Carves part_acc/part_m/part_l/counters out of a workspace of attn_workspace_bytes().
void attn_bind_workspace(AttnParams &p, void *workspace);
hipError_t launch_attn_decode(uint32_t dtype, const AttnParams &p, hipStream_t stream);

// Prompt block: rounds and writes the K and V rows of `tokens` consecutive positions
// (position .. position + tokens - 1) into the cache - bias, per-head RMSNorm (k_norm) and RoPE
// as in the decode kernel - so that a following launch_attn_decode with append = 0 and the same
// token block finds every row of the block in place. head_dim 128 only. Uses qkv, k_norm, k_bias,
// v_bias, the caches and table, rope_freq / rope_cs and the token strides of `p`.
hipError_t launch_kv_publish_rows(uint32_t dtype, const AttnParams &p, hipStream_t stream);

// Attention of a prompt block with the K/V tiles of the prefix shared by the block's tokens
// (attn_prompt.hip): same inputs and outputs as launch_attn_decode for a block (tokens consecutive
// positions from `position`, rows already in the cache, append = 0, per-token strides, per-token split
// workspaces, rotation tables per token row), head_dim 128 and GQA factor 1/2/4/8 only.
// p.splits = 0 lets the launcher choose.
hipError_t launch_attn_prompt(uint32_t dtype, const AttnParams &p, hipStream_t stream);

}  // namespace nv
