// Fused decode attention for one new token:
//   bias -> per-head RMSNorm (q_norm/k_norm) -> half-split RoPE -> K/V rounded to
//   16 bits and appended to the paged cache -> split-KV online-softmax attention
//   over keys 0..pos -> merge of the splits -> 16-bit attention output.
// Reference: hf_layer_qkv_prepare_kernel / chunk kernels / reduce kernel
// (kernels.cu:287-555, attention_kernels.cu:263-760), per_head_rms_norm
// (precision/block/ops.rs:52-73), apply_rotary_to_heads (common/rope.rs:54-79),
// exact_blockwise_attention_into (attention/exact/run.rs:13-127).
//
// gfx950 mapping of the fast path (head_dim 128, G = heads/kv_heads in {1,2,4,8}):
//   grid (kv_heads, splits), 8 waves per workgroup; a wave owns whole 16-token KV
//   tiles of its workgroup's token range and runs q.K^T and P.V on the matrix cores
//   (details at attn_fast_body). The cache keeps each tile in matrix-operand order,
//   so a tile is eight coalesced 1 KiB loads straight into operand registers; two tiles
//   are in flight per wave. LDS only carries q, the new K/V row and the cross-wave
//   merge. The last workgroup to finish a kv head merges its split partials (arrival
//   counter; nobody waits), so a layer needs no separate reduce launch.
#include <stdlib.h>

#include "attn_decode.cuh"
#include "attn_tile.cuh"

namespace nv {

namespace {

using namespace attn;

// Parameters of token z of a block launch.
__device__ __forceinline__ void token_view(AttnParams &p, uint32_t z) {
  if (p.seqs != nullptr) {
    const AttnSeq seq = p.seqs[z];
    p.k_cache = seq.k_cache;
    p.v_cache = seq.v_cache;
    p.table = seq.table;
    p.block_count = seq.block_count;
    p.position = seq.position;
  } else {
    p.position += z;
  }
  p.qkv += static_cast<uint64_t>(z) * p.qkv_token_stride;
  p.out16 += attn_out_token(p, z);
  if (p.out_f32 != nullptr) p.out_f32 += static_cast<uint64_t>(z) * p.out_token_stride;
  if (p.rope_cs != nullptr) p.rope_cs += static_cast<uint64_t>(z) * p.rope_token_stride;
  const uint64_t ws = z * p.ws_token_stride;
  p.part_acc = reinterpret_cast<float *>(reinterpret_cast<char *>(p.part_acc) + ws);
  p.part_m = reinterpret_cast<float *>(reinterpret_cast<char *>(p.part_m) + ws);
  p.part_l = reinterpret_cast<float *>(reinterpret_cast<char *>(p.part_l) + ws);
  p.counters = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(p.counters) + ws);
}

// K and V rows of a prompt block into the cache: grid (kv head, token), two waves (key, value).
template <uint32_t DT>
__global__ __launch_bounds__(2 * kWave) void kv_publish_rows_kernel(AttnParams p) {
  __shared__ __align__(16) uint16_t row16[2][kHD];
  const uint32_t kvh = blockIdx.x, z = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  uint32_t pos = p.position + z;
  if (p.seqs != nullptr) {
    const AttnSeq seq = p.seqs[z];
    p.k_cache = seq.k_cache;
    p.v_cache = seq.v_cache;
    p.table = seq.table;
    p.block_count = seq.block_count;
    pos = seq.position;
  }
  const uint32_t A = p.heads * kHD, KV = p.kv_heads * kHD;
  const float *qkv = p.qkv + static_cast<uint64_t>(z) * p.qkv_token_stride;
  const float *rope_cs = p.rope_cs != nullptr ? p.rope_cs + static_cast<uint64_t>(z) * p.rope_token_stride : nullptr;
  const uint32_t off = (wave == 0 ? A : A + KV) + kvh * kHD;
  const uint16_t *bias = wave == 0 ? p.k_bias : p.v_bias;
  prep_head128<DT>(qkv[off + lane], qkv[off + lane + 64], bias ? bias + kvh * kHD : nullptr, wave == 0 ? p.k_norm : nullptr,
                   wave == 0 ? p.rope_freq : nullptr, rope_cs, pos, p.eps, lane, nullptr, row16[wave]);
  __syncthreads();
  const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, p.table[pos / kKvBlockTokens], kvh);
  const uint32_t row = pos % kKvBlockTokens;
  if (wave == 0) {
    if (lane < 16)  // K: 16 pieces of 8 consecutive dims
      *reinterpret_cast<uint4 *>(p.k_cache + tile + kv_k_elem(kHD, row, lane * 8)) =
          *reinterpret_cast<const uint4 *>(row16[0] + lane * 8);
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // V: one 16-bit element per dim
      const uint32_t d = lane + i * kWave;
      p.v_cache[tile + kv_v_elem(kHD, row, d)] = row16[1][d];
    }
  }
}

// Launch of the matrix-core attention body (attn_fast_body) for token blocks and batch steps: grid (kv_heads,
// splits, tokens); the lean variant, two workgroups per CU.
template <uint32_t DT, int G, int W>
__global__ __launch_bounds__(W *kWave, W / 2) void attn_block_kernel(AttnParams p) {
  __shared__ AttnShared<G, W> sh;
  if (blockIdx.z != 0 || p.seqs != nullptr) token_view(p, blockIdx.z);
  const RawHeads<G, W> raw = attn_request_raw<G, W>(p, blockIdx.x);
  attn_fast_body<DT, G, W, 1>(p, p.position, blockIdx.x, blockIdx.y, gridDim.y, sh, raw);
}

// ---------------------------------------------------------------------------------------------
// The decode step's launch: one token, grid (kv_heads, splits), 8 waves, G = 1, 2, 4 or 8 query heads per
// kv head. Same arithmetic as attn_fast_body (same tile step, same merges); what differs is the order
// in which a wave asks for things, because at decode sizes - a wave owns two or three 8 KiB tiles of an
// 8k-token context - the launch is one burst of requests and a chain of latencies, not a stream:
//   1. the head inputs (raw q / k / v, bias, norm weights, rotation) are requested first but NOT
//      awaited; 2. position and block-table entries come through the scalar path; 3. the wave's tiles
//      (up to four) are requested right behind the inputs; 4. the wave waits for the inputs only:
//      loads return in request order, so "at most 8 x tiles requests outstanding" means the inputs have
//      arrived while every tile is still in flight. All of these requests are issued by hand with
//      explicit outstanding-request counts: a count the compiler derives stops at the first
//      conditional request and falls back to waiting for everything.
//   5. head preparation (bias, RMSNorm, RoPE, scaling, hi/lo split) runs under the tiles' flight; the
//      query operand of the first product is written to LDS once per workgroup, as 16-bit hi and lo
//      rows, and every wave reads its operand registers back with four 16-byte LDS reads.
//   6. tiles are consumed in request order with counted waits; a wave with more than four tiles
//      re-requests into the registers it has just consumed. A wait is a bare instruction chosen by a
//      scalar branch on the number of tiles requested behind the awaited one; the statement that hands
//      the awaited registers to the compiler comes after the branch has joined, so nothing that reads
//      them (not even a register copy) can precede the wait.
// A split takes ceil(blocks / splits) blocks - not rounded up to a multiple of the wave count: at 8k
// tokens that keeps 31 of 32 splits busy instead of 22 - and a wave without a tile simply contributes
// nothing to the merge.
// ---------------------------------------------------------------------------------------------
// Loads through the scalar path (position, block-table entries: the same for every lane, and read-only
// while the launch runs). The compiler takes the vector path for them - it cannot prove that the
// launch does not write there - and a vector load would have to be awaited with everything requested
// before it.
__device__ __forceinline__ uint32_t sload(const uint32_t *ptr) {
  uint32_t v;
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(ptr) : "memory");
  return v;
}
__device__ __forceinline__ void sload4(const uint32_t *p0, const uint32_t *p1, const uint32_t *p2, const uint32_t *p3,
                                       uint32_t (&v)[4]) {
  asm volatile(
      "s_load_dword %0, %4, 0x0\n\ts_load_dword %1, %5, 0x0\n\ts_load_dword %2, %6, 0x0\n\ts_load_dword %3, %7, 0x0\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(v[0]), "=&s"(v[1]), "=&s"(v[2]), "=&s"(v[3])
      : "s"(p0), "s"(p1), "s"(p2), "s"(p3)
      : "memory");
}

// The splits' partials of the step kernel, as (f32 value, tag) words. One (head, split) record is cut
// into kStepParts parts of 32 dims, each followed by its own copy of the split's m and l, so that a part
// is read - and its tags cleared - by exactly one merging workgroup.
constexpr uint32_t kStepParts = 4, kStepPartDims = kHD / kStepParts, kStepPartWords = kStepPartDims + 2;
constexpr uint32_t kStepRecord = kStepParts * kStepPartWords;
// One part (32 dims of one head) merged by one workgroup of 512 threads. Thread (dl = t % 32,
// q = t / 32) takes the splits q, q + 16, q + 32, q + 48: it polls their accumulator word and their m
// and l words until every tag is up and folds them in split order; the two groups of a wave meet by a lane
// exchange and the eight waves in LDS, in wave order - a fixed order, whatever the arrival order was. A CU sustains only a few hundred
// device-coherent cache lines per microsecond, which is why a head is spread over several merging
// workgroups. Last of all every word that was read gets its tag cleared for the next launch (launches
// are ordered by the stream). A wait that runs out (a split that never stored: cannot happen on a
// healthy device with every split resident, which the launcher sees to) ends after the launch's spin limit: the
// fault word is set - the session hands it out with the token, the operator entry point through its status call -
// and the outputs it feeds become NaN. A word counts only with this launch's tag, so a partial that lands after
// its merge gave up is never taken for a later launch's.
template <uint32_t DT, int G>
__device__ __forceinline__ void merge_part_tagged(const AttnParams &p, uint32_t kvh, uint32_t g, uint32_t part, uint32_t S,
                                                  uint32_t active, float *lds_o, float *lds_m, float *lds_l, bool first_part,
                                                  uint32_t tag) {
  const uint32_t spin_limit = p.merge_spin_limit != 0 ? p.merge_spin_limit : kAttnMergeSpinLimit;
  constexpr uint32_t kGroups = 16, kPer = kAttnMaxSplits / kGroups;  // 4 splits per thread at most
  const uint32_t h = kvh * G + g;
  uint64_t *rec = p.part_tagged + static_cast<uint64_t>(h) * S * kStepRecord + part * kStepPartWords;
  const uint32_t dl = threadIdx.x % kStepPartDims, q = threadIdx.x / kStepPartDims;
  uint64_t av[kPer], mv[kPer], lv[kPer];
  uint32_t spins = 0;
  for (;;) {
    bool ok = true;
#pragma unroll
    for (uint32_t i = 0; i < kPer; ++i) {
      // unconditional loads (index clamped): a load under a branch would serialise the round
      const uint64_t *r = rec + static_cast<uint64_t>(min(q + i * kGroups, active - 1)) * kStepRecord;
      av[i] = load_tagged(r + dl);
      mv[i] = load_tagged(r + kStepPartDims);
      lv[i] = load_tagged(r + kStepPartDims + 1);
    }
#pragma unroll
    for (uint32_t i = 0; i < kPer; ++i)  // (a clamped repeat of the last split belongs to another thread: not awaited)
      if (q + i * kGroups < active) ok = ok && tag_is(av[i], tag) && tag_is(mv[i], tag) && tag_is(lv[i], tag);
    if (__all(ok) || ++spins > spin_limit) break;
  }
  const bool gave_up = spins > spin_limit;  // per wave; poisons the outputs this wave contributes to
  if (gave_up && p.fault != nullptr && (threadIdx.x & (kWave - 1)) == 0)
    __hip_atomic_store(p.fault, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  float M = -INFINITY, L = 0.0f, o = 0.0f;
#pragma unroll
  for (uint32_t i = 0; i < kPer; ++i)
    if (q + i * kGroups < active) M = fmaxf(M, tag_value(mv[i]));
#pragma unroll
  for (uint32_t i = 0; i < kPer; ++i) {
    if (q + i * kGroups < active) {
      const float f = attn_exp2(tag_value(mv[i]) - M);  // every active split saw a key: its m is finite
      L = fmaf(tag_value(lv[i]), f, L);
      o = fmaf(tag_value(av[i]), f, o);
    }
  }
  // the two groups of a wave (its lanes 0-31 and 32-63) meet by a lane exchange, the even group's sum first;
  // the eight waves meet in LDS (arrays of their own: no barrier before they are written, except between parts)
  {
    const float Mo = __shfl_xor(M, static_cast<int>(kStepPartDims), kWave), Lo = __shfl_xor(L, static_cast<int>(kStepPartDims), kWave),
                oo = __shfl_xor(o, static_cast<int>(kStepPartDims), kWave);
    const bool even = (q & 1u) == 0;
    const float Ma = even ? M : Mo, La = even ? L : Lo, oa = even ? o : oo;
    const float Mb = even ? Mo : M, Lb = even ? Lo : L, ob = even ? oo : o;
    const float Mw = fmaxf(Ma, Mb);
    const float fa = Ma > -INFINITY ? attn_exp2(Ma - Mw) : 0.0f, fb = Mb > -INFINITY ? attn_exp2(Mb - Mw) : 0.0f;   // a group without a split
    M = Mw;
    L = fmaf(Lb, fb, La * fa);
    o = fmaf(ob, fb, oa * fa);
  }
  constexpr uint32_t kWaves = kGroups / 2;
  const uint32_t w = q / 2;
  if (!first_part) __syncthreads();   // the previous part's last reads
  if ((q & 1u) == 0) {
    lds_o[w * kStepPartDims + dl] = gave_up ? NAN : o;
    if (dl == 0) {
      lds_m[w] = M;
      lds_l[w] = L;
    }
  }
  __syncthreads();
  if (q == 0) {
    float Mt = -INFINITY;
#pragma unroll
    for (uint32_t k = 0; k < kWaves; ++k) Mt = fmaxf(Mt, lds_m[k]);
    float Lt = 0.0f, ot = 0.0f;
#pragma unroll
    for (uint32_t k = 0; k < kWaves; ++k) {
      const float f = lds_m[k] > -INFINITY ? attn_exp2(lds_m[k] - Mt) : 0.0f;  // a wave without a split
      Lt = fmaf(lds_l[k], f, Lt);
      ot = fmaf(lds_o[k * kStepPartDims + dl], f, ot);
    }
    if (Lt > 0.0f && isfinite(Lt)) ot /= Lt;
    const uint32_t e = h * kHD + part * kStepPartDims + dl;
    if (p.out_f32 != nullptr) p.out_f32[e] = ot;
    p.out16[attn_out_elem(p, e)] = enc16<DT>(ot);
  }
  // The words are left as they are: they carry this launch's tag, which no later launch on this workspace uses
  // (attn_launch_tag), so nothing has to be cleared behind the reads.
}

typedef uint32_t u32x8_t __attribute__((ext_vector_type(8)));
__device__ __forceinline__ void sload8x2(const uint32_t *a, const uint32_t *b, u32x8_t &va, u32x8_t &vb) {
  asm volatile("s_load_dwordx8 %0, %2, 0x0\n\ts_load_dwordx8 %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(va), "=&s"(vb)
               : "s"(a), "s"(b)
               : "memory");
}

template <int G>
struct StepShared {
  static constexpr int kRow = kHD + 8;     // 272-byte rows: the operand reads of a lane group spread over the banks
  alignas(16) uint16_t qhl[2 * G][kRow];   // Qx columns: rows 0..G-1 the hi halves of the scaled query heads, G..2G-1 the lo halves
  alignas(16) uint16_t knew[kHD];
  alignas(16) uint16_t vnew[kHD];
  float wm[8][G], wl[8][G];
  alignas(16) float wacc[8][G][kHD];
  float merge_o[8][32], merge_m[8], merge_l[8];   // the splits' merge: one entry per wave
  uint32_t is_last;
};

#define NV_AT_LD32(DST, PTR, OFF) asm volatile("global_load_dword %0, %1, off offset:" #OFF : "=v"(DST) : "v"(PTR) : "memory")
#define NV_AT_LD16(DST, PTR, OFF) asm volatile("global_load_ushort %0, %1, off offset:" #OFF : "=v"(DST) : "v"(PTR) : "memory")
#define NV_AT_TILE_LOAD(F, PHYS)                                                                                 \
  do {                                                                                                           \
    const uint64_t t_ = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, (PHYS), kvh) + lane * 8;          \
    const uint16_t *kp_ = p.k_cache + t_, *vp_ = p.v_cache + t_;                                                  \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(kr[F][0]) : "v"(kp_) : "memory");                    \
    asm volatile("global_load_dwordx4 %0, %1, off offset:1024 nt" : "=v"(kr[F][1]) : "v"(kp_) : "memory");        \
    asm volatile("global_load_dwordx4 %0, %1, off offset:2048 nt" : "=v"(kr[F][2]) : "v"(kp_) : "memory");        \
    asm volatile("global_load_dwordx4 %0, %1, off offset:3072 nt" : "=v"(kr[F][3]) : "v"(kp_) : "memory");        \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(vr[F][0]) : "v"(vp_) : "memory");                    \
    asm volatile("global_load_dwordx4 %0, %1, off offset:1024 nt" : "=v"(vr[F][1]) : "v"(vp_) : "memory");        \
    asm volatile("global_load_dwordx4 %0, %1, off offset:2048 nt" : "=v"(vr[F][2]) : "v"(vp_) : "memory");        \
    asm volatile("global_load_dwordx4 %0, %1, off offset:3072 nt" : "=v"(vr[F][3]) : "v"(vp_) : "memory");        \
  } while (0)
// Waits until at most 8 * TILES of this wave's requests are outstanding (TILES uniform, 0..4).
#define NV_AT_WAIT_BEHIND(TILES)                                                \
  do {                                                                          \
    switch (TILES) {                                                            \
      case 0u: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;          \
      case 1u: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;          \
      case 2u: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;         \
      case 3u: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;         \
      default: asm volatile("s_waitcnt vmcnt(32)" ::: "memory"); break;         \
    }                                                                           \
  } while (0)
// Hands registers that a wait has just covered to the compiler: every later use depends on this statement.
#define NV_AT_TAKE_INPUTS()                                                                                        \
  asm volatile(""                                                                                                  \
               : "+v"(qx0), "+v"(qx1), "+v"(ex0), "+v"(ex1), "+v"(qb0), "+v"(qb1), "+v"(eb0), "+v"(eb1), "+v"(qg0), \
                 "+v"(qg1), "+v"(kg0), "+v"(kg1), "+v"(ra), "+v"(rb))
#define NV_AT_TAKE_TILE(F)                                                                                         \
  asm volatile(""                                                                                                  \
               : "+v"(kr[F][0]), "+v"(kr[F][1]), "+v"(kr[F][2]), "+v"(kr[F][3]), "+v"(vr[F][0]), "+v"(vr[F][1]),   \
                 "+v"(vr[F][2]), "+v"(vr[F][3]))
#define NV_AT_U4(V) make_uint4((V).x, (V).y, (V).z, (V).w)

template <uint32_t DT, int G>
__global__ __launch_bounds__(8 * kWave) void attn_step_kernel(AttnParams p) {
  constexpr int W = 8;
  constexpr int kThreads = W * kWave;
  __shared__ StepShared<G> sh;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t kvh = blockIdx.x, split = blockIdx.y, S = gridDim.y;
  const uint32_t A = p.heads * kHD, KV = p.kv_heads * kHD;
  uint64_t *const tr = kvh == 0 && split == 0 ? p.trace : nullptr;
  uint64_t *const trm = kvh == 0 ? p.trace : nullptr;
  link_mark(tr, 7);

  // ---- 1. head inputs, every one of them requested unconditionally (a missing bias / weight / table
  // reads a stand-in address inside the projection vector and is ignored below)
  const bool q_wave = wave < G, key_wave = wave == (G % W), value_wave = wave == ((G + 1) % W);
  const uint32_t qoff = (kvh * G + (q_wave ? wave : 0)) * kHD;
  const uint32_t eoff = (value_wave ? A + KV : A) + kvh * kHD;
  const uint16_t *stand_in = reinterpret_cast<const uint16_t *>(p.qkv);
  const uint16_t *ebias = value_wave ? p.v_bias : p.k_bias;
  const float *qp = p.qkv + qoff + lane, *ep = p.qkv + eoff + lane;
  const uint16_t *qbp = (p.q_bias != nullptr ? p.q_bias + qoff : stand_in) + lane;
  const uint16_t *ebp = (ebias != nullptr ? ebias + kvh * kHD : stand_in) + lane;
  const uint16_t *qgp = (p.q_norm != nullptr ? p.q_norm : stand_in) + lane;
  const uint16_t *kgp = (p.k_norm != nullptr ? p.k_norm : stand_in) + lane;
  const float *rap = (p.rope_cs != nullptr ? p.rope_cs : (p.rope_freq != nullptr ? p.rope_freq : p.qkv)) + lane;
  const float *rbp = p.rope_cs != nullptr ? p.rope_cs + 64 + lane : rap;
  float qx0, qx1, ex0, ex1, ra, rb;
  uint32_t qb0, qb1, eb0, eb1, qg0, qg1, kg0, kg1;
  NV_AT_LD32(qx0, qp, 0);
  NV_AT_LD32(qx1, qp, 256);
  NV_AT_LD32(ex0, ep, 0);
  NV_AT_LD32(ex1, ep, 256);
  NV_AT_LD16(qb0, qbp, 0);
  NV_AT_LD16(qb1, qbp, 128);
  NV_AT_LD16(eb0, ebp, 0);
  NV_AT_LD16(eb1, ebp, 128);
  NV_AT_LD16(qg0, qgp, 0);
  NV_AT_LD16(qg1, qgp, 128);
  NV_AT_LD16(kg0, kgp, 0);
  NV_AT_LD16(kg1, kgp, 128);
  NV_AT_LD32(ra, rap, 0);
  NV_AT_LD32(rb, rbp, 0);

  // ---- 2. position, this split's blocks, this wave's tiles (scalar path)
  uint32_t pos, nblk, bps, active, first, nt, phys[4], launch_seq = p.launch_seq;
  if (p.plan != nullptr) {
    // this step's plan: everything above in one round trip
    u32x8_t head, mine;
    sload8x2(p.plan, p.plan + kAttnPlanHeader + (split * W + wave) * kAttnPlanEntry, head, mine);
    pos = head[0], nblk = head[1], bps = head[2], active = head[3], launch_seq = head[4];
    nt = mine[0], first = mine[1];
    phys[0] = mine[2], phys[1] = mine[3], phys[2] = mine[4], phys[3] = mine[5];
    if (pos >= p.max_steps) return;
  } else {
    pos = p.cursor != nullptr ? sload(p.cursor) : p.position;
    if (p.cursor != nullptr && pos >= p.max_steps) return;
    attn_split_geometry(pos, S, p.single_split_blocks, nblk, bps, active);
    first = split * bps + wave;
    const uint32_t end = min(nblk, split * bps + bps);
    nt = first < end ? (end - first + W - 1) / W : 0u;  // tiles first, first + W, ...
    if (split < active)
      sload4(p.table + min(first, nblk - 1), p.table + min(first + W, nblk - 1), p.table + min(first + 2 * W, nblk - 1),
             p.table + min(first + 3 * W, nblk - 1), phys);
  }
  if (split >= active) return;  // idle splits neither store a partial nor take a ticket
  const uint32_t n_keys = pos + 1;
  const uint32_t b0 = split * bps;
  const uint32_t b1 = min(nblk, b0 + bps);
  const uint32_t new_block = pos / kKvBlockTokens, new_row = pos % kKvBlockTokens;
  const bool owns_new = p.append != 0 && new_block >= b0 && new_block < b1;
  const uint32_t tag = attn_launch_tag(launch_seq, p.layer);

  // ---- 3. the wave's first tile. Only the first: at long contexts the launch is one burst of requests, the
  // memory path fills up, and a wave that goes on requesting sits in its request instructions until the burst
  // has drained enough (3 us at 8k tokens) - with its head inputs long there and its head preparation not
  // started. So: one tile out, the head preparation under its flight, then the rest (the burst takes its
  // 4-5 us either way; what is requested a microsecond later is not served later).
  link_mark(tr, 6);
  u32x4_t kr[4][4], vr[4][4];
  if (nt > 0) NV_AT_TILE_LOAD(0, phys[0]);
  link_mark(tr, 8);

  // ---- 4. the inputs have arrived once at most the first tile's requests are outstanding
  NV_AT_WAIT_BEHIND(min(nt, 1u));
  NV_AT_TAKE_INPUTS();
  link_mark(tr, 14);

  // ---- 5. head preparation under the tiles' flight
  const bool has_rope = p.rope_freq != nullptr;
  float rc = ra, rs = rb;
  if (has_rope && p.rope_cs == nullptr) sincosf(static_cast<float>(pos) / ra, &rs, &rc);
  if (q_wave) {
    float x0 = qx0, x1 = qx1;
    head_values<DT>(x0, x1, p.q_bias != nullptr, dec16<DT>(static_cast<uint16_t>(qb0)), dec16<DT>(static_cast<uint16_t>(qb1)),
                    p.q_norm != nullptr, dec16<DT>(static_cast<uint16_t>(qg0)), dec16<DT>(static_cast<uint16_t>(qg1)),
                    has_rope, rc, rs, p.eps);
    // softmax runs in base 2 on scores scaled by 1/sqrt(d): both folded into the query
    const float scale = kLog2e / sqrtf(static_cast<float>(kHD));
    uint16_t h0, l0, h1, l1;
    split16<DT>(x0 * scale, h0, l0);
    split16<DT>(x1 * scale, h1, l1);
    sh.qhl[wave][lane] = h0;
    sh.qhl[wave][lane + 64] = h1;
    sh.qhl[G + wave][lane] = l0;
    sh.qhl[G + wave][lane + 64] = l1;
  }
  if (owns_new && (key_wave || value_wave)) {
    float x0 = ex0, x1 = ex1;
    const bool norm = key_wave && p.k_norm != nullptr;
    head_values<DT>(x0, x1, ebias != nullptr, dec16<DT>(static_cast<uint16_t>(eb0)), dec16<DT>(static_cast<uint16_t>(eb1)), norm,
                    dec16<DT>(static_cast<uint16_t>(kg0)), dec16<DT>(static_cast<uint16_t>(kg1)), key_wave && has_rope, rc, rs,
                    p.eps);
    uint16_t *row = key_wave ? sh.knew : sh.vnew;
    row[lane] = enc16<DT>(x0);
    row[lane + 64] = enc16<DT>(x1);
  }
  // the wave's other tiles of the first four, behind its own head work and before it waits for the others'
  if (nt > 1) NV_AT_TILE_LOAD(1, phys[1]);
  if (nt > 2) NV_AT_TILE_LOAD(2, phys[2]);
  if (nt > 3) NV_AT_TILE_LOAD(3, phys[3]);
  link_mark(tr, 15);
  __syncthreads();
  link_mark(tr, 9);
  if (owns_new && wave == W - 1) {
    // publish the rounded row to the cache in operand order
    const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, sload(p.table + new_block), kvh);
    if (lane < 16)  // K: 16 pieces of 8 consecutive dims
      *reinterpret_cast<uint4 *>(p.k_cache + tile + kv_k_elem(kHD, new_row, lane * 8)) =
          *reinterpret_cast<const uint4 *>(sh.knew + lane * 8);
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // V: one 16-bit element per dim
      const uint32_t d = lane + i * kWave;
      p.v_cache[tile + kv_v_elem(kHD, new_row, d)] = sh.vnew[d];
    }
  }

  // ---- B operand of the first product: column `col` of Qx for dims j*32 + grp*8 .. +7
  const int col = lane & 15, grp = lane >> 4;
  uint4 qx[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4 v = *reinterpret_cast<const uint4 *>(&sh.qhl[col < 2 * G ? col : 0][j * 32 + grp * 8]);
    qx[j] = col < 2 * G ? v : make_uint4(0u, 0u, 0u, 0u);
  }
  link_mark(tr, 10);

  // ---- 6. tiles in request order
  float m = -INFINITY, l = 0.0f;  // of column `col` (both copies of a head track the same values)
  f32x4_t acc[8];                  // O^T[dims s*16 + grp*4 .. +3][col]
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) acc[s2] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#define NV_AT_STEP(F)                                                                                              \
  do {                                                                                                             \
    const uint32_t t_idx = done + F;                                                                               \
    if (t_idx < nt) {                                                                                              \
      /* tiles requested behind this one and not yet consumed: at most three */                                   \
      NV_AT_WAIT_BEHIND(min(nt - t_idx - 1u, 3u));                                                                 \
      NV_AT_TAKE_TILE(F);                                                                                          \
      uint4 kk[4], vv[4];                                                                                          \
      _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                              \
        kk[j] = NV_AT_U4(kr[F][j]);                                                                                \
        vv[j] = NV_AT_U4(vr[F][j]);                                                                                \
      }                                                                                                            \
      const uint32_t bb = first + t_idx * W;                                                                       \
      attn_tile<DT, G, false>(kk, vv, qx, nullptr, bb, n_keys, col, grp, owns_new && bb == new_block, new_row,     \
                              sh.knew, sh.vnew, m, l, acc);                                                        \
      if (t_idx + 4u < nt) NV_AT_TILE_LOAD(F, sload(p.table + first + (t_idx + 4u) * W));                          \
    }                                                                                                              \
  } while (0)
  for (uint32_t done = 0; done < nt; done += 4) {
    NV_AT_STEP(0);
    NV_AT_STEP(1);
    NV_AT_STEP(2);
    NV_AT_STEP(3);
  }
#undef NV_AT_STEP
  link_mark(tr, 11);

  // ---- 7. wave result: tokens of the four lane groups, then hi + lo columns; then the W waves
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) {
    float4 o;
    o.x = acc[s2][0] + row_shl<G>(acc[s2][0]);
    o.y = acc[s2][1] + row_shl<G>(acc[s2][1]);
    o.z = acc[s2][2] + row_shl<G>(acc[s2][2]);
    o.w = acc[s2][3] + row_shl<G>(acc[s2][3]);
    if (col < G) *reinterpret_cast<float4 *>(&sh.wacc[wave][col][s2 * 16 + grp * 4]) = o;
  }
  if (lane < G) {
    sh.wm[wave][lane] = m;
    sh.wl[wave][lane] = l;
  }
  __syncthreads();
  // every thread owns output elements (g, d): the W waves' scale factors are recomputed per thread
  // (eight exponentials) instead of being shared through another barrier
  for (int e = threadIdx.x; e < G * kHD; e += kThreads) {
    const int g = e / kHD, d = e % kHD;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < W; ++w) M = fmaxf(M, sh.wm[w][g]);
    float L = 0.0f, o = 0.0f;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const float mw = sh.wm[w][g];
      const float f = mw > -INFINITY ? attn_exp2(mw - M) : 0.0f;  // a wave without a tile contributes nothing
      L = fmaf(sh.wl[w][g], f, L);
      o = fmaf(sh.wacc[w][g][d], f, o);
    }
    const uint32_t h = kvh * G + g;
    if (active == 1) {
      // a single split holds every key: this is the final result, nothing to exchange
      if (L > 0.0f && isfinite(L)) o /= L;
      if (p.out_f32 != nullptr) p.out_f32[h * kHD + d] = o;
      p.out16[attn_out_elem(p, h * kHD + d)] = enc16<DT>(o);
    } else {
      // The partial leaves as tagged words through device-coherent stores (written through, no cache
      // flush, nobody waits for them to be performed).
      const uint32_t part = d / kStepPartDims, dl = d % kStepPartDims;
      uint64_t *rec = p.part_tagged + (static_cast<uint64_t>(h) * S + split) * kStepRecord + part * kStepPartWords;
      if (p.withhold_split != split + 1u) {
        store_tagged(rec + dl, o, tag);
        if (dl == 0) {
          store_tagged(rec + kStepPartDims, M, tag);
          store_tagged(rec + kStepPartDims + 1, L, tag);
        }
      }
    }
  }
  if (active == 1) return;
  link_mark(tr, 12);
  // ---- 8. the splits' merge: part j = (head g, 32 dims) of this kv head is merged by split j (mod the
  // active splits), which polls the other splits' words until every tag is up - two memory round
  // trips after the slowest split's tiles (store, then the poll that finds it), where a ticket taken
  // after the stores have been performed and a merge by the last arriver needed four.
  for (uint32_t j = split; j < G * kStepParts; j += active) {
    link_mark(trm, 16);
    merge_part_tagged<DT, G>(p, kvh, j % G, j / G, S, active, sh.merge_o[0], sh.merge_m, sh.merge_l, j == split, tag);
    link_mark(trm, 17);
  }
}
#undef NV_AT_LD32
#undef NV_AT_LD16
#undef NV_AT_TILE_LOAD
#undef NV_AT_WAIT_BEHIND
#undef NV_AT_TAKE_INPUTS
#undef NV_AT_TAKE_TILE
#undef NV_AT_U4

// Any head_dim (even when RoPE is on) / any group size: one workgroup per query
// head, waves stride over tokens, lanes over dims. Used for shapes the fast path
// does not cover (the tiny known-answer models).
template <uint32_t DT>
__global__ __launch_bounds__(kBlock) void attn_generic_kernel(AttnParams p) {
  extern __shared__ __align__(16) float sm[];
  __shared__ float red[kWavesPerBlock];
  __shared__ float wm[kWavesPerBlock], wl[kWavesPerBlock];
  const uint32_t hd = p.head_dim, half = hd / 2;
  float *q = sm;                 // [hd]
  float *kn = sm + hd;           // [hd] rounded new key
  float *vn = sm + 2 * hd;       // [hd] rounded new value
  float *wacc = sm + 3 * hd;     // [waves][hd]

  const uint32_t pos = p.cursor != nullptr ? *p.cursor : p.position;
  if (p.cursor != nullptr && pos >= p.max_steps) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t h = blockIdx.x, group = p.heads / p.kv_heads, kvh = h / group;
  const uint32_t A = p.heads * hd, KV = p.kv_heads * hd;
  const uint32_t n_keys = pos + 1;

  // q: bias -> per-head norm -> RoPE
  float ss = 0.0f;
  for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
    float v = p.qkv[h * hd + d];
    if (p.q_bias) v += dec16<DT>(p.q_bias[h * hd + d]);
    q[d] = v;
    ss += v * v;
  }
  ss = block_sum(ss, red);
  if (p.q_norm) {
    const float sc = 1.0f / sqrtf(ss / static_cast<float>(hd) + p.eps);
    for (uint32_t d = threadIdx.x; d < hd; d += kBlock) q[d] *= sc * dec16<DT>(p.q_norm[d]);
  }
  __syncthreads();
  if (p.rope_freq) {
    for (uint32_t i = threadIdx.x; i < half; i += kBlock) {
      const float angle = static_cast<float>(pos) / p.rope_freq[i];
      float s, c;
      sincosf(angle, &s, &c);
      const float a = q[i], b = q[i + half];
      q[i] = a * c - b * s;
      q[i + half] = b * c + a * s;
    }
  }
  if (p.append) {
    float ks = 0.0f;
    for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
      float kv = p.qkv[A + kvh * hd + d];
      if (p.k_bias) kv += dec16<DT>(p.k_bias[kvh * hd + d]);
      kn[d] = kv;
      ks += kv * kv;
      float vv = p.qkv[A + KV + kvh * hd + d];
      if (p.v_bias) vv += dec16<DT>(p.v_bias[kvh * hd + d]);
      vn[d] = vv;
    }
    ks = block_sum(ks, red);
    if (p.k_norm) {
      const float sc = 1.0f / sqrtf(ks / static_cast<float>(hd) + p.eps);
      for (uint32_t d = threadIdx.x; d < hd; d += kBlock) kn[d] *= sc * dec16<DT>(p.k_norm[d]);
    }
    __syncthreads();
    if (p.rope_freq) {
      for (uint32_t i = threadIdx.x; i < half; i += kBlock) {
        const float angle = static_cast<float>(pos) / p.rope_freq[i];
        float s, c;
        sincosf(angle, &s, &c);
        const float a = kn[i], b = kn[i + half];
        kn[i] = a * c - b * s;
        kn[i + half] = b * c + a * s;
      }
    }
    __syncthreads();
    const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, hd, p.layer,
                                         p.table[pos / kKvBlockTokens], kvh);
    const uint32_t prow = pos % kKvBlockTokens;
    for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
      const uint16_t k16 = enc16<DT>(kn[d]), v16 = enc16<DT>(vn[d]);
      if (h % group == 0) {
        p.k_cache[tile + kv_k_elem(hd, prow, d)] = k16;
        p.v_cache[tile + kv_v_elem(hd, prow, d)] = v16;
      }
      kn[d] = dec16<DT>(k16);
      vn[d] = dec16<DT>(v16);
    }
  }
  __syncthreads();

  constexpr int kMaxPerLane = 8;  // head_dim <= 512
  float acc[kMaxPerLane];
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) acc[j] = 0.0f;
  float m = -INFINITY, l = 0.0f;
  const float scale = 1.0f / sqrtf(static_cast<float>(hd));
  for (uint32_t t = wave; t < n_keys; t += kWavesPerBlock) {
    const bool fresh = p.append && t == pos;
    const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, hd, p.layer,
                                         p.table[t / kKvBlockTokens], kvh);
    const uint32_t trow = t % kKvBlockTokens;
    float partial = 0.0f;
    for (uint32_t d = lane; d < hd; d += kWave)
      partial = fmaf(q[d], fresh ? kn[d] : dec16<DT>(p.k_cache[tile + kv_k_elem(hd, trow, d)]), partial);
    const float score = wave_sum(partial) * scale;
    const float m_new = fmaxf(m, score);
    const float alpha = l == 0.0f ? 0.0f : expf(m - m_new);
    const float pnew = expf(score - m_new);
#pragma unroll
    for (int j = 0; j < kMaxPerLane; ++j) {
      const uint32_t d = lane + j * kWave;
      if (d < hd) acc[j] = acc[j] * alpha + (fresh ? vn[d] : dec16<DT>(p.v_cache[tile + kv_v_elem(hd, trow, d)])) * pnew;
    }
    l = l * alpha + pnew;
    m = m_new;
  }
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) {
    const uint32_t d = lane + j * kWave;
    if (d < hd) wacc[wave * hd + d] = acc[j];
  }
  if (lane == 0) {
    wm[wave] = m;
    wl[wave] = l;
  }
  __syncthreads();
  float M = -INFINITY;
  for (int w = 0; w < kWavesPerBlock; ++w) M = fmaxf(M, wm[w]);
  for (uint32_t d = threadIdx.x; d < hd; d += kBlock) {
    float L = 0.0f, o = 0.0f;
    for (int w = 0; w < kWavesPerBlock; ++w) {
      if (wm[w] > -INFINITY) {
        const float f = expf(wm[w] - M);
        L += wl[w] * f;
        o += wacc[w * hd + d] * f;
      }
    }
    if (L > 0.0f && isfinite(L)) o /= L;
    if (p.out_f32) p.out_f32[h * hd + d] = o;
    p.out16[h * hd + d] = enc16<DT>(o);
  }
}

template <uint32_t DT>
hipError_t launch_dt(const AttnParams &p, hipStream_t stream) {
  const uint32_t group = p.heads / p.kv_heads;
  const bool fast = p.head_dim == kHD && (group == 1 || group == 2 || group == 4 || group == 8) &&
                    p.part_acc != nullptr && p.splits >= 1;
  if (fast) {
    const dim3 grid(p.kv_heads, p.splits, p.tokens > 1 ? p.tokens : 1);
    if (p.tokens > 1 || p.seqs != nullptr) {
      switch (group) {
        case 1: hipLaunchKernelGGL((attn_block_kernel<DT, 1, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((attn_block_kernel<DT, 2, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
        case 4: hipLaunchKernelGGL((attn_block_kernel<DT, 4, kAttnWaves>), grid, dim3(kAttnWaves * kWave), 0, stream, p); break;
        default: hipLaunchKernelGGL((attn_block_kernel<DT, 8, kAttnWaves / 2>), grid, dim3(kAttnWaves / 2 * kWave), 0, stream, p); break;
      }
      return hipGetLastError();
    }
    if (p.part_tagged == nullptr) return hipErrorInvalidValue;
    // every active split of a kv head has to be resident while the merges poll: a larger split factor is refused
    // here, never launched (callers size theirs with attn_default_splits)
    if (p.splits > 1 && p.splits > attn_resident_splits(p.kv_heads)) return hipErrorInvalidValue;
    switch (group) {
      case 1: hipLaunchKernelGGL((attn_step_kernel<DT, 1>), grid, dim3(8 * kWave), 0, stream, p); break;
      case 2: hipLaunchKernelGGL((attn_step_kernel<DT, 2>), grid, dim3(8 * kWave), 0, stream, p); break;
      case 4: hipLaunchKernelGGL((attn_step_kernel<DT, 4>), grid, dim3(8 * kWave), 0, stream, p); break;
      default: hipLaunchKernelGGL((attn_step_kernel<DT, 8>), grid, dim3(8 * kWave), 0, stream, p); break;
    }
  } else {
    if (p.head_dim > 512) return hipErrorInvalidValue;
    const size_t lds = static_cast<size_t>(3 + kWavesPerBlock) * p.head_dim * sizeof(float);
    hipLaunchKernelGGL((attn_generic_kernel<DT>), dim3(p.heads), dim3(kBlock), lds, stream, p);
  }
  return hipGetLastError();
}

}  // namespace

uint32_t attn_resident_splits(uint32_t kv_heads) {
  static const uint32_t cus = [] {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) {
      (void)hipGetLastError();
      return 256u;   // no device to ask: the part this library is written for
    }
    return static_cast<uint32_t>(count);
  }();
  const uint32_t splits = cus / (kv_heads == 0 ? 1 : kv_heads);
  return splits == 0 ? 1 : splits;
}

uint64_t attn_step_workspace_bytes(uint32_t heads) {
  return static_cast<uint64_t>(heads) * kAttnMaxSplits * kStepRecord * sizeof(uint64_t);
}

uint64_t attn_workspace_bytes(uint32_t heads, uint32_t head_dim) {
  const uint64_t acc = static_cast<uint64_t>(heads) * kAttnMaxSplits * head_dim * sizeof(float);
  const uint64_t ml = static_cast<uint64_t>(heads) * kAttnMaxSplits * sizeof(float) * 2;
  return acc + ml + 1024 * sizeof(uint32_t);
}

void attn_bind_workspace(AttnParams &p, void *workspace) {
  char *base = static_cast<char *>(workspace);
  const uint64_t acc = static_cast<uint64_t>(p.heads) * kAttnMaxSplits * p.head_dim * sizeof(float);
  const uint64_t ml = static_cast<uint64_t>(p.heads) * kAttnMaxSplits * sizeof(float);
  p.part_acc = reinterpret_cast<float *>(base);
  p.part_m = reinterpret_cast<float *>(base + acc);
  p.part_l = reinterpret_cast<float *>(base + acc + ml);
  p.counters = reinterpret_cast<uint32_t *>(base + acc + 2 * ml);
}

hipError_t launch_kv_publish_rows(uint32_t dtype, const AttnParams &p, hipStream_t stream) {
  const bool caches = p.seqs != nullptr || (p.k_cache != nullptr && p.v_cache != nullptr && p.table != nullptr);
  if (p.qkv == nullptr || !caches || p.tokens == 0 || p.head_dim != static_cast<uint32_t>(kHD) || p.kv_heads == 0)
    return hipErrorInvalidValue;
  if (p.seqs == nullptr &&
      static_cast<uint64_t>(p.position) + p.tokens > static_cast<uint64_t>(p.block_count) * kKvBlockTokens)
    return hipErrorInvalidValue;
  const dim3 grid(p.kv_heads, p.tokens);
  if (dtype == kBF16) hipLaunchKernelGGL(kv_publish_rows_kernel<kBF16>, grid, dim3(2 * kWave), 0, stream, p);
  else if (dtype == kF16) hipLaunchKernelGGL(kv_publish_rows_kernel<kF16>, grid, dim3(2 * kWave), 0, stream, p);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_attn_decode(uint32_t dtype, const AttnParams &p, hipStream_t stream) {
  const bool caches = p.seqs != nullptr || (p.k_cache != nullptr && p.v_cache != nullptr && p.table != nullptr);
  if (p.qkv == nullptr || !caches || p.out16 == nullptr) return hipErrorInvalidValue;
  if (p.heads == 0 || p.kv_heads == 0 || p.head_dim == 0 || p.heads % p.kv_heads != 0 ||
      (p.seqs == nullptr && p.block_count == 0) || p.kv_heads > 1024)
    return hipErrorInvalidValue;
  if (p.rope_freq != nullptr && p.head_dim % 2 != 0) return hipErrorInvalidValue;
  if (p.splits > kAttnMaxSplits) return hipErrorInvalidValue;
  // partial sums instead of values: only the launch for a batch of sequences reads them
  if (p.qkv_slices > 1 && (p.qkv_slices > 4 || p.seqs == nullptr || p.append == 0 || p.qkv_slice_stride == 0)) return hipErrorInvalidValue;
  if (p.cursor == nullptr && p.seqs == nullptr &&
      static_cast<uint64_t>(p.position) >= static_cast<uint64_t>(p.block_count) * kKvBlockTokens)
    return hipErrorInvalidValue;
  if (p.out_packed_tiles != 0 && (!(p.tokens > 1 || p.seqs != nullptr) || p.out_packed_tiles * 16u < p.tokens || p.out_f32 != nullptr))
    return hipErrorInvalidValue;
  if (p.tokens > 1 || p.seqs != nullptr) {
    // a block of positions or of sequences: host-given positions, matrix-core kernel only
    const uint32_t group = p.heads / p.kv_heads;
    const bool fast = p.head_dim == 128 && (group == 1 || group == 2 || group == 4 || group == 8) && p.part_acc != nullptr;
    // (rows of consecutive positions have to be in the cache before the launch; rows of different
    // sequences can be appended by the launch itself, as the single-token kernel does)
    if (p.cursor != nullptr || (p.append != 0 && p.seqs == nullptr) || !fast || p.tokens == 0 || p.tokens > 65535 ||
        (p.seqs == nullptr &&
         static_cast<uint64_t>(p.position) + p.tokens > static_cast<uint64_t>(p.block_count) * kKvBlockTokens))
      return hipErrorInvalidValue;
  }
  if (dtype == kBF16) return launch_dt<kBF16>(p, stream);
  if (dtype == kF16) return launch_dt<kF16>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace nv
