// Attention of a prompt block: consecutive positions of one sequence (64 in the session's prefill) in one launch, every
// K/V tile of the prefix fetched once per workgroup and used by all its tokens.
// Reference: the chunked prefill's attention (session_decode_prefill.inc.cu:1879-2243) over the
// arithmetic of exact_blockwise_attention_into (attention/exact/run.rs:13-127) per token; the rows
// of the block itself are in the cache already (launch_kv_publish_rows), so token t simply attends to
// keys 0 .. position + t.
//
// gfx950 mapping (head_dim 128, G = heads / kv_heads in {1, 2, 4, 8}): the 16-column matrix-core tile
// of the decode kernel holds the G query heads of ONE token as hi/lo column pairs and leaves the
// rest of its columns empty; here a wave fills all 16 columns with 16 (token, head) pairs - 16 / G tokens
// of the kv head's G query heads - and the hi and lo halves of a query (and of a tile's probabilities) are
// two products into the same accumulators (attn_tile_wide), with the causal limit n_keys chosen per column.
// The 8 waves of a workgroup take 8 * 16 / G consecutive tokens and walk the SAME tiles: a tile (4 KiB of K,
// 4 KiB of V) is requested once
// by the workgroup - one 16-byte piece per lane - parked in LDS (two stages, one barrier per tile) and
// read back by every wave as matrix operands. Grid (kv head, split of the prefix, token group); split
// partials go to the per-token workspaces the decode kernel uses and a small second launch merges them.
#include <algorithm>

#include "attn_decode.cuh"
#include "attn_tile.cuh"

namespace nv {

namespace {

using namespace attn;

constexpr int kPW = 8;    // waves per workgroup
constexpr int kVG = 16;   // (token, head) pairs per wave: one per column of the matrix-core tile

// Split geometry of a token group, the same on both launches: tiles per split, active splits.
__device__ __forceinline__ void prompt_splits(uint32_t last_pos, uint32_t S, uint32_t &bps, uint32_t &active, uint32_t &nblk) {
  nblk = last_pos / kKvBlockTokens + 1;
  bps = (nblk + S - 1) / S;
  active = (nblk + bps - 1) / bps;
}

template <uint32_t DT, int G>
__global__ __launch_bounds__(kPW *kWave) void attn_prompt_kernel(AttnParams p) {
  constexpr int kTokensPerWave = kVG / G;
  constexpr uint32_t kGroupTokens = kPW * kTokensPerWave;
  __shared__ uint4 stage[2][8][kWave];          // K pieces 0..3, V pieces 4..7 of a tile, twice
  __shared__ __align__(16) float q_s[kPW][kVG][kHD];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t kvh = blockIdx.x, split = blockIdx.y, S = gridDim.y, T = p.tokens;
  const uint32_t group_first = blockIdx.z * kGroupTokens;
  const uint32_t group_last = min(T, group_first + kGroupTokens) - 1;
  uint32_t bps, active, nblk;
  prompt_splits(p.position + group_last, S, bps, active, nblk);
  if (split >= active) return;
  const uint32_t b0 = split * bps, b1 = min(nblk, b0 + bps);

  // the workgroup's first tile is on its way while the queries are prepared
  const uint16_t *cache = wave < 4 ? p.k_cache : p.v_cache;
  const uint32_t piece = (wave & 3) * 512 + lane * 8;
  auto tile_piece = [&](uint32_t b) {
    return load_stream(cache + kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, p.table[b], kvh) + piece);
  };
  uint4 inflight = tile_piece(b0);

  // ---- this wave's eight (token, head) pairs: bias, norm, rotation -> f32 q in LDS
  const uint32_t wave_first = group_first + wave * kTokensPerWave;   // may lie past the block: clamped, never stored
  // (every input of all eight requested first, unconditionally: one round trip instead of eight)
  const bool has_bias = p.q_bias != nullptr, has_gamma = p.q_norm != nullptr, has_rope = p.rope_freq != nullptr;
  const uint16_t *bias_base = has_bias ? p.q_bias : p.k_cache;    // any readable address when unused
  const float *rope_base = has_rope ? p.rope_cs : p.qkv;
  const uint32_t rope_stride = has_rope ? p.rope_token_stride : 0u;
  const uint16_t *gamma_base = has_gamma ? p.q_norm : p.k_cache;
  const float g0 = dec16<DT>(gamma_base[lane]), g1 = dec16<DT>(gamma_base[lane + 64]);
#pragma unroll
  for (int part = 0; part < kVG / 8; ++part) {   // eight pairs at a time: their inputs in one round trip
    float x0[8], x1[8], rc[8], rs[8];
    uint16_t qb0[8], qb1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int vh = part * 8 + i;
      const uint32_t tok = min(wave_first + vh / G, T - 1);
      const uint32_t h = kvh * G + vh % G;
      const float *src = p.qkv + static_cast<uint64_t>(tok) * p.qkv_token_stride + h * kHD;
      x0[i] = src[lane];
      x1[i] = src[lane + 64];
      qb0[i] = bias_base[h * kHD + lane];
      qb1[i] = bias_base[h * kHD + lane + 64];
      rc[i] = rope_base[static_cast<uint64_t>(tok) * rope_stride + lane];
      rs[i] = rope_base[static_cast<uint64_t>(tok) * rope_stride + 64 + lane];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      prep_head128_core<DT>(x0[i], x1[i], has_bias, dec16<DT>(qb0[i]), dec16<DT>(qb1[i]), has_gamma, g0, g1, has_rope,
                            rc[i], rs[i], p.eps, lane, q_s[wave][part * 8 + i], nullptr);
  }
  __syncthreads();

  const int col = lane & 15, grp = lane >> 4;
  const float scale = kLog2e / sqrtf(static_cast<float>(kHD));
  uint4 qhi[4], qlo[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float *src = &q_s[wave][col][j * 32 + grp * 8];
    uint32_t wh[4], wl[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint16_t h0, l0, h1, l1;
      split16<DT>(src[2 * e] * scale, h0, l0);
      split16<DT>(src[2 * e + 1] * scale, h1, l1);
      wh[e] = h0 | (static_cast<uint32_t>(h1) << 16);
      wl[e] = l0 | (static_cast<uint32_t>(l1) << 16);
    }
    qhi[j] = make_uint4(wh[0], wh[1], wh[2], wh[3]);
    qlo[j] = make_uint4(wl[0], wl[1], wl[2], wl[3]);
  }
  // causal limit of this lane's column, and the last tile any of the wave's tokens can see
  const uint32_t my_tok = min(wave_first + col / G, T - 1);
  const uint32_t n_keys = p.position + my_tok + 1;
  const uint32_t wave_last_tile = (p.position + min(wave_first + kTokensPerWave - 1, T - 1)) / kKvBlockTokens;
  const bool wave_on = wave_first < T;

  float m = -INFINITY, l = 0.0f;
  f32x4_t acc[8];
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) acc[s2] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  for (uint32_t b = b0; b < b1; ++b) {
    const int st = (b - b0) & 1;
    stage[st][wave][lane] = inflight;
    inflight = tile_piece(min(b + 1, b1 - 1));   // unconditional: a load under a branch would serialise
    __syncthreads();                             // the tile is complete; the other stage is free again
    if (wave_on && b <= wave_last_tile) {
      uint4 kreg[4], vreg[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        kreg[j] = stage[st][j][lane];
        vreg[j] = stage[st][4 + j][lane];
      }
      attn_tile_wide<DT>(kreg, vreg, qhi, qlo, b, n_keys, grp, m, l, acc);
    }
  }
  if (!wave_on) return;

  // ---- results of the wave's pairs: token rows of the four lane groups
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  const uint32_t tok = wave_first + col / G;
  const uint32_t h = kvh * G + col % G;
  const bool writer = tok < T;
  const float inv = l > 0.0f && isfinite(l) ? 1.0f / l : 1.0f;
  char *ws = reinterpret_cast<char *>(p.part_acc) + static_cast<uint64_t>(tok) * p.ws_token_stride;
  const uint64_t ml_off = reinterpret_cast<char *>(p.part_m) - reinterpret_cast<char *>(p.part_acc);
  const uint64_t l_off = reinterpret_cast<char *>(p.part_l) - reinterpret_cast<char *>(p.part_acc);
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) {
    if (!writer) continue;
    const float4 o = make_float4(acc[s2][0], acc[s2][1], acc[s2][2], acc[s2][3]);
    const uint32_t d = s2 * 16 + grp * 4;
    if (active == 1) {
      // a single split holds every key: final
      uint2 packed;
      packed.x = enc16<DT>(o.x * inv) | (static_cast<uint32_t>(enc16<DT>(o.y * inv)) << 16);
      packed.y = enc16<DT>(o.z * inv) | (static_cast<uint32_t>(enc16<DT>(o.w * inv)) << 16);
      *reinterpret_cast<uint2 *>(p.out16 + attn_out_token(p, tok) + attn_out_elem(p, h * kHD + d)) = packed;   // d % 4 == 0
    } else {
      *reinterpret_cast<float4 *>(reinterpret_cast<float *>(ws) + (static_cast<uint64_t>(h) * S + split) * kHD + d) = o;
    }
  }
  if (active != 1 && writer && grp == 0) {
    reinterpret_cast<float *>(ws + ml_off)[h * S + split] = m;
    reinterpret_cast<float *>(ws + l_off)[h * S + split] = l;
  }
}

// Second launch: grid (head, token), one lane per dim; splits in order, kRound of them requested at a time
// (4 where the launch has no more splits than that: the same sums in the same order with a quarter of the loads).
template <uint32_t DT, int kRound>
__global__ __launch_bounds__(kHD) void attn_prompt_merge_kernel(AttnParams p, uint32_t S, uint32_t group_tokens) {
  const uint32_t h = blockIdx.x, tok = blockIdx.y, d = threadIdx.x;
  const uint32_t group_last = min(p.tokens, (tok / group_tokens + 1) * group_tokens) - 1;
  uint32_t bps, active, nblk;
  prompt_splits(p.position + group_last, S, bps, active, nblk);
  if (active == 1) return;   // the first launch wrote the final rows
  const char *ws = reinterpret_cast<const char *>(p.part_acc) + static_cast<uint64_t>(tok) * p.ws_token_stride;
  const float *acc = reinterpret_cast<const float *>(ws) + static_cast<uint64_t>(h) * S * kHD + d;
  const float *pm = reinterpret_cast<const float *>(ws + (reinterpret_cast<const char *>(p.part_m) - reinterpret_cast<const char *>(p.part_acc))) + h * S;
  const float *pl = reinterpret_cast<const float *>(ws + (reinterpret_cast<const char *>(p.part_l) - reinterpret_cast<const char *>(p.part_acc))) + h * S;
  // rounds of kRound splits, every load of a round unconditional (index clamped) and in flight at once
  float M = -INFINITY, L = 0.0f, o = 0.0f;
  for (uint32_t s0 = 0; s0 < active; s0 += kRound) {
    float mm[kRound], ll[kRound], aa[kRound];
#pragma unroll
    for (int i = 0; i < kRound; ++i) {
      const uint32_t si = min(s0 + i, active - 1);
      mm[i] = pm[si];
      ll[i] = pl[si];
      aa[i] = acc[static_cast<uint64_t>(si) * kHD];
    }
    float Mc = M;
#pragma unroll
    for (int i = 0; i < kRound; ++i) {
      // a split past this token's position saw no key: m = -inf, and its accumulator may hold anything
      const bool on = s0 + i < active && mm[i] > -INFINITY;
      mm[i] = on ? mm[i] : -INFINITY;
      ll[i] = on ? ll[i] : 0.0f;
      aa[i] = on ? aa[i] : 0.0f;
      Mc = fmaxf(Mc, mm[i]);
    }
    const float keep = M > -INFINITY ? attn_exp2(M - Mc) : 0.0f;
    L *= keep;
    o *= keep;
#pragma unroll
    for (int i = 0; i < kRound; ++i) {
      const float f = mm[i] > -INFINITY ? attn_exp2(mm[i] - Mc) : 0.0f;
      L = fmaf(ll[i], f, L);
      o = fmaf(aa[i], f, o);
    }
    M = Mc;
  }
  if (L > 0.0f && isfinite(L)) o /= L;
  p.out16[attn_out_token(p, tok) + attn_out_elem(p, h * kHD + d)] = enc16<DT>(o);
}

template <uint32_t DT>
hipError_t launch_dt(const AttnParams &p, uint32_t splits, hipStream_t stream) {
  const uint32_t group = p.heads / p.kv_heads;
  const uint32_t group_tokens = kPW * (kVG / group);
  const dim3 grid(p.kv_heads, splits, (p.tokens + group_tokens - 1) / group_tokens);
  switch (group) {
    case 1: hipLaunchKernelGGL((attn_prompt_kernel<DT, 1>), grid, dim3(kPW * kWave), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((attn_prompt_kernel<DT, 2>), grid, dim3(kPW * kWave), 0, stream, p); break;
    case 4: hipLaunchKernelGGL((attn_prompt_kernel<DT, 4>), grid, dim3(kPW * kWave), 0, stream, p); break;
    default: hipLaunchKernelGGL((attn_prompt_kernel<DT, 8>), grid, dim3(kPW * kWave), 0, stream, p); break;
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess || splits == 1) return err;
  if (splits <= 4)
    hipLaunchKernelGGL((attn_prompt_merge_kernel<DT, 4>), dim3(p.heads, p.tokens), dim3(kHD), 0, stream, p, splits, group_tokens);
  else
    hipLaunchKernelGGL((attn_prompt_merge_kernel<DT, 16>), dim3(p.heads, p.tokens), dim3(kHD), 0, stream, p, splits, group_tokens);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_attn_prompt(uint32_t dtype, const AttnParams &p, hipStream_t stream) {
  const uint32_t group = p.kv_heads != 0 ? p.heads / p.kv_heads : 0;
  if (p.qkv == nullptr || p.k_cache == nullptr || p.v_cache == nullptr || p.table == nullptr || p.out16 == nullptr ||
      p.part_acc == nullptr || p.part_m == nullptr || p.part_l == nullptr)
    return hipErrorInvalidValue;
  if (p.head_dim != static_cast<uint32_t>(kHD) || p.kv_heads == 0 || p.heads != group * p.kv_heads ||
      !(group == 1 || group == 2 || group == 4 || group == 8) || p.tokens == 0 || p.tokens > 65535 || p.block_count == 0)
    return hipErrorInvalidValue;
  if (static_cast<uint64_t>(p.position) + p.tokens > static_cast<uint64_t>(p.block_count) * kKvBlockTokens)
    return hipErrorInvalidValue;
  if (p.rope_freq != nullptr && p.rope_cs == nullptr) return hipErrorInvalidValue;   // rotation tables per token row
  if (p.out_packed_tiles != 0 && p.out_packed_tiles * 16u < p.tokens) return hipErrorInvalidValue;
  // enough splits of the prefix to spread the block over the chip, at least eight tiles each
  const uint32_t group_tokens = kPW * (kVG / group);
  const uint32_t groups = (p.tokens + group_tokens - 1) / group_tokens;
  const uint32_t nblk = (p.position + p.tokens - 1) / kKvBlockTokens + 1;
  uint32_t splits = p.splits != 0 ? p.splits : (512u + p.kv_heads * groups - 1) / (p.kv_heads * groups);
  splits = std::min(splits, std::max(1u, nblk / 8));
  splits = std::max(1u, std::min<uint32_t>(splits, kAttnMaxSplits));
  if (dtype == kBF16) return launch_dt<kBF16>(p, splits, stream);
  if (dtype == kF16) return launch_dt<kF16>(p, splits, stream);
  return hipErrorInvalidValue;
}

}  // namespace nv
