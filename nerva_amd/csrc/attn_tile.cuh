// Device-side building blocks of the matrix-core decode attention (head_dim 128): head
// preparation (bias, per-head RMSNorm, RoPE), operand helpers, coherent accesses for data
// exchanged between workgroups of one launch, and the 16-token tile step. Shared by the
// stand-alone attention kernel (attn_decode.hip) and the fused layer-front kernel
// (layer_front.hip).
#pragma once

#include "attn_decode.cuh"

namespace nv {
namespace attn {

constexpr int kHD = 128;
constexpr int kAttnWaves = 8;   // waves per workgroup of the fast path (group 8 uses half)

// One wave prepares one 128-wide head: lane l owns the RoPE pair (l, l+64).
// out[] receives f32; when out16 != null the value is rounded first and the 16-bit
// copy is stored too (K/V that go to the cache).
// rope_cs (optional): cos at [i], sin at [64 + i] of this step's angles, computed once
// per step; without it the angle pos / rope_freq[i] is evaluated here.
template <uint32_t DT, bool COHERENT = false>
__device__ __forceinline__ void prep_head128(const float *src, const uint16_t *bias,
                                             const uint16_t *gamma, const float *rope_freq,
                                             const float *rope_cs, uint32_t pos, float eps, int lane,
                                             float *out, uint16_t *out16) {
  float x0, x1;
  if constexpr (COHERENT) {  // src was written by another workgroup of this launch
    x0 = __hip_atomic_load(src + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    x1 = __hip_atomic_load(src + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    x0 = src[lane];
    x1 = src[lane + 64];
  }
  if (bias != nullptr) {
    x0 += dec16<DT>(bias[lane]);
    x1 += dec16<DT>(bias[lane + 64]);
  }
  if (gamma != nullptr) {
    const float ss = wave_sum(x0 * x0 + x1 * x1);
    const float scale = 1.0f / sqrtf(ss / 128.0f + eps);
    x0 *= scale * dec16<DT>(gamma[lane]);
    x1 *= scale * dec16<DT>(gamma[lane + 64]);
  }
  if (rope_freq != nullptr) {
    float s, c;
    if (rope_cs != nullptr) {
      c = rope_cs[lane];
      s = rope_cs[64 + lane];
    } else {
      sincosf(static_cast<float>(pos) / rope_freq[lane], &s, &c);
    }
    const float r0 = x0 * c - x1 * s;
    const float r1 = x1 * c + x0 * s;
    x0 = r0;
    x1 = r1;
  }
  if (out16 != nullptr) {
    out16[lane] = enc16<DT>(x0);
    out16[lane + 64] = enc16<DT>(x1);
    x0 = round16<DT>(x0);
    x1 = round16<DT>(x1);
  }
  if (out != nullptr) {
    out[lane] = x0;
    out[lane + 64] = x1;
  }
}

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// D(16x16) += A(16x32) . B(32x16): lane l holds A[l%16][8*(l/16)..+7], B[8*(l/16)..+7][l%16] and
// D[4*(l/16)..+3][l%16].
template <uint32_t DT>
__device__ __forceinline__ f32x4_t mfma_k32(const uint4 &a, const uint4 &b, f32x4_t c) {
  if constexpr (DT == kBF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}
// D(16x16) += A(16x16) . B(16x16): four contraction elements per lane, 4*(l/16)..+3.
template <uint32_t DT>
__device__ __forceinline__ f32x4_t mfma_k16(const uint2 &a, const uint2 &b, f32x4_t c) {
  if constexpr (DT == kBF16)
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a),
                                                     __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a),
                                                 __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
}

// Lane i of a 16-lane row receives lane i + N (shl) / i - N (shr); lanes without a source get 0.
template <int N>
__device__ __forceinline__ float row_shl(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x100 + N, 0xF, 0xF, true));
}
template <int N>
__device__ __forceinline__ float row_shr(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x110 + N, 0xF, 0xF, true));
}

// v = hi + lo with hi, lo 16-bit: the pair carries 16 (bf16) / 22 (f16) mantissa bits, so a
// matrix-core product against exact 16-bit K/V data loses nothing that matters to f32 math.
template <uint32_t DT>
__device__ __forceinline__ void split16(float v, uint16_t &hi, uint16_t &lo) {
  hi = enc16<DT>(v);
  lo = enc16<DT>(v - dec16<DT>(hi));
}

// Device-scope coherent accesses: written through / read around the XCD-local L2, so data
// exchanged between workgroups inside one kernel needs no cache flush or invalidate.
__device__ __forceinline__ void store_coherent(float *ptr, float v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float *ptr) {
  return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_coherent(uint32_t *ptr, uint32_t v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t load_coherent(const uint32_t *ptr) {
  return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Returns when every store this wave has issued has been performed.
__device__ __forceinline__ void wait_stores_performed() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Requests one (block, kv head) tile: four 1 KiB loads each for K and V.
__device__ __forceinline__ void attn_load_tile(const AttnParams &p, uint32_t b, uint32_t kvh, int lane,
                                               uint4 (&k)[4], uint4 (&v)[4]) {
  const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, p.table[b], kvh);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    k[i] = load_stream(p.k_cache + tile + i * 512 + lane * 8);
    v[i] = load_stream(p.v_cache + tile + i * 512 + lane * 8);
  }
}

// One 16-token tile against the G query heads of the kv head (see attn_fast_kernel).
template <uint32_t DT, int G, bool QX_LDS>
__device__ __forceinline__ void attn_tile(uint4 (&kreg)[4], uint4 (&vreg)[4], const uint4 (&qx)[4],
                                          const uint4 *qx_lds, uint32_t b,
                                          uint32_t n_keys, int col, int grp, bool splice, uint32_t new_row,
                                          const uint16_t *knew, const uint16_t *vnew, float &m, float &l,
                                          f32x4_t (&acc)[8]) {
  if (splice) {
    // the row published by this workgroup may not be visible to its own loads yet: take it from LDS
    if (static_cast<uint32_t>(col) == new_row) {  // K operand: lane = (token col, dims grp*8..)
#pragma unroll
      for (int j = 0; j < 4; ++j) kreg[j] = *reinterpret_cast<const uint4 *>(knew + j * 32 + grp * 8);
    }
    if (static_cast<uint32_t>(grp) == new_row / 4) {  // V operand: lane = (dim col of a slab, tokens grp*4..)
      const uint32_t e = new_row % 4;
      const uint32_t sh = (e & 1u) * 16u, keep = ~(0xffffu << sh);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t v0 = vnew[(2 * j) * 16 + col], v1 = vnew[(2 * j + 1) * 16 + col];
        if (e < 2) {
          vreg[j].x = (vreg[j].x & keep) | (v0 << sh);
          vreg[j].z = (vreg[j].z & keep) | (v1 << sh);
        } else {
          vreg[j].y = (vreg[j].y & keep) | (v0 << sh);
          vreg[j].w = (vreg[j].w & keep) | (v1 << sh);
        }
      }
    }
  }
  // scores of tokens b*16 + grp*4 + r for column col
  f32x4_t c{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if constexpr (QX_LDS) c = mfma_k32<DT>(kreg[j], qx_lds[j * kWave], c);  // qx_lds: this lane's first operand
    else c = mfma_k32<DT>(kreg[j], qx[j], c);
  }
  float sc[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    // hi column + lo column of the same head (either order: one f32 add). Both shifts run
    // with every lane active: a lane-crossing read from a lane that sits out returns 0.
    const float from_up = row_shl<G>(c[r]), from_down = row_shr<G>(c[r]);
    const float other = col < G ? from_up : from_down;
    const bool valid = b * kKvBlockTokens + grp * 4 + r < n_keys;
    sc[r] = valid ? c[r] + other : -INFINITY;
  }
  float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
  mb = fmaxf(mb, __shfl_xor(mb, 16, kWave));
  mb = fmaxf(mb, __shfl_xor(mb, 32, kWave));
  const float m_new = fmaxf(m, mb);   // finite: every processed tile has a valid token
  const float alpha = expf(m - m_new);
  uint32_t px[2];
  float psum = 0.0f;
#pragma unroll
  for (int r = 0; r < 4; r += 2) {
    const float p0 = expf(sc[r] - m_new), p1 = expf(sc[r + 1] - m_new);
    psum += p0 + p1;
    uint16_t h0, l0, h1, l1;
    split16<DT>(p0, h0, l0);
    split16<DT>(p1, h1, l1);
    px[r / 2] = col < G ? (h0 | (static_cast<uint32_t>(h1) << 16)) : (l0 | (static_cast<uint32_t>(l1) << 16));
  }
  l = l * alpha + psum;
  m = m_new;
  const uint2 pb = make_uint2(px[0], px[1]);
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) {
    acc[s2] *= alpha;
    const uint4 &vr = vreg[s2 / 2];
    const uint2 va = (s2 & 1) ? make_uint2(vr.z, vr.w) : make_uint2(vr.x, vr.y);
    acc[s2] = mfma_k16<DT>(va, pb, acc[s2]);
  }
}

template <int G, int W>
struct AttnShared {
  alignas(16) float q_s[G][kHD];
  alignas(16) uint16_t knew[kHD];
  alignas(16) uint16_t vnew[kHD];
  float wm[W][G];
  float wl[W][G];
  alignas(16) float wacc[W][G][kHD];
  float wf[W][G];   // exp(m_w - M_g), 0 for idle waves
  float bM[G];
  uint32_t is_last;
  alignas(16) uint4 qx_s[4][kWave];  // linked launches: the query operand of the first product
};

// Connections of an attention workgroup to the other roles of a fused launch.
struct AttnLink {
  const uint32_t *wait_flags;  // [wait_count <= 64] producer flags to wait for, or null
  uint32_t wait_count;
  uint32_t *done_flag;         // this kv head's flag, raised to `epoch` when its output is visible
  float *out_coherent;         // [heads * 128] f32 output for the consumer role
  uint32_t *abort_flag;        // raised when a bounded wait ran out
  uint32_t epoch;
  uint64_t *trace;             // tuning aid: device timestamps of this workgroup's stages, or null
  uint64_t *trace_merge;       // same for the workgroup that merges this kv head's splits
};
__device__ __forceinline__ void link_mark(uint64_t *trace, int slot) {
  if (trace != nullptr && threadIdx.x == 0) trace[slot] = wall_clock64();
}
constexpr uint32_t kLinkSpinLimit = 1u << 20;

// Every wave's output stores have to be performed before one lane raises the flag.
__device__ __forceinline__ void attn_publish(const AttnLink &link, uint32_t kvh) {
  wait_stores_performed();
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(link.done_flag, link.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  (void)kvh;
}

// W waves per workgroup. A workgroup owns one kv head and one contiguous range of
// 16-token tiles; wave w takes tiles b0+w, b0+w+W, ...  Both products of a tile run on
// the matrix cores:
//   S^T[token][col] = K[token][dim] . Qx[dim][col]   4 x mfma 16x16x32 (contraction: 128 dims)
//   O^T[dim][col]  += V^T[dim][token] . Px[token][col]   8 x mfma 16x16x16 (one per 16 dims)
// with 16 columns = G query heads x {hi, lo}: the f32 q (pre-scaled by 1/sqrt(d)) and the f32
// probabilities are split into two 16-bit parts that occupy columns g and g + G, so products
// against the 16-bit K/V stay f32-accurate. The S^T result layout (lane = column, 4 tokens of
// its lane group) is exactly the B-operand layout of the second product, and the O^T
// accumulators are indexed by the same column, so m, l and the rescale never cross lanes.
// The cache stores tiles in operand order (kv_k_elem / kv_v_elem): every load is one coalesced
// 1 KiB instruction and lands in the registers the matrix core reads.
//
// LINKED = the workgroup is the attention role of a launch that also holds its producer and/or
// consumer (AttnLink): it may wait for flags before it reads q/k/v (its first tiles are already
// requested by then), reads q/k/v with device-coherent loads, publishes the final output with
// device-coherent stores as well and raises the kv head's flag once they have been performed.
template <uint32_t DT, int G, int W, bool LINKED>
__device__ __forceinline__ void attn_fast_body(const AttnParams &p, const uint32_t pos, const uint32_t kvh,
                                               const uint32_t split, const uint32_t S, AttnShared<G, W> &sh,
                                               const AttnLink &link) {
  constexpr int kThreads = W * kWave;
  auto &q_s = sh.q_s;
  auto &knew = sh.knew;
  auto &vnew = sh.vnew;
  auto &wm = sh.wm;
  auto &wl = sh.wl;
  auto &wacc = sh.wacc;
  auto &wf = sh.wf;
  auto &bM = sh.bM;

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t n_keys = pos + 1;
  const uint32_t nblk = (n_keys + kKvBlockTokens - 1) / kKvBlockTokens;
  // at least W tiles per active split so that every wave of a workgroup has work
  uint32_t bps = (nblk + S - 1) / S;
  bps = ((bps + W - 1) / W) * W;
  const uint32_t active = (nblk + bps - 1) / bps;
  if (split >= active) return;  // idle splits neither store a partial nor take a ticket
  const uint32_t b0 = split * bps;
  const uint32_t b1 = min(nblk, b0 + bps);
  const uint32_t A = p.heads * kHD, KV = p.kv_heads * kHD;
  const uint32_t new_block = pos / kKvBlockTokens, new_row = pos % kKvBlockTokens;
  const bool owns_new = p.append != 0 && new_block >= b0 && new_block < b1;

  // ---- first tile of every wave: issue its loads before anything else
  // Two tiles in flight per wave (roles swap); a linked workgroup keeps one, to fit the register
  // budget that lets two 8-wave workgroups share a CU, and its launch uses more splits instead.
  constexpr int kInFlight = LINKED ? 1 : 2;
  uint4 kreg[4], vreg[4], kreg1[kInFlight == 2 ? 4 : 1], vreg1[kInFlight == 2 ? 4 : 1];
  uint32_t b = b0 + wave;
  if (b < b1) attn_load_tile(p, b, kvh, lane, kreg, vreg);

  if constexpr (LINKED) link_mark(link.trace, 8);
  if constexpr (LINKED) {
    // ---- the producer of q/k/v runs in the same launch: wait for its rows (bounded)
    if (link.wait_flags != nullptr) {
      if (wave == 0) {
        uint32_t spins = 0;
        bool ok = true;
        for (;;) {
          const bool mine = static_cast<uint32_t>(lane) >= link.wait_count ||
                            static_cast<int32_t>(load_coherent(link.wait_flags + lane) - link.epoch) >= 0;
          if (__all(mine)) break;
          if (++spins > kLinkSpinLimit || load_coherent(link.abort_flag) != 0u) {
            ok = false;
            break;
          }
        }
        if (!ok && lane == 0) store_coherent(link.abort_flag, 1u);
      }
      __syncthreads();
    }
    link_mark(link.trace, 9);
  }
  // ---- q (all workgroups) and the new K/V row (the workgroup whose range holds pos)
  for (int g = wave; g < G; g += W) {
    const uint32_t h = kvh * G + g;
    prep_head128<DT, LINKED>(p.qkv + h * kHD, p.q_bias ? p.q_bias + h * kHD : nullptr, p.q_norm, p.rope_freq,
                     p.rope_cs, pos, p.eps, lane, q_s[g], nullptr);
  }
  if (owns_new) {
    if (wave == (G % W)) {
      prep_head128<DT, LINKED>(p.qkv + A + kvh * kHD, p.k_bias ? p.k_bias + kvh * kHD : nullptr, p.k_norm,
                       p.rope_freq, p.rope_cs, pos, p.eps, lane, nullptr, knew);
    } else if (wave == ((G + 1) % W)) {
      prep_head128<DT, LINKED>(p.qkv + A + KV + kvh * kHD, p.v_bias ? p.v_bias + kvh * kHD : nullptr, nullptr,
                       nullptr, nullptr, pos, p.eps, lane, nullptr, vnew);
    }
  }
  __syncthreads();
  if (owns_new && wave == 0) {
    // publish the rounded row to the cache in operand order
    const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, p.table[new_block], kvh);
    if (lane < 16) {  // K: 16 pieces of 8 consecutive dims
      *reinterpret_cast<uint4 *>(p.k_cache + tile + kv_k_elem(kHD, new_row, lane * 8)) =
          *reinterpret_cast<const uint4 *>(knew + lane * 8);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // V: one 16-bit element per dim
      const uint32_t d = lane + i * kWave;
      p.v_cache[tile + kv_v_elem(kHD, new_row, d)] = vnew[d];
    }
  }

  const int col = lane & 15, grp = lane >> 4;
  const float scale = 1.0f / sqrtf(static_cast<float>(kHD));

  // B operand of the first product: column `col` of Qx for dims j*32 + grp*8 .. +7
  uint4 qx[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (col < 2 * G) {
      const float *src = &q_s[col < G ? col : col - G][j * 32 + grp * 8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint16_t h0, l0, h1, l1;
        split16<DT>(src[2 * e] * scale, h0, l0);
        split16<DT>(src[2 * e + 1] * scale, h1, l1);
        w[e] = col < G ? (h0 | (static_cast<uint32_t>(h1) << 16)) : (l0 | (static_cast<uint32_t>(l1) << 16));
      }
    }
    qx[j] = make_uint4(w[0], w[1], w[2], w[3]);
  }
  // A linked workgroup runs under a tighter register budget: it parks the operand in LDS (every
  // wave writes the same values, and reads them back after its own writes).
  const uint4 *qx_lds = nullptr;
  if constexpr (LINKED) {
#pragma unroll
    for (int j = 0; j < 4; ++j) sh.qx_s[j][lane] = qx[j];
    qx_lds = &sh.qx_s[0][lane];
  }

  if constexpr (LINKED) link_mark(link.trace, 10);
  float m = -INFINITY, l = 0.0f;  // of column `col` (both copies of a head track the same values)
  f32x4_t acc[8];                  // O^T[dims s*16 + grp*4 .. +3][col]
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) acc[s2] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  if constexpr (kInFlight == 2) {
    if (b + W < b1) attn_load_tile(p, b + W, kvh, lane, kreg1, vreg1);
    for (; b < b1; b += 2 * W) {
      attn_tile<DT, G, LINKED>(kreg, vreg, qx, qx_lds, b, n_keys, col, grp, owns_new && b == new_block, new_row, knew, vnew, m, l, acc);
      if (b + 2 * W < b1) attn_load_tile(p, b + 2 * W, kvh, lane, kreg, vreg);
      if (b + W < b1) {
        attn_tile<DT, G, LINKED>(kreg1, vreg1, qx, qx_lds, b + W, n_keys, col, grp, owns_new && b + W == new_block, new_row, knew, vnew, m, l, acc);
        if (b + 3 * W < b1) attn_load_tile(p, b + 3 * W, kvh, lane, kreg1, vreg1);
      }
    }
  } else {
    for (; b < b1; b += W) {
      attn_tile<DT, G, LINKED>(kreg, vreg, qx, qx_lds, b, n_keys, col, grp, owns_new && b == new_block, new_row, knew, vnew, m, l, acc);
      if (b + W < b1) attn_load_tile(p, b + W, kvh, lane, kreg, vreg);
    }
  }

  if constexpr (LINKED) link_mark(link.trace, 11);
  // ---- wave result: tokens of the four lane groups, then hi + lo columns; then the W waves
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) {
    float4 o;
    o.x = acc[s2][0] + row_shl<G>(acc[s2][0]);
    o.y = acc[s2][1] + row_shl<G>(acc[s2][1]);
    o.z = acc[s2][2] + row_shl<G>(acc[s2][2]);
    o.w = acc[s2][3] + row_shl<G>(acc[s2][3]);
    if (col < G) *reinterpret_cast<float4 *>(&wacc[wave][col][s2 * 16 + grp * 4]) = o;
  }
  if (lane < G) {
    wm[wave][lane] = m;
    wl[wave][lane] = l;
  }
  __syncthreads();
  // ---- merge of the W waves: W*G scale factors once, then every thread owns (g, d) pairs
  if (threadIdx.x < W * G) {
    const int w = threadIdx.x / G, g = threadIdx.x % G;
    float M = -INFINITY;
#pragma unroll
    for (int w2 = 0; w2 < W; ++w2) M = fmaxf(M, wm[w2][g]);
    wf[w][g] = wm[w][g] > -INFINITY ? expf(wm[w][g] - M) : 0.0f;
    if (w == 0) bM[g] = M;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < G * kHD; e += kThreads) {
    const int g = e / kHD, d = e % kHD;
    float L = 0.0f, o = 0.0f;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      L = fmaf(wl[w][g], wf[w][g], L);
      o = fmaf(wacc[w][g][d], wf[w][g], o);
    }
    const uint32_t h = kvh * G + g;
    if (active == 1) {
      // a single split holds every key: this is the final result, nothing to exchange
      if (L > 0.0f && isfinite(L)) o /= L;
      if (p.out_f32 != nullptr) p.out_f32[h * kHD + d] = o;
      p.out16[h * kHD + d] = enc16<DT>(o);
      if constexpr (LINKED) store_coherent(link.out_coherent + h * kHD + d, o);
    } else {
      // The partial leaves through device-coherent stores (written through, no cache flush).
      store_coherent(p.part_acc + (static_cast<uint64_t>(h) * S + split) * kHD + d, o);
      if (d == 0) {
        store_coherent(p.part_m + h * S + split, bM[g]);
        store_coherent(p.part_l + h * S + split, L);
      }
    }
  }
  if (active == 1) {
    if constexpr (LINKED) attn_publish(link, kvh);
    return;
  }
  // Every wave waits until its own stores have been performed, the barrier collects the waves,
  // and only then one lane takes the arrival ticket of this kv head.
  wait_stores_performed();
  __syncthreads();
  if constexpr (LINKED) link_mark(link.trace, 12);
  if (threadIdx.x == 0) {
    const uint32_t ticket =
        __hip_atomic_fetch_add(p.counters + kvh, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh.is_last = ticket == active - 1 ? 1u : 0u;
  }
  __syncthreads();
  if constexpr (LINKED) link_mark(link.trace, 13);
  if (!sh.is_last) return;
  if constexpr (LINKED) link_mark(link.trace_merge, 16);
  // ---- the last workgroup of this kv head merges the splits. Each thread owns (g, d) and reads
  // the partials with device-coherent loads, sixteen splits per round trip, in split order.
  for (int e = threadIdx.x; e < G * kHD; e += kThreads) {
    const int g = e / kHD, d = e % kHD;
    const uint32_t h = kvh * G + g;
    const float *pm = p.part_m + h * S, *pl = p.part_l + h * S;
    const float *src = p.part_acc + static_cast<uint64_t>(h) * S * kHD + d;
    float M = -INFINITY, L = 0.0f, o = 0.0f;
    for (uint32_t s0 = 0; s0 < active; s0 += 16) {
      float mm[16], ll[16], aa[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const bool on = s0 + i < active;
        mm[i] = on ? load_coherent(pm + s0 + i) : -INFINITY;
        ll[i] = on ? load_coherent(pl + s0 + i) : 0.0f;
        aa[i] = on ? load_coherent(src + static_cast<uint64_t>(s0 + i) * kHD) : 0.0f;
      }
      float Mc = M;
#pragma unroll
      for (int i = 0; i < 16; ++i) Mc = fmaxf(Mc, mm[i]);
      const float keep = M > -INFINITY ? expf(M - Mc) : 0.0f;
      L *= keep;
      o *= keep;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float f = mm[i] > -INFINITY ? expf(mm[i] - Mc) : 0.0f;
        L = fmaf(ll[i], f, L);
        o = fmaf(aa[i], f, o);
      }
      M = Mc;
    }
    if (L > 0.0f && isfinite(L)) o /= L;
    if (p.out_f32 != nullptr) p.out_f32[h * kHD + d] = o;
    p.out16[h * kHD + d] = enc16<DT>(o);
    if constexpr (LINKED) store_coherent(link.out_coherent + h * kHD + d, o);
  }
  if (threadIdx.x == 0) __hip_atomic_store(p.counters + kvh, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if constexpr (LINKED) {
    link_mark(link.trace_merge, 17);
    attn_publish(link, kvh);
    link_mark(link.trace_merge, 18);
  }
}

}  // namespace attn
}  // namespace nv
