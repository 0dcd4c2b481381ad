// Device-side building blocks of the matrix-core decode attention (head_dim 128): head
// preparation (bias, per-head RMSNorm, RoPE), operand helpers, coherent accesses for data
// exchanged between workgroups of one launch, and the 16-token tile step. Shared by the
// decode attention kernel (attn_decode.hip) and the prompt-block kernel (attn_prompt.hip).
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
// (x0, x1) = raw projection values of dims (lane, lane + 64); bias / gamma / rotation of the
// same two dims, already in registers.
template <uint32_t DT>
__device__ __forceinline__ void prep_head128_core(float x0, float x1, bool has_bias, float b0, float b1,
                                                  bool has_gamma, float g0, float g1, bool has_rope, float c,
                                                  float s, float eps, int lane, float *out, uint16_t *out16) {
  if (has_bias) {
    x0 += b0;
    x1 += b1;
  }
  if (has_gamma) {
    const float ss = wave_sum(x0 * x0 + x1 * x1);
    const float scale = 1.0f / sqrtf(ss / 128.0f + eps);
    x0 *= scale * g0;
    x1 *= scale * g1;
  }
  if (has_rope) {
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
// The same arithmetic on values that stay in registers: (x0, x1) = dims (lane, lane + 64) of one head.
template <uint32_t DT>
__device__ __forceinline__ void head_values(float &x0, float &x1, bool has_bias, float b0, float b1, bool has_gamma,
                                            float g0, float g1, bool has_rope, float c, float s, float eps) {
  if (has_bias) {
    x0 += b0;
    x1 += b1;
  }
  if (has_gamma) {
    const float ss = wave_sum(x0 * x0 + x1 * x1);
    const float scale = 1.0f / sqrtf(ss / 128.0f + eps);
    x0 *= scale * g0;
    x1 *= scale * g1;
  }
  if (has_rope) {
    const float r0 = x0 * c - x1 * s;
    const float r1 = x1 * c + x0 * s;
    x0 = r0;
    x1 = r1;
  }
}
// Same with bias / gamma / rotation fetched here.
template <uint32_t DT>
__device__ __forceinline__ void prep_head128(float x0, float x1, const uint16_t *bias,
                                             const uint16_t *gamma, const float *rope_freq,
                                             const float *rope_cs, uint32_t pos, float eps, int lane,
                                             float *out, uint16_t *out16) {
  float b0 = 0.0f, b1 = 0.0f, g0 = 0.0f, g1 = 0.0f, c = 1.0f, s = 0.0f;
  if (bias != nullptr) {
    b0 = dec16<DT>(bias[lane]);
    b1 = dec16<DT>(bias[lane + 64]);
  }
  if (gamma != nullptr) {
    g0 = dec16<DT>(gamma[lane]);
    g1 = dec16<DT>(gamma[lane + 64]);
  }
  if (rope_freq != nullptr) {
    if (rope_cs != nullptr) {
      c = rope_cs[lane];
      s = rope_cs[64 + lane];
    } else {
      sincosf(static_cast<float>(pos) / rope_freq[lane], &s, &c);
    }
  }
  prep_head128_core<DT>(x0, x1, bias != nullptr, b0, b1, gamma != nullptr, g0, g1, rope_freq != nullptr, c, s, eps,
                        lane, out, out16);
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
// Finite inputs only (the hardware conversions round to nearest even like enc16; they differ
// from it in the NaN bit pattern alone, and neither a scaled query nor a probability is NaN).
template <uint32_t DT>
__device__ __forceinline__ uint16_t enc16_finite(float v) {
  if constexpr (DT == kBF16) return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));  // v_cvt_pk_bf16_f32
  else return f32_to_f16(v);
}
template <uint32_t DT>
__device__ __forceinline__ void split16(float v, uint16_t &hi, uint16_t &lo) {
  hi = enc16_finite<DT>(v);
  lo = enc16_finite<DT>(v - dec16<DT>(hi));
}
// Softmax arithmetic runs in base 2: the query is pre-scaled by log2(e) / sqrt(d), so scores, the
// running maxima m and every exchanged partial maximum are log2-domain numbers and
// exp(s - m) is one v_exp_f32. exp2(-inf) = 0.
__device__ __forceinline__ float attn_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
constexpr float kLog2e = 1.4426950408889634f;

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

// Requests one (physical block, kv head) tile: four 1 KiB loads each for K and V.
__device__ __forceinline__ void attn_load_tile(const AttnParams &p, uint32_t physical_block, uint32_t kvh, int lane,
                                               uint4 (&k)[4], uint4 (&v)[4]) {
  const uint64_t tile = kv_tile_offset(p.block_count, p.kv_heads, kHD, p.layer, physical_block, kvh);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    k[i] = load_stream(p.k_cache + tile + i * 512 + lane * 8);
    v[i] = load_stream(p.v_cache + tile + i * 512 + lane * 8);
  }
}

// One 16-token tile against the G query heads of the kv head (see attn_fast_body).
// n_keys may differ from lane to lane (by column: the prompt kernel's columns belong to tokens at
// different positions). COLUMN_MASKS = a column may find a whole tile masked, even its first one: the
// running maximum then stays at minus infinity, and the exponentials are taken against a finite stand-in
// so that they come out as 0 instead of NaN.
// LAZY_RESCALE = the accumulators are multiplied by alpha only in tiles where some lane's alpha is not 1 (a
// running maximum that did not move gives exp2(0) = 1 exactly, so the result is the same bits): worth a branch
// where a wave walks many tiles and the vector ALU is what it waits for (prompt blocks).
template <uint32_t DT, int G, bool QX_LDS, bool COLUMN_MASKS = false, bool LAZY_RESCALE = false>
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
  const float m_new = fmaxf(m, mb);   // finite: every processed tile has a valid token (without column masks)
  const float m_ref = COLUMN_MASKS ? fmaxf(m_new, -3.0e38f) : m_new;
  const float alpha = attn_exp2(m - m_ref);
  uint32_t px[2];
  float psum = 0.0f;
#pragma unroll
  for (int r = 0; r < 4; r += 2) {
    const float p0 = attn_exp2(sc[r] - m_ref), p1 = attn_exp2(sc[r + 1] - m_ref);
    psum += p0 + p1;
    uint16_t h0, l0, h1, l1;
    split16<DT>(p0, h0, l0);
    split16<DT>(p1, h1, l1);
    px[r / 2] = col < G ? (h0 | (static_cast<uint32_t>(h1) << 16)) : (l0 | (static_cast<uint32_t>(l1) << 16));
  }
  l = l * alpha + psum;
  m = m_new;
  const uint2 pb = make_uint2(px[0], px[1]);
  if constexpr (LAZY_RESCALE) {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int s2 = 0; s2 < 8; ++s2) acc[s2] *= alpha;
    }
  }
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) {
    if constexpr (!LAZY_RESCALE) acc[s2] *= alpha;
    const uint4 &vr = vreg[s2 / 2];
    const uint2 va = (s2 & 1) ? make_uint2(vr.z, vr.w) : make_uint2(vr.x, vr.y);
    acc[s2] = mfma_k16<DT>(va, pb, acc[s2]);
  }
}

// The same tile step for sixteen independent columns (prompt blocks: sixteen (token, head) pairs of a wave). The
// hi and lo halves of a query, and of a tile's probabilities, are two operands of two products that accumulate in the
// same registers instead of two columns that meet by a lane exchange: the same number of matrix instructions per
// pair, but the softmax arithmetic of a lane - the maximum, five exponentials, four hi/lo splits - serves a pair of
// its own instead of being done twice, and a K/V tile read from LDS meets twice as many pairs. Columns are masked
// individually (n_keys by column; a column may find a whole tile masked) and the accumulators are rescaled only
// in tiles where some running maximum moved.
template <uint32_t DT>
__device__ __forceinline__ void attn_tile_wide(const uint4 (&kreg)[4], const uint4 (&vreg)[4], const uint4 (&qhi)[4],
                                               const uint4 (&qlo)[4], uint32_t b, uint32_t n_keys, int grp, float &m,
                                               float &l, f32x4_t (&acc)[8]) {
  // scores of tokens b*16 + grp*4 + r for this lane's column
  f32x4_t c{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) c = mfma_k32<DT>(kreg[j], qhi[j], c);
#pragma unroll
  for (int j = 0; j < 4; ++j) c = mfma_k32<DT>(kreg[j], qlo[j], c);
  float sc[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) sc[r] = b * kKvBlockTokens + grp * 4 + r < n_keys ? c[r] : -INFINITY;
  float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
  mb = fmaxf(mb, __shfl_xor(mb, 16, kWave));
  mb = fmaxf(mb, __shfl_xor(mb, 32, kWave));
  const float m_new = fmaxf(m, mb);
  const float m_ref = fmaxf(m_new, -3.0e38f);   // a column with nothing to see yet: exponentials against a finite stand-in
  const float alpha = attn_exp2(m - m_ref);
  uint32_t ph[2], pl[2];
  float psum = 0.0f;
#pragma unroll
  for (int r = 0; r < 4; r += 2) {
    const float p0 = attn_exp2(sc[r] - m_ref), p1 = attn_exp2(sc[r + 1] - m_ref);
    psum += p0 + p1;
    uint16_t h0, l0, h1, l1;
    split16<DT>(p0, h0, l0);
    split16<DT>(p1, h1, l1);
    ph[r / 2] = h0 | (static_cast<uint32_t>(h1) << 16);
    pl[r / 2] = l0 | (static_cast<uint32_t>(l1) << 16);
  }
  l = l * alpha + psum;
  m = m_new;
  const uint2 pbh = make_uint2(ph[0], ph[1]), pbl = make_uint2(pl[0], pl[1]);
  if (__any(alpha != 1.0f)) {
#pragma unroll
    for (int s2 = 0; s2 < 8; ++s2) acc[s2] *= alpha;
  }
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) {
    const uint4 &vr = vreg[s2 / 2];
    const uint2 va = (s2 & 1) ? make_uint2(vr.z, vr.w) : make_uint2(vr.x, vr.y);
    acc[s2] = mfma_k16<DT>(va, pbh, acc[s2]);
    acc[s2] = mfma_k16<DT>(va, pbl, acc[s2]);
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
  alignas(16) uint4 qx_s[4][kWave];  // lean variant: the query operand of the first product
};

// ---- hand-over between workgroups of one launch ------------------------------------------
// A value that another workgroup of the same launch consumes travels as one 8-byte word
// (f32 value, tag): the consumer polls the word with device-coherent loads until the tag is the
// expected one. A single aligned 8-byte store is indivisible, so a matching tag proves the value;
// no flag, no "stores performed" wait, no cache flush is needed on either side. The consumer
// clears the tag once it has taken the value (launches are ordered by the stream).
__device__ __forceinline__ void store_tagged(uint64_t *ptr, float v, uint32_t epoch) {
  __hip_atomic_store(ptr, (static_cast<uint64_t>(epoch) << 32) | __float_as_uint(v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t load_tagged(const uint64_t *ptr) {
  return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool tag_is(uint64_t word, uint32_t epoch) {
  return static_cast<uint32_t>(word >> 32) == epoch;
}
__device__ __forceinline__ float tag_value(uint64_t word) { return __uint_as_float(static_cast<uint32_t>(word)); }

__device__ __forceinline__ void link_mark(uint64_t *trace, int slot) {
  if (trace != nullptr && threadIdx.x == 0) trace[slot] = wall_clock64();
}

// Everything a wave needs to prepare its heads - raw projections of its query heads
// (g = wave, wave + W, ...) and, on two designated waves, of the new key / value row, with the
// bias, norm weight and rotation of the same dims - requested by the stand-alone kernel before
// anything else and awaited before the first KV tile is requested: loads return in order, so a
// value requested after the tiles could only be used once all of their data had arrived.
struct HeadInputs {
  float x0, x1;
  uint16_t b0, b1;  // bias bits (valid when the bias pointer is set)
};
template <int G, int W>
struct RawHeads {
  HeadInputs q[(G + W - 1) / W];
  HeadInputs e;                  // new key row (wave G % W) or new value row (wave (G + 1) % W)
  uint16_t qg0, qg1, kg0, kg1;   // q_norm / k_norm weight bits
  float rope_a, rope_b;          // cos, sin of this step; without a table: the frequency of the pair
};
template <int G, int W>
__device__ __forceinline__ RawHeads<G, W> attn_request_raw(const AttnParams &p, uint32_t kvh) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t A = p.heads * kHD, KV = p.kv_heads * kHD;
  RawHeads<G, W> r{};
  // one value, or the sum of its K-slice partials in slice order (all requested at once; a slice that does not
  // exist reads slice 0 again and is left out of the sum)
  const uint32_t slices = p.qkv_slices;
  auto raw_value = [&](uint32_t at) {
    if (slices <= 1) return p.qkv[at];
    float part[4];
#pragma unroll
    for (uint32_t s = 0; s < 4; ++s) part[s] = p.qkv[at + (s < slices ? s : 0u) * static_cast<uint64_t>(p.qkv_slice_stride)];
    float sum = 0.0f;
#pragma unroll
    for (uint32_t s = 0; s < 4; ++s) sum = s < slices ? sum + part[s] : sum;
    return sum;
  };
#pragma unroll
  for (int i = 0; i < (G + W - 1) / W; ++i) {
    const uint32_t off = (kvh * G + min(wave + i * W, G - 1)) * kHD;  // clamped: the loads are unconditional
    r.q[i].x0 = raw_value(off + lane);
    r.q[i].x1 = raw_value(off + lane + 64);
    if (p.q_bias != nullptr) {
      r.q[i].b0 = p.q_bias[off + lane];
      r.q[i].b1 = p.q_bias[off + lane + 64];
    }
  }
  const bool value_wave = wave == ((G + 1) % W);
  const uint32_t off = (value_wave ? A + KV : A) + kvh * kHD;
  r.e.x0 = raw_value(off + lane);
  r.e.x1 = raw_value(off + lane + 64);
  const uint16_t *eb = value_wave ? p.v_bias : p.k_bias;
  if (eb != nullptr) {
    r.e.b0 = eb[kvh * kHD + lane];
    r.e.b1 = eb[kvh * kHD + lane + 64];
  }
  if (p.q_norm != nullptr) {
    r.qg0 = p.q_norm[lane];
    r.qg1 = p.q_norm[lane + 64];
  }
  if (p.k_norm != nullptr) {
    r.kg0 = p.k_norm[lane];
    r.kg1 = p.k_norm[lane + 64];
  }
  if (p.rope_freq != nullptr) {
    if (p.rope_cs != nullptr) {
      r.rope_a = p.rope_cs[lane];
      r.rope_b = p.rope_cs[64 + lane];
    } else {
      r.rope_a = p.rope_freq[lane];
    }
  }
  return r;
}

constexpr int kTicketRound = 32;           // splits read per round by the last workgroup of the ticket protocol
// The last workgroup of a kv head merges the splits' partials. Each thread owns output elements (g, d)
// and reads the partials with device-coherent loads, kTicketRound splits per round trip, in split
// order, so the result does not depend on which workgroup arrived last.
template <uint32_t DT, int G, int THREADS>
__device__ __forceinline__ void merge_splits(const AttnParams &p, uint32_t kvh, uint32_t S, uint32_t active, int lane) {
  for (int e = threadIdx.x; e < G * kHD; e += THREADS) {
    const int g = e / kHD, d = e % kHD;
    const uint32_t h = kvh * G + g;
    const float *pm = p.part_m + h * S, *pl = p.part_l + h * S;
    const float *src = p.part_acc + static_cast<uint64_t>(h) * S * kHD + d;
    float M = -INFINITY, L = 0.0f, o = 0.0f;
    for (uint32_t s0 = 0; s0 < active; s0 += kTicketRound) {
      float mm[kTicketRound], ll[kTicketRound], aa[kTicketRound];
      // m and l of this head's splits: the head is the same for all lanes of a wave, so lane i fetches
      // m of split s0 + i and lane kTicketRound + i its l (one load a lane instead of two per split),
      // and the values are handed round with lane reads below.
      static_assert(2 * kTicketRound == kWave && kHD % kWave == 0, "one (m, l) pair per lane pair, one head per wave");
      const uint32_t si_ml = min(s0 + static_cast<uint32_t>(lane & (kTicketRound - 1)), active - 1);
      const float ml = load_coherent((lane < kTicketRound ? pm : pl) + si_ml);
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        // unconditional loads (index clamped): a load under a branch would serialise the round
        const uint32_t si = min(s0 + i, active - 1);
        aa[i] = load_coherent(src + static_cast<uint64_t>(si) * kHD);
      }
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        mm[i] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(ml), i));
        ll[i] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(ml), kTicketRound + i));
      }
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        const bool on = s0 + i < active;
        mm[i] = on ? mm[i] : -INFINITY;
        ll[i] = on ? ll[i] : 0.0f;
        aa[i] = on ? aa[i] : 0.0f;
      }
      float Mc = M;
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) Mc = fmaxf(Mc, mm[i]);
      const float keep = M > -INFINITY ? attn_exp2(M - Mc) : 0.0f;
      L *= keep;
      o *= keep;
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        const float f = mm[i] > -INFINITY ? attn_exp2(mm[i] - Mc) : 0.0f;
        L = fmaf(ll[i], f, L);
        o = fmaf(aa[i], f, o);
      }
      M = Mc;
    }
    if (L > 0.0f && isfinite(L)) o /= L;
    if (p.out_f32 != nullptr) p.out_f32[h * kHD + d] = o;
    p.out16[attn_out_elem(p, h * kHD + d)] = enc16<DT>(o);
  }
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
template <uint32_t DT, int G, int W, int IN_FLIGHT = 4>
__device__ __forceinline__ void attn_fast_body(const AttnParams &p, const uint32_t pos, const uint32_t kvh,
                                               const uint32_t split, const uint32_t S, AttnShared<G, W> &sh,
                                               const RawHeads<G, W> &raw) {
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
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // uniform: block-table reads stay scalar
  // tuning aid: stage timestamps of workgroup (kv head 0, split 0) and of kv head 0's merging workgroup
  uint64_t *const tr = kvh == 0 && split == 0 ? p.trace : nullptr;
  uint64_t *const trm = kvh == 0 ? p.trace : nullptr;
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
  // Up to four tiles in flight per wave (one 8-wave workgroup per CU leaves 256 registers a lane;
  // at the default split factor a wave's whole share of an 8k context is requested at once). The
  // lean variant keeps one, to fit the 128 registers that let two 8-wave workgroups share a CU:
  // prompt blocks, whose launches hold thousands of workgroups and are bound by how many of them a
  // CU can run at a time.
  constexpr int kInFlight = IN_FLIGHT;
  constexpr bool kLean = IN_FLIGHT == 1;  // 128-register budget: the query operand is parked in LDS
  uint4 kreg[kInFlight][4], vreg[kInFlight][4];
  uint32_t b = b0 + wave;
  // the block-table entries first, all of them, so that no tile request waits behind another tile's data
  uint32_t phys[kInFlight];
#pragma unroll
  for (int f = 0; f < kInFlight; ++f) phys[f] = p.table[min(b + f * W, nblk - 1)];
  // the head inputs requested at kernel start have to be in registers before the tiles go out
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int f = 0; f < kInFlight; ++f)
    if (b + f * W < b1) attn_load_tile(p, phys[f], kvh, lane, kreg[f], vreg[f]);

  link_mark(tr, 8);
  // ---- q (all workgroups) and the new K/V row (the workgroup whose range holds pos)
  {
    // every input is in registers already: pure arithmetic while the tiles are in flight
    const bool has_rope = p.rope_freq != nullptr;
    float rc = raw.rope_a, rs = raw.rope_b;
    if (has_rope && p.rope_cs == nullptr) sincosf(static_cast<float>(pos) / raw.rope_a, &rs, &rc);
#pragma unroll
    for (int i = 0; i < (G + W - 1) / W; ++i) {
      const int g = wave + i * W;
      if (g < G)
        prep_head128_core<DT>(raw.q[i].x0, raw.q[i].x1, p.q_bias != nullptr, dec16<DT>(raw.q[i].b0),
                              dec16<DT>(raw.q[i].b1), p.q_norm != nullptr, dec16<DT>(raw.qg0), dec16<DT>(raw.qg1),
                              has_rope, rc, rs, p.eps, lane, q_s[g], nullptr);
    }
    if (owns_new) {
      if (wave == (G % W)) {
        prep_head128_core<DT>(raw.e.x0, raw.e.x1, p.k_bias != nullptr, dec16<DT>(raw.e.b0), dec16<DT>(raw.e.b1),
                              p.k_norm != nullptr, dec16<DT>(raw.kg0), dec16<DT>(raw.kg1), has_rope, rc, rs, p.eps,
                              lane, nullptr, knew);
      } else if (wave == ((G + 1) % W)) {
        prep_head128_core<DT>(raw.e.x0, raw.e.x1, p.v_bias != nullptr, dec16<DT>(raw.e.b0), dec16<DT>(raw.e.b1), false,
                              0.0f, 0.0f, false, 1.0f, 0.0f, p.eps, lane, nullptr, vnew);
      }
    }
  }
  __syncthreads();
  link_mark(tr, 9);
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
  const float scale = kLog2e / sqrtf(static_cast<float>(kHD));

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
  // Under the tighter register budget the operand is parked in LDS (every wave writes the same
  // values, and reads them back after its own writes).
  const uint4 *qx_lds = nullptr;
  if constexpr (kLean) {
#pragma unroll
    for (int j = 0; j < 4; ++j) sh.qx_s[j][lane] = qx[j];
    qx_lds = &sh.qx_s[0][lane];
  }

  link_mark(tr, 10);
  float m = -INFINITY, l = 0.0f;  // of column `col` (both copies of a head track the same values)
  f32x4_t acc[8];                  // O^T[dims s*16 + grp*4 .. +3][col]
#pragma unroll
  for (int s2 = 0; s2 < 8; ++s2) acc[s2] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  for (; b < b1; b += kInFlight * W) {
#pragma unroll
    for (int f = 0; f < kInFlight; ++f) {
      const uint32_t bb = b + f * W;
      if (bb < b1) {
        attn_tile<DT, G, kLean>(kreg[f], vreg[f], qx, qx_lds, bb, n_keys, col, grp, owns_new && bb == new_block, new_row,
                                 knew, vnew, m, l, acc);
        if (bb + kInFlight * W < b1) attn_load_tile(p, p.table[bb + kInFlight * W], kvh, lane, kreg[f], vreg[f]);
      }
    }
  }

  link_mark(tr, 11);
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
    wf[w][g] = wm[w][g] > -INFINITY ? attn_exp2(wm[w][g] - M) : 0.0f;
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
      const uint16_t o16 = enc16<DT>(o);
      p.out16[attn_out_elem(p, h * kHD + d)] = o16;
    } else {
      // The partial leaves through device-coherent stores (written through, no cache flush).
      store_coherent(p.part_acc + (static_cast<uint64_t>(h) * S + split) * kHD + d, o);
      if (d == 0) {
        store_coherent(p.part_m + h * S + split, bM[g]);
        store_coherent(p.part_l + h * S + split, L);
      }
    }
  }
  if (active == 1) return;
  // Every wave waits until its own stores have been performed, the barrier collects the waves,
  // and only then one lane takes the arrival ticket of this kv head.
  wait_stores_performed();
  __syncthreads();
  link_mark(tr, 12);
  if (threadIdx.x == 0) {
    const uint32_t ticket =
        __hip_atomic_fetch_add(p.counters + kvh, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh.is_last = ticket == active - 1 ? 1u : 0u;
  }
  __syncthreads();
  link_mark(tr, 13);
  if (!sh.is_last) return;
  link_mark(trm, 16);
  // ---- the last workgroup of this kv head merges the splits. Each thread owns (g, d) and reads
  // the partials with device-coherent loads, kTicketRound splits per round trip, in split order.
  for (int e = threadIdx.x; e < G * kHD; e += kThreads) {
    const int g = e / kHD, d = e % kHD;
    const uint32_t h = kvh * G + g;
    const float *pm = p.part_m + h * S, *pl = p.part_l + h * S;
    const float *src = p.part_acc + static_cast<uint64_t>(h) * S * kHD + d;
    float M = -INFINITY, L = 0.0f, o = 0.0f;
    for (uint32_t s0 = 0; s0 < active; s0 += kTicketRound) {
      float mm[kTicketRound], ll[kTicketRound], aa[kTicketRound];
      // m and l of this head's splits: the head is the same for all lanes of a wave, so lane i fetches
      // m of split s0 + i and lane kTicketRound + i its l (one load a lane instead of two per split),
      // and the values are handed round with lane reads below.
      static_assert(2 * kTicketRound == kWave && kHD % kWave == 0, "one (m, l) pair per lane pair, one head per wave");
      const uint32_t si_ml = min(s0 + static_cast<uint32_t>(lane & (kTicketRound - 1)), active - 1);
      const float ml = load_coherent((lane < kTicketRound ? pm : pl) + si_ml);
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        // unconditional loads (index clamped): a load under a branch would serialise the round
        const uint32_t si = min(s0 + i, active - 1);
        aa[i] = load_coherent(src + static_cast<uint64_t>(si) * kHD);
      }
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        mm[i] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(ml), i));
        ll[i] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(ml), kTicketRound + i));
      }
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        const bool on = s0 + i < active;
        mm[i] = on ? mm[i] : -INFINITY;
        ll[i] = on ? ll[i] : 0.0f;
        aa[i] = on ? aa[i] : 0.0f;
      }
      float Mc = M;
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) Mc = fmaxf(Mc, mm[i]);
      const float keep = M > -INFINITY ? attn_exp2(M - Mc) : 0.0f;
      L *= keep;
      o *= keep;
#pragma unroll
      for (int i = 0; i < kTicketRound; ++i) {
        const float f = mm[i] > -INFINITY ? attn_exp2(mm[i] - Mc) : 0.0f;
        L = fmaf(ll[i], f, L);
        o = fmaf(aa[i], f, o);
      }
      M = Mc;
    }
    if (L > 0.0f && isfinite(L)) o /= L;
    if (p.out_f32 != nullptr) p.out_f32[h * kHD + d] = o;
    p.out16[attn_out_elem(p, h * kHD + d)] = enc16<DT>(o);
  }
  if (threadIdx.x == 0) __hip_atomic_store(p.counters + kvh, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  link_mark(trm, 17);
}

}  // namespace attn
}  // namespace nv
