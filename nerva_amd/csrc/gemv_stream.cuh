// Weight-streaming GEMV for batch-1 decode: y = W.x, W row-major [rows x cols]
// 16-bit, f32 accumulation. HBM-bound: the only goal is to keep as many 16-byte
// loads of W in flight per CU as the memory system can absorb, and to fold the
// element-wise work of the decode step into the prologue/epilogue so that a
// transformer layer is 4 GEMV launches + 1 attention launch.
//
// Mapping (gfx950, wave64):
//   * one wave owns NR rows at a time and walks the full K extent with
//     64 lanes x 16 B = 1 KiB per load instruction; U x NR loads are issued
//     back to back before the first FMA (U*NR KiB in flight per wave);
//   * x lives in LDS as packed 16-bit values (<= 24 KiB at K = 12288), written
//     once per block by the prologue, read with ds_read_b128;
//   * partial sums are reduced with wave shuffles; lane 0 runs the epilogue.
//
// Reference contracts: mat_vec_encoded_row_major (precision/block/ops.rs:75-91),
// rms_norm_to_encoded (device_ops.cuh:317-332), mlp-norm/ff/finish kernels
// (kernels.cu:577-612,651-687), greedy sampler (sampler.cu:89-119,394-407).
#pragma once

#include "nerva_hip_api.h"
#include "nv_common.cuh"

namespace nv {

enum : int { kProX16 = 0, kProRmsNorm = 1 };
enum : int { kEpiF32 = 0, kEpiResidual = 1, kEpiSwiglu = 2, kEpiOut16 = 3, kEpiArgmax = 4 };

struct SampleParams {
  float *part_value;       // [grid] per-block best
  uint32_t *part_index;    // [grid]
  uint32_t *part_has;      // [grid]
  uint32_t *counter;       // arrival counter, zero between launches
  NervaHipSyntheticTokenSlot *slots;  // optional: publish slot[pos] and bump the cursor
  uint32_t *cursor_rw;
  uint32_t *token_out;     // optional: plain token output (operator entry point)
};

struct GemvParams {
  const uint16_t *w;
  const uint16_t *x16;
  const float *xf;
  const uint16_t *gamma;
  const uint16_t *bias;
  const float *residual;
  float *out_f32;
  uint16_t *out16;
  uint32_t rows;   // output rows (kEpiSwiglu: pairs; W holds 2*rows rows, gate first)
  uint32_t cols;
  float eps;
  uint32_t round_out;
  const uint32_t *cursor;  // optional step guard: skip when *cursor >= max_steps
  uint32_t max_steps;
  SampleParams sample;
};

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

template <uint32_t DT, bool DOT2>
__device__ __forceinline__ float dot2w(uint32_t w, uint32_t x, float acc) {
  if constexpr (DOT2) {
    if constexpr (DT == kBF16)
      return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w),
                                             __builtin_bit_cast(bf16x2_t, x), acc, false);
    else
      return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, w), __builtin_bit_cast(f16x2_t, x),
                                    acc, false);
  } else {
    float w0, w1, x0, x1;
    unpack2<DT>(w, w0, w1);
    unpack2<DT>(x, x0, x1);
    acc = fmaf(w0, x0, acc);
    return fmaf(w1, x1, acc);
  }
}
template <uint32_t DT, bool DOT2>
__device__ __forceinline__ float dot8(const uint4 &w, const uint4 &x, float acc) {
  acc = dot2w<DT, DOT2>(w.x, x.x, acc);
  acc = dot2w<DT, DOT2>(w.y, x.y, acc);
  acc = dot2w<DT, DOT2>(w.z, x.z, acc);
  return dot2w<DT, DOT2>(w.w, x.w, acc);
}

// Final stage of the device sampler: called by every block after it has stored
// its per-block best; the last block to arrive reduces all partials, publishes
// the token and re-arms the counter. No block waits on another.
__device__ __forceinline__ void sample_finish(const SampleParams &s, Best block_best, float *red_v,
                                              uint32_t *red_i, uint32_t *red_h) {
  __shared__ uint32_t is_last;
  const uint32_t nblocks = gridDim.x;
  if (threadIdx.x == 0) {
    s.part_value[blockIdx.x] = block_best.value;
    s.part_index[blockIdx.x] = block_best.index;
    s.part_has[blockIdx.x] = block_best.has;
    __threadfence();
    uint32_t ticket = __hip_atomic_fetch_add(s.counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    is_last = ticket == nblocks - 1 ? 1u : 0u;
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();
  Best b{0.0f, 0u, 0u};
  for (uint32_t i = threadIdx.x; i < nblocks; i += kBlock) {
    Best o;
    o.value = __hip_atomic_load(s.part_value + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    o.index = __hip_atomic_load(s.part_index + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    o.has = __hip_atomic_load(s.part_has + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (better(o, b)) b = o;
  }
  b = wave_best(b);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    red_v[wave] = b.value;
    red_i[wave] = b.index;
    red_h[wave] = b.has;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    Best t{red_v[0], red_i[0], red_h[0]};
    for (int w = 1; w < kWavesPerBlock; ++w) {
      Best o{red_v[w], red_i[w], red_h[w]};
      if (better(o, t)) t = o;
    }
    const uint32_t token = t.has ? t.index : 0u;
    if (s.token_out != nullptr) *s.token_out = token;
    if (s.slots != nullptr) {
      const uint32_t pos = *s.cursor_rw;
      NervaHipSyntheticTokenSlot slot;
      slot.request_id = NERVA_HIP_SLOT_REQUEST_ID;
      slot.sequence_id = NERVA_HIP_SLOT_SEQUENCE_ID;
      slot.token_index = pos;
      slot.token = token;
      slot.version = static_cast<uint64_t>(pos) + 1u;
      slot.completion = NERVA_HIP_SLOT_DEVICE_COMPLETE;
      slot.host_copied = 0;
      s.slots[pos] = slot;
      *s.cursor_rw = pos + 1u;
    }
    __hip_atomic_store(s.counter, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// UU consecutive 512-column chunks of NR rows: all UU*NR loads are issued before
// the first FMA so that the wave keeps UU*NR KiB in flight.
template <uint32_t DT, int NR, int UU, bool DOT2>
__device__ __forceinline__ void row_chunks(const uint16_t *const (&wrow)[NR], const uint16_t *xs,
                                           uint32_t chunk, int lane, float (&acc)[NR]) {
  uint4 wv[NR][UU];
  const uint32_t c0 = chunk * (kWave * 8) + lane * 8;
#pragma unroll
  for (int u = 0; u < UU; ++u)
#pragma unroll
    for (int k = 0; k < NR; ++k) wv[k][u] = load_stream(wrow[k] + c0 + u * (kWave * 8));
#pragma unroll
  for (int u = 0; u < UU; ++u) {
    const uint4 xv = *reinterpret_cast<const uint4 *>(xs + c0 + u * (kWave * 8));
#pragma unroll
    for (int k = 0; k < NR; ++k) acc[k] = dot8<DT, DOT2>(wv[k][u], xv, acc[k]);
  }
}

enum : int { kScalar = 0, kVecGuarded = 1, kVecFull = 2 };

// MODE kVecFull: cols % 512 == 0 and 16-byte aligned rows (every production
// shape). kVecGuarded: cols % 8 == 0. kScalar: anything (tiny known-answer
// models with hidden = 2 take it).
template <uint32_t DT, int PRO, int EPI, int NR, int U, int MODE, bool DOT2>
__global__ __launch_bounds__(kBlock) void gemv_kernel(GemvParams p) {
  extern __shared__ __align__(16) uint16_t xs[];  // cols (rounded up to 8) 16-bit values
  __shared__ float red[kWavesPerBlock];
  __shared__ uint32_t red_i[kWavesPerBlock];
  __shared__ uint32_t red_h[kWavesPerBlock];

  if (p.cursor != nullptr && *p.cursor >= p.max_steps) return;

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t cols = p.cols;

  // ---- prologue: x -> LDS as 16-bit ------------------------------------
  if constexpr (PRO == kProX16) {
    if constexpr (MODE != kScalar) {
      for (uint32_t c = threadIdx.x * 8; c < cols; c += kBlock * 8)
        *reinterpret_cast<uint4 *>(xs + c) = *reinterpret_cast<const uint4 *>(p.x16 + c);
    } else {
      for (uint32_t c = threadIdx.x; c < cols; c += kBlock) xs[c] = p.x16[c];
    }
  } else {
    // x = round16(v * rsqrt(mean(v^2) + eps) * gamma)
    float ss = 0.0f;
    if constexpr (MODE != kScalar) {
      for (uint32_t c = threadIdx.x * 4; c < cols; c += kBlock * 4) {
        const float4 v = *reinterpret_cast<const float4 *>(p.xf + c);
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
    } else {
      for (uint32_t c = threadIdx.x; c < cols; c += kBlock) ss += p.xf[c] * p.xf[c];
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / static_cast<float>(cols) + p.eps);
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock)
      xs[c] = enc16<DT>(p.xf[c] * scale * dec16<DT>(p.gamma[c]));
  }
  __syncthreads();

  // ---- main loop: each wave owns NR rows per iteration -------------------
  const uint32_t units = (EPI == kEpiSwiglu) ? p.rows : (p.rows + NR - 1) / NR;
  const uint32_t wave_global = blockIdx.x * kWavesPerBlock + wave;
  const uint32_t wave_stride = gridDim.x * kWavesPerBlock;
  Best best{0.0f, 0u, 0u};

  for (uint32_t unit = wave_global; unit < units; unit += wave_stride) {
    uint32_t row[NR];
    const uint16_t *wrow[NR];
    bool live[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      if constexpr (EPI == kEpiSwiglu) {
        row[k] = unit + k * p.rows;  // k = 0 gate row, k = 1 up row
        live[k] = true;
      } else {
        row[k] = unit * NR + k;
        live[k] = row[k] < p.rows;
      }
      wrow[k] = p.w + static_cast<uint64_t>(live[k] ? row[k] : 0u) * cols;
    }
    float acc[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) acc[k] = 0.0f;

    if constexpr (MODE == kVecFull) {
      // cols % 512 == 0: every lane has a full 16-byte chunk in every step, no guards.
      uint32_t chunk = 0;
      const uint32_t nchunks = cols / (kWave * 8);
      for (; chunk + U <= nchunks; chunk += U) row_chunks<DT, NR, U, DOT2>(wrow, xs, chunk, lane, acc);
      if constexpr (U > 4) {
        if (chunk + 4 <= nchunks) {
          row_chunks<DT, NR, 4, DOT2>(wrow, xs, chunk, lane, acc);
          chunk += 4;
        }
      }
      if constexpr (U > 2) {
        if (chunk + 2 <= nchunks) {
          row_chunks<DT, NR, 2, DOT2>(wrow, xs, chunk, lane, acc);
          chunk += 2;
        }
      }
      if constexpr (U > 1) {
        if (chunk < nchunks) row_chunks<DT, NR, 1, DOT2>(wrow, xs, chunk, lane, acc);
      }
    } else if constexpr (MODE == kVecGuarded) {
      for (uint32_t base = 0; base < cols; base += kWave * 8 * U) {
        uint4 wv[NR][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t c = base + u * (kWave * 8) + lane * 8;
#pragma unroll
          for (int k = 0; k < NR; ++k)
            wv[k][u] = (c < cols) ? load_stream(wrow[k] + c) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const uint32_t c = base + u * (kWave * 8) + lane * 8;
          if (c < cols) {
            const uint4 xv = *reinterpret_cast<const uint4 *>(xs + c);
#pragma unroll
            for (int k = 0; k < NR; ++k) acc[k] = dot8<DT, DOT2>(wv[k][u], xv, acc[k]);
          }
        }
      }
    } else {
      for (uint32_t c = lane; c < cols; c += kWave) {
        const float xv = dec16<DT>(xs[c]);
#pragma unroll
        for (int k = 0; k < NR; ++k) acc[k] = fmaf(dec16<DT>(wrow[k][c]), xv, acc[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) acc[k] = wave_sum(acc[k]);

    // ---- epilogue (lane 0) ------------------------------------------------
    if (lane == 0) {
      if constexpr (EPI == kEpiSwiglu) {
        float g = acc[0], u = acc[1];
        if (p.bias != nullptr) {
          g += dec16<DT>(p.bias[row[0]]);
          u += dec16<DT>(p.bias[row[1]]);
        }
        p.out16[unit] = enc16<DT>(silu(g) * u);
      } else {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
          if (!live[k]) continue;
          float y = acc[k];
          if (p.bias != nullptr) y += dec16<DT>(p.bias[row[k]]);
          if constexpr (EPI == kEpiF32) {
            p.out_f32[row[k]] = y;
          } else if constexpr (EPI == kEpiResidual) {
            y += p.residual[row[k]];
            if (p.round_out) y = round16<DT>(y);
            p.out_f32[row[k]] = y;
          } else if constexpr (EPI == kEpiOut16) {
            p.out16[row[k]] = enc16<DT>(y);
          } else if constexpr (EPI == kEpiArgmax) {
            p.out_f32[row[k]] = y;
            Best cand{y, row[k], isfinite(y) ? 1u : 0u};
            if (better(cand, best)) best = cand;
          }
        }
      }
    }
  }

  if constexpr (EPI == kEpiArgmax) {
    if (lane == 0) {
      red[wave] = best.value;
      red_i[wave] = best.index;
      red_h[wave] = best.has;
    }
    __syncthreads();
    Best block_best{red[0], red_i[0], red_h[0]};
    for (int w = 1; w < kWavesPerBlock; ++w) {
      Best o{red[w], red_i[w], red_h[w]};
      if (better(o, block_best)) block_best = o;
    }
    __syncthreads();
    sample_finish(p.sample, block_best, red, red_i, red_h);
  }
}

// Host-side tuning knobs (set by the launcher; overridable for sweeps).
struct GemvTuning {
  int rows_per_wave = 2;   // NR for non-swiglu epilogues (1 or 2)
  int unroll = 8;          // U (4 or 8)
  int dot2 = 0;
  int max_blocks = 0;      // 0 = automatic
};

hipError_t launch_gemv(uint32_t dtype, int prologue, int epilogue, const GemvParams &p,
                       hipStream_t stream, const GemvTuning *tuning = nullptr);
uint32_t gemv_grid_blocks(int epilogue, uint32_t rows, int rows_per_wave, int max_blocks);
constexpr uint32_t kSampleMaxBlocks = 4096;  // capacity of SampleParams::part_* arrays

}  // namespace nv
