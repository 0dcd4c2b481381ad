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
//   * the first U chunks of a wave's rows are requested BEFORE the prologue
//     touches x: the weight stream does not depend on x, so the HBM latency of
//     the first loads overlaps the norm / LDS staging instead of following it;
//   * x lives in LDS as packed 16-bit values (<= 24 KiB at K = 12288), written
//     once per block by the prologue, read with ds_read_b128;
//   * partial sums are reduced with wave shuffles; lane 0 runs the epilogue;
//   * the grid is capped at a few workgroups per CU and waves loop over units
//     with the next unit's head already requested, so the per-workgroup prologue
//     (x staging, RMSNorm) is paid a few hundred times per launch, not per 4 rows.
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

// Device sampler state. The LM-head GEMV (or the stand-alone argmax kernel) stores
// one candidate per workgroup; sample_finish_kernel (one workgroup) reduces them
// and publishes the token. Single-address atomics serialise at ~0.1 us each on
// this part, so thousands of workgroups must not take tickets on one counter.
struct SampleParams {
  float *part_value;       // [kSampleMaxBlocks] per-workgroup best
  uint32_t *part_index;
  uint32_t *part_has;
  NervaHipSyntheticTokenSlot *slots;  // optional: publish slot[pos] and bump the cursor
  uint32_t *cursor_rw;
  uint32_t *token_out;     // optional: plain token output (operator entry point)
  const uint32_t *fault;   // optional: a word that a kernel of this step sets when a bounded wait of its gave up
};

// One lane: hands the step's token out - plain output word and/or slot[pos] in the reference's
// slot format (nerva_cuda_api.h:29-37, sampler.cu:394-407) plus the cursor bump.
__device__ __forceinline__ void publish_token(const SampleParams &s, uint32_t token) {
  if (s.token_out != nullptr) *s.token_out = token;
  if (s.slots != nullptr) {
    const uint32_t pos = *s.cursor_rw;
    NervaHipSyntheticTokenSlot slot;
    slot.request_id = NERVA_HIP_SLOT_REQUEST_ID;
    slot.sequence_id = NERVA_HIP_SLOT_SEQUENCE_ID;
    slot.token_index = pos;
    slot.token = token;
    slot.version = static_cast<uint64_t>(pos) + 1u;
    // a step that gave up somewhere says so in the slot it publishes: the host hands the error out with the token
    slot.completion = s.fault != nullptr && *s.fault != 0u ? NERVA_HIP_SLOT_DEVICE_FAULT : NERVA_HIP_SLOT_DEVICE_COMPLETE;
    slot.host_copied = 0;
    s.slots[pos] = slot;
    *s.cursor_rw = pos + 1u;
  }
}

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
  uint32_t pair_gap;  // kEpiSwiglu: elements left unused between the last gate row and the first up row
  float eps;
  uint32_t round_out;
  const uint32_t *cursor;  // optional step guard: skip when *cursor >= max_steps
  uint32_t max_steps;
  SampleParams sample;
  // test hook of the RMSNorm prologue: when set, workgroup 0 also writes the 16-bit vector the rows
  // are multiplied with (the prologue's output, which otherwise exists in LDS only) to [cols]
  uint16_t *x16_dump;
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

// Issue UU consecutive 512-column chunks of NR rows (loads only).
template <int NR, int UU, int CAP>
__device__ __forceinline__ void chunks_load(const uint16_t *const (&wrow)[NR], uint32_t chunk, int lane,
                                            uint4 (&wv)[NR][CAP]) {
  const uint32_t c0 = chunk * (kWave * 8) + lane * 8;
#pragma unroll
  for (int u = 0; u < UU; ++u)
#pragma unroll
    for (int k = 0; k < NR; ++k) wv[k][u] = load_stream(wrow[k] + c0 + u * (kWave * 8));
}
// Consume them against x in LDS.
template <uint32_t DT, int NR, int UU, int CAP, bool DOT2>
__device__ __forceinline__ void chunks_fma(const uint4 (&wv)[NR][CAP], const uint16_t *xs, uint32_t chunk,
                                           int lane, float (&acc)[NR]) {
  const uint32_t c0 = chunk * (kWave * 8) + lane * 8;
#pragma unroll
  for (int u = 0; u < UU; ++u) {
    const uint4 xv = *reinterpret_cast<const uint4 *>(xs + c0 + u * (kWave * 8));
#pragma unroll
    for (int k = 0; k < NR; ++k) acc[k] = dot8<DT, DOT2>(wv[k][u], xv, acc[k]);
  }
}
template <uint32_t DT, int NR, int UU, bool DOT2>
__device__ __forceinline__ void row_chunks(const uint16_t *const (&wrow)[NR], const uint16_t *xs,
                                           uint32_t chunk, int lane, float (&acc)[NR]) {
  uint4 wv[NR][UU];
  chunks_load<NR, UU, UU>(wrow, chunk, lane, wv);
  chunks_fma<DT, NR, UU, UU, DOT2>(wv, xs, chunk, lane, acc);
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
  const uint32_t units = (EPI == kEpiSwiglu) ? p.rows : (p.rows + NR - 1) / NR;
  const uint32_t wave_global = blockIdx.x * kWavesPerBlock + wave;
  const uint32_t wave_stride = gridDim.x * kWavesPerBlock;
  const uint32_t nchunks = cols / (kWave * 8);

  auto unit_rows = [&](uint32_t unit, uint32_t (&row)[NR], const uint16_t *(&wrow)[NR], bool (&live)[NR]) {
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      if constexpr (EPI == kEpiSwiglu) {
        row[k] = unit + k * p.rows;  // k = 0 gate row, k = 1 up row
        live[k] = true;
      } else {
        row[k] = unit * NR + k;
        live[k] = row[k] < p.rows;
      }
      wrow[k] = p.w + static_cast<uint64_t>(live[k] ? row[k] : 0u) * cols + (EPI == kEpiSwiglu ? k * p.pair_gap : 0u);
    }
  };

  // ---- request the head of this wave's first rows before x is touched -------
  // head = the first min(U, nchunks) chunks (a power of two), the same for every unit.
  const uint32_t head = nchunks >= static_cast<uint32_t>(U) ? U : (U > 4 && nchunks >= 4) ? 4u : (U > 2 && nchunks >= 2) ? 2u : 1u;
  // (a macro, not a lambda: the buffers must stay in VGPRs, and an array that is handed to a
  // closure by reference ends up in scratch memory)
#define NV_GEMV_HEAD_LOAD(UNIT, DST)                                                              \
  do {                                                                                            \
    uint32_t row_[NR];                                                                            \
    const uint16_t *wrow_[NR];                                                                    \
    bool live_[NR];                                                                               \
    unit_rows((UNIT), row_, wrow_, live_);                                                        \
    if (head == static_cast<uint32_t>(U)) chunks_load<NR, U, U>(wrow_, 0, lane, DST);             \
    else if (U > 4 && head == 4) chunks_load<NR, (U > 4 ? 4 : 1), U>(wrow_, 0, lane, DST);        \
    else if (U > 2 && head == 2) chunks_load<NR, (U > 2 ? 2 : 1), U>(wrow_, 0, lane, DST);        \
    else chunks_load<NR, 1, U>(wrow_, 0, lane, DST);                                              \
  } while (0)
  // Two head buffers that swap roles every unit (no register copies: a copy would wait for
  // the very loads it is meant to overlap).
  uint4 buf[2][NR][U];
  if constexpr (MODE == kVecFull) {
    if (wave_global < units) NV_GEMV_HEAD_LOAD(wave_global, buf[0]);
  }

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
      for (uint32_t c = threadIdx.x * 8; c < cols; c += kBlock * 8) {
        const float4 a = *reinterpret_cast<const float4 *>(p.xf + c);
        const float4 b = *reinterpret_cast<const float4 *>(p.xf + c + 4);
        ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
      }
    } else {
      for (uint32_t c = threadIdx.x; c < cols; c += kBlock) ss += p.xf[c] * p.xf[c];
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / static_cast<float>(cols) + p.eps);
    if constexpr (MODE != kScalar) {
      for (uint32_t c = threadIdx.x * 8; c < cols; c += kBlock * 8) {
        const float4 a = *reinterpret_cast<const float4 *>(p.xf + c);   // second touch: L1/L2 hit
        const float4 b = *reinterpret_cast<const float4 *>(p.xf + c + 4);
        const uint4 g = *reinterpret_cast<const uint4 *>(p.gamma + c);
        float g0, g1, g2, g3, g4, g5, g6, g7;
        unpack2<DT>(g.x, g0, g1);
        unpack2<DT>(g.y, g2, g3);
        unpack2<DT>(g.z, g4, g5);
        unpack2<DT>(g.w, g6, g7);
        uint4 o;
        o.x = enc16<DT>(a.x * scale * g0) | (static_cast<uint32_t>(enc16<DT>(a.y * scale * g1)) << 16);
        o.y = enc16<DT>(a.z * scale * g2) | (static_cast<uint32_t>(enc16<DT>(a.w * scale * g3)) << 16);
        o.z = enc16<DT>(b.x * scale * g4) | (static_cast<uint32_t>(enc16<DT>(b.y * scale * g5)) << 16);
        o.w = enc16<DT>(b.z * scale * g6) | (static_cast<uint32_t>(enc16<DT>(b.w * scale * g7)) << 16);
        *reinterpret_cast<uint4 *>(xs + c) = o;
      }
    } else {
      for (uint32_t c = threadIdx.x; c < cols; c += kBlock)
        xs[c] = enc16<DT>(p.xf[c] * scale * dec16<DT>(p.gamma[c]));
    }
  }
  __syncthreads();
  if constexpr (PRO == kProRmsNorm) {
    if (p.x16_dump != nullptr && blockIdx.x == 0)
      for (uint32_t c = threadIdx.x; c < cols; c += kBlock) p.x16_dump[c] = xs[c];
  }

  // ---- main loop: each wave owns NR rows per iteration -------------------
  Best best{0.0f, 0u, 0u};

  // One unit of NR rows per phase. buf[ph] holds the unit's head (requested earlier); the
  // head of the unit after it goes into buf[ph ^ 1] before buf[ph] is consumed, so the
  // wave's load queue is never empty between rows.
  for (uint32_t unit0 = wave_global; unit0 < units; unit0 += 2 * wave_stride) {
#pragma unroll
  for (int ph = 0; ph < 2; ++ph) {
    const uint32_t unit = unit0 + ph * wave_stride;
    if (unit >= units) break;
    uint32_t row[NR];
    const uint16_t *wrow[NR];
    bool live[NR];
    unit_rows(unit, row, wrow, live);
    float acc[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) acc[k] = 0.0f;

    if constexpr (MODE == kVecFull) {
      // cols % 512 == 0: every lane has a full 16-byte chunk in every step, no guards.
      // The head of the NEXT unit is requested before this unit's head is consumed, so the
      // wave never sits with an empty load queue between rows.
      if (unit + wave_stride < units) NV_GEMV_HEAD_LOAD(unit + wave_stride, buf[ph ^ 1]);
      if (head == static_cast<uint32_t>(U)) chunks_fma<DT, NR, U, U, DOT2>(buf[ph], xs, 0, lane, acc);
      else if (U > 4 && head == 4) chunks_fma<DT, NR, (U > 4 ? 4 : 1), U, DOT2>(buf[ph], xs, 0, lane, acc);
      else if (U > 2 && head == 2) chunks_fma<DT, NR, (U > 2 ? 2 : 1), U, DOT2>(buf[ph], xs, 0, lane, acc);
      else chunks_fma<DT, NR, 1, U, DOT2>(buf[ph], xs, 0, lane, acc);
      uint32_t chunk = head;
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
  }
#undef NV_GEMV_HEAD_LOAD

  if constexpr (EPI == kEpiArgmax) {
    // one candidate per workgroup; sample_finish_kernel reduces them
    if (lane == 0) {
      red[wave] = best.value;
      red_i[wave] = best.index;
      red_h[wave] = best.has;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      Best block_best{red[0], red_i[0], red_h[0]};
      for (int w = 1; w < kWavesPerBlock; ++w) {
        Best o{red[w], red_i[w], red_h[w]};
        if (better(o, block_best)) block_best = o;
      }
      p.sample.part_value[blockIdx.x] = block_best.value;
      p.sample.part_index[blockIdx.x] = block_best.index;
      p.sample.part_has[blockIdx.x] = block_best.has;
    }
  }
}

// ---------------------------------------------------------------------------
// Production-shape kernel: cols % (512 * B) == 0, 16-byte aligned rows, cols <= 12288 (30720 with a 16-bit input).
// Same contract as gemv_kernel, leaner register budget (about 64 VGPRs instead of
// ~150) so that 6-8 workgroups stay resident per CU and a whole 4096-row matrix is
// on the machine at once. A wave walks a flat list of request batches - (its 1st
// row, columns 0..512B), (1st row, next 512B columns), ..., (2nd row, ...) - with two
// batches in flight in two register buffers that swap roles (fully unrolled, no
// register copies). The activation vector and the first two weight batches are
// requested before anything waits, the step guard is read after that, and the
// residual element of a row is requested together with the row's first batch. A 16-byte chunk meets its
// eight activations in four packed dot instructions (v_dot2_f32_bf16 / _f16: exact products, f32
// accumulation, 16-bit denormals kept) instead of eight unpack pairs and eight FMAs: a wave's whole share
// arrives at about the same time as its SIMD neighbours', so the arithmetic behind the last data is on the
// launch's critical path (gate_up 32.6 -> 31.8 us, down 17.5 -> 17.1, o 7.45 -> 7.2, LM head 191 -> 187).
// ---------------------------------------------------------------------------
// Register budget as resident waves per SIMD (= workgroups per CU): 6 with a 16-bit input,
// 5 with the RMSNorm prologue, which holds the f32 activations and the norm weights in
// registers across the first weight requests (a budget of 6 makes it spill).
constexpr int fast_waves_per_simd(int prologue) { return prologue == kProRmsNorm ? 5 : 6; }
constexpr int kFastMaxCols = 12288;  // x staged through at most 6 x 16 B per lane in registers ...
constexpr int kFastMaxColsLoop = 30720;  // ... or, with a 16-bit input, copied into LDS behind the first weight requests

// EXACT (short launches: a wave's whole share is the two batches requested up front, so the start-up is
// the launch): the first two batches and the residual element are requested unconditionally - a wave
// without a row asks for the last row's data and drops it - so that the compiler can count the requests
// behind the activation loads and waits for exactly those before the prologue, which then runs under
// the weights' latency. With the requests under `if (total > n)` it waits for everything.
// WG: waves per workgroup (4 or 16). Every workgroup fetches the whole input vector (and for the RMSNorm
// prologue the norm weights) for itself, so fewer, larger workgroups move that much less through the L2s ahead of
// the weights; the waves' work is the same whatever the size (wave_global = workgroup x WG + wave).
// ROT: a unit's walk over its columns starts at batch (unit mod batches per row) and wraps, so the waves of a
// workgroup - and of the launch, which move through their rows at about the same pace - ask for different
// column ranges at any one time instead of all for the same one. Rows are a multiple of the memory channels'
// interleave apart, so without it the launch's requests of a moment land on a part of the channels. Measured
// with the matrices on 2 KiB boundaries (a batch is then whole interleave units; the session's arena and
// hipMalloc'ed buffers are): gate/up pair 32.8 -> 30.8 us (31.5 was the best the plain walk reached at any base),
// qkv at two chunks a batch on 1024 workgroups 10.05 -> 9.65, LM head at one chunk a batch 183.6 -> 178.1; the
// down and o launches do not move (a wave's two 4 KiB batches cover every phase already). The sum over a row
// starts at another column, so results differ from the plain walk's in the last bits (each is deterministic).
// XREG (4096 columns only): a lane's share of the input vector - the eight 16-byte pieces that meet its eight
// weight pieces of a row - is read from LDS once, right after the prologue, and kept in registers, so the
// products behind a batch's arrival do not wait for LDS reads (a wave gets one 1 KiB LDS read through every
// ~30 cycles: eight of them a row were twice the time of the row's 32 dot instructions). Costs 32 registers:
// one wave per SIMD less.
template <uint32_t DT, int PRO, int EPI, int NR, int B, bool EXACT = false, int WG = kWavesPerBlock, bool XREG = false,
          bool ROT = false>
__global__ __launch_bounds__(WG *kWave, XREG ? 4 : fast_waves_per_simd(PRO)) void gemv_fast_kernel(GemvParams p) {
  static_assert(!(ROT && (XREG || EXACT)), "the rotated walk has no exact-start or register-input variant");
  constexpr int TB = WG * kWave;
  constexpr uint32_t kXregBpr = 8 / B;   // batches per 4096-column row
  extern __shared__ __align__(16) uint16_t xs[];
  __shared__ float red[WG];
  __shared__ uint32_t red_i[WG];
  __shared__ uint32_t red_h[WG];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t cols = p.cols;
  const uint32_t units = p.rows;  // NR == 1: rows; kEpiSwiglu (NR == 2): gate/up pairs
  const uint32_t wave_global = blockIdx.x * WG + wave;
  const uint32_t wave_stride = gridDim.x * WG;
  const uint32_t bpr = cols / (kWave * 8 * B);  // request batches per row
  const uint32_t my_units = wave_global < units ? (units - wave_global + wave_stride - 1) / wave_stride : 0u;
  const uint32_t total = my_units * bpr;

  // ---- 1. activation loads (L2 hits), kept in registers until the weights are requested
  constexpr int kXV = (kFastMaxCols + TB * 8 - 1) / (TB * 8);  // 6 with four waves
  uint4 xraw[PRO == kProX16 ? kXV : 1];
  float4 xa[PRO == kProRmsNorm ? 2 : 1], xb[PRO == kProRmsNorm ? 2 : 1];
  uint4 gw[PRO == kProRmsNorm ? 2 : 1];
  const bool norm_in_regs = cols <= TB * 16;
  // (the same for every wave of the launch; a constant in the variant with exact start-up waits, which only
  // runs at 4096 columns, so its request counts stay countable)
  const bool x_in_regs = EXACT || cols <= static_cast<uint32_t>(kFastMaxCols);
  if constexpr (PRO == kProX16) {
    if (x_in_regs) {
#pragma unroll
      for (int i = 0; i < kXV; ++i) {
        const uint32_t c = (i * TB + threadIdx.x) * 8;
        xraw[i] = make_uint4(0u, 0u, 0u, 0u);
        if (c < cols) xraw[i] = *reinterpret_cast<const uint4 *>(p.x16 + c);
      }
    }
  } else {
    if (norm_in_regs) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t c = (i * TB + threadIdx.x) * 8;
        if (c < cols) {
          xa[i] = *reinterpret_cast<const float4 *>(p.xf + c);
          xb[i] = *reinterpret_cast<const float4 *>(p.xf + c + 4);
          gw[i] = *reinterpret_cast<const uint4 *>(p.gamma + c);
        }
      }
    }
  }

  // ---- 2. weight request state + the first two batches
  uint32_t iu = EXACT ? min(wave_global, units - 1) : wave_global, ib = 0;  // next batch to request: unit, batch within the row
  uint32_t ic = 0, cc = 0;            // ROT: column batch being requested / consumed (ic stays 0 otherwise)
  constexpr uint32_t kBatchElems = B * kWave * 8;
  const uint16_t *wp[NR];
  uint4 buf0[NR][B], buf1[NR][B];
  float res0 = 0.0f, res1 = 0.0f;     // residual element requested with a row's first batch
#define NV_FAST_ISSUE(DST, RES)                                                                   \
  do {                                                                                            \
    if (ib == 0) {                                                                                \
      if constexpr (ROT) ic = iu % bpr;                                                           \
      _Pragma("unroll") for (int k = 0; k < NR; ++k)                                              \
        wp[k] = p.w + static_cast<uint64_t>(iu + k * p.rows) * cols + k * p.pair_gap + ic * kBatchElems + lane * 8; \
      if constexpr (EPI == kEpiResidual) {                                                        \
        if (EXACT || lane == 0) RES = p.residual[iu];                                             \
      }                                                                                           \
    }                                                                                             \
    _Pragma("unroll") for (int u = 0; u < B; ++u)                                                 \
      _Pragma("unroll") for (int k = 0; k < NR; ++k) DST[k][u] = load_stream(wp[k] + u * (kWave * 8)); \
    _Pragma("unroll") for (int k = 0; k < NR; ++k) wp[k] += kBatchElems;                              \
    if constexpr (ROT) {                                                                          \
      if (++ic == bpr) {                                                                          \
        ic = 0;                                                                                   \
        _Pragma("unroll") for (int k = 0; k < NR; ++k) wp[k] -= cols;                             \
      }                                                                                           \
    }                                                                                             \
    if (++ib == bpr) {                                                                            \
      ib = 0;                                                                                     \
      iu += wave_stride;                                                                          \
    }                                                                                             \
  } while (0)
  if constexpr (EXACT) {  // the launcher guarantees two batches per row at least
    NV_FAST_ISSUE(buf0, res0);
    NV_FAST_ISSUE(buf1, res1);
  } else {
    if (total > 0) NV_FAST_ISSUE(buf0, res0);
    if (total > 1) NV_FAST_ISSUE(buf1, res1);
  }

  // ---- 3. step guard (after the requests: they do not depend on it and are always in bounds)
  if (p.cursor != nullptr && *p.cursor >= p.max_steps) return;

  // ---- 4. prologue: x -> LDS as 16-bit
  if constexpr (PRO == kProX16) {
    if (x_in_regs) {
#pragma unroll
      for (int i = 0; i < kXV; ++i) {
        const uint32_t c = (i * TB + threadIdx.x) * 8;
        if (c < cols) *reinterpret_cast<uint4 *>(xs + c) = xraw[i];
      }
    } else {
      // rows of more than kFastMaxCols columns (MLP widths above 12288): such a launch is long, its start-up is not
      // what it costs, and the vector would not fit the register budget
      for (uint32_t c = threadIdx.x * 8; c < cols; c += TB * 8)
        *reinterpret_cast<uint4 *>(xs + c) = *reinterpret_cast<const uint4 *>(p.x16 + c);
    }
  } else {
    float ss = 0.0f;
    if (norm_in_regs) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t c = (i * TB + threadIdx.x) * 8;
        if (c < cols)
          ss += xa[i].x * xa[i].x + xa[i].y * xa[i].y + xa[i].z * xa[i].z + xa[i].w * xa[i].w +
                xb[i].x * xb[i].x + xb[i].y * xb[i].y + xb[i].z * xb[i].z + xb[i].w * xb[i].w;
      }
    } else {
      for (uint32_t c = threadIdx.x * 8; c < cols; c += TB * 8) {
        const float4 a = *reinterpret_cast<const float4 *>(p.xf + c);
        const float4 b = *reinterpret_cast<const float4 *>(p.xf + c + 4);
        ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
      }
    }
    ss = block_sum_n<WG>(ss, red);
    const float scale = 1.0f / sqrtf(ss / static_cast<float>(cols) + p.eps);
    auto emit = [&](uint32_t c, const float4 &a, const float4 &b, const uint4 &g) {
      float g0, g1, g2, g3, g4, g5, g6, g7;
      unpack2<DT>(g.x, g0, g1);
      unpack2<DT>(g.y, g2, g3);
      unpack2<DT>(g.z, g4, g5);
      unpack2<DT>(g.w, g6, g7);
      uint4 o;
      o.x = enc16<DT>(a.x * scale * g0) | (static_cast<uint32_t>(enc16<DT>(a.y * scale * g1)) << 16);
      o.y = enc16<DT>(a.z * scale * g2) | (static_cast<uint32_t>(enc16<DT>(a.w * scale * g3)) << 16);
      o.z = enc16<DT>(b.x * scale * g4) | (static_cast<uint32_t>(enc16<DT>(b.y * scale * g5)) << 16);
      o.w = enc16<DT>(b.z * scale * g6) | (static_cast<uint32_t>(enc16<DT>(b.w * scale * g7)) << 16);
      *reinterpret_cast<uint4 *>(xs + c) = o;
    };
    if (norm_in_regs) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t c = (i * TB + threadIdx.x) * 8;
        if (c < cols) emit(c, xa[i], xb[i], gw[i]);
      }
    } else {
      for (uint32_t c = threadIdx.x * 8; c < cols; c += TB * 8)
        emit(c, *reinterpret_cast<const float4 *>(p.xf + c), *reinterpret_cast<const float4 *>(p.xf + c + 4),
             *reinterpret_cast<const uint4 *>(p.gamma + c));
    }
  }
  __syncthreads();
  if constexpr (PRO == kProRmsNorm) {
    if (p.x16_dump != nullptr && blockIdx.x == 0)
      for (uint32_t c = threadIdx.x; c < cols; c += TB) p.x16_dump[c] = xs[c];
  }

  // ---- 5. main loop
  uint4 xr[XREG ? 8 : 1];
  if constexpr (XREG) {
#pragma unroll
    for (int i = 0; i < 8; ++i) xr[i] = *reinterpret_cast<const uint4 *>(xs + i * (kWave * 8) + lane * 8);
  }
  Best best{0.0f, 0u, 0u};
  uint32_t cu = wave_global, cb = 0;  // batch being consumed: unit, batch within the row
  float acc[NR];
  float res_cur = 0.0f;
#define NV_FAST_CONSUME(SRC, RES)                                                                 \
  do {                                                                                            \
    if (cb == 0) {                                                                                \
      _Pragma("unroll") for (int k = 0; k < NR; ++k) acc[k] = 0.0f;                               \
      res_cur = RES;                                                                              \
      if constexpr (ROT) cc = cu % bpr;                                                           \
    }                                                                                             \
    const uint32_t c0 = (ROT ? cc : cb) * (B * kWave * 8) + lane * 8;                             \
    if constexpr (ROT) {                                                                          \
      if (++cc == bpr) cc = 0;                                                                    \
    }                                                                                             \
    _Pragma("unroll") for (int u = 0; u < B; ++u) {                                               \
      uint4 xv;                                                                                   \
      if constexpr (XREG) xv = xr[cb * B + u]; /* cb is a constant at every use in this mode */   \
      else xv = *reinterpret_cast<const uint4 *>(xs + c0 + u * (kWave * 8));                      \
      _Pragma("unroll") for (int k = 0; k < NR; ++k) acc[k] = dot8<DT, true>(SRC[k][u], xv, acc[k]);  \
    }                                                                                             \
    if (++cb == (XREG ? kXregBpr : bpr)) {                                                        \
      cb = 0;                                                                                     \
      _Pragma("unroll") for (int k = 0; k < NR; ++k) acc[k] = wave_sum(acc[k]);                   \
      if (lane == 0) {                                                                            \
        if constexpr (EPI == kEpiSwiglu) {                                                        \
          float g = acc[0], u = acc[NR - 1];                                                      \
          if (p.bias != nullptr) {                                                                \
            g += dec16<DT>(p.bias[cu]);                                                           \
            u += dec16<DT>(p.bias[cu + p.rows]);                                                  \
          }                                                                                       \
          p.out16[cu] = enc16<DT>(silu(g) * u);                                                   \
        } else {                                                                                  \
          float y = acc[0];                                                                       \
          if (p.bias != nullptr) y += dec16<DT>(p.bias[cu]);                                      \
          if constexpr (EPI == kEpiF32) {                                                         \
            p.out_f32[cu] = y;                                                                    \
          } else if constexpr (EPI == kEpiResidual) {                                             \
            y += res_cur;                                                                         \
            if (p.round_out) y = round16<DT>(y);                                                  \
            p.out_f32[cu] = y;                                                                    \
          } else if constexpr (EPI == kEpiOut16) {                                                \
            p.out16[cu] = enc16<DT>(y);                                                           \
          } else if constexpr (EPI == kEpiArgmax) {                                               \
            p.out_f32[cu] = y;                                                                    \
            Best cand{y, cu, isfinite(y) ? 1u : 0u};                                              \
            if (better(cand, best)) best = cand;                                                  \
          }                                                                                       \
        }                                                                                         \
      }                                                                                           \
      cu += wave_stride;                                                                          \
    }                                                                                             \
  } while (0)

  if constexpr (XREG) {
    // one unit per turn: its batches alternate between the two buffers, the batch index is a constant
    for (uint32_t t = 0; t < total; t += kXregBpr) {
      cb = 0;
      NV_FAST_CONSUME(buf0, res0);
      if (t + 2 < total) NV_FAST_ISSUE(buf0, res0);
      cb = 1;
      NV_FAST_CONSUME(buf1, res1);
      if (t + 3 < total) NV_FAST_ISSUE(buf1, res1);
      if constexpr (kXregBpr == 4) {
        cb = 2;
        NV_FAST_CONSUME(buf0, res0);
        if (t + 4 < total) NV_FAST_ISSUE(buf0, res0);
        cb = 3;
        NV_FAST_CONSUME(buf1, res1);
        if (t + 5 < total) NV_FAST_ISSUE(buf1, res1);
      }
    }
  } else {
    for (uint32_t t = 0; t < total; t += 2) {
      NV_FAST_CONSUME(buf0, res0);
      if (t + 2 < total) NV_FAST_ISSUE(buf0, res0);
      if (t + 1 < total) {
        NV_FAST_CONSUME(buf1, res1);
        if (t + 3 < total) NV_FAST_ISSUE(buf1, res1);
      }
    }
  }
#undef NV_FAST_ISSUE
#undef NV_FAST_CONSUME

  if constexpr (EPI == kEpiArgmax) {
    if (lane == 0) {
      red[wave] = best.value;
      red_i[wave] = best.index;
      red_h[wave] = best.has;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      Best block_best{red[0], red_i[0], red_h[0]};
      for (int w = 1; w < WG; ++w) {
        Best o{red[w], red_i[w], red_h[w]};
        if (better(o, block_best)) block_best = o;
      }
      p.sample.part_value[blockIdx.x] = block_best.value;
      p.sample.part_index[blockIdx.x] = block_best.index;
      p.sample.part_has[blockIdx.x] = block_best.has;
    }
  }
}

// Host-side tuning knobs (overridable for sweeps).
struct GemvTuning {
  int max_blocks = 0;      // 0 = library default (a few workgroups per CU)
  bool force_generic = false;  // never take the lean production-shape kernel
};

// `blocks_used`, when given, receives the number of workgroups launched: an LM-head launch leaves
// exactly that many sampler candidates, so the finishing launch takes its count from here.
hipError_t launch_gemv(uint32_t dtype, int prologue, int epilogue, const GemvParams &p,
                       hipStream_t stream, const GemvTuning *tuning = nullptr, uint32_t *blocks_used = nullptr);
// Kernel variant and grid of a launch (shared by the launcher and by callers that size
// per-workgroup outputs). `vec16` = every pointer is 16-byte aligned.
struct GemvPlan {
  int mode;         // kScalar / kVecGuarded / kVecFull / kFast
  uint32_t blocks;  // four-wave workgroups' worth of waves
  int wg_waves;     // waves per workgroup the launch uses (kFast: 4 or 16)
  uint32_t grid;    // workgroups launched: ceil(blocks * 4 / wg_waves)
  bool rotated;     // kFast: the rotated walk (see gemv_fast_kernel)
  int chunks;       // kFast: 1 KiB chunks per row and request batch
};
constexpr int kFast = 3;  // the lean production-shape kernel
GemvPlan gemv_plan(int prologue, int epilogue, uint32_t rows, uint32_t cols, bool vec16,
                   const struct GemvTuning *tuning);
// Reduce `count` per-workgroup candidates and publish the token (one workgroup).
hipError_t launch_sample_finish(const SampleParams &s, uint32_t count, const uint32_t *cursor,
                                uint32_t max_steps, hipStream_t stream);
constexpr uint32_t kSampleMaxBlocks = 65536;  // capacity of SampleParams::part_* arrays

}  // namespace nv
