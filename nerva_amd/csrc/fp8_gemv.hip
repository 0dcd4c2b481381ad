// FP8-e4m3fn weight-streaming GEMV with f32 block scales, and the MoE expert
// kernels built on it. Weights are dequantised in f32 registers
// (value = e4m3(W[r,c]) * S[r/br][c/bc], no 16-bit rounding in between), which
// is the contract of the reference's own check
// (crates/nerva-cuda/src/tests/deepseek_quant.rs:689-713); the reference CUDA
// kernel's extra bf16 rounding (deepseek/projection.inc.cu:19-23) is not reproduced.
//
// Mapping: one wave owns NR rows; a load instruction covers 64 lanes x 16 B =
// 1024 columns; a lane's 16 weights share one block scale when block_cols is a
// multiple of 16, so the scale multiplies a 16-term partial sum once.
// Kernels, from general to lean: fp8_gemv_kernel / moe_gate_up_kernel / moe_down_kernel (any shape; several
// tokens; f32 or 16-bit activations, kept in LDS as f32 or - K a multiple of 1024 - as they came), then
// lean_pair_stream with its two users fp8_gemv_lean_kernel (one token, 16-bit activations, K a multiple of 16)
// and moe_gate_up_lean_kernel, and moe_down_lean_kernel: hand-issued request rings with exact waits.
#include "fp8_gemv.cuh"

#include <algorithm>

#include "fp8_codec.cuh"

namespace nv {

namespace {

__device__ __forceinline__ float dot16_fp8(const uint4 &w, const float *x) {
  float f[4];
  float acc = 0.0f;
  const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    fp8x4_to_f32(words[i], f);
    const float4 xv = *reinterpret_cast<const float4 *>(x + 4 * i);
    acc = fmaf(f[0], xv.x, acc);
    acc = fmaf(f[1], xv.y, acc);
    acc = fmaf(f[2], xv.z, acc);
    acc = fmaf(f[3], xv.w, acc);
  }
  return acc;
}

// Lean-kernel operand order in LDS. A lane owns 16 consecutive columns of every 1024-column chunk
// (the 16 weights of its 16-byte request). Stored column after column, the lanes of a wave would read
// 16-byte pieces 64 bytes apart (32 for 16-bit values) and collide on the banks; instead a chunk is
// kept as planes of one 16-byte piece per lane - piece j of lane l at [chunk][j][l] - so that a wave's
// read of piece j is 1 KiB in a row.
//   f32 values: 4 planes of 4 columns; 16-bit values: 2 planes of 8 columns.
__device__ __forceinline__ uint32_t lean_slot_f32(uint32_t c) {
  const uint32_t i = c & 15u, lane = (c >> 4) & 63u;
  return (c & ~1023u) + (i >> 2) * 256u + lane * 4u + (i & 3u);
}
__device__ __forceinline__ uint32_t lean_slot_16(uint32_t c) {
  const uint32_t i = c & 15u, lane = (c >> 4) & 63u;
  return (c & ~1023u) + (i >> 3) * 512u + lane * 8u + (i & 7u);
}

// 16 e4m3fn weights times the lane's 16 f32 activations in lean order (xp -> piece 0 of the lane).
__device__ __forceinline__ float dot16_fp8_lean(const uint4 &w, const float *xp) {
  float f[4];
  float acc = 0.0f;
  const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    fp8x4_to_f32(words[i], f);
    const float4 xv = *reinterpret_cast<const float4 *>(xp + 256 * i);
    acc = fmaf(f[0], xv.x, acc);
    acc = fmaf(f[1], xv.y, acc);
    acc = fmaf(f[2], xv.z, acc);
    acc = fmaf(f[3], xv.w, acc);
  }
  return acc;
}

// The same against 16-bit activations: e4m3fn values are exact in bf16 and in f16, so two weights
// become one packed 16-bit pair (gfx950 scaled conversion, scale 1) and meet their activation pair in
// one dot2 with f32 accumulation - half the instructions and half the LDS bytes of the f32 route.
typedef __bf16 lean_bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 lean_f16x2_t __attribute__((ext_vector_type(2)));
template <uint32_t DT>
__device__ __forceinline__ float dot4_fp8_x16(uint32_t w, uint32_t x01, uint32_t x23, float acc) {
  if constexpr (DT == kBF16) {
    const lean_bf16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
    const lean_bf16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
    acc = __builtin_amdgcn_fdot2_f32_bf16(lo, __builtin_bit_cast(lean_bf16x2_t, x01), acc, false);
    return __builtin_amdgcn_fdot2_f32_bf16(hi, __builtin_bit_cast(lean_bf16x2_t, x23), acc, false);
  } else {
    const lean_f16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
    const lean_f16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
    acc = __builtin_amdgcn_fdot2(lo, __builtin_bit_cast(lean_f16x2_t, x01), acc, false);
    return __builtin_amdgcn_fdot2(hi, __builtin_bit_cast(lean_f16x2_t, x23), acc, false);
  }
}
template <uint32_t DT>
__device__ __forceinline__ float dot16_fp8_x16(const uint4 &w, const uint4 &xa, const uint4 &xb) {
  float acc = dot4_fp8_x16<DT>(w.x, xa.x, xa.y, 0.0f);
  acc = dot4_fp8_x16<DT>(w.y, xa.z, xa.w, acc);
  acc = dot4_fp8_x16<DT>(w.z, xb.x, xb.y, acc);
  return dot4_fp8_x16<DT>(w.w, xb.z, xb.w, acc);
}

// Stage x (16-bit or f32) into LDS. ORDER 0: f32, column after column; 1: f32 in lean order; 2: the
// 16-bit values as they came, in lean order (x16 only, 16-byte aligned, cols % 8 == 0).
constexpr int kXColumns = 0, kXLeanF32 = 1, kXLean16 = 2;
template <uint32_t DT, int ORDER = kXColumns>
__device__ __forceinline__ void stage_x(float *xs, const uint16_t *x16, const float *xf, uint32_t cols) {
  if constexpr (ORDER == kXLean16) {
    uint16_t *xs16 = reinterpret_cast<uint16_t *>(xs);
    for (uint32_t c = threadIdx.x * 8; c < cols; c += kBlock * 8)
      *reinterpret_cast<uint4 *>(xs16 + lean_slot_16(c)) = *reinterpret_cast<const uint4 *>(x16 + c);
  } else if (x16 != nullptr) {
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock)
      xs[ORDER == kXLeanF32 ? lean_slot_f32(c) : c] = dec16<DT>(x16[c]);
  } else {
    for (uint32_t c = threadIdx.x; c < cols; c += kBlock) xs[ORDER == kXLeanF32 ? lean_slot_f32(c) : c] = xf[c];
  }
}

// UU consecutive 1024-column chunks of NR rows, all loads issued before the first use. XT says how the
// activations lie in LDS (lean orders: see lean_slot_f32 / lean_slot_16).
template <uint32_t DT, int NR, int UU, int XT>
__device__ __forceinline__ void fp8_chunks(const uint8_t *const (&wrow)[NR], const float *const (&srow)[NR],
                                           const float *xs, uint32_t chunk, uint32_t block_cols,
                                           int lane, float (&acc)[NR]) {
  uint4 wv[NR][UU];
  const uint32_t c0 = chunk * 1024u + lane * 16;
#pragma unroll
  for (int u = 0; u < UU; ++u)
#pragma unroll
    for (int k = 0; k < NR; ++k) wv[k][u] = load_stream(wrow[k] + c0 + u * 1024u);
#pragma unroll
  for (int u = 0; u < UU; ++u) {
    const uint32_t c = c0 + u * 1024u;
    const uint32_t sidx = c / block_cols;
    if constexpr (XT == kXLean16) {
      const uint16_t *xp = reinterpret_cast<const uint16_t *>(xs) + (chunk + u) * 1024u + lane * 8;
      const uint4 xa = *reinterpret_cast<const uint4 *>(xp), xb = *reinterpret_cast<const uint4 *>(xp + 512);
#pragma unroll
      for (int k = 0; k < NR; ++k) acc[k] = fmaf(srow[k][sidx], dot16_fp8_x16<DT>(wv[k][u], xa, xb), acc[k]);
    } else if constexpr (XT == kXLeanF32) {
      const float *xp = xs + (chunk + u) * 1024u + lane * 4;
#pragma unroll
      for (int k = 0; k < NR; ++k) acc[k] = fmaf(srow[k][sidx], dot16_fp8_lean(wv[k][u], xp), acc[k]);
    } else {
#pragma unroll
      for (int k = 0; k < NR; ++k) acc[k] = fmaf(srow[k][sidx], dot16_fp8(wv[k][u], xs + c), acc[k]);
    }
  }
}

// NR rows x all columns for one wave; FAST: cols % 1024 == 0, block_cols % 16 == 0,
// 16-byte aligned rows, activations in a lean order (XT); otherwise column order.
template <uint32_t DT, int NR, bool FAST, int XT>
__device__ __forceinline__ void fp8_rows(const uint8_t *const (&wrow)[NR], const float *const (&srow)[NR],
                                         const float *xs, uint32_t cols, uint32_t block_cols, int lane,
                                         float (&acc)[NR]) {
  static_assert(FAST ? XT != kXColumns : XT == kXColumns, "lean orders belong to the chunked path");
  if constexpr (FAST) {
    const uint32_t nchunks = cols / 1024u;
    uint32_t chunk = 0;
    for (; chunk + 4 <= nchunks; chunk += 4) fp8_chunks<DT, NR, 4, XT>(wrow, srow, xs, chunk, block_cols, lane, acc);
    if (chunk + 2 <= nchunks) {
      fp8_chunks<DT, NR, 2, XT>(wrow, srow, xs, chunk, block_cols, lane, acc);
      chunk += 2;
    }
    if (chunk < nchunks) fp8_chunks<DT, NR, 1, XT>(wrow, srow, xs, chunk, block_cols, lane, acc);
  } else {
    for (uint32_t c = lane; c < cols; c += kWave) {
#pragma unroll
      for (int k = 0; k < NR; ++k) {
        const float w = fp8_e4m3fn_to_f32_sw(wrow[k][c]) * srow[k][c / block_cols];
        acc[k] = fmaf(w, xs[c], acc[k]);
      }
    }
  }
}

template <uint32_t DT, int NR, bool FAST, int XT = FAST ? kXLeanF32 : kXColumns>
__global__ __launch_bounds__(kBlock) void fp8_gemv_kernel(Fp8GemvParams p) {
  extern __shared__ __align__(16) float xsf[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (uint32_t token = 0; token < p.tokens; ++token) {
    if (token != 0) __syncthreads();
    stage_x<DT, XT>(xsf, p.x16 ? p.x16 + static_cast<uint64_t>(token) * p.cols : nullptr,
                    p.xf ? p.xf + static_cast<uint64_t>(token) * p.cols : nullptr, p.cols);
    __syncthreads();
    const uint32_t scale_cols = (p.cols + p.block_cols - 1) / p.block_cols;
    const uint32_t units = (p.rows + NR - 1) / NR;
    for (uint32_t unit = blockIdx.x * kWavesPerBlock + wave; unit < units;
         unit += gridDim.x * kWavesPerBlock) {
      const uint8_t *wrow[NR];
      const float *srow[NR];
      float acc[NR];
#pragma unroll
      for (int k = 0; k < NR; ++k) {
        const uint32_t r = min(unit * NR + k, p.rows - 1);
        wrow[k] = p.w + static_cast<uint64_t>(r) * p.cols;
        srow[k] = p.scales + static_cast<uint64_t>(r / p.block_rows) * scale_cols;
        acc[k] = 0.0f;
      }
      fp8_rows<DT, NR, FAST, XT>(wrow, srow, xsf, p.cols, p.block_cols, lane, acc);
#pragma unroll
      for (int k = 0; k < NR; ++k) {
        const float y = wave_sum(acc[k]);
        const uint32_t r = unit * NR + k;
        if (lane == 0 && r < p.rows) p.out[static_cast<uint64_t>(token) * p.rows + r] = y;
      }
    }
  }
}

// MoE gate/up: unit = (slot k, row i); the wave computes gate.x and up.x of expert
// e_k and stores act[k][i] = silu(g) * u as f32.
template <uint32_t DT, bool FAST>
__global__ __launch_bounds__(kBlock) void moe_gate_up_kernel(MoeFp8Params p) {
  extern __shared__ __align__(16) float xsf[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  stage_x<DT, FAST ? kXLeanF32 : kXColumns>(xsf, p.x16, nullptr, p.hidden);
  __syncthreads();
  const uint32_t slots = p.top_k + (p.shared_index >= 0 ? 1u : 0u);
  const uint32_t units = slots * p.inter;
  const uint32_t sc = (p.hidden + p.block - 1) / p.block;
  const uint64_t scale_stride = static_cast<uint64_t>((p.inter + p.block - 1) / p.block) * sc;
  const uint64_t w_stride = static_cast<uint64_t>(p.inter) * p.hidden;
  for (uint32_t unit = blockIdx.x * kWavesPerBlock + wave; unit < units;
       unit += gridDim.x * kWavesPerBlock) {
    const uint32_t k = unit / p.inter, i = unit % p.inter;
    uint32_t e = k < p.top_k ? p.expert_ids[k] : static_cast<uint32_t>(p.shared_index);
    if (e >= p.num_experts) e = 0;  // stay in bounds; the down kernel turns such a slot into NaN outputs
    const uint8_t *wrow[2] = {p.w_gate + e * w_stride + static_cast<uint64_t>(i) * p.hidden,
                              p.w_up + e * w_stride + static_cast<uint64_t>(i) * p.hidden};
    const float *srow[2] = {p.s_gate + e * scale_stride + static_cast<uint64_t>(i / p.block) * sc,
                            p.s_up + e * scale_stride + static_cast<uint64_t>(i / p.block) * sc};
    float acc[2] = {0.0f, 0.0f};
    fp8_rows<DT, 2, FAST, FAST ? kXLeanF32 : kXColumns>(wrow, srow, xsf, p.hidden, p.block, lane, acc);
    const float g = wave_sum(acc[0]);
    const float u = wave_sum(acc[1]);
    if (lane == 0) p.act[static_cast<uint64_t>(k) * p.inter + i] = silu(g) * u;
  }
}

// MoE down + combine: the wave owns NR output rows h and walks the selected
// experts in slot order, so out[h] = sum_k w_k * (Wd_k[h,:] . act[k]) is summed in
// a fixed order (no atomics). act[k] is staged through LDS one expert at a time.
template <int NR, bool FAST>
__global__ __launch_bounds__(kBlock) void moe_down_kernel(MoeFp8Params p) {
  extern __shared__ __align__(16) float acts[];  // 2 x inter floats (double buffer)
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t slots = p.top_k + (p.shared_index >= 0 ? 1u : 0u);
  const uint32_t sc = (p.inter + p.block - 1) / p.block;
  const uint64_t scale_stride = static_cast<uint64_t>((p.hidden + p.block - 1) / p.block) * sc;
  const uint64_t w_stride = static_cast<uint64_t>(p.hidden) * p.inter;
  const uint32_t unit = blockIdx.x * kWavesPerBlock + wave;  // grid covers all rows exactly
  float total[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) total[r] = 0.0f;
  for (uint32_t k = 0; k < slots; ++k) {
    float *buf = acts + (k & 1u) * p.inter;
    for (uint32_t c = threadIdx.x; c < p.inter; c += kBlock)
      buf[FAST ? lean_slot_f32(c) : c] = p.act[static_cast<uint64_t>(k) * p.inter + c];
    __syncthreads();  // double buffer: the previous expert's readers are at most one step behind
    uint32_t e = k < p.top_k ? p.expert_ids[k] : static_cast<uint32_t>(p.shared_index);
    float weight = k < p.top_k ? p.expert_weights[k] : 1.0f;
    if (e >= p.num_experts) {  // an id outside the bank: read expert 0 (in bounds), poison the result
      e = 0;
      weight = __builtin_nanf("");
    }
    const uint8_t *wrow[NR];
    const float *srow[NR];
    float acc[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const uint32_t h = min(unit * NR + r, p.hidden - 1);
      wrow[r] = p.w_down + e * w_stride + static_cast<uint64_t>(h) * p.inter;
      srow[r] = p.s_down + e * scale_stride + static_cast<uint64_t>(h / p.block) * sc;
      acc[r] = 0.0f;
    }
    fp8_rows<kBF16, NR, FAST, FAST ? kXLeanF32 : kXColumns>(wrow, srow, buf, p.inter, p.block, lane, acc);
#pragma unroll
    for (int r = 0; r < NR; ++r) total[r] = fmaf(weight, wave_sum(acc[r]), total[r]);
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const uint32_t h = unit * NR + r;
    if (lane == 0 && h < p.hidden) p.out[h] = total[r];
  }
}

// ---------------------------------------------------------------------------
// Lean MoE kernels for the production shapes (hidden, inter multiples of 1024; block a
// multiple of 16; 16-byte aligned weights). Same arithmetic as the kernels above; the
// difference is the request pipeline: a wave walks a flat list of batches (one 1 KiB
// chunk of each of its two rows, plus the two block scales) with four batches in
// flight in four register buffers that are refilled as soon as they are consumed
// (fully unrolled, no register copies), so rows, and in the down kernel experts,
// follow each other without a bubble.
// ---------------------------------------------------------------------------
constexpr uint32_t kLeanMaxSlots = 65;  // top_k <= 64 routed experts + the shared one

// The lean streaming loop over ROW PAIRS against 16-bit activations in LDS (lean order): a wave walks a flat
// list of batches - one 1 KiB chunk of each row of its pair plus the two block scales - through a ring of four.
// The requests are issued by hand and each batch is awaited with an explicit count of the newer requests that
// may stay in flight (requests return in issue order). With the compiler's own bookkeeping the refills under
// `if (t + n < total)` made every use wait for the whole ring: four batches per round trip instead of a
// rolling window. A pair's results are stored by ordinary stores between the requests; the counts ignore
// them, which is safe whichever way stores and loads complete relative to each other.
// What a pair is comes from the policy:
//   rows<TABLE>(unit, w0, w1, s0, s1)  the two weight rows and their scale rows (TABLE: tables in LDS may be
//                                      read - false for the requests in front of the workgroup's barrier)
//   finish(unit, a, b, lane)           the two dot products, reduced over the wave
constexpr uint32_t kLeanPairMaxWaves = 8;
constexpr uint32_t kLeanPairMinCols = 256;  // shorter rows keep the general kernels
template <uint32_t DT, class Policy>
__device__ __forceinline__ void lean_pair_stream(const Policy &pol, const uint16_t *x16, uint32_t cols,
                                                 uint32_t block_cols, uint32_t units, uint16_t *xs16, bool x_ahead) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t waves = blockDim.x / kWave;   // the host picks the workgroup size (lean_pair_grid)
  const uint32_t wave_global = blockIdx.x * waves + wave;
  const uint32_t wave_stride = gridDim.x * waves;
  // cols is a multiple of 16; a last chunk of fewer than 1024 columns has idle lanes: they ask for the row's first
  // bytes again, meet zeros in LDS and take a zero scale
  const uint32_t bpr = (cols + 1023u) / 1024u;
  const bool ragged = (cols & 1023u) != 0;
  const uint32_t my_units = wave_global < units ? (units - wave_global + wave_stride - 1) / wave_stride : 0u;
  const uint32_t total = my_units * bpr;

  typedef uint32_t lp_u32x4_t __attribute__((ext_vector_type(4)));
  uint32_t iu = wave_global, ib = 0;
  const uint8_t *wa = nullptr, *wb = nullptr;
  const float *sa = nullptr, *sb = nullptr;
  lp_u32x4_t ba0, ba1, ba2, ba3, bb0, bb1, bb2, bb3;
  float fa0, fa1, fa2, fa3, fb0, fb1, fb2, fb3;
#define NV_LP_ISSUE(J, TABLE)                                                                 \
  do {                                                                                        \
    if (ib == 0) pol.template rows<TABLE>(iu, wa, wb, sa, sb);                                \
    uint32_t col_ = ib * 1024u + lane * 16;                                                   \
    if (col_ >= cols) col_ = 0;                                                               \
    const uint8_t *q0_ = wa + col_, *q1_ = wb + col_;                                         \
    const float *r0_ = sa + col_ / block_cols;                                                \
    const float *r1_ = sb + col_ / block_cols;                                                \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(ba##J) : "v"(q0_) : "memory");   \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(bb##J) : "v"(q1_) : "memory");   \
    asm volatile("global_load_dword %0, %1, off" : "=v"(fa##J) : "v"(r0_) : "memory");        \
    asm volatile("global_load_dword %0, %1, off" : "=v"(fb##J) : "v"(r1_) : "memory");        \
    if (++ib == bpr) {                                                                        \
      ib = 0;                                                                                 \
      iu += wave_stride;                                                                      \
    }                                                                                         \
  } while (0)
  // The wait and the hand-over of a batch to compiler-visible registers are one asm statement: the moves read
  // the request's destination registers after the wait whatever registers the compiler picks for either side.
  lp_u32x4_t ua, ub;
  float ga, gb;
#define NV_LP_TAKE(WAIT, J)                                                                   \
  asm volatile(WAIT "\n\tv_mov_b32 %0, %10\n\tv_mov_b32 %1, %11\n\tv_mov_b32 %2, %12\n\tv_mov_b32 %3, %13" \
               "\n\tv_mov_b32 %4, %14\n\tv_mov_b32 %5, %15\n\tv_mov_b32 %6, %16\n\tv_mov_b32 %7, %17"     \
               "\n\tv_mov_b32 %8, %18\n\tv_mov_b32 %9, %19"                                       \
               : "=&v"(ua.x), "=&v"(ua.y), "=&v"(ua.z), "=&v"(ua.w), "=&v"(ub.x), "=&v"(ub.y),     \
                 "=&v"(ub.z), "=&v"(ub.w), "=&v"(ga), "=&v"(gb)                                    \
               : "v"(ba##J.x), "v"(ba##J.y), "v"(ba##J.z), "v"(ba##J.w), "v"(bb##J.x),             \
                 "v"(bb##J.y), "v"(bb##J.z), "v"(bb##J.w), "v"(fa##J), "v"(fb##J)                  \
               : "memory")
#define NV_LP_AWAIT(J, NEWER)                                                                 \
  do {                                                                                        \
    const uint32_t newer_ = (NEWER);                                                          \
    if (newer_ >= 3u) NV_LP_TAKE("s_waitcnt vmcnt(12)", J);                                   \
    else if (newer_ == 2u) NV_LP_TAKE("s_waitcnt vmcnt(8)", J);                               \
    else if (newer_ == 1u) NV_LP_TAKE("s_waitcnt vmcnt(4)", J);                               \
    else NV_LP_TAKE("s_waitcnt vmcnt(0)", J);                                                 \
  } while (0)

  uint32_t cu = wave_global, cb = 0;
  float aa = 0.0f, ab = 0.0f;
  bool pair_done = false;
#define NV_LP_CONSUME()                                                                       \
  do {                                                                                        \
    const uint16_t *xp = xs16 + cb * 1024u + lane * 8;                                        \
    const uint4 xa = *reinterpret_cast<const uint4 *>(xp);                                    \
    const uint4 xb = *reinterpret_cast<const uint4 *>(xp + 512);                              \
    if (ragged && cb == bpr - 1u && cb * 1024u + lane * 16 >= cols) {                         \
      ga = 0.0f;                                                                              \
      gb = 0.0f;                                                                              \
    }                                                                                         \
    aa = fmaf(ga, dot16_fp8_x16<DT>(make_uint4(ua.x, ua.y, ua.z, ua.w), xa, xb), aa);         \
    ab = fmaf(gb, dot16_fp8_x16<DT>(make_uint4(ub.x, ub.y, ub.z, ub.w), xa, xb), ab);         \
    pair_done = ++cb == bpr;                                                                  \
  } while (0)
  // a pair's reduction and store come BEHIND the refill of the ring slot that its last batch left (the wave
  // issues in order: a reduction in front of the refill keeps the request back for its whole length)
#define NV_LP_FINISH()                                                                        \
  do {                                                                                        \
    if (pair_done) {                                                                          \
      cb = 0;                                                                                 \
      pol.finish(cu, wave_sum(aa), wave_sum(ab), lane);                                       \
      aa = 0.0f;                                                                              \
      ab = 0.0f;                                                                              \
      cu += wave_stride;                                                                      \
    }                                                                                         \
  } while (0)

  // Start: the activations are requested FIRST (up to kXHold 16-byte pieces a thread, in registers), the ring's
  // first four batches right behind them, and the thread then waits for the activations alone - they are the
  // oldest requests - and writes them to LDS while the weights are on their way. (Requested behind the ring,
  // as a loop would, the activations arrive after 8 KiB of weights per wave, and the ring stands still until
  // the barrier behind them.) Vectors with more pieces a thread take the loop.
  constexpr uint32_t kXHold = 5;
  const uint32_t pieces = cols / 8u;  // 8 columns = one piece of one lane
  const uint32_t slots_x = bpr * 128u;  // pieces of the LDS copy (zeros behind a ragged end)
  const uint32_t nx = (slots_x + blockDim.x - 1) / blockDim.x;
  const bool x_first = nx <= kXHold && x_ahead;
  lp_u32x4_t xh0 = {0u, 0u, 0u, 0u}, xh1 = xh0, xh2 = xh0, xh3 = xh0, xh4 = xh0;   // (a piece that is not requested is never stored)
#define NV_LP_XREQ(I)                                                                              \
  if (x_first && (I##u) < nx) {                                                                       \
    const uint16_t *src_ = x16 + static_cast<uint64_t>(min(threadIdx.x + (I##u) * blockDim.x, pieces - 1u)) * 8u; \
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xh##I) : "v"(src_) : "memory");          \
  }
  NV_LP_XREQ(0)
  NV_LP_XREQ(1)
  NV_LP_XREQ(2)
  NV_LP_XREQ(3)
  NV_LP_XREQ(4)
#undef NV_LP_XREQ
  if (total > 0) NV_LP_ISSUE(0, false);
  if (total > 1) NV_LP_ISSUE(1, false);
  if (total > 2) NV_LP_ISSUE(2, false);
  if (total > 3) NV_LP_ISSUE(3, false);
  if (x_first) {
    switch (min(total, 4u)) {  // four requests a batch stay in flight
      case 4: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
    asm volatile("" : "+v"(xh0), "+v"(xh1), "+v"(xh2), "+v"(xh3), "+v"(xh4));
#define NV_LP_XPUT(I)                                                                              \
  if ((I##u) < nx && threadIdx.x + (I##u) * blockDim.x < slots_x)                                 \
    *reinterpret_cast<uint4 *>(xs16 + lean_slot_16((threadIdx.x + (I##u) * blockDim.x) * 8u)) =    \
        threadIdx.x + (I##u) * blockDim.x < pieces ? make_uint4(xh##I.x, xh##I.y, xh##I.z, xh##I.w) \
                                                   : make_uint4(0u, 0u, 0u, 0u);
    NV_LP_XPUT(0)
    NV_LP_XPUT(1)
    NV_LP_XPUT(2)
    NV_LP_XPUT(3)
    NV_LP_XPUT(4)
#undef NV_LP_XPUT
  } else {
    for (uint32_t c = threadIdx.x * 8; c < slots_x * 8u; c += blockDim.x * 8)
      *reinterpret_cast<uint4 *>(xs16 + lean_slot_16(c)) =
          c < cols ? *reinterpret_cast<const uint4 *>(x16 + c) : make_uint4(0u, 0u, 0u, 0u);
  }
  __syncthreads();
  uint32_t t = 0;
  for (; t + 8 <= total; t += 4) {  // steady state: three newer batches behind every use
    NV_LP_AWAIT(0, 3u);
    NV_LP_CONSUME();
    NV_LP_ISSUE(0, true);
    NV_LP_FINISH();
    NV_LP_AWAIT(1, 3u);
    NV_LP_CONSUME();
    NV_LP_ISSUE(1, true);
    NV_LP_FINISH();
    NV_LP_AWAIT(2, 3u);
    NV_LP_CONSUME();
    NV_LP_ISSUE(2, true);
    NV_LP_FINISH();
    NV_LP_AWAIT(3, 3u);
    NV_LP_CONSUME();
    NV_LP_ISSUE(3, true);
    NV_LP_FINISH();
  }
  // the last four to seven batches: batch b is used with the batches up to min(b + 3, total - 1) requested
  for (; t < total; t += 4) {
    NV_LP_AWAIT(0, total - 1u - t);
    NV_LP_CONSUME();
    if (t + 4 < total) NV_LP_ISSUE(0, true);
    NV_LP_FINISH();
    if (t + 1 < total) {
      NV_LP_AWAIT(1, total - 2u - t);
      NV_LP_CONSUME();
      if (t + 5 < total) NV_LP_ISSUE(1, true);
      NV_LP_FINISH();
    }
    if (t + 2 < total) {
      NV_LP_AWAIT(2, total - 3u - t);
      NV_LP_CONSUME();
      if (t + 6 < total) NV_LP_ISSUE(2, true);
      NV_LP_FINISH();
    }
    if (t + 3 < total) {
      NV_LP_AWAIT(3, total - 4u - t);
      NV_LP_CONSUME();
      if (t + 7 < total) NV_LP_ISSUE(3, true);
      NV_LP_FINISH();
    }
  }
#undef NV_LP_ISSUE
#undef NV_LP_TAKE
#undef NV_LP_AWAIT
#undef NV_LP_CONSUME
#undef NV_LP_FINISH
}

// MoE gate/up: pair = (gate row i, up row i) of slot k's expert, unit = k * inter + i; act[unit] = silu(g) * u.
struct MoeGateUpPairs {
  const MoeFp8Params &p;
  const uint32_t *table;  // LDS: expert of a slot (an id outside the bank reads expert 0)
  uint32_t sc_cols;
  uint64_t scale_stride, w_stride;
  template <bool TABLE>
  __device__ __forceinline__ void rows(uint32_t unit, const uint8_t *&wg, const uint8_t *&wu, const float *&sg,
                                       const float *&su) const {
    const uint32_t k = unit / p.inter, i = unit % p.inter;
    uint32_t e;
    if constexpr (TABLE) {
      e = table[k];
    } else {
      // through the scalar path: a vector load here would be awaited together with every request in front of it
      e = static_cast<uint32_t>(p.shared_index);
      if (k < p.top_k)
        asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e) : "s"(p.expert_ids + k) : "memory");
      if (e >= p.num_experts) e = 0;
    }
    const uint64_t row = e * w_stride + static_cast<uint64_t>(i) * p.hidden;
    wg = p.w_gate + row;
    wu = p.w_up + row;
    const uint64_t srow = e * scale_stride + static_cast<uint64_t>(i / p.block) * sc_cols;
    sg = p.s_gate + srow;
    su = p.s_up + srow;
  }
  __device__ __forceinline__ void finish(uint32_t unit, float g, float u, int lane) const {
    if (lane == 0) p.act[unit] = silu(g) * u;  // act is [slot][inter] = flat unit index
  }
};
template <uint32_t DT>
__global__ __launch_bounds__(kLeanPairMaxWaves * kWave, 5) void moe_gate_up_lean_kernel(MoeFp8Params p) {
  extern __shared__ __align__(16) uint16_t xs16[];  // the 16-bit activations as they came, in lean order
  __shared__ uint32_t sh_expert[kLeanMaxSlots];
  const uint32_t slots = p.top_k + (p.shared_index >= 0 ? 1u : 0u);
  if (threadIdx.x < slots) {
    const uint32_t e = threadIdx.x < p.top_k ? p.expert_ids[threadIdx.x] : static_cast<uint32_t>(p.shared_index);
    sh_expert[threadIdx.x] = e < p.num_experts ? e : 0u;
  }
  const uint32_t sc_cols = (p.hidden + p.block - 1) / p.block;
  const MoeGateUpPairs pol{p, sh_expert, sc_cols, static_cast<uint64_t>((p.inter + p.block - 1) / p.block) * sc_cols,
                           static_cast<uint64_t>(p.inter) * p.hidden};
  lean_pair_stream<DT>(pol, p.x16, p.hidden, p.block, slots * p.inter, xs16, false);
}

// One FP8 GEMV, one token, 16-bit activations: pair = rows 2u and 2u + 1 (the last row doubles where the row
// count is odd).
struct GemvRowPairs {
  const Fp8GemvParams &p;
  uint32_t scale_cols;
  template <bool TABLE>
  __device__ __forceinline__ void rows(uint32_t unit, const uint8_t *&w0, const uint8_t *&w1, const float *&s0,
                                       const float *&s1) const {
    const uint32_t r0 = min(unit * 2u, p.rows - 1u), r1 = min(unit * 2u + 1u, p.rows - 1u);
    w0 = p.w + static_cast<uint64_t>(r0) * p.cols;
    w1 = p.w + static_cast<uint64_t>(r1) * p.cols;
    s0 = p.scales + static_cast<uint64_t>(r0 / p.block_rows) * scale_cols;
    s1 = p.scales + static_cast<uint64_t>(r1 / p.block_rows) * scale_cols;
  }
  __device__ __forceinline__ void finish(uint32_t unit, float a, float b, int lane) const {
    if (lane == 0) {
      p.out[unit * 2u] = a;
      if (unit * 2u + 1u < p.rows) p.out[unit * 2u + 1u] = b;
    }
  }
};
template <uint32_t DT>
__global__ __launch_bounds__(kLeanPairMaxWaves * kWave, 5) void fp8_gemv_lean_kernel(Fp8GemvParams p) {
  extern __shared__ __align__(16) uint16_t xs16[];
  const GemvRowPairs pol{p, (p.cols + p.block_cols - 1) / p.block_cols};
  lean_pair_stream<DT>(pol, p.x16, p.cols, p.block_cols, (p.rows + 1u) / 2u, xs16, p.x_first != 0);
}

// Down + combine, lean. Four consumer waves each own output rows 2u and 2u+1 and walk (expert, chunk)
// batches through a ring of four request buffers; a fifth wave does nothing but move act[k] into a
// two-slot LDS buffer one expert ahead (lean order) - loads return in order, so a consumer that
// fetched activations itself would have to wait for every weight batch it had requested before them,
// once per expert. Expert ids and weights sit in LDS from the start for the same reason: the loop of a
// consumer holds no vector load besides the ring's. P = inter / 1024 chunks per expert and row; P
// divides the ring, so which ring slot starts or ends an expert is known at compile time and the
// steady-state loop body is straight-line code: the compiler can count exactly how many younger
// requests may stay in flight at each use instead of waiting for all of them.
constexpr int kDownLeanMaxConsumers = 7;    // consumer waves of a workgroup (+ 1 staging wave: 512 threads at most)
constexpr int kDownLeanMaxThreads = (kDownLeanMaxConsumers + 1) * kWave;
constexpr uint32_t kDownLeanMaxSlots = kLeanMaxSlots;
template <int P>
__global__ __launch_bounds__(kDownLeanMaxThreads, 5) void moe_down_lean_kernel(MoeFp8Params p) {
  static_assert(P == 1 || P == 2 || P == 4, "P must divide the ring of four");
  extern __shared__ __align__(16) float acts[];  // 2 x inter floats, lean order
  __shared__ uint32_t sh_expert[kDownLeanMaxSlots];
  __shared__ float sh_weight[kDownLeanMaxSlots];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t slots = p.top_k + (p.shared_index >= 0 ? 1u : 0u);
  const bool has_shared = p.shared_index >= 0 && p.shared_last == 0;   // "the shared expert is slot 0"
  constexpr uint32_t inter = P * 1024u;
  // Slot order: the shared expert FIRST, then the routed ones in their order. The shared expert's index is a
  // launch argument, so every wave can request its first weights at once; the routed ids are a dependent read
  // from memory (a microsecond at the start of a launch) which then arrives under those weights' latency.
  // source(slot): where the slot's activations and routing entry sit in the caller's order (routed.., shared).
  const uint32_t first_routed = has_shared ? 1u : 0u;
  if (threadIdx.x < slots) {
    const bool routed = threadIdx.x >= first_routed && threadIdx.x < first_routed + p.top_k;
    uint32_t e = routed ? p.expert_ids[threadIdx.x - first_routed] : static_cast<uint32_t>(p.shared_index);
    float weight = routed ? p.expert_weights[threadIdx.x - first_routed] : 1.0f;
    if (e >= p.num_experts) {  // an id outside the bank: read expert 0 (in bounds), poison the result
      e = 0;
      weight = __builtin_nanf("");
    }
    sh_expert[threadIdx.x] = e;
    sh_weight[threadIdx.x] = weight;
  }
  const int consumers = static_cast<int>(blockDim.x) / kWave - 1;  // the last wave stages
  if (wave == consumers) {
    // ---- the staging wave: act[k] -> LDS slot k & 1, published by the barrier that starts expert k
    for (uint32_t k = 0; k < slots; ++k) {
      float4 st[P * 4];
#pragma unroll
      for (int i = 0; i < P * 4; ++i)
        st[i] = *reinterpret_cast<const float4 *>(p.act + static_cast<uint64_t>(has_shared ? (k == 0 ? p.top_k : k - 1) : k) * inter +
                                                  (i * kWave + lane) * 4);
      float *dst = acts + (k & 1u) * inter;
#pragma unroll
      for (int i = 0; i < P * 4; ++i)
        *reinterpret_cast<float4 *>(dst + lean_slot_f32((i * kWave + lane) * 4)) = st[i];
      __syncthreads();  // barrier k: expert k may be read; everyone has left slot (k + 1) & 1
    }
    return;
  }
  const uint32_t sc_cols = (inter + p.block - 1) / p.block;
  const uint64_t scale_stride = static_cast<uint64_t>((p.hidden + p.block - 1) / p.block) * sc_cols;
  const uint64_t w_stride = static_cast<uint64_t>(p.hidden) * inter;
  const uint32_t unit = blockIdx.x * consumers + wave;  // the grid covers all row pairs
  const uint32_t h0 = min(unit * 2, p.hidden - 1), h1 = min(unit * 2 + 1, p.hidden - 1);
  const uint32_t total = slots * P;

  uint32_t ik = 0;  // expert slot of the next request
  // slot 0's expert without the table: the shared expert's index is an argument; without a shared expert
  // it is the first routed id, read here directly (the same dependent read the table would have waited for)
  uint32_t first_e = has_shared ? static_cast<uint32_t>(p.shared_index) : p.expert_ids[0];
  if (first_e >= p.num_experts) first_e = 0;   // (the table entry carries the NaN weight for this case)
  const uint8_t *w0 = nullptr, *w1 = nullptr;
  const float *s0 = nullptr, *s1 = nullptr;
  // The ring's requests are asynchronous loads issued by hand, and each batch is awaited with an
  // explicit outstanding-request count just before its use (requests return in issue order: with
  // four requests a batch, "at most 4 n outstanding" means the batch is complete once n newer batches
  // have been requested). Left to the compiler's own bookkeeping the loop waited for the whole ring at
  // every batch. These waves issue no other vector-memory instruction inside the loop.
  typedef uint32_t dn_u32x4_t __attribute__((ext_vector_type(4)));
  dn_u32x4_t ba0, ba1, ba2, ba3, bb0, bb1, bb2, bb3;
  float fa0, fa1, fa2, fa3, fb0, fb1, fb2, fb3;
  // ring slot J always carries chunk J % P of an expert
#define NV_DN_ISSUE(J)                                                                        \
  do {                                                                                        \
    constexpr uint32_t ib_ = (J) % P;                                                         \
    if constexpr (ib_ == 0) {                                                                 \
      const uint32_t e = ik == 0 ? first_e : sh_expert[ik];                                   \
      w0 = p.w_down + e * w_stride + static_cast<uint64_t>(h0) * inter + lane * 16;           \
      w1 = p.w_down + e * w_stride + static_cast<uint64_t>(h1) * inter + lane * 16;           \
      s0 = p.s_down + e * scale_stride + static_cast<uint64_t>(h0 / p.block) * sc_cols;       \
      s1 = p.s_down + e * scale_stride + static_cast<uint64_t>(h1 / p.block) * sc_cols;       \
    }                                                                                         \
    const uint8_t *q0_ = w0 + ib_ * 1024u, *q1_ = w1 + ib_ * 1024u;                           \
    const float *r0_ = s0 + (ib_ * 1024u + lane * 16) / p.block;                              \
    const float *r1_ = s1 + (ib_ * 1024u + lane * 16) / p.block;                              \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(ba##J) : "v"(q0_) : "memory");   \
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(bb##J) : "v"(q1_) : "memory");   \
    asm volatile("global_load_dword %0, %1, off" : "=v"(fa##J) : "v"(r0_) : "memory");        \
    asm volatile("global_load_dword %0, %1, off" : "=v"(fb##J) : "v"(r1_) : "memory");        \
    if constexpr (ib_ == P - 1) ++ik;                                                         \
  } while (0)
  // The wait and the hand-over of a batch to compiler-visible registers are one asm statement: the
  // moves read the request's destination registers after the wait whatever registers the compiler
  // picks for either side (a wait with the registers as in/out operands leaves it free to copy them
  // before the wait).
  dn_u32x4_t ua, ub;
  float ga, gb;
#define NV_DN_TAKE(WAIT, J)                                                                   \
  asm volatile(WAIT "\n\tv_mov_b32 %0, %10\n\tv_mov_b32 %1, %11\n\tv_mov_b32 %2, %12\n\tv_mov_b32 %3, %13" \
               "\n\tv_mov_b32 %4, %14\n\tv_mov_b32 %5, %15\n\tv_mov_b32 %6, %16\n\tv_mov_b32 %7, %17"     \
               "\n\tv_mov_b32 %8, %18\n\tv_mov_b32 %9, %19"                                       \
               : "=&v"(ua.x), "=&v"(ua.y), "=&v"(ua.z), "=&v"(ua.w), "=&v"(ub.x), "=&v"(ub.y),     \
                 "=&v"(ub.z), "=&v"(ub.w), "=&v"(ga), "=&v"(gb)                                    \
               : "v"(ba##J.x), "v"(ba##J.y), "v"(ba##J.z), "v"(ba##J.w), "v"(bb##J.x),             \
                 "v"(bb##J.y), "v"(bb##J.z), "v"(bb##J.w), "v"(fa##J), "v"(fb##J)                  \
               : "memory")
#define NV_DN_AWAIT(J, NEWER)                                                                 \
  do {                                                                                        \
    const uint32_t newer_ = (NEWER);                                                          \
    if (newer_ >= 3u) NV_DN_TAKE("s_waitcnt vmcnt(12)", J);                                   \
    else if (newer_ == 2u) NV_DN_TAKE("s_waitcnt vmcnt(8)", J);                               \
    else if (newer_ == 1u) NV_DN_TAKE("s_waitcnt vmcnt(4)", J);                               \
    else NV_DN_TAKE("s_waitcnt vmcnt(0)", J);                                                 \
  } while (0)
#define NV_DN_U4(V) make_uint4((V).x, (V).y, (V).z, (V).w)

  uint32_t ck = 0;  // expert slot being consumed
  float a0 = 0.0f, a1 = 0.0f, t0 = 0.0f, t1 = 0.0f;
#define NV_DN_CONSUME(J)                                                                      \
  do {                                                                                        \
    constexpr uint32_t cb_ = (J) % P;                                                         \
    if constexpr (cb_ == 0) {                                                                 \
      if (ck != 0) __syncthreads(); /* barrier ck; barrier 0 was taken above */               \
    }                                                                                         \
    const float *xp = acts + (ck & 1u) * inter + cb_ * 1024u + lane * 4;                      \
    a0 = fmaf(ga, dot16_fp8_lean(NV_DN_U4(ua), xp), a0);                                      \
    a1 = fmaf(gb, dot16_fp8_lean(NV_DN_U4(ub), xp), a1);                                      \
  } while (0)
  // an expert's reduction comes BEHIND the refill of the ring slot its last batch left (the wave issues in
  // order: a reduction in front of the refill keeps the request back for its whole length)
#define NV_DN_FINISH(J)                                                                       \
  do {                                                                                        \
    if constexpr ((J) % P == P - 1) {                                                         \
      const float weight = sh_weight[ck];                                                     \
      t0 = fmaf(weight, wave_sum(a0), t0);                                                    \
      t1 = fmaf(weight, wave_sum(a1), t1);                                                    \
      a0 = 0.0f;                                                                              \
      a1 = 0.0f;                                                                              \
      ++ck;                                                                                   \
    }                                                                                         \
  } while (0)

  // the shared expert's batches (the first P of the ring) go out before anything is awaited; barrier 0 then
  // publishes the expert table and the first activations, and the rest of the ring follows
  // (every ring register has ONE place where it is requested first: two places would meet in a copy of a
  // register whose data is still on its way)
  NV_DN_ISSUE(0);
  if constexpr (P >= 2) NV_DN_ISSUE(1);
  if constexpr (P == 4) {
    NV_DN_ISSUE(2);
    NV_DN_ISSUE(3);
  }
  __syncthreads();  // barrier 0
  if constexpr (P == 1) {
    if (total > 1) NV_DN_ISSUE(1);
  }
  if constexpr (P <= 2) {
    if (total > 2) NV_DN_ISSUE(2);
    if (total > 3) NV_DN_ISSUE(3);
  }
  uint32_t t = 0;
  for (; t + 8 <= total; t += 4) {  // steady state: three newer batches behind every use
    NV_DN_AWAIT(0, 3u);
    NV_DN_CONSUME(0);
    NV_DN_ISSUE(0);
    NV_DN_FINISH(0);
    NV_DN_AWAIT(1, 3u);
    NV_DN_CONSUME(1);
    NV_DN_ISSUE(1);
    NV_DN_FINISH(1);
    NV_DN_AWAIT(2, 3u);
    NV_DN_CONSUME(2);
    NV_DN_ISSUE(2);
    NV_DN_FINISH(2);
    NV_DN_AWAIT(3, 3u);
    NV_DN_CONSUME(3);
    NV_DN_ISSUE(3);
    NV_DN_FINISH(3);
  }
  // the last four to seven batches: batch b is used with the batches up to min(b + 3, total - 1) requested,
  // so it may leave that many newer ones in flight (waiting for everything here put the round trips of the
  // last two refills on the wave's path)
  for (; t < total; t += 4) {
    NV_DN_AWAIT(0, total - 1u - t);
    NV_DN_CONSUME(0);
    if (t + 4 < total) NV_DN_ISSUE(0);
    NV_DN_FINISH(0);
    if (t + 1 < total) {
      NV_DN_AWAIT(1, total - 2u - t);
      NV_DN_CONSUME(1);
      if (t + 5 < total) NV_DN_ISSUE(1);
      NV_DN_FINISH(1);
    }
    if (t + 2 < total) {
      NV_DN_AWAIT(2, total - 3u - t);
      NV_DN_CONSUME(2);
      if (t + 6 < total) NV_DN_ISSUE(2);
      NV_DN_FINISH(2);
    }
    if (t + 3 < total) {
      NV_DN_AWAIT(3, total - 4u - t);
      NV_DN_CONSUME(3);
      if (t + 7 < total) NV_DN_ISSUE(3);
      NV_DN_FINISH(3);
    }
  }
#undef NV_DN_AWAIT
#undef NV_DN_TAKE
#undef NV_DN_U4
#undef NV_DN_ISSUE
#undef NV_DN_CONSUME
#undef NV_DN_FINISH
  if (lane == 0) {
    if (unit * 2 < p.hidden) p.out[unit * 2] = t0;
    if (unit * 2 + 1 < p.hidden) p.out[unit * 2 + 1] = t1;
  }
}

// softmax over E logits, top-k by (probability desc, index asc), optional
// renormalisation (precision/block/moe.rs:1107-1155,1254-1268,1303-1326).
// One workgroup; E <= 1024. Selection is k rounds of a block-wide argmax.
__global__ __launch_bounds__(kBlock) void moe_route_kernel(MoeRouteParams p) {
  __shared__ float probs[1024];
  __shared__ float red[kWavesPerBlock];
  __shared__ uint32_t red_i[kWavesPerBlock];
  __shared__ uint32_t red_h[kWavesPerBlock];
  __shared__ float sel_w[64];
  float m = -INFINITY;
  for (uint32_t i = threadIdx.x; i < p.num_experts; i += kBlock) m = fmaxf(m, p.logits[i]);
  m = wave_max(m);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < p.num_experts; i += kBlock) probs[i] = expf(p.logits[i] - m);
  __syncthreads();
  // The reference sums probabilities sequentially; do the same on one thread so
  // that ties and ordering see identical values (E is tiny).
  if (threadIdx.x == 0) {
    float sum = 0.0f;
    for (uint32_t i = 0; i < p.num_experts; ++i) sum += probs[i];
    red[0] = sum;
  }
  __syncthreads();
  const float sum = red[0];
  __syncthreads();
  if (sum > 0.0f && isfinite(sum))
    for (uint32_t i = threadIdx.x; i < p.num_experts; i += kBlock) probs[i] = probs[i] / sum;
  __syncthreads();
  for (uint32_t k = 0; k < p.top_k; ++k) {
    Best b{0.0f, 0u, 0u};
    for (uint32_t i = threadIdx.x; i < p.num_experts; i += kBlock) {
      Best c{probs[i], i, probs[i] >= 0.0f ? 1u : 0u};  // taken entries are marked -1
      if (better(c, b)) b = c;
    }
    b = wave_best(b);
    if ((threadIdx.x & (kWave - 1)) == 0) {
      red[threadIdx.x / kWave] = b.value;
      red_i[threadIdx.x / kWave] = b.index;
      red_h[threadIdx.x / kWave] = b.has;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      Best t{red[0], red_i[0], red_h[0]};
      for (int w = 1; w < kWavesPerBlock; ++w) {
        Best o{red[w], red_i[w], red_h[w]};
        if (better(o, t)) t = o;
      }
      p.expert_ids[k] = t.index;
      sel_w[k] = t.value;
      probs[t.index] = -1.0f;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    float selected = 0.0f;
    for (uint32_t k = 0; k < p.top_k; ++k) selected += sel_w[k];
    const bool norm = p.normalize && selected > 0.0f && isfinite(selected);
    for (uint32_t k = 0; k < p.top_k; ++k) p.expert_weights[k] = norm ? sel_w[k] / selected : sel_w[k];
  }
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

namespace {
// Launch shape of lean_pair_stream: waves per workgroup and workgroups such that every workgroup is resident at
// once (20 waves a CU at the kernels' register budget, LDS permitting) and the busiest CU holds as few pairs as
// possible - 7168 rows are 14 pairs a CU, which two workgroups of seven waves hold exactly where workgroups of
// four leave half the CUs with 16. Among equal loads the fewest pairs per wave (most requests in flight).
struct LeanPairGrid {
  uint32_t waves, blocks;
};
LeanPairGrid lean_pair_grid(uint32_t units, size_t lds_bytes) {
  const uint32_t lds_fit = std::max<uint32_t>(1u, static_cast<uint32_t>((156u * 1024u) / (lds_bytes + 1024u)));
  LeanPairGrid best{kWavesPerBlock, 256u * std::min<uint32_t>(5u, lds_fit)};  // (looping grid if nothing fits)
  uint32_t best_load = ~0u;
  const uint32_t ideal = (units + 255u) / 256u;
  for (uint32_t per_wave = 1; per_wave <= 64u && best_load > ideal; ++per_wave) {
    for (uint32_t c = kLeanPairMaxWaves; c >= 1; --c) {
      const uint32_t wgs = (units + c * per_wave - 1) / (c * per_wave), per_cu = std::min(20u / c, lds_fit);
      if (wgs > 256u * per_cu) continue;
      const uint32_t load = (wgs + 255u) / 256u * c * per_wave;
      if (load < best_load) {
        best_load = load;
        best = LeanPairGrid{c, wgs};
      }
    }
  }
  return best;
}
}  // namespace

hipError_t launch_fp8_gemv(const Fp8GemvParams &p, hipStream_t stream) {
  if (p.w == nullptr || p.scales == nullptr || p.out == nullptr || (p.x16 == nullptr && p.xf == nullptr))
    return hipErrorInvalidValue;
  if (p.rows == 0 || p.cols == 0 || p.block_rows == 0 || p.block_cols == 0 || p.tokens == 0)
    return hipErrorInvalidValue;
  if (p.input_dtype > kBF16) return hipErrorInvalidValue;
  const bool fast = p.cols % 1024u == 0 && p.block_cols % 16u == 0 && aligned16(p.w);
  // 16-bit activations stay 16 bit in LDS on the chunked path (half the bytes, and K up to 30720)
  const bool x16_lean = fast && p.x16 != nullptr && aligned16(p.x16);
  // one token of 16-bit activations, rows of whole 16-byte pieces: row pairs through the hand-issued ring
  const bool pair_lean = p.tokens == 1 && p.x16 != nullptr && aligned16(p.x16) && aligned16(p.w) &&
                         p.cols % 16u == 0 && p.block_cols % 16u == 0 && p.cols >= kLeanPairMinCols;
  const size_t lds = pair_lean ? static_cast<size_t>((p.cols + 1023u) / 1024u) * 1024u * sizeof(uint16_t)
                               : static_cast<size_t>(p.cols) * (x16_lean ? sizeof(uint16_t) : sizeof(float));
  if (lds > 60 * 1024) return hipErrorInvalidValue;
  const bool bf = p.input_dtype == kBF16;
  if (pair_lean) {
    const LeanPairGrid g = lean_pair_grid((p.rows + 1) / 2, lds);
    Fp8GemvParams q = p;
    // Activations requested ahead of the weights where the vector is long (measured: 16384 columns 21.7 ->
    // 21.0 us, 7168 columns 22.2 -> 22.5 us)
    q.x_first = p.cols >= 8192u ? 1u : 0u;
    if (bf) hipLaunchKernelGGL(fp8_gemv_lean_kernel<kBF16>, dim3(g.blocks), dim3(g.waves * kWave), lds, stream, q);
    else hipLaunchKernelGGL(fp8_gemv_lean_kernel<kF16>, dim3(g.blocks), dim3(g.waves * kWave), lds, stream, q);
  } else if (fast) {
    // short rows: more rows per wave to keep the same number of bytes in flight
    const bool four = p.cols <= 2048u;
    const uint32_t units = four ? (p.rows + 3) / 4 : (p.rows + 1) / 2;
    const uint32_t blocks = std::min<uint32_t>((units + kWavesPerBlock - 1) / kWavesPerBlock, 256u * 8u);
#define NV_FP8_GEMV_LAUNCH(DT, NR, XT) \
  hipLaunchKernelGGL((fp8_gemv_kernel<DT, NR, true, XT>), dim3(blocks), dim3(kBlock), lds, stream, p)
    if (x16_lean) {
      if (four) { if (bf) NV_FP8_GEMV_LAUNCH(kBF16, 4, kXLean16); else NV_FP8_GEMV_LAUNCH(kF16, 4, kXLean16); }
      else { if (bf) NV_FP8_GEMV_LAUNCH(kBF16, 2, kXLean16); else NV_FP8_GEMV_LAUNCH(kF16, 2, kXLean16); }
    } else {
      if (four) { if (bf) NV_FP8_GEMV_LAUNCH(kBF16, 4, kXLeanF32); else NV_FP8_GEMV_LAUNCH(kF16, 4, kXLeanF32); }
      else { if (bf) NV_FP8_GEMV_LAUNCH(kBF16, 2, kXLeanF32); else NV_FP8_GEMV_LAUNCH(kF16, 2, kXLeanF32); }
    }
#undef NV_FP8_GEMV_LAUNCH
  } else {
    const uint32_t blocks = std::min<uint32_t>((p.rows + kWavesPerBlock - 1) / kWavesPerBlock, 256u * 8u);
    if (bf)
      hipLaunchKernelGGL((fp8_gemv_kernel<kBF16, 1, false>), dim3(blocks), dim3(kBlock), lds, stream, p);
    else
      hipLaunchKernelGGL((fp8_gemv_kernel<kF16, 1, false>), dim3(blocks), dim3(kBlock), lds, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_moe_fp8(const MoeFp8Params &p, hipStream_t stream) {
  if (p.x16 == nullptr || p.expert_ids == nullptr || p.expert_weights == nullptr ||
      p.w_gate == nullptr || p.w_up == nullptr || p.w_down == nullptr || p.s_gate == nullptr ||
      p.s_up == nullptr || p.s_down == nullptr || p.act == nullptr || p.out == nullptr)
    return hipErrorInvalidValue;
  if (p.hidden == 0 || p.inter == 0 || p.num_experts == 0 || p.top_k == 0 || p.block == 0 ||
      p.top_k > p.num_experts || p.input_dtype > kBF16)
    return hipErrorInvalidValue;
  if (p.shared_index >= static_cast<int32_t>(p.num_experts)) return hipErrorInvalidValue;
  const uint32_t slots = p.top_k + (p.shared_index >= 0 ? 1u : 0u);
  if (static_cast<size_t>(p.hidden) * 4 > 60 * 1024 || static_cast<size_t>(p.inter) * 8 > 60 * 1024)
    return hipErrorInvalidValue;
  const bool fast_gu = p.hidden % 1024u == 0 && p.block % 16u == 0 && aligned16(p.w_gate) && aligned16(p.w_up);
  const bool fast_dn = p.inter % 1024u == 0 && p.block % 16u == 0 && aligned16(p.w_down);
  if (p.phases > 2) return hipErrorInvalidValue;
  if (p.phases != 2) {
    const uint64_t units = static_cast<uint64_t>(slots) * p.inter;
    const uint32_t blocks =
        static_cast<uint32_t>(std::min<uint64_t>((units + kWavesPerBlock - 1) / kWavesPerBlock, 256u * 32u));
    const size_t lds = static_cast<size_t>(p.hidden) * sizeof(float);
    if (fast_gu && aligned16(p.act) && aligned16(p.x16) && slots <= kLeanMaxSlots && units <= 0xffffffffull) {
      // lean kernel: the activations stay 16 bit in LDS
      const size_t lean_lds = static_cast<size_t>(p.hidden) * sizeof(uint16_t);
      // (grid: more workgroups than fit at once, handed out as others finish - measured 1 us ahead of the
      // all-resident balanced grid the single GEMV takes)
      const LeanPairGrid g{kWavesPerBlock, static_cast<uint32_t>(std::min<uint64_t>((units + kWavesPerBlock - 1) / kWavesPerBlock, 256u * 8u))};
      if (p.input_dtype == kBF16)
        hipLaunchKernelGGL((moe_gate_up_lean_kernel<kBF16>), dim3(g.blocks), dim3(g.waves * kWave), lean_lds, stream, p);
      else
        hipLaunchKernelGGL((moe_gate_up_lean_kernel<kF16>), dim3(g.blocks), dim3(g.waves * kWave), lean_lds, stream, p);
    } else if (p.input_dtype == kBF16) {
      if (fast_gu) hipLaunchKernelGGL((moe_gate_up_kernel<kBF16, true>), dim3(blocks), dim3(kBlock), lds, stream, p);
      else hipLaunchKernelGGL((moe_gate_up_kernel<kBF16, false>), dim3(blocks), dim3(kBlock), lds, stream, p);
    } else {
      if (fast_gu) hipLaunchKernelGGL((moe_gate_up_kernel<kF16, true>), dim3(blocks), dim3(kBlock), lds, stream, p);
      else hipLaunchKernelGGL((moe_gate_up_kernel<kF16, false>), dim3(blocks), dim3(kBlock), lds, stream, p);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  if (p.phases != 1) {
    constexpr int NR = 2;
    const uint32_t units = (p.hidden + NR - 1) / NR;
    const uint32_t blocks = (units + kWavesPerBlock - 1) / kWavesPerBlock;
    const size_t lds = static_cast<size_t>(p.inter) * 2 * sizeof(float);
    const bool lean_dn = fast_dn && aligned16(p.act) && slots <= kDownLeanMaxSlots &&
                         (p.inter == 1024u || p.inter == 2048u || p.inter == 4096u);  // whole experts per ring of four chunks
    if (lean_dn) {
      // Consumer waves per workgroup: the count that puts the fewest row pairs on the busiest CU while
      // every workgroup is resident at once (20 waves a CU at this kernel's register budget); hidden 7168
      // = 14 pairs a CU = two workgroups of 7 + 1 waves.
      uint32_t consumers = 4, best = ~0u;
      for (uint32_t c = kDownLeanMaxConsumers; c >= 1; --c) {
        const uint32_t wgs = (units + c - 1) / c, per_cu = 20u / (c + 1);
        if (wgs > 256u * per_cu) continue;
        const uint32_t load = (wgs + 255u) / 256u * c;
        if (load < best) {
          best = load;
          consumers = c;
        }
      }
      const uint32_t wgs = (units + consumers - 1) / consumers;
      const dim3 block((consumers + 1) * kWave);
      MoeFp8Params q = p;
      q.shared_last = tuning(kTuneMoeDownSharedFirst) == 2 ? 1u : 0u;
      if (p.inter == 1024u) hipLaunchKernelGGL(moe_down_lean_kernel<1>, dim3(wgs), block, lds, stream, q);
      else if (p.inter == 2048u) hipLaunchKernelGGL(moe_down_lean_kernel<2>, dim3(wgs), block, lds, stream, q);
      else hipLaunchKernelGGL(moe_down_lean_kernel<4>, dim3(wgs), block, lds, stream, q);
    }
    else if (fast_dn) hipLaunchKernelGGL((moe_down_kernel<NR, true>), dim3(blocks), dim3(kBlock), lds, stream, p);
    else hipLaunchKernelGGL((moe_down_kernel<NR, false>), dim3(blocks), dim3(kBlock), lds, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_moe_route(const MoeRouteParams &p, hipStream_t stream) {
  if (p.logits == nullptr || p.expert_ids == nullptr || p.expert_weights == nullptr)
    return hipErrorInvalidValue;
  if (p.num_experts == 0 || p.num_experts > 1024 || p.top_k == 0 || p.top_k > p.num_experts ||
      p.top_k > 64)
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(kBlock), 0, stream, p);
  return hipGetLastError();
}

}  // namespace nv
