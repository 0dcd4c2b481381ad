// Multi-row projection on the matrix cores (see gemm_rows.cuh).
#include "gemm_rows.cuh"

#include <stdlib.h>

#include <mutex>

namespace nv {

namespace {

constexpr int kGW = 8;                          // waves per workgroup: they split K
constexpr int kGThreads = kGW * kWave;
constexpr int kKB = 256;                        // columns per staged block (512 B per row)
constexpr int kRowStride = kKB + 8;             // LDS row stride in elements: 16 B of padding keeps
                                                // the 16 rows of an operand read on distinct banks
constexpr int kTileElems = 16 * kRowStride;     // one 16-row block of W in LDS
constexpr int kSteps = kKB / 32;                // matrix-core K-steps per block
constexpr uint32_t kTwoTileMinWorkgroups = 512; // two row tiles per workgroup from this many workgroups on

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// D(16x16) += A(16x32) . B(32x16): lane l holds A[l%16][8*(l/16)..+7], B[8*(l/16)..+7][l%16] and
// D[4*(l/16)..+3][l%16].
template <uint32_t DT>
__device__ __forceinline__ f32x4_t mfma_k32(const uint4 &a, const uint4 &b, f32x4_t c) {
  if constexpr (DT == kBF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                  0, 0);
}

template <int NR>
constexpr size_t gemm_lds_bytes() {
  const size_t tiles = static_cast<size_t>(kGW) * NR * kTileElems * sizeof(uint16_t);
  const size_t partials = static_cast<size_t>(kGW) * NR * 16 * kGemmMaxTokens * sizeof(float);
  return tiles > partials ? tiles : partials;
}

// RT: 16-row tiles of W per workgroup for the plain epilogues (the X pieces a wave fetches serve all of
// them, so two tiles halve the X traffic per weight byte; the grid halves with it).
// KW: waves of a workgroup along K (8, or 4: the workgroup then holds two row groups of four waves, and
// the two waves that walk the same K range fetch the same X pieces at about the same time, so the
// second fetch is served by the CU's own cache instead of L2).
// TT: 16-token tiles a wave keeps accumulators for (2: up to 32 token rows; 4: up to 64; 8: up to 128 -
// every W operand then serves that many products).
// XP: the X operand lies in matrix-operand order (gemm_x_packed_index with TT tiles) instead of row-major:
// the 64 lanes' pieces of a (K-step, token tile) are then 1 KiB in a row and one load instruction
// touches 8 full cache lines instead of 16 half lines of 16 different rows. Measured at 32 / 64 token
// rows: gate_up 56 -> 45 / 84 -> 57 us, down 41 -> 30 / 64 -> 48, qkv 20 -> 16 / 29 -> 20.
template <uint32_t DT, int EPI, int RT, int KW, int TT, bool XP>
__global__ __launch_bounds__(kGThreads) void gemm_rows_kernel(GemmRowsParams p) {
  constexpr uint32_t kTokCap = 16u * TT;
  constexpr int NR = EPI == kGemmSwiglu ? 2 : RT;  // SwiGLU: the gate rows and the up rows of the same outputs
  constexpr uint32_t kGroupRows = EPI == kGemmSwiglu ? 16u : 16u * RT;   // output rows of one row group
  constexpr int kGroups = kGW / KW;
  constexpr uint32_t kWgRows = kGroupRows * kGroups;
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  uint16_t *tile = reinterpret_cast<uint16_t *>(smem) + static_cast<size_t>(wave) * NR * kTileElems;
  const uint32_t cols = p.cols, T = p.tokens;
  // the last workgroup of a row count that is no multiple of 16 moves back to the last 16 rows: the
  // rows it shares with its neighbour are computed and stored twice, with the same value
  const int kslice = wave % KW, group = wave / KW;
  const uint32_t row0 = min(blockIdx.x * kWgRows, p.rows - kWgRows) + group * kGroupRows;
  const uint32_t tile_rows = EPI == kGemmSwiglu ? p.rows : 16u;   // rows between a wave's tiles
  const uint32_t kper = cols / KW, nblk = kper / kKB, kbase = kslice * kper;

  // W block -> registers: instruction i covers rows 2i and 2i + 1, 32 lanes x 16 B each
  const uint16_t *wp[NR];
#pragma unroll
  for (int j = 0; j < NR; ++j)
    wp[j] = p.w + static_cast<uint64_t>(row0 + j * tile_rows + (lane >> 5)) * cols + kbase + (lane & 31) * 8 +
            (EPI == kGemmSwiglu ? j * p.pair_gap : 0u);
  uint4 areg[NR][8];
#define NV_GEMM_REQUEST(BLK)                                                                        \
  _Pragma("unroll") for (int j = 0; j < NR; ++j) _Pragma("unroll") for (int i = 0; i < 8; ++i)      \
      areg[j][i] = load_stream(wp[j] + static_cast<uint64_t>(2 * i) * cols + (BLK) * kKB)
  uint16_t *park_at = tile + (lane >> 5) * kRowStride + (lane & 31) * 8;
#define NV_GEMM_PARK()                                                                              \
  _Pragma("unroll") for (int j = 0; j < NR; ++j) _Pragma("unroll") for (int i = 0; i < 8; ++i)      \
      *reinterpret_cast<uint4 *>(park_at + j * kTileElems + 2 * i * kRowStride) = areg[j][i]

  // X operand: token of this lane in each of the token tiles (clamped: columns past T are dropped later)
  const uint32_t n = lane & 15, q = lane >> 4;
  // Row-major X: lane (n, q) of token tile c reads 16 bytes of row n + 16c at column k + 8q. Operand
  // order: piece `lane` of (K-step, tile c). Either way rows past T are clamped to the last one (those
  // columns are dropped later), so a small block touches few cache lines.
  const uint16_t *xp[TT];
  constexpr uint32_t x_step = XP ? TT * 512u : 32u;   // elements between K-steps
#pragma unroll
  for (int c = 0; c < TT; ++c) {
    const uint32_t tok = min(n + 16u * c, T - 1);   // lanes past the block's tokens re-read its last token
    xp[c] = XP ? p.x16 + (static_cast<uint64_t>(kbase / 32u) * TT + tok / 16u) * 512u + (q * 16u + tok % 16u) * 8u
               : p.x16 + static_cast<uint64_t>(tok) * cols + kbase + q * 8;
  }
  const uint16_t *a_read = tile + n * kRowStride + q * 8;

  f32x4_t acc[NR][TT];
#pragma unroll
  for (int j = 0; j < NR; ++j)
#pragma unroll
    for (int c = 0; c < TT; ++c) acc[j][c] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  uint4 breg[kSteps][TT];
#define NV_GEMM_LOAD_X(BLK)                                                                         \
  _Pragma("unroll") for (int s = 0; s < kSteps; ++s) _Pragma("unroll") for (int c = 0; c < TT; ++c)  \
      breg[s][c] = *reinterpret_cast<const uint4 *>(xp[c] + ((BLK) * kSteps + s) * x_step)
#define NV_GEMM_COMPUTE()                                                                           \
  _Pragma("unroll") for (int s = 0; s < kSteps; ++s) _Pragma("unroll") for (int j = 0; j < NR; ++j) { \
    const uint4 a = *reinterpret_cast<const uint4 *>(a_read + j * kTileElems + s * 32);             \
    _Pragma("unroll") for (int c = 0; c < TT; ++c) acc[j][c] = mfma_k32<DT>(a, breg[s][c], acc[j][c]); \
  }

  // Order of requests per block: this block's X pieces, then the next block of W. Loads return in
  // order, so the X pieces are usable while the next W block is still on its way. No request sits
  // under a branch (the last block is peeled off), so the compiler's waits stay exact.
  NV_GEMM_REQUEST(0);
  uint32_t blk = 0;
  for (; blk + 1 < nblk; ++blk) {
    NV_GEMM_PARK();
    NV_GEMM_LOAD_X(blk);
    NV_GEMM_REQUEST(blk + 1);
    NV_GEMM_COMPUTE();
  }
  NV_GEMM_PARK();
  NV_GEMM_LOAD_X(blk);
  NV_GEMM_COMPUTE();
#undef NV_GEMM_REQUEST
#undef NV_GEMM_PARK
#undef NV_GEMM_LOAD_X
#undef NV_GEMM_COMPUTE

  // ---- partial sums of the 8 waves meet in LDS (the W tiles are done with)
  __syncthreads();
  float *red = reinterpret_cast<float *>(smem);  // [wave][j][row 16][token kTokCap]
#pragma unroll
  for (int j = 0; j < NR; ++j)
#pragma unroll
    for (int c = 0; c < TT; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        red[((wave * NR + j) * 16 + q * 4 + r) * kTokCap + c * 16 + n] = acc[j][c][r];
  __syncthreads();
  // one thread per output element of a row group: 16 rows x 32 tokens at a time, rows fastest (contiguous
  // stores per token); the row groups in turn
  const uint32_t r = threadIdx.x & 15u;
  const uint32_t wg_row0 = row0 - group * kGroupRows;
#pragma unroll
  for (int half = 0; half < TT / 2; ++half) {
  const uint32_t t = (threadIdx.x >> 4) + 32u * half;
  if (t >= T) break;
#pragma unroll
  for (int gq = 0; gq < kGroups; ++gq) {
    const uint32_t grow0 = wg_row0 + gq * kGroupRows;
    float y[NR];
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < KW; ++w) sum += red[(((gq * KW + w) * NR + j) * 16 + r) * kTokCap + t];
      if (p.bias != nullptr) sum += dec16<DT>(p.bias[grow0 + j * tile_rows + r]);
      y[j] = sum;
    }
    const uint64_t at = static_cast<uint64_t>(t) * p.rows + grow0 + r;
    if constexpr (EPI == kGemmSwiglu) {
      const uint64_t at16 = p.out_packed_tiles != 0 ? gemm_x_packed_index(p.out_packed_tiles, t, grow0 + r) : at;
      p.out16[at16] = enc16<DT>(silu(y[0]) * y[NR - 1]);
    } else {
#pragma unroll
      for (int j = 0; j < NR; ++j) {
        float v = y[j];
        if constexpr (EPI == kGemmResidual) {
          v += p.residual[at + j * 16];
          if (p.round_out) v = round16<DT>(v);
        }
        p.out_f32[at + j * 16] = v;
      }
    }
  }
  }
}

// One workgroup of 1024 lanes per token row; a lane keeps its values in registers between the sum of
// squares and the scaling (cols <= 16384), so the row is read once.
constexpr int kNormThreads = 1024;
constexpr int kNormPerLane = 4;  // float4 pieces per lane
template <uint32_t DT>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_rows_kernel(const float *x, const uint16_t *gamma, float eps,
                                                                    uint32_t cols, uint16_t *out16, uint32_t packed_tiles) {
  __shared__ float red[kNormThreads / kWave];
  const float *row = x + static_cast<uint64_t>(blockIdx.x) * cols;
  float4 v[kNormPerLane];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < kNormPerLane; ++i) {
    const uint32_t c = (i * kNormThreads + threadIdx.x) * 4;
    v[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (c < cols) v[i] = *reinterpret_cast<const float4 *>(row + c);
    ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = ss;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < kNormThreads / kWave; ++w) total += red[w];
  const float scale = 1.0f / sqrtf(total / static_cast<float>(cols) + eps);
  uint16_t *out = out16 + static_cast<uint64_t>(blockIdx.x) * cols;
#pragma unroll
  for (int i = 0; i < kNormPerLane; ++i) {
    const uint32_t c = (i * kNormThreads + threadIdx.x) * 4;
    if (c < cols) {
      const uint2 g = *reinterpret_cast<const uint2 *>(gamma + c);
      float g0, g1, g2, g3;
      unpack2<DT>(g.x, g0, g1);
      unpack2<DT>(g.y, g2, g3);
      uint2 o;
      o.x = enc16<DT>(v[i].x * scale * g0) | (static_cast<uint32_t>(enc16<DT>(v[i].y * scale * g1)) << 16);
      o.y = enc16<DT>(v[i].z * scale * g2) | (static_cast<uint32_t>(enc16<DT>(v[i].w * scale * g3)) << 16);
      // four consecutive columns stay together in operand order too (c % 8 is 0 or 4)
      if (packed_tiles != 0) *reinterpret_cast<uint2 *>(out16 + gemm_x_packed_index(packed_tiles, blockIdx.x, c)) = o;
      else *reinterpret_cast<uint2 *>(out + c) = o;
    }
  }
}

template <uint32_t DT, int EPI, int RT, int KW, int TT, bool XP>
hipError_t launch_xp(const GemmRowsParams &p, hipStream_t stream) {
  constexpr int NR = EPI == kGemmSwiglu ? 2 : RT;
  constexpr uint32_t kWgRows = (EPI == kGemmSwiglu ? 16u : 16u * RT) * (kGW / KW);
  constexpr size_t lds = gemm_lds_bytes<NR>();
  if (lds > 64 * 1024) {
    // more than the default dynamic LDS limit: raise it once per kernel (never under stream capture)
    static std::once_flag once;
    static hipError_t raised = hipSuccess;
    std::call_once(once, [] {
      raised = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_rows_kernel<DT, EPI, RT, KW, TT, XP>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    });
    if (raised != hipSuccess) return raised;
  }
  hipLaunchKernelGGL((gemm_rows_kernel<DT, EPI, RT, KW, TT, XP>), dim3((p.rows + kWgRows - 1) / kWgRows), dim3(kGThreads), lds, stream, p);
  return hipGetLastError();
}

template <uint32_t DT, int EPI, int RT, int KW, int TT>
hipError_t launch_tt(const GemmRowsParams &p, hipStream_t stream) {
  return p.x_packed != 0 ? launch_xp<DT, EPI, RT, KW, TT, true>(p, stream) : launch_xp<DT, EPI, RT, KW, TT, false>(p, stream);
}

// More than 32 token rows: four token tiles (eight waves along K only).
template <uint32_t DT, int EPI, int RT, int KW>
hipError_t launch_one(const GemmRowsParams &p, hipStream_t stream) {
  if (p.tokens > 64) return launch_tt<DT, EPI, RT, 8, 8>(p, stream);
  if (p.tokens > 32) return launch_tt<DT, EPI, RT, 8, 4>(p, stream);
  return launch_tt<DT, EPI, RT, KW, 2>(p, stream);
}

template <uint32_t DT>
hipError_t launch_dt(int epilogue, const GemmRowsParams &p, hipStream_t stream) {
  // Two row tiles per workgroup where that still leaves the chip full of workgroups and there are
  // enough token rows for the X traffic to matter. Measured on MI355X at T = 1 / 8 / 32 (one tile vs
  // two, microseconds): LM head 151936x4096 198 / 223 / 383 vs 207 / 218 / 314; qkv 6144x4096
  // 12.4 / 14.1 / 23.6 vs 14.7 / 15.3 / 20.1; o and down (4096 rows: 128 workgroups with two tiles) lose.
  const int forced = tuning(kTuneGemmRowTiles) == 1 || tuning(kTuneGemmRowTiles) == 2 ? tuning(kTuneGemmRowTiles) : 0;
  const bool two = forced != 0 ? forced == 2
                               : (p.rows >= 32u * kTwoTileMinWorkgroups ? p.tokens >= 8 : (p.tokens > 16 && p.rows >= 32u * 192u));
  const bool can_two = p.rows >= 32 && !(epilogue == kGemmResidual && p.rows % 32 != 0 && p.residual == p.out_f32);
  const int forced_kw = tuning(kTuneGemmKWaves) == 4 || tuning(kTuneGemmKWaves) == 8 ? tuning(kTuneGemmKWaves) : 0;
  // Four waves along K (two row groups per workgroup): measured at T = 1 / 8 / 32 against eight, LM head
  // 202 / 208 / 299 vs 199 / 219 / 315 us; gate_up 39.8 / 41.9 / 60.1 vs 36.5 / 38.3 / 53.1, down and o
  // lose more (half the workgroups). So: only for matrices with thousands of row tiles.
  const bool kw4 = (forced_kw != 0 ? forced_kw == 4 : (p.rows >= 32u * kTwoTileMinWorkgroups && p.tokens >= 8)) &&
                   p.rows >= 64 && !(epilogue == kGemmResidual && p.residual == p.out_f32);
  switch (epilogue) {
    case kGemmF32:
      if (kw4) return two && can_two ? launch_one<DT, kGemmF32, 2, 4>(p, stream) : launch_one<DT, kGemmF32, 1, 4>(p, stream);
      return two && can_two ? launch_one<DT, kGemmF32, 2, 8>(p, stream) : launch_one<DT, kGemmF32, 1, 8>(p, stream);
    case kGemmResidual:
      if (kw4) return launch_one<DT, kGemmResidual, 1, 4>(p, stream);
      return two && can_two ? launch_one<DT, kGemmResidual, 2, 8>(p, stream) : launch_one<DT, kGemmResidual, 1, 8>(p, stream);
    case kGemmSwiglu: return kw4 ? launch_one<DT, kGemmSwiglu, 1, 4>(p, stream) : launch_one<DT, kGemmSwiglu, 1, 8>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

bool gemm_rows_supported(uint32_t rows, uint32_t cols, uint32_t tokens) {
  return rows >= 16 && cols != 0 && cols % (kGW * kKB) == 0 && tokens >= 1 && tokens <= kGemmMaxTokens;
}

hipError_t launch_gemm_rows(uint32_t dtype, int epilogue, const GemmRowsParams &p, hipStream_t stream) {
  // more than kGemmMaxTokens rows: only in operand order and only where the kernel for wide blocks takes the shape
  const uint32_t wide_slices = p.tokens > kGemmMaxTokens && p.tokens <= kGemmWideMaxTokens && p.x_packed != 0
                                   ? gemm_wide_slices(epilogue, p.rows, p.cols, p.tokens, p.workspace != nullptr ? p.workspace_bytes : 0)
                                   : 0u;
  const uint32_t deep_slices = p.tokens > kGemmWideMaxTokens && p.x_packed != 0
                                   ? gemm_deep_slices(epilogue, p.rows, p.cols, p.tokens, p.workspace != nullptr ? p.workspace_bytes : 0)
                                   : 0u;
  if (p.w == nullptr || p.x16 == nullptr) return hipErrorInvalidValue;
  if (wide_slices == 0 && deep_slices == 0 && !gemm_rows_supported(p.rows, p.cols, p.tokens)) return hipErrorInvalidValue;
  if (!aligned16(p.w) || !aligned16(p.x16)) return hipErrorInvalidValue;
  if ((epilogue == kGemmF32 || epilogue == kGemmResidual) && p.out_f32 == nullptr) return hipErrorInvalidValue;
  if (epilogue == kGemmResidual && p.residual == nullptr) return hipErrorInvalidValue;
  // rows shared by the last two workgroups are written twice: an in-place residual would be added twice
  if (epilogue == kGemmResidual && p.rows % 16 != 0 && p.residual == p.out_f32) return hipErrorInvalidValue;
  if (epilogue == kGemmSwiglu && p.out16 == nullptr) return hipErrorInvalidValue;
  // (operand order is defined in runs of 32 columns: an output of another width has no such layout)
  if (p.out_packed_tiles != 0 && (epilogue != kGemmSwiglu || p.out_packed_tiles * 16u < p.tokens || p.rows % 32 != 0))
    return hipErrorInvalidValue;
  if (p.x_packed != 0 && p.x_packed != gemm_packed_tiles(p.tokens)) return hipErrorInvalidValue;   // tiles the kernel will assume
  if (dtype != kBF16 && dtype != kF16) return hipErrorInvalidValue;
  if (p.keep_partials != 0 &&   // partial sums for a reader only where the launch leaves them; never silently summed
      (epilogue != kGemmF32 || p.bias != nullptr ||
       gemm_rows_partial_slices(p.rows, p.cols, p.tokens, p.x_packed, p.workspace != nullptr ? p.workspace_bytes : 0, nullptr) == 0))
    return hipErrorInvalidValue;
  if (p.norm_gamma != nullptr &&   // a fused norm only where the shape has one; never silently dropped
      (p.norm_out16 == nullptr || !gemm_rows_fuses_norm(epilogue, p.rows, p.cols, p.tokens, p.x_packed, p.workspace != nullptr ? p.workspace_bytes : 0)))
    return hipErrorInvalidValue;
  if (deep_slices != 0) return launch_gemm_deep(dtype, epilogue, p, deep_slices, stream);
  if (wide_slices != 0) return launch_gemm_wide(dtype, epilogue, p, wide_slices, stream);
  if (p.x_packed != 0) {   // blocks in operand order: the kernel that shares X through LDS, where its plan takes the shape
    const GemmBlockPlan plan = gemm_block_plan(epilogue, p.rows, p.cols, p.tokens, p.workspace != nullptr ? p.workspace_bytes : 0);
    if (plan.kslices != 0) return launch_gemm_block(dtype, epilogue, p, plan, stream);
  }
  if (dtype == kBF16) return launch_dt<kBF16>(epilogue, p, stream);
  return launch_dt<kF16>(epilogue, p, stream);
}

hipError_t launch_rmsnorm_rows(uint32_t dtype, const float *x, const uint16_t *gamma, float eps, uint32_t tokens,
                               uint32_t cols, uint16_t *out16, hipStream_t stream, uint32_t packed_tiles) {
  if (packed_tiles != 0 && (packed_tiles * 16u < tokens || cols % 32 != 0)) return hipErrorInvalidValue;
  if (x == nullptr || gamma == nullptr || out16 == nullptr || tokens == 0 || cols == 0 || cols % 4 != 0 ||
      cols > static_cast<uint32_t>(kNormThreads * kNormPerLane * 4) || !aligned16(x) || (reinterpret_cast<uintptr_t>(gamma) & 7u) != 0 ||
      (reinterpret_cast<uintptr_t>(out16) & 7u) != 0)
    return hipErrorInvalidValue;
  if (dtype == kBF16)
    hipLaunchKernelGGL(rmsnorm_rows_kernel<kBF16>, dim3(tokens), dim3(kNormThreads), 0, stream, x, gamma, eps, cols, out16,
                       packed_tiles);
  else if (dtype == kF16)
    hipLaunchKernelGGL(rmsnorm_rows_kernel<kF16>, dim3(tokens), dim3(kNormThreads), 0, stream, x, gamma, eps, cols, out16,
                       packed_tiles);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace nv
