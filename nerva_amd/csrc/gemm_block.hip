// Multi-row projection for token blocks of 17..256 rows with X in matrix-operand order: the X operand is
// shared through LDS instead of being fetched by every wave (see gemm_rows.cuh). Two kernels: up to 128 rows
// (gemm_block_kernel) and 129..256 rows (gemm_wide_kernel, further down).
//
// gemm_rows_kernel gives a workgroup 16 weight rows over the whole K and lets its 8 waves split K, so
// every wave fetches its own X pieces from L2: per matrix instruction 0.6 vector-memory reads, and the
// matrix cores are busy 8-13 % of the time. Here the waves of a workgroup split the ROWS and walk the
// same K range, so a K-block of X (128 columns x 128 tokens = 32 KiB, contiguous in operand order) is
// copied into LDS once per workgroup and read from there by all four waves as B operands; the weight
// rows go from global memory straight into A-operand registers (16 rows x 64 bytes per request), two
// K-blocks in flight per wave. A wave holds NR row tiles x 8 token tiles of f32 accumulators.
// Projections with few rows get their parallelism from K: grid (row groups, K slices); with more than
// one slice the workgroups write f32 partial sums and gemm_block_finish_kernel adds them in slice order
// (deterministic) and applies the epilogue.
#include "gemm_rows.cuh"

#include <stdlib.h>

#include <algorithm>
#include <mutex>

namespace nv {

namespace {

constexpr int kBW = 4;                       // waves per workgroup: they split the rows
constexpr int kBThreads = kBW * kWave;
constexpr int kBK = 128;                     // columns per K-block
constexpr int kBSteps = kBK / 32;            // matrix-core K-steps per block
constexpr int kBRing = 4;                    // W blocks a wave requests ahead at most (two with one row tile per wave)
constexpr uint32_t kBTokCap = 128;           // token rows at most; also the token stride of the partial sums
constexpr int kBRowStride = kBK + 16;        // LDS row stride of a W tile in elements: 32 B of padding. A 16-byte LDS read is
                                             // served 16 lanes at a time - lanes 0-3, 12-15, 20-23, 24-27 first, i.e. rows 0-3 and
                                             // 12-15 of one K quarter with rows 4-11 of the next - and with 16 B of padding two
                                             // lanes of every such group met in the same banks (4 extra cycles per operand read,
                                             // a third of the kernel's LDS time by the bank-conflict counter); with 32 B they do not
constexpr int kBWTile = 16 * kBRowStride;    // one 16-row block of W in LDS

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // a 16-byte piece as a first-class value

template <uint32_t DT>
__device__ __forceinline__ f32x4_t mfma_k32(u32x4_t a, u32x4_t b, f32x4_t c) {
  if constexpr (DT == kBF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                  0, 0);
}

// Epilogue of four consecutive output rows (row .. row + 3) of token t. For SwiGLU `up` holds the up
// rows' sums, otherwise it is unused.
template <uint32_t DT, int EPI>
__device__ __forceinline__ void block_epilogue(const GemmRowsParams &p, uint32_t t, uint32_t row, f32x4_t y, f32x4_t up) {
  if (p.bias != nullptr) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      y[r] += dec16<DT>(p.bias[row + r]);
      if constexpr (EPI == kGemmSwiglu) up[r] += dec16<DT>(p.bias[p.rows + row + r]);
    }
  }
  const uint64_t at = static_cast<uint64_t>(t) * p.rows + row;
  if constexpr (EPI == kGemmSwiglu) {
    uint16_t h[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) h[r] = enc16<DT>(silu(y[r]) * up[r]);
    const uint64_t at16 = p.out_packed_tiles != 0 ? gemm_x_packed_index(p.out_packed_tiles, t, row) : at;
    *reinterpret_cast<uint2 *>(p.out16 + at16) =
        make_uint2(h[0] | (static_cast<uint32_t>(h[1]) << 16), h[2] | (static_cast<uint32_t>(h[3]) << 16));
  } else {
    if constexpr (EPI == kGemmResidual) {
      const float4 res = *reinterpret_cast<const float4 *>(p.residual + at);
      y[0] += res.x;
      y[1] += res.y;
      y[2] += res.z;
      y[3] += res.w;
      if (p.round_out) {
#pragma unroll
        for (int r = 0; r < 4; ++r) y[r] = round16<DT>(y[r]);
      }
    }
    *reinterpret_cast<float4 *>(p.out_f32 + at) = make_float4(y[0], y[1], y[2], y[3]);
  }
}

// Grid (row groups, K slices). NR: row tiles per wave (SwiGLU: 2 = the gate tile and its up tile).
// cols / gridDim.y must be a multiple of kBRing * kBK (the block loop is unrolled by the ring depth, so
// that no load sits under a branch and every register index is static).
// One row tile per wave: two W blocks requested ahead, two workgroups share a CU. Two row tiles: a wave
// takes more than 256 registers, a CU holds one workgroup, and four W blocks are requested ahead to make
// up for it (measured: gate_up 62.5 -> 54.4 us with four; the one-tile projections lose 5-8 % with four).
template <uint32_t DT, int EPI, int NR, int TT>
__global__ __launch_bounds__(kBThreads, NR == 1 ? 2 : 1) void gemm_block_kernel(GemmRowsParams p, float *partials) {
  constexpr int kTiles = TT;                              // 16-token tiles of the block (X in operand order with TT tiles)
  constexpr int kStageVec = kBSteps * kTiles * kWave;     // 16-byte pieces of one X block (TT = 8: 2048 = 32 KiB)
  constexpr int kFill = kStageVec / kBThreads;            // pieces per thread and block
  extern __shared__ __align__(16) unsigned char smem[];
  u32x4_t *stage = reinterpret_cast<u32x4_t *>(smem);   // [kStageVec]: the X block, shared by the four waves
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  uint16_t *wtile = reinterpret_cast<uint16_t *>(smem + kStageVec * sizeof(u32x4_t)) + wave * NR * kBWTile;   // wave-private
  const uint32_t n = lane & 15, q = lane >> 4;
  const uint32_t cols = p.cols, T = p.tokens;
  const uint32_t kslices = gridDim.y, kper = cols / kslices, k0 = blockIdx.y * kper, nblk = kper / kBK;

  // W row of tile j (index into W; for SwiGLU the up tile lies p.rows further down)
  uint32_t trow[NR];
#pragma unroll
  for (int j = 0; j < NR; ++j)
    trow[j] = EPI == kGemmSwiglu ? j * p.rows + blockIdx.x * (16u * kBW) + wave * 16u
                                 : blockIdx.x * (16u * kBW * NR) + (wave * NR + j) * 16u;
  // W block -> registers: request i of a tile covers its rows 4i .. 4i + 3, 16 lanes x 16 B = 256 contiguous
  // bytes per row (whole cache lines, like the GEMV's stream)
  // Addresses are a wave-uniform 64-bit base (scalar registers, scalar arithmetic) plus a 32-bit per-lane
  // offset that never changes, so a request costs no vector ALU work.
  const char *wbase[NR];
#pragma unroll
  for (int j = 0; j < NR; ++j)
    wbase[j] = reinterpret_cast<const char *>(p.w) +
               (static_cast<uint64_t>(trow[j]) * cols + k0 + (EPI == kGemmSwiglu ? j * p.pair_gap : 0u)) * sizeof(uint16_t);
  const uint32_t wlane = (q * cols + n * 8u) * static_cast<uint32_t>(sizeof(uint16_t));
  uint16_t *park_at = wtile + q * kBRowStride + n * 8;
  const uint16_t *a_read = wtile + n * kBRowStride + q * 8;
  // X block b of this slice: kStageVec pieces in a row
  const char *xbase = reinterpret_cast<const char *>(p.x16) + static_cast<uint64_t>(k0 / 32u) * (kTiles * kWave) * sizeof(u32x4_t);
  const uint32_t xlane = threadIdx.x * static_cast<uint32_t>(sizeof(u32x4_t));

  constexpr int kRing = NR == 1 ? 2 : kBRing;   // W blocks requested ahead: what the register budget holds
  u32x4_t areg[kRing][NR][4];
  u32x4_t xreg[2][kFill];   // the X blocks one and two ahead
  f32x4_t acc[NR][kTiles];
#pragma unroll
  for (int j = 0; j < NR; ++j)
#pragma unroll
    for (int c = 0; c < kTiles; ++c) acc[j][c] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

#define NV_BLK_W(BUF, BLK)                                                                          \
  _Pragma("unroll") for (int j = 0; j < NR; ++j) _Pragma("unroll") for (int i = 0; i < 4; ++i)       \
      areg[BUF][j][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(               \
          wbase[j] + (static_cast<uint64_t>(4 * i) * cols + static_cast<uint64_t>(BLK) * kBK) * sizeof(uint16_t) + wlane))
#define NV_BLK_WPARK(BUF)                                                                           \
  _Pragma("unroll") for (int j = 0; j < NR; ++j) _Pragma("unroll") for (int i = 0; i < 4; ++i)       \
      *reinterpret_cast<u32x4_t *>(park_at + j * kBWTile + 4 * i * kBRowStride) = areg[BUF][j][i]
#define NV_BLK_X(XB, BLK)                                                                           \
  _Pragma("unroll") for (int i = 0; i < kFill; ++i)                                                 \
      xreg[XB][i] = *reinterpret_cast<const u32x4_t *>(                                              \
          xbase + (static_cast<uint64_t>(BLK) * kStageVec + i * kBThreads) * sizeof(u32x4_t) + xlane)
#define NV_BLK_XPARK(XB)                                                                            \
  _Pragma("unroll") for (int i = 0; i < kFill; ++i) stage[i * kBThreads + threadIdx.x] = xreg[XB][i]
  // LDS operand reads run one half K-step ahead of the products that use them: once the products of token
  // tiles 0..3 have been issued their B registers take the next K-step's pieces, likewise tiles 4..7, so a
  // read has the other half's products (128 cycles of matrix-core time per row tile) to arrive in. The
  // scheduling barriers keep the compiler from folding this back into read-wait-multiply pairs.
#define NV_BLK_READ_A(S, A)                                                                         \
  _Pragma("unroll") for (int j = 0; j < NR; ++j)                                                     \
      A[j] = *reinterpret_cast<const u32x4_t *>(a_read + j * kBWTile + (S) * 32)
#define NV_BLK_READ_B(S, C0)                                                                        \
  _Pragma("unroll") for (int c = C0; c < C0 + kTiles / 2; ++c) b[c] = stage[((S) * kTiles + c) * kWave + lane]
#define NV_BLK_PRODUCTS(A, C0)                                                                      \
  _Pragma("unroll") for (int c = C0; c < C0 + kTiles / 2; ++c)                                      \
      _Pragma("unroll") for (int j = 0; j < NR; ++j) acc[j][c] = mfma_k32<DT>(A[j], b[c], acc[j][c])
  // The requests for the blocks ahead go out between the products, two per half K-step (first the X pieces,
  // then the W rows: the order they are awaited in): the CU's vector-memory path takes 64 bytes a cycle, and
  // four waves handing it their 16 requests at once spent 550-1000 cycles issuing them before any product ran.
#define NV_BLK_W1(BUF, BLK, J, I)                                                                   \
  areg[BUF][J][I] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(                   \
      wbase[J] + (static_cast<uint64_t>(4 * (I)) * cols + static_cast<uint64_t>(BLK) * kBK) * sizeof(uint16_t) + wlane))
#define NV_BLK_X1(XB, BLK, I)                                                                       \
  xreg[XB][I] = *reinterpret_cast<const u32x4_t *>(                                                  \
      xbase + (static_cast<uint64_t>(BLK) * kStageVec + (I) * kBThreads) * sizeof(u32x4_t) + xlane)
#define NV_BLK_SLOT(K, BUF, XB, XEN, XBLK, WEN, WBLK)                                               \
  if constexpr ((K) < 4) {                                                                          \
    if constexpr (XEN && 2 * (K) < kFill) {                                                         \
      NV_BLK_X1(XB, XBLK, 2 * (K));                                                                 \
      NV_BLK_X1(XB, XBLK, 2 * (K) + 1);                                                             \
    }                                                                                               \
  } else if constexpr (WEN && 2 * ((K) - 4) < NR * 4) {                                             \
    NV_BLK_W1(BUF, WBLK, (2 * ((K) - 4)) / 4, (2 * ((K) - 4)) % 4);                                 \
    NV_BLK_W1(BUF, WBLK, (2 * ((K) - 4) + 1) / 4, (2 * ((K) - 4) + 1) % 4);                         \
  }
#define NV_BLK_STEP(S, ACUR, ANEXT, LAST, BUF, XB, XEN, XBLK, WEN, WBLK)                            \
  if (!(LAST)) { NV_BLK_READ_A((S) + 1, ANEXT); }                                                   \
  NV_BLK_PRODUCTS(ACUR, 0);                                                                         \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  if (!(LAST)) { NV_BLK_READ_B((S) + 1, 0); }                                                       \
  NV_BLK_SLOT(2 * (S), BUF, XB, XEN, XBLK, WEN, WBLK)                                               \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_BLK_PRODUCTS(ACUR, kTiles / 2);                                                               \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  if (!(LAST)) { NV_BLK_READ_B((S) + 1, kTiles / 2); }                                             \
  NV_BLK_SLOT(2 * (S) + 1, BUF, XB, XEN, XBLK, WEN, WBLK)                                           \
  __builtin_amdgcn_sched_barrier(0)
#define NV_BLK_COMPUTE(BUF, XB, XEN, XBLK, WEN, WBLK)                                               \
  do {                                                                                              \
    u32x4_t a0[NR], a1[NR], b[kTiles];                                                             \
    NV_BLK_READ_A(0, a0);                                                                           \
    NV_BLK_READ_B(0, 0);                                                                            \
    NV_BLK_READ_B(0, kTiles / 2);                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    NV_BLK_STEP(0, a0, a1, false, BUF, XB, XEN, XBLK, WEN, WBLK);                                   \
    NV_BLK_STEP(1, a1, a0, false, BUF, XB, XEN, XBLK, WEN, WBLK);                                   \
    NV_BLK_STEP(2, a0, a1, false, BUF, XB, XEN, XBLK, WEN, WBLK);                                   \
    NV_BLK_STEP(3, a1, a0, true, BUF, XB, XEN, XBLK, WEN, WBLK);                                    \
  } while (0)
  // One block: the wave parks its W rows (wave-private tile, read back in operand order) and re-uses those
  // registers for the block kRing further on; the workgroup swaps the X block in LDS (barrier: everyone has
  // finished the previous block; barrier: the new block is complete); then the products run, with the
  // requests for the X block after next (XEN: block XBLK) and the W block kRing ahead (WEN: block WBLK)
  // between them. Loads return in order, so the order of the requests is pinned (scheduling barriers) to
  // the order their data is awaited in.
#define NV_BLK_ITER(BUF, XB, XEN, XBLK, WEN, WBLK)                                                  \
  NV_BLK_WPARK(BUF);                                                                                \
  __syncthreads();                                                                                  \
  NV_BLK_XPARK(XB);                                                                                 \
  __syncthreads();                                                                                  \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_BLK_COMPUTE(BUF, XB, XEN, XBLK, WEN, WBLK)

  NV_BLK_W(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  NV_BLK_X(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  NV_BLK_X(1, 1);
  __builtin_amdgcn_sched_barrier(0);
  uint32_t blk = 0;
  if constexpr (kRing == 4) {
    NV_BLK_W(1, 1);
    NV_BLK_W(2, 2);
    NV_BLK_W(3, 3);
    __builtin_amdgcn_sched_barrier(0);
    for (; blk + 4 < nblk; blk += 4) {
      NV_BLK_ITER(0, 0, true, blk + 2, true, blk + 4);
      NV_BLK_ITER(1, 1, true, blk + 3, true, blk + 5);
      NV_BLK_ITER(2, 0, true, blk + 4, true, blk + 6);
      NV_BLK_ITER(3, 1, true, blk + 5, true, blk + 7);
    }
    NV_BLK_ITER(0, 0, true, blk + 2, false, 0);
    NV_BLK_ITER(1, 1, true, blk + 3, false, 0);
    NV_BLK_ITER(2, 0, false, 0, false, 0);
    NV_BLK_ITER(3, 1, false, 0, false, 0);
  } else {
    NV_BLK_W(1, 1);
    __builtin_amdgcn_sched_barrier(0);
    for (; blk + 2 < nblk; blk += 2) {
      NV_BLK_ITER(0, 0, true, blk + 2, true, blk + 2);
      NV_BLK_ITER(1, 1, true, blk + 3, true, blk + 3);
    }
    NV_BLK_ITER(0, 0, false, 0, false, 0);
    NV_BLK_ITER(1, 1, false, 0, false, 0);
  }
#undef NV_BLK_W
#undef NV_BLK_WPARK
#undef NV_BLK_X
#undef NV_BLK_XPARK
#undef NV_BLK_COMPUTE
#undef NV_BLK_READ_A
#undef NV_BLK_READ_B
#undef NV_BLK_PRODUCTS
#undef NV_BLK_STEP
#undef NV_BLK_SLOT
#undef NV_BLK_W1
#undef NV_BLK_X1
#undef NV_BLK_ITER

  // D layout: lane (n, q) holds rows q*4 .. q*4+3 of a row tile for token n of a token tile
  if (kslices == 1) {
#pragma unroll
    for (int c = 0; c < kTiles; ++c) {
      const uint32_t t = c * 16u + n;
      if (t < T) {
        if constexpr (EPI == kGemmSwiglu) {
          block_epilogue<DT, EPI>(p, t, trow[0] + q * 4u, acc[0][c], acc[NR - 1][c]);
        } else {
#pragma unroll
          for (int j = 0; j < NR; ++j) block_epilogue<DT, EPI>(p, t, trow[j] + q * 4u, acc[j][c], acc[j][c]);
        }
      }
    }
  } else {
    const uint32_t wrows = EPI == kGemmSwiglu ? 2u * p.rows : p.rows;
    float *part = partials + static_cast<uint64_t>(blockIdx.y) * kBTokCap * wrows;
#pragma unroll
    for (int c = 0; c < kTiles; ++c) {
      const uint32_t t = c * 16u + n;
      if (t < T) {
#pragma unroll
        for (int j = 0; j < NR; ++j)
          *reinterpret_cast<float4 *>(part + static_cast<uint64_t>(t) * wrows + trow[j] + q * 4u) =
              make_float4(acc[j][c][0], acc[j][c][1], acc[j][c][2], acc[j][c][3]);
      }
    }
  }
}

// One thread per token and four consecutive output rows: partial sums in slice order, then the epilogue.
template <uint32_t DT, int EPI>
__global__ __launch_bounds__(256) void gemm_block_finish_kernel(GemmRowsParams p, const float *partials, uint32_t kslices,
                                                                uint32_t tokcap) {
  const uint32_t quads = p.rows / 4u;
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= quads * p.tokens) return;
  const uint32_t t = i / quads, row = (i % quads) * 4u;
  const uint32_t wrows = EPI == kGemmSwiglu ? 2u * p.rows : p.rows;
  f32x4_t y = {0.0f, 0.0f, 0.0f, 0.0f}, up = {0.0f, 0.0f, 0.0f, 0.0f};
  for (uint32_t s = 0; s < kslices; ++s) {
    const float *at = partials + (static_cast<uint64_t>(s) * tokcap + t) * wrows + row;
    const float4 a = *reinterpret_cast<const float4 *>(at);
    y[0] += a.x;
    y[1] += a.y;
    y[2] += a.z;
    y[3] += a.w;
    if constexpr (EPI == kGemmSwiglu) {
      const float4 b = *reinterpret_cast<const float4 *>(at + p.rows);
      up[0] += b.x;
      up[1] += b.y;
      up[2] += b.z;
      up[3] += b.w;
    }
  }
  block_epilogue<DT, EPI>(p, t, row, y, up);
}

// The slice-adding launch of a residual projection with the RMSNorm of the result in the same pass: one workgroup
// of 1024 lanes per token, a lane's values, sum of squares, reduction and scaling laid out exactly as in
// rmsnorm_rows_kernel (gemm_rows.hip), so norm_out16 equals what that kernel writes for out_f32.
constexpr int kFinNormThreads = 1024, kFinNormPerLane = 4;
template <uint32_t DT>
__global__ __launch_bounds__(kFinNormThreads) void gemm_finish_norm_kernel(GemmRowsParams p, const float *partials, uint32_t kslices,
                                                                         uint32_t tokcap) {
  __shared__ float red[kFinNormThreads / kWave];
  const uint32_t t = blockIdx.x, rows = p.rows;
  float4 v[kFinNormPerLane];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < kFinNormPerLane; ++i) {
    const uint32_t row = (i * kFinNormThreads + threadIdx.x) * 4;
    v[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (row < rows) {
      float4 y = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      for (uint32_t s = 0; s < kslices; ++s) {
        const float4 a = *reinterpret_cast<const float4 *>(partials + (static_cast<uint64_t>(s) * tokcap + t) * rows + row);
        y.x += a.x;
        y.y += a.y;
        y.z += a.z;
        y.w += a.w;
      }
      if (p.bias != nullptr) {
        y.x += dec16<DT>(p.bias[row]);
        y.y += dec16<DT>(p.bias[row + 1]);
        y.z += dec16<DT>(p.bias[row + 2]);
        y.w += dec16<DT>(p.bias[row + 3]);
      }
      const uint64_t at = static_cast<uint64_t>(t) * rows + row;
      const float4 res = *reinterpret_cast<const float4 *>(p.residual + at);
      y.x += res.x;
      y.y += res.y;
      y.z += res.z;
      y.w += res.w;
      if (p.round_out) {
        y.x = round16<DT>(y.x);
        y.y = round16<DT>(y.y);
        y.z = round16<DT>(y.z);
        y.w = round16<DT>(y.w);
      }
      *reinterpret_cast<float4 *>(p.out_f32 + at) = y;
      v[i] = y;
    }
    ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = ss;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < kFinNormThreads / kWave; ++w) total += red[w];
  const float scale = 1.0f / sqrtf(total / static_cast<float>(rows) + p.norm_eps);
#pragma unroll
  for (int i = 0; i < kFinNormPerLane; ++i) {
    const uint32_t c = (i * kFinNormThreads + threadIdx.x) * 4;
    if (c < rows) {
      const uint2 g = *reinterpret_cast<const uint2 *>(p.norm_gamma + c);
      float g0, g1, g2, g3;
      unpack2<DT>(g.x, g0, g1);
      unpack2<DT>(g.y, g2, g3);
      uint2 o;
      o.x = enc16<DT>(v[i].x * scale * g0) | (static_cast<uint32_t>(enc16<DT>(v[i].y * scale * g1)) << 16);
      o.y = enc16<DT>(v[i].z * scale * g2) | (static_cast<uint32_t>(enc16<DT>(v[i].w * scale * g3)) << 16);
      if (p.norm_packed_tiles != 0) *reinterpret_cast<uint2 *>(p.norm_out16 + gemm_x_packed_index(p.norm_packed_tiles, t, c)) = o;
      else *reinterpret_cast<uint2 *>(p.norm_out16 + static_cast<uint64_t>(t) * rows + c) = o;
    }
  }
}

template <int NR, int TT>
constexpr size_t block_lds_bytes() {
  return static_cast<size_t>(kBSteps) * TT * kWave * sizeof(u32x4_t) + static_cast<size_t>(kBW) * NR * kBWTile * sizeof(uint16_t);
}

template <uint32_t DT, int EPI, int NR, int TT>
hipError_t launch_block_tt(const GemmRowsParams &p, float *partials, uint32_t kslices, hipStream_t stream) {
  const uint32_t wg_rows = EPI == kGemmSwiglu ? 16u * kBW : 16u * kBW * NR;
  constexpr size_t lds = block_lds_bytes<NR, TT>();
  if (lds > 64 * 1024) {
    // more than the default dynamic LDS limit: raise it once per kernel (never under stream capture)
    static std::once_flag once;
    static hipError_t raised = hipSuccess;
    std::call_once(once, [] {
      raised = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_block_kernel<DT, EPI, NR, TT>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    });
    if (raised != hipSuccess) return raised;
  }
  hipLaunchKernelGGL((gemm_block_kernel<DT, EPI, NR, TT>), dim3(p.rows / wg_rows, kslices), dim3(kBThreads), lds, stream,
                     p, partials);
  hipError_t err = hipGetLastError();
  if (err == hipSuccess && kslices > 1) {
    if (EPI == kGemmResidual && p.norm_gamma != nullptr) {   // (the caller asked gemm_rows_fuses_norm first)
      hipLaunchKernelGGL((gemm_finish_norm_kernel<DT>), dim3(p.tokens), dim3(kFinNormThreads), 0, stream, p,
                         static_cast<const float *>(partials), kslices, kBTokCap);
    } else {
      const uint32_t threads = p.rows / 4u * p.tokens;
      hipLaunchKernelGGL((gemm_block_finish_kernel<DT, EPI>), dim3((threads + 255u) / 256u), dim3(256), 0, stream, p,
                         static_cast<const float *>(partials), kslices, kBTokCap);
    }
    err = hipGetLastError();
  }
  return err;
}

template <uint32_t DT, int EPI, int NR>
hipError_t launch_block_nr(const GemmRowsParams &p, float *partials, uint32_t kslices, hipStream_t stream) {
  switch (p.x_packed) {   // token tiles of the block = tiles of its operand-order layout
    case 2: return launch_block_tt<DT, EPI, NR, 2>(p, partials, kslices, stream);
    case 4: return launch_block_tt<DT, EPI, NR, 4>(p, partials, kslices, stream);
    case 8: return launch_block_tt<DT, EPI, NR, 8>(p, partials, kslices, stream);
    default: return hipErrorInvalidValue;
  }
}

// ---------------------------------------------------------------------------------------------
// Token blocks of 129..256 rows (X in operand order with 16 token tiles). At 128 rows a byte of W meets 128
// tokens and the kernel above waits for HBM four fifths of the time; here it meets 256, and the matrix cores
// and the weight stream take about the same time. A workgroup is four PAIRS of waves. A pair owns two 16-row
// tiles of W (SwiGLU: a gate tile and its up tile) in LDS: each of its waves fetches one of them (global memory
// -> registers, four K-blocks requested ahead) and parks it there, and both read both back as A operands - one
// wave for the block's token tiles 0..7, the other for tiles 8..15, so a wave holds 2 x 8 tiles of f32
// accumulators like the kernel above, in under 256 registers: two waves per SIMD, one of which multiplies while
// the other waits for LDS. The K-block of X (128 columns x 256 tokens = 64 KiB, contiguous in operand order) is
// copied into LDS once per workgroup by all eight waves, requested one block ahead (L2 hits).
// Per block: barrier (everyone has finished the previous block's products), the waves park their W tile and
// their X pieces, barrier, products - with the requests for the next X block and for the W block four ahead
// between them, in the order they are awaited in.
// Pairs per workgroup: 4 or 3, whichever divides the rows (plain projections take 3 first: the qkv projection
// of Qwen3-8B width is then 64 row groups x 4 K slices = 256 workgroups, 30.0 us against 31.1 with 48 x 4; a
// gate/up pair takes 4 first: 192 workgroups of 64 + 64 rows measured 74.1 us, 256 of 48 + 48 rows 77.9 - every
// workgroup fetches the whole X block, whatever its rows).
constexpr int kWTiles = 16;                  // token tiles of the block's operand-order layout
constexpr uint32_t kWTokCap = 256;           // token rows at most; the token stride of this kernel's partial sums
constexpr size_t wide_lds_bytes(int pairs) {
  return static_cast<size_t>(kBSteps) * kWTiles * kWave * sizeof(u32x4_t) + static_cast<size_t>(pairs) * 2 * kBWTile * sizeof(uint16_t);
}
constexpr uint32_t wide_wg_rows(int epilogue, int pairs) { return (epilogue == kGemmSwiglu ? 16u : 32u) * pairs; }
inline int wide_pairs(int epilogue, uint32_t rows) {
  const int first = epilogue == kGemmSwiglu ? 4 : 3, second = 7 - first;
  return rows % wide_wg_rows(epilogue, first) == 0 ? first : rows % wide_wg_rows(epilogue, second) == 0 ? second : 0;
}

template <uint32_t DT, int EPI, int PAIRS>
__global__ __launch_bounds__(PAIRS * 2 * kWave, 2) void gemm_wide_kernel(GemmRowsParams p, float *partials) {
  constexpr int kWPairs = PAIRS;
  constexpr int kWThreads = kWPairs * 2 * kWave;
  constexpr int kStageVec = kBSteps * kWTiles * kWave;   // 16-byte pieces of one X block: 4096 = 64 KiB
  constexpr int kFill = (kStageVec + kWThreads - 1) / kWThreads;   // pieces per thread and block (the last one only
  constexpr bool kFillRagged = kStageVec % kWThreads != 0;         // for the first threads when the count does not divide)
  constexpr int kXPer = (kFill + 3) / 4;                 // X requests per slot
  constexpr int kHalf = kWTiles / 2;                     // token tiles per wave
  extern __shared__ __align__(16) unsigned char smem[];
  u32x4_t *stage = reinterpret_cast<u32x4_t *>(smem);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int pair = wave % kWPairs, half = wave / kWPairs;
  uint16_t *wtile = reinterpret_cast<uint16_t *>(smem + kStageVec * sizeof(u32x4_t)) + pair * 2 * kBWTile;   // the pair's two tiles
  const uint32_t n = lane & 15, q = lane >> 4;
  const uint32_t cols = p.cols, T = p.tokens;
  const uint32_t kslices = gridDim.y, kper = cols / kslices, k0 = blockIdx.y * kper, nblk = kper / kBK;

  uint32_t trow[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    trow[j] = EPI == kGemmSwiglu ? j * p.rows + blockIdx.x * (16u * kWPairs) + pair * 16u
                                 : blockIdx.x * (32u * kWPairs) + (pair * 2 + j) * 16u;
  // the tile this wave fetches: a wave-uniform base plus a per-lane offset that never changes
  const char *wbase = reinterpret_cast<const char *>(p.w) +
                      (static_cast<uint64_t>(trow[half]) * cols + k0 + (EPI == kGemmSwiglu ? half * p.pair_gap : 0u)) * sizeof(uint16_t);
  const uint32_t wlane = (q * cols + n * 8u) * static_cast<uint32_t>(sizeof(uint16_t));
  uint16_t *park_at = wtile + half * kBWTile + q * kBRowStride + n * 8;
  const uint16_t *a_read = wtile + n * kBRowStride + q * 8;
  const char *xbase = reinterpret_cast<const char *>(p.x16) + static_cast<uint64_t>(k0 / 32u) * (kWTiles * kWave) * sizeof(u32x4_t);
  const uint32_t xlane = threadIdx.x * static_cast<uint32_t>(sizeof(u32x4_t));
  const u32x4_t *b_read = stage + half * kHalf * kWave + lane;

  constexpr int kRing = 2;   // W blocks requested ahead (a block is about two microseconds of products)
  u32x4_t areg[kRing][4];
  u32x4_t xreg[kFill];
  f32x4_t acc[2][kHalf];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int c = 0; c < kHalf; ++c) acc[j][c] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

#define NV_WD_W1(BUF, BLK, I)                                                                       \
  areg[BUF][I] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(                      \
      wbase + (static_cast<uint64_t>(4 * (I)) * cols + static_cast<uint64_t>(BLK) * kBK) * sizeof(uint16_t) + wlane))
#define NV_WD_W(BUF, BLK) _Pragma("unroll") for (int i = 0; i < 4; ++i) NV_WD_W1(BUF, BLK, i)
#define NV_WD_WPARK(BUF) \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4_t *>(park_at + 4 * i * kBRowStride) = areg[BUF][i]
#define NV_WD_XLIVE(I) (!kFillRagged || (I) + 1 < kFill || (I) * kWThreads + threadIdx.x < static_cast<uint32_t>(kStageVec))
#define NV_WD_X1(BLK, I)                                                                            \
  if (NV_WD_XLIVE(I))                                                                               \
  xreg[I] = *reinterpret_cast<const u32x4_t *>(                                                      \
      xbase + (static_cast<uint64_t>(BLK) * kStageVec + (I) * kWThreads) * sizeof(u32x4_t) + xlane)
#define NV_WD_X(BLK) _Pragma("unroll") for (int i = 0; i < kFill; ++i) { NV_WD_X1(BLK, i); }
#define NV_WD_XPARK() \
  _Pragma("unroll") for (int i = 0; i < kFill; ++i) { if (NV_WD_XLIVE(i)) stage[i * kWThreads + threadIdx.x] = xreg[i]; }
#define NV_WD_READ_A(S, A) \
  _Pragma("unroll") for (int j = 0; j < 2; ++j) A[j] = *reinterpret_cast<const u32x4_t *>(a_read + j * kBWTile + (S) * 32)
#define NV_WD_READ_B(S, B) \
  _Pragma("unroll") for (int c = 0; c < kHalf; ++c) B[c] = b_read[((S) * kWTiles + c) * kWave]
#define NV_WD_PRODUCTS(A, B, C0)                                                                    \
  _Pragma("unroll") for (int c = C0; c < C0 + kHalf / 2; ++c)                                       \
      _Pragma("unroll") for (int j = 0; j < 2; ++j) acc[j][c] = mfma_k32<DT>(A[j], B[c], acc[j][c])
  // request slots between the products: slots 0..3 the next X block's pieces (two or three each), slots
  // 4 and 5 the four rows-of-four of the W block kRing ahead, two each (the order they are awaited in)
#define NV_WD_SLOT(K, BUF, XEN, XBLK, WEN, WBLK)                                                    \
  if constexpr ((K) < 4) {                                                                          \
    if constexpr (XEN) {                                                                            \
      _Pragma("unroll") for (int xi = kXPer * (K); xi < kXPer * ((K) + 1); ++xi) {                  \
        if (xi < kFill) { NV_WD_X1(XBLK, xi); }                                                     \
      }                                                                                             \
    }                                                                                               \
  } else if constexpr (WEN && (K) < 6) {                                                            \
    NV_WD_W1(BUF, WBLK, 2 * ((K) - 4));                                                             \
    NV_WD_W1(BUF, WBLK, 2 * ((K) - 4) + 1);                                                         \
  }
  // The operands of K-step s + 1 (two A pieces, eight B pieces) are requested from LDS before the sixteen
  // products of step s are issued: a wave gets a 1 KiB LDS read through about every 30 cycles, so ten reads
  // take longer than half a step's products.
#define NV_WD_STEP(S, ACUR, ANEXT, BCUR, BNEXT, LAST, BUF, XEN, XBLK, WEN, WBLK)                    \
  if (!(LAST)) {                                                                                    \
    NV_WD_READ_A((S) + 1, ANEXT);                                                                   \
    NV_WD_READ_B((S) + 1, BNEXT);                                                                   \
  }                                                                                                 \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_WD_PRODUCTS(ACUR, BCUR, 0);                                                                    \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_WD_SLOT(2 * (S), BUF, XEN, XBLK, WEN, WBLK)                                                    \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_WD_PRODUCTS(ACUR, BCUR, kHalf / 2);                                                            \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_WD_SLOT(2 * (S) + 1, BUF, XEN, XBLK, WEN, WBLK)                                                \
  __builtin_amdgcn_sched_barrier(0)
#define NV_WD_ITER(BUF, XEN, XBLK, WEN, WBLK)                                                       \
  do {                                                                                              \
    __syncthreads();                                                                                \
    NV_WD_WPARK(BUF);                                                                               \
    NV_WD_XPARK();                                                                                  \
    __syncthreads();                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    u32x4_t a0[2], a1[2], b0[kHalf], b1[kHalf];                                                     \
    NV_WD_READ_A(0, a0);                                                                            \
    NV_WD_READ_B(0, b0);                                                                            \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    NV_WD_STEP(0, a0, a1, b0, b1, false, BUF, XEN, XBLK, WEN, WBLK);                                \
    NV_WD_STEP(1, a1, a0, b1, b0, false, BUF, XEN, XBLK, WEN, WBLK);                                \
    NV_WD_STEP(2, a0, a1, b0, b1, false, BUF, XEN, XBLK, WEN, WBLK);                                \
    NV_WD_STEP(3, a1, a0, b1, b0, true, BUF, XEN, XBLK, WEN, WBLK);                                 \
  } while (0)

  NV_WD_W(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  NV_WD_X(0);
  __builtin_amdgcn_sched_barrier(0);
  NV_WD_W(1, 1);
  __builtin_amdgcn_sched_barrier(0);
  uint32_t blk = 0;
  for (; blk + 2 < nblk; blk += 2) {
    NV_WD_ITER(0, true, blk + 1, true, blk + 2);
    NV_WD_ITER(1, true, blk + 2, true, blk + 3);
  }
  NV_WD_ITER(0, true, blk + 1, false, 0);
  NV_WD_ITER(1, false, 0, false, 0);
#undef NV_WD_W1
#undef NV_WD_W
#undef NV_WD_WPARK
#undef NV_WD_X1
#undef NV_WD_XLIVE
#undef NV_WD_X
#undef NV_WD_XPARK
#undef NV_WD_READ_A
#undef NV_WD_READ_B
#undef NV_WD_PRODUCTS
#undef NV_WD_SLOT
#undef NV_WD_STEP
#undef NV_WD_ITER

  // D layout: lane (n, q) holds rows q*4 .. q*4+3 of a row tile for token n of a token tile
  if (kslices == 1) {
#pragma unroll
    for (int c = 0; c < kHalf; ++c) {
      const uint32_t t = (half * kHalf + c) * 16u + n;
      if (t < T) {
        if constexpr (EPI == kGemmSwiglu) {
          block_epilogue<DT, EPI>(p, t, trow[0] + q * 4u, acc[0][c], acc[1][c]);
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) block_epilogue<DT, EPI>(p, t, trow[j] + q * 4u, acc[j][c], acc[j][c]);
        }
      }
    }
  } else {
    const uint32_t wrows = EPI == kGemmSwiglu ? 2u * p.rows : p.rows;
    float *part = partials + static_cast<uint64_t>(blockIdx.y) * kWTokCap * wrows;
#pragma unroll
    for (int c = 0; c < kHalf; ++c) {
      const uint32_t t = (half * kHalf + c) * 16u + n;
      if (t < T) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
          *reinterpret_cast<float4 *>(part + static_cast<uint64_t>(t) * wrows + trow[j] + q * 4u) =
              make_float4(acc[j][c][0], acc[j][c][1], acc[j][c][2], acc[j][c][3]);
      }
    }
  }
}

template <uint32_t DT, int EPI, int PAIRS>
hipError_t launch_wide_pairs(const GemmRowsParams &p, float *partials, uint32_t kslices, hipStream_t stream) {
  constexpr uint32_t wg_rows = wide_wg_rows(EPI, PAIRS);
  constexpr size_t lds = wide_lds_bytes(PAIRS);
  // more than the default dynamic LDS limit: raised once per kernel (never under stream capture)
  static std::once_flag once;
  static hipError_t raised = hipSuccess;
  std::call_once(once, [] {
    raised = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_wide_kernel<DT, EPI, PAIRS>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  });
  if (raised != hipSuccess) return raised;
  hipLaunchKernelGGL((gemm_wide_kernel<DT, EPI, PAIRS>), dim3(p.rows / wg_rows, kslices), dim3(PAIRS * 2 * kWave), lds, stream, p,
                     partials);
  return hipGetLastError();
}

template <uint32_t DT, int EPI>
hipError_t launch_wide(const GemmRowsParams &p, float *partials, uint32_t kslices, hipStream_t stream) {
  const int pairs = wide_pairs(EPI, p.rows);
  hipError_t err = pairs == 3   ? launch_wide_pairs<DT, EPI, 3>(p, partials, kslices, stream)
                   : pairs == 4 ? launch_wide_pairs<DT, EPI, 4>(p, partials, kslices, stream)
                                : hipErrorInvalidValue;
  if (err == hipSuccess && kslices > 1) {
    if (EPI == kGemmResidual && p.norm_gamma != nullptr) {   // (the caller asked gemm_rows_fuses_norm first)
      hipLaunchKernelGGL((gemm_finish_norm_kernel<DT>), dim3(p.tokens), dim3(kFinNormThreads), 0, stream, p,
                         static_cast<const float *>(partials), kslices, kWTokCap);
    } else {
      const uint32_t threads = p.rows / 4u * p.tokens;
      hipLaunchKernelGGL((gemm_block_finish_kernel<DT, EPI>), dim3((threads + 255u) / 256u), dim3(256), 0, stream, p,
                         static_cast<const float *>(partials), kslices, kWTokCap);
    }
    err = hipGetLastError();
  }
  return err;
}

template <uint32_t DT>
hipError_t launch_wide_dt(int epilogue, const GemmRowsParams &p, uint32_t kslices, hipStream_t stream) {
  float *partials = static_cast<float *>(p.workspace);
  switch (epilogue) {
    case kGemmF32: return launch_wide<DT, kGemmF32>(p, partials, kslices, stream);
    case kGemmResidual: return launch_wide<DT, kGemmResidual>(p, partials, kslices, stream);
    case kGemmSwiglu: return launch_wide<DT, kGemmSwiglu>(p, partials, kslices, stream);
    default: return hipErrorInvalidValue;
  }
}

template <uint32_t DT>
hipError_t launch_block_dt(int epilogue, const GemmRowsParams &p, const GemmBlockPlan &plan, hipStream_t stream) {
  float *partials = static_cast<float *>(p.workspace);
  switch (epilogue) {
    case kGemmF32:
      return plan.row_tiles == 2 ? launch_block_nr<DT, kGemmF32, 2>(p, partials, plan.kslices, stream)
                                 : launch_block_nr<DT, kGemmF32, 1>(p, partials, plan.kslices, stream);
    case kGemmResidual:
      return plan.row_tiles == 2 ? launch_block_nr<DT, kGemmResidual, 2>(p, partials, plan.kslices, stream)
                                 : launch_block_nr<DT, kGemmResidual, 1>(p, partials, plan.kslices, stream);
    case kGemmSwiglu: return launch_block_nr<DT, kGemmSwiglu, 2>(p, partials, plan.kslices, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

GemmBlockPlan gemm_block_plan(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes) {
  GemmBlockPlan plan{};
  const int mode = tuning(kTuneGemmBlockOff) == 1 ? 0 : 1;   // "gemm_block_off" override: never the shared-X kernel
  const int want_slices = tuning(kTuneGemmBlockSlices);
  const int want_tiles = tuning(kTuneGemmBlockRowTiles);
  const uint32_t min_tokens = tuning(kTuneGemmBlockMinTokens) > 0 ? static_cast<uint32_t>(tuning(kTuneGemmBlockMinTokens)) : 17u;
  if (mode == 0 || tokens < min_tokens || tokens > kBTokCap || rows % (16u * kBW) != 0 || cols % (kBRing * kBK) != 0) return plan;
  const uint32_t wrows = epilogue == kGemmSwiglu ? 2u * rows : rows;
  // Row tiles per wave: two where that still leaves a workgroup for most CUs.
  uint32_t tiles = epilogue == kGemmSwiglu ? 2u : (rows / (16u * kBW * 2u) >= 96u && rows % (16u * kBW * 2u) == 0 ? 2u : 1u);
  if (epilogue != kGemmSwiglu && (want_tiles == 1 || (want_tiles == 2 && rows % (16u * kBW * 2u) == 0))) tiles = want_tiles;
  const uint32_t groups = rows / (epilogue == kGemmSwiglu ? 16u * kBW : 16u * kBW * tiles);
  // K slices: enough workgroups for two per CU, each slice a whole number of rings of K-blocks.
  // (A sliced gate/up pair would write and re-read 12.6 MB of partial sums per slice: measured no faster.)
  uint32_t slices = 1;
  while (epilogue != kGemmSwiglu && groups * slices < 384u && cols % (slices * 2u * kBRing * kBK) == 0) slices *= 2u;
  // A projection that would need eight or more slices of four K-blocks each (the o projection, 4096 x 4096)
  // stays with gemm_rows_kernel: pipelines that short plus the second launch measured 12.6 / 15.9 / 20.0 us
  // against 10.4 / 13.9 / 19.5 at 32 / 64 / 128 rows.
  if (want_slices == 0 && slices >= 8 && cols / slices <= 4u * kBK) return plan;
  if (want_slices > 0 && cols % (static_cast<uint32_t>(want_slices) * kBRing * kBK) == 0) slices = want_slices;
  if (slices > 1 && static_cast<uint64_t>(slices) * kBTokCap * wrows * sizeof(float) > workspace_bytes) {
    // not enough room for the partial sums: as many slices as fit (a power of two), or none
    while (slices > 1 && static_cast<uint64_t>(slices) * kBTokCap * wrows * sizeof(float) > workspace_bytes) slices /= 2u;
  }
  plan.row_tiles = tiles;
  plan.kslices = slices;
  return plan;
}

// Blocks of 129..256 rows: K slices of the kernel with wave pairs, or 0 where it does not take the shape.
// Enough workgroups for three quarters of the CUs (a gate/up pair of Qwen3-8B width has 192 row groups and
// runs unsliced), each slice a whole number of rings of K-blocks, the partial sums within the workspace.
uint32_t gemm_wide_slices(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes) {
  const int pairs = wide_pairs(epilogue, rows);
  if (tokens <= kBTokCap || tokens > kWTokCap || pairs == 0 || cols % (kBRing * kBK) != 0) return 0;
  const uint32_t wg_rows = wide_wg_rows(epilogue, pairs);
  const uint32_t wrows = epilogue == kGemmSwiglu ? 2u * rows : rows;
  const uint32_t groups = rows / wg_rows;
  uint32_t slices = 1;
  const int want = tuning(kTuneGemmBlockSlices);
  if (want > 0 && cols % (static_cast<uint32_t>(want) * kBRing * kBK) == 0) {
    slices = static_cast<uint32_t>(want);
  } else {
    while (groups * slices < 192u && slices < 8u && cols % (slices * 2u * kBRing * kBK) == 0) slices *= 2u;
  }
  while (slices > 1 && static_cast<uint64_t>(slices) * kWTokCap * wrows * sizeof(float) > workspace_bytes) slices /= 2u;
  return slices;
}

bool gemm_rows_fuses_norm(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint32_t x_packed, uint64_t workspace_bytes) {
  if (epilogue != kGemmResidual || x_packed == 0 || rows % 4 != 0 ||
      rows > static_cast<uint32_t>(kFinNormThreads * kFinNormPerLane * 4))
    return false;
  // wherever a launch of its own adds the K slices: the wide kernel's, or the shared-X kernel's for smaller blocks
  if (tokens > kBTokCap) return gemm_wide_slices(epilogue, rows, cols, tokens, workspace_bytes) > 1;
  return gemm_block_plan(epilogue, rows, cols, tokens, workspace_bytes).kslices > 1;
}

uint64_t gemm_block_workspace_bytes(uint32_t rows_max) {
  // room for 8 slices of the widest plain projection (or 2 of a gate/up pair of that width) at the wide kernel's
  // token stride
  return static_cast<uint64_t>(8) * kWTokCap * rows_max * sizeof(float);
}

hipError_t launch_gemm_wide(uint32_t dtype, int epilogue, const GemmRowsParams &p, uint32_t kslices, hipStream_t stream) {
  if (kslices == 0 || p.x_packed != static_cast<uint32_t>(kWTiles) || p.tokens <= kBTokCap || p.tokens > kWTokCap)
    return hipErrorInvalidValue;
  if (kslices > 1 && p.workspace == nullptr) return hipErrorInvalidValue;
  if (dtype == kBF16) return launch_wide_dt<kBF16>(epilogue, p, kslices, stream);
  if (dtype == kF16) return launch_wide_dt<kF16>(epilogue, p, kslices, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_gemm_block(uint32_t dtype, int epilogue, const GemmRowsParams &p, const GemmBlockPlan &plan,
                             hipStream_t stream) {
  if (plan.kslices == 0 || p.x_packed == 0 || p.x_packed != gemm_packed_tiles(p.tokens)) return hipErrorInvalidValue;
  if (plan.kslices > 1 && p.workspace == nullptr) return hipErrorInvalidValue;
  if (dtype == kBF16) return launch_block_dt<kBF16>(epilogue, p, plan, stream);
  if (dtype == kF16) return launch_block_dt<kF16>(epilogue, p, plan, stream);
  return hipErrorInvalidValue;
}

}  // namespace nv
