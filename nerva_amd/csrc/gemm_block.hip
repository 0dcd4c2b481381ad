// Multi-row projection for token blocks of 2..256 rows with X in matrix-operand order: the X operand is
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

constexpr int kBW = 4;                       // waves per workgroup: they split the rows (three where that fills the chip)
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
// BW: waves per workgroup. With three, the X block is not a whole number of rounds of the workgroup's threads: the
// last round wraps and fetches pieces of the first again (same bytes to the same place), so that no request sits
// under a branch.
template <uint32_t DT, int EPI, int NR, int TT, int BW>
__global__ __launch_bounds__(BW * kWave, NR == 1 ? 2 : 1) void gemm_block_kernel(GemmRowsParams p, float *partials, uint32_t rotate) {
  constexpr int kBThreads = BW * kWave;
  constexpr int kTiles = TT;                              // 16-token tiles of the block (X in operand order with TT tiles)
  constexpr int kStageVec = kBSteps * kTiles * kWave;     // 16-byte pieces of one X block (TT = 8: 2048 = 32 KiB)
  constexpr int kFill = (kStageVec + kBThreads - 1) / kBThreads;   // pieces per thread and block
  static_assert(kFill <= 8, "the X requests of a block go out in the first four half K-steps, two at a time");
  extern __shared__ __align__(16) unsigned char smem[];
  u32x4_t *stage = reinterpret_cast<u32x4_t *>(smem);   // [kStageVec]: the X block, shared by the four waves
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  uint16_t *wtile = reinterpret_cast<uint16_t *>(smem + kStageVec * sizeof(u32x4_t)) + wave * NR * kBWTile;   // wave-private
  const uint32_t n = lane & 15, q = lane >> 4;
  const uint32_t cols = p.cols, T = p.tokens;
  const uint32_t kslices = gridDim.y, kper = cols / kslices, k0 = blockIdx.y * kper, nblk = kper / kBK;
  // Row groups start their walk over the K-blocks at different places (and wrap): when every workgroup asks for the
  // same columns of its rows at the same time, rows that are a multiple of 8 KiB apart crowd a part of the memory
  // channels (the request pattern alone, gate/up of 32 token rows: 39 us from a common start, 33-35 rotated).
  const uint32_t rot_off = (blockIdx.x * rotate) % nblk;
#define NV_BLK_AT(BLK) ((BLK) + rot_off >= nblk ? (BLK) + rot_off - nblk : (BLK) + rot_off)

  // W row of tile j (index into W; for SwiGLU the up tile lies p.rows further down)
  uint32_t trow[NR];
#pragma unroll
  for (int j = 0; j < NR; ++j)
    trow[j] = EPI == kGemmSwiglu ? j * p.rows + blockIdx.x * (16u * BW) + wave * 16u
                                 : blockIdx.x * (16u * BW * NR) + (wave * NR + j) * 16u;
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
          wbase[j] + (static_cast<uint64_t>(4 * i) * cols + static_cast<uint64_t>(NV_BLK_AT(BLK)) * kBK) * sizeof(uint16_t) + wlane))
#define NV_BLK_WPARK(BUF)                                                                           \
  _Pragma("unroll") for (int j = 0; j < NR; ++j) _Pragma("unroll") for (int i = 0; i < 4; ++i)       \
      *reinterpret_cast<u32x4_t *>(park_at + j * kBWTile + 4 * i * kBRowStride) = areg[BUF][j][i]
#define NV_BLK_XPIECE(I) ((static_cast<uint32_t>(I) * kBThreads + threadIdx.x) & static_cast<uint32_t>(kStageVec - 1))
#define NV_BLK_X(XB, BLK)                                                                           \
  _Pragma("unroll") for (int i = 0; i < kFill; ++i)                                                 \
      xreg[XB][i] = *reinterpret_cast<const u32x4_t *>(                                              \
          xbase + (static_cast<uint64_t>(NV_BLK_AT(BLK)) * kStageVec + NV_BLK_XPIECE(i)) * sizeof(u32x4_t))
#define NV_BLK_XPARK(XB)                                                                            \
  _Pragma("unroll") for (int i = 0; i < kFill; ++i) stage[NV_BLK_XPIECE(i)] = xreg[XB][i]
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
      wbase[J] + (static_cast<uint64_t>(4 * (I)) * cols + static_cast<uint64_t>(NV_BLK_AT(BLK)) * kBK) * sizeof(uint16_t) + wlane))
#define NV_BLK_X1(XB, BLK, I)                                                                       \
  if constexpr ((I) < kFill)                                                                        \
    xreg[XB][I] = *reinterpret_cast<const u32x4_t *>(                                                \
        xbase + (static_cast<uint64_t>(NV_BLK_AT(BLK)) * kStageVec + NV_BLK_XPIECE(I)) * sizeof(u32x4_t))
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
#undef NV_BLK_XPIECE
#undef NV_BLK_AT
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

// K-blocks by which consecutive row groups start their walk apart (the "gemm_block_rotate" override: value - 1)
inline uint32_t block_rotation() {
  const int want = tuning(kTuneGemmBlockRotate);
  return want > 0 ? static_cast<uint32_t>(want - 1) : 5u;
}

template <int NR, int TT, int BW>
constexpr size_t block_lds_bytes() {
  return static_cast<size_t>(kBSteps) * TT * kWave * sizeof(u32x4_t) + static_cast<size_t>(BW) * NR * kBWTile * sizeof(uint16_t);
}

template <uint32_t DT, int EPI, int NR, int TT, int BW = kBW>
hipError_t launch_block_tt(const GemmRowsParams &p, float *partials, uint32_t kslices, hipStream_t stream) {
  const uint32_t wg_rows = EPI == kGemmSwiglu ? 16u * BW : 16u * BW * NR;
  constexpr size_t lds = block_lds_bytes<NR, TT, BW>();
  if (lds > 64 * 1024) {
    // more than the default dynamic LDS limit: raise it once per kernel (never under stream capture)
    static std::once_flag once;
    static hipError_t raised = hipSuccess;
    std::call_once(once, [] {
      raised = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_block_kernel<DT, EPI, NR, TT, BW>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    });
    if (raised != hipSuccess) return raised;
  }
  hipLaunchKernelGGL((gemm_block_kernel<DT, EPI, NR, TT, BW>), dim3(p.rows / wg_rows, kslices), dim3(BW * kWave), lds, stream,
                     p, partials, block_rotation());
  hipError_t err = hipGetLastError();
  if (err == hipSuccess && kslices > 1 && !(EPI == kGemmF32 && p.keep_partials != 0)) {
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
hipError_t launch_block_nr(const GemmRowsParams &p, float *partials, uint32_t kslices, uint32_t waves, hipStream_t stream) {
  if constexpr (EPI == kGemmSwiglu) {
    if (waves == 3) {   // (the plan offers it for blocks of up to 64 rows)
      switch (p.x_packed) {
        case 2: return launch_block_tt<DT, EPI, NR, 2, 3>(p, partials, kslices, stream);
        case 4: return launch_block_tt<DT, EPI, NR, 4, 3>(p, partials, kslices, stream);
        default: return hipErrorInvalidValue;
      }
    }
  }
  if (waves != kBW) return hipErrorInvalidValue;
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

// ---------------------------------------------------------------------------------------------
// Token blocks of 257..512 rows (X in operand order with 32 token tiles). What bounds the kernel above is what a
// CU has to pull in, not its matrix cores: every workgroup of 128 weight rows fetches the whole X block from L2
// (twice the weight bytes per launch), ten operand pieces cross the LDS port for every sixteen products, and every
// X block is written to LDS through registers. A block of 512 tokens lets a workgroup take 256 weight rows (a
// gate/up pair: 128 + 128) x 256 tokens - one half of the block - so that a byte of X is fetched by half as many
// workgroups and a byte of W still by two (the two halves of a row group run on the same XCD, next to each other
// in dispatch order: the second finds the rows in that L2):
//   * grid: one dimension, workgroup L -> XCD L % 8 (the hardware deals them round robin), and within an XCD
//     (unit, half) with the half running fastest; unit = (row group, K slice);
//   * 8 waves = 4 row quarters x 2 token halves of 128, a wave holds 4 row tiles x 8 token tiles of accumulators
//     (128 registers) and reads 4 + 8 operand pieces for 32 products;
//   * K-blocks of 64 columns; X and W go from global memory to LDS directly (global_load_lds_dwordx4, 1 KiB a
//     request, no registers, no LDS write instructions): X in two buffers of 32 KiB (the block in use and the next
//     one), W in three (the W block two ahead is in flight from HBM): 160 KiB, all of a CU's LDS. A W tile is 16
//     rows of 128 bytes; the 16-byte pieces of a row are XORed with the row number (mod 8) on the way in - a lane
//     asks for the piece that belongs in its LDS slot - which makes the operand reads conflict-free;
//   * one barrier per K-block: a wave waits for its own requests of this block, everyone meets (the block is
//     complete and nobody reads the previous one any more), the requests for the block ahead go out, 64 products.
//     The barrier is a bare s_barrier with the waits it needs written out - a fence would wait for the requests
//     in flight - and every LDS operand read is issued by hand with a counted wait (the compiler's own
//     bookkeeping falls back to "everything" once direct-to-LDS requests are pending).
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kDTokCap = 512;                      // token rows at most; the token stride of this kernel's partial sums
constexpr int kDK = 64;                                 // columns per K-block
constexpr int kDXBuf = 2 * 16 * kWave * static_cast<int>(sizeof(u32x4_t));   // one X block of a half: 2 K-steps x 16 tiles = 32 KiB
constexpr int kDWTile = 16 * kDK * static_cast<int>(sizeof(uint16_t));       // one W tile of a block: 2 KiB
constexpr size_t deep_lds_bytes(int tpw) { return 2 * static_cast<size_t>(kDXBuf) + 3 * static_cast<size_t>(4 * tpw * kDWTile); }
#define NV_LDS_PTR(P) ((__attribute__((address_space(3))) void *)(P))

// TPW: row tiles a wave takes, 4 (256 rows a workgroup, 160 KiB of LDS) or 3 (192 rows: where that many rows make
// the launch fill the chip - a gate/up pair of 12288 + 12288 rows is 96 workgroups of 128 + 128 rows per token half,
// 192 in all on 256 CUs, but 128 of 96 + 96). With three tiles a wave the gate tiles and the up tiles of a pair end
// in different waves (row parts 0, 1: gate, 2, 3: their up tiles), and the up sums cross through LDS at the end.
template <uint32_t DT, int EPI, int TPW>
__global__ __launch_bounds__(8 * kWave, 2) void gemm_deep_kernel(GemmRowsParams p, float *partials, uint32_t units,
                                                                  uint32_t kslices) {
  static_assert(TPW == 3 || TPW == 4, "three or four row tiles a wave");
  constexpr int kTiles = 4 * TPW;                 // W tiles of the workgroup
  constexpr int kWBuf = kTiles * kDWTile;         // one W buffer
  constexpr int kWReq = kTiles * 2 / 8;           // W requests a wave and block (half a tile each)
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int th = wave & 1, rq = wave >> 1;   // token half of the workgroup's 256, row part of its 16 TPW rows
  const uint32_t n = lane & 15, q = lane >> 4;
  const uint32_t cols = p.cols, T = p.tokens;
  const uint32_t halves = (T + 255u) / 256u;
  const uint32_t in_xcd = blockIdx.x >> 3;
  const uint32_t half = in_xcd % halves, unit = (in_xcd / halves) * 8u + (blockIdx.x & 7u);
  if (unit >= units) return;
  const uint32_t group = unit / kslices, slice = unit % kslices;
  const uint32_t kper = cols / kslices, k0 = slice * kper, nblk = kper / kDK;

  // LDS tile slot s = TPW * (row part) + j. Plain: rows 16 s .. of the workgroup's rows. SwiGLU, four tiles a
  // wave: j = 0, 1 the gate tiles 2 rq + j of the workgroup's 128 gate rows, j = 2, 3 their up tiles - a wave's
  // tiles end in the wave that runs the epilogue. SwiGLU, three tiles a wave: parts 0, 1 the six gate tiles of
  // the workgroup's 96 gate rows, parts 2, 3 their up tiles.
  auto slot_row = [&](int s) -> uint32_t {
    if constexpr (EPI == kGemmSwiglu && TPW == 4)
      return ((s >> 1) & 1) * p.rows + group * 128u + (2u * (s >> 2) + (s & 1)) * 16u;
    else if constexpr (EPI == kGemmSwiglu)
      return (s / 6) * p.rows + group * 96u + (s % 6) * 16u;
    else
      return group * (16u * kTiles) + s * 16u;
  };
  auto slot_is_up = [&](int s) -> bool { return EPI == kGemmSwiglu && (TPW == 4 ? ((s >> 1) & 1) != 0 : s >= 6); };
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(NV_LDS_PTR(smem)));   // X buffers, then W buffers
  // W requests of this wave: requests kWReq wave .. + kWReq - 1 of the block's 2 kTiles (tile m / 2, rows 8 (m % 2)
  // .. + 7, 128 bytes a row). Lane (r, c) of a request asks for piece c ^ r of row r: a wave-uniform base per
  // request and one lane offset for all.
  const char *wsrc[kWReq];
#pragma unroll
  for (int i = 0; i < kWReq; ++i) {
    const int m = kWReq * wave + i, s_ = m >> 1;
    wsrc[i] = reinterpret_cast<const char *>(p.w) +
              (static_cast<uint64_t>(slot_row(s_) + (m & 1) * 8u) * cols + k0 + (slot_is_up(s_) ? p.pair_gap : 0u)) * sizeof(uint16_t);
  }
  const uint32_t wlane = ((lane >> 3) * cols) * static_cast<uint32_t>(sizeof(uint16_t)) + (((lane & 7) ^ (lane >> 3)) << 4);
  // X requests of this wave: four consecutive token tiles of one K-step of the half's block
  const uint32_t xtiles = p.x_packed;   // token tiles of the whole block per K-step (32 above 256 tokens)
  const char *xsrc = reinterpret_cast<const char *>(p.x16) +
                     ((static_cast<uint64_t>(k0 / 32u + (wave >> 2)) * xtiles + half * 16u + (wave & 3) * 4u) * kWave + lane) * sizeof(u32x4_t);
  const uint64_t xstep = static_cast<uint64_t>(2u * xtiles) * kWave * sizeof(u32x4_t);   // one K-block further
  // A operand of K-step e of the block, lane (row n, quarter q): piece 4 e + q of row n, at piece ^ (n & 7)
  uint32_t a_off[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) a_off[e] = lds0 + 2 * kDXBuf + (TPW * rq) * kDWTile + n * 128 + (((e * 4 + q) ^ (n & 7)) << 4);
  // B operand of K-step e, token tile c of this wave's eight: piece (e * 16 + th * 8 + c) * 64 + lane of the buffer
  uint32_t b_addr[2];
#pragma unroll
  for (int xb = 0; xb < 2; ++xb) b_addr[xb] = lds0 + xb * kDXBuf + ((th * 8) * kWave + lane) * static_cast<uint32_t>(sizeof(u32x4_t));

  f32x4_t acc[TPW][8];
#pragma unroll
  for (int j = 0; j < TPW; ++j)
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[j][c] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  // W block BLK -> W buffer at byte offset WOFF (wave-uniform); X block BLK -> X buffer XB
#define NV_DP_W1(WOFF, BLK, I)                                                                      \
  __builtin_amdgcn_global_load_lds(                                                                 \
      reinterpret_cast<const u32x4_t *>(wsrc[I] + static_cast<uint64_t>(BLK) * (kDK * sizeof(uint16_t)) + wlane), \
      NV_LDS_PTR(smem + 2 * kDXBuf + (WOFF) + (kWReq * wave + (I)) * 1024), 16, 0, 0)
#define NV_DP_X1(XB, BLK, I)                                                                        \
  __builtin_amdgcn_global_load_lds(                                                                 \
      reinterpret_cast<const u32x4_t *>(xsrc + static_cast<uint64_t>(BLK) * xstep + (I) * 1024),    \
      NV_LDS_PTR(smem + (XB) * kDXBuf + (wave * 4 + (I)) * 1024), 16, 0, 0)
#define NV_DP_LDS_READ(DST, ADDR, OFF) \
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(DST) : "v"(ADDR), "n"(OFF) : "memory")
#define NV_DP_READ_B(XB, IDX) NV_DP_LDS_READ(bq[(IDX) % 3], b_addr[XB], ((((IDX) >> 3) * 16 + ((IDX) & 7)) * kWave * 16))
#define NV_DP_READ_A(E, J) NV_DP_LDS_READ(aq[E][J], a_cur[E], (J) * kDWTile)
  // Operand reads of a block, in issue order: bq0, aq[0][0..TPW-1], bq1; then product group i issues bq(i + 2) and,
  // for i < TPW, aq[1][i]. LDS reads return in order, so group i waits until at most this many younger reads are
  // outstanding: (behind aq[0][TPW-1]) 3, then 4, 5, then 5, 4, 3 (four tiles a wave) or 4, 3, 2 (three), and 2 from
  // there on, 1 and 0 for the last two. The awaited registers are in/out operands of the wait, so that their use
  // cannot move in front of it.
#define NV_DP_AWAIT(N_, B_) asm volatile("s_waitcnt lgkmcnt(" #N_ ")" : "+v"(B_) :: "memory")
#define NV_DP_AWAIT_A(N_, B_, E_)                                                                   \
  do {                                                                                              \
    if constexpr (TPW == 4)                                                                         \
      asm volatile("s_waitcnt lgkmcnt(" #N_ ")" : "+v"(B_), "+v"(aq[E_][0]), "+v"(aq[E_][1]), "+v"(aq[E_][2]), "+v"(aq[E_][TPW - 1]) :: "memory"); \
    else                                                                                            \
      asm volatile("s_waitcnt lgkmcnt(" #N_ ")" : "+v"(B_), "+v"(aq[E_][0]), "+v"(aq[E_][1]), "+v"(aq[E_][2]) :: "memory"); \
  } while (0)
#define NV_DP_WAIT(IDX)                                                                             \
  if constexpr ((IDX) == 0) NV_DP_AWAIT_A(3, bq[0], 0);                                             \
  else if constexpr ((IDX) == 1) NV_DP_AWAIT(4, bq[(IDX) % 3]);                                     \
  else if constexpr ((IDX) == 2) NV_DP_AWAIT(5, bq[(IDX) % 3]);                                     \
  else if constexpr ((IDX) == 3) { if constexpr (TPW == 4) NV_DP_AWAIT(5, bq[(IDX) % 3]); else NV_DP_AWAIT(4, bq[(IDX) % 3]); } \
  else if constexpr ((IDX) == 4) { if constexpr (TPW == 4) NV_DP_AWAIT(4, bq[(IDX) % 3]); else NV_DP_AWAIT(3, bq[(IDX) % 3]); } \
  else if constexpr ((IDX) == 5) { if constexpr (TPW == 4) NV_DP_AWAIT(3, bq[(IDX) % 3]); else NV_DP_AWAIT(2, bq[(IDX) % 3]); } \
  else if constexpr ((IDX) == 8) NV_DP_AWAIT_A(2, bq[(IDX) % 3], 1);                                \
  else if constexpr ((IDX) == 14) NV_DP_AWAIT(1, bq[(IDX) % 3]);                                    \
  else if constexpr ((IDX) == 15) NV_DP_AWAIT(0, bq[(IDX) % 3]);                                    \
  else NV_DP_AWAIT(2, bq[(IDX) % 3])
  // request slots between the products: first the next X block's four pieces, then the W block two ahead
#define NV_DP_SLOT(IDX, XB, XEN, WEN)                                                               \
  if constexpr ((IDX) < 4) {                                                                        \
    if constexpr (XEN) { NV_DP_X1((XB) ^ 1, blk_ + 1u, IDX); }                                      \
  } else if constexpr ((IDX) < 4 + kWReq) {                                                         \
    if constexpr (WEN) { NV_DP_W1(w_ahead, blk_ + 2u, (IDX) - 4); }                                 \
  }
#define NV_DP_ITEM(IDX, XB, XEN, WEN)                                                               \
  if constexpr ((IDX) + 2 < 16) { NV_DP_READ_B(XB, (IDX) + 2); }                                    \
  if constexpr ((IDX) < TPW) { NV_DP_READ_A(1, IDX); }                                              \
  NV_DP_WAIT(IDX);                                                                                  \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  _Pragma("unroll") for (int j = 0; j < TPW; ++j)                                                   \
      acc[j][(IDX) & 7] = mfma_k32<DT>(aq[(IDX) >> 3][j], bq[(IDX) % 3], acc[j][(IDX) & 7]);        \
  __builtin_amdgcn_sched_barrier(0);                                                                \
  NV_DP_SLOT(IDX, XB, XEN, WEN)                                                                     \
  __builtin_amdgcn_sched_barrier(0)
  // Block BLK in X buffer XB and the W buffer at w_cur. LAST: nothing younger than this block's requests is in
  // flight; otherwise the W requests of the block after it are.
#define NV_DP_BLOCK(BLK, XB, LAST, XEN, WEN)                                                        \
  do {                                                                                              \
    const uint32_t blk_ = (BLK);                                                                    \
    if constexpr (LAST) asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");               \
    else if constexpr (kWReq == 4) asm volatile("s_waitcnt vmcnt(4)\n\ts_barrier" ::: "memory");    \
    else asm volatile("s_waitcnt vmcnt(3)\n\ts_barrier" ::: "memory");                              \
    const uint32_t a_cur[2] = {a_off[0] + w_cur, a_off[1] + w_cur};                                 \
    const uint32_t w_ahead = w_cur >= static_cast<uint32_t>(kWBuf) ? w_cur - kWBuf : w_cur + 2 * kWBuf;   /* (b + 2) % 3 */ \
    u32x4_t aq[2][TPW], bq[3];                                                                      \
    NV_DP_READ_B(XB, 0);                                                                            \
    _Pragma("unroll") for (int j = 0; j < TPW; ++j) { NV_DP_READ_A(0, j); }                         \
    NV_DP_READ_B(XB, 1);                                                                            \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    NV_DP_ITEM(0, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(1, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(2, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(3, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(4, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(5, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(6, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(7, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(8, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(9, XB, XEN, WEN);                                                                    \
    NV_DP_ITEM(10, XB, XEN, WEN);                                                                   \
    NV_DP_ITEM(11, XB, XEN, WEN);                                                                   \
    NV_DP_ITEM(12, XB, XEN, WEN);                                                                   \
    NV_DP_ITEM(13, XB, XEN, WEN);                                                                   \
    NV_DP_ITEM(14, XB, XEN, WEN);                                                                   \
    NV_DP_ITEM(15, XB, XEN, WEN);                                                                   \
    w_cur = w_cur == static_cast<uint32_t>(2 * kWBuf) ? 0u : w_cur + kWBuf;                          \
  } while (0)

  // start: X block 0, W blocks 0 and 1, in the order they are awaited in (nblk is even and at least 2)
  uint32_t w_cur = 0;   // byte offset of the W buffer of the block being multiplied (wave-uniform)
  {
    const uint32_t blk_ = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) NV_DP_X1(0, blk_, i);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < kWReq; ++i) NV_DP_W1(0u, 0u, i);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < kWReq; ++i) NV_DP_W1(static_cast<uint32_t>(kWBuf), 1u, i);
  __builtin_amdgcn_sched_barrier(0);
  uint32_t blk = 0;
  for (; blk + 2 < nblk; blk += 2) {
    NV_DP_BLOCK(blk, 0, false, true, true);
    NV_DP_BLOCK(blk + 1, 1, false, true, true);
  }
  NV_DP_BLOCK(blk, 0, false, true, false);
  NV_DP_BLOCK(blk + 1, 1, true, false, false);
#undef NV_DP_W1
#undef NV_DP_X1
#undef NV_DP_LDS_READ
#undef NV_DP_READ_B
#undef NV_DP_READ_A
#undef NV_DP_AWAIT
#undef NV_DP_AWAIT_A
#undef NV_DP_WAIT
#undef NV_DP_SLOT
#undef NV_DP_ITEM
#undef NV_DP_BLOCK

  // D layout: lane (n, q) holds rows q*4 .. q*4+3 of a row tile for token n of a token tile
  if constexpr (EPI == kGemmSwiglu && TPW == 3) {
    // the up sums (row parts 2, 3) cross to the waves that hold their gate tiles (parts 0, 1, same token half)
    // through LDS, which everyone has finished with
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    f32x4_t *meet = reinterpret_cast<f32x4_t *>(smem) + (((rq & 1) * 2 + th) * (TPW * 8)) * kWave + lane;
    if (rq >= 2) {
#pragma unroll
      for (int j = 0; j < TPW; ++j)
#pragma unroll
        for (int c = 0; c < 8; ++c) meet[(j * 8 + c) * kWave] = acc[j][c];
    }
    __syncthreads();
    if (rq >= 2) return;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t t = half * 256u + (th * 8 + c) * 16u + n;
      if (t < T) {
#pragma unroll
        for (int j = 0; j < TPW; ++j) block_epilogue<DT, EPI>(p, t, slot_row(TPW * rq + j) + q * 4u, acc[j][c], meet[(j * 8 + c) * kWave]);
      }
    }
  } else if (kslices == 1) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t t = half * 256u + (th * 8 + c) * 16u + n;
      if (t < T) {
        if constexpr (EPI == kGemmSwiglu) {
#pragma unroll
          for (int j = 0; j < 2; ++j) block_epilogue<DT, EPI>(p, t, slot_row(4 * rq + j) + q * 4u, acc[j][c], acc[j + 2][c]);
        } else {
#pragma unroll
          for (int j = 0; j < TPW; ++j) block_epilogue<DT, EPI>(p, t, slot_row(TPW * rq + j) + q * 4u, acc[j][c], acc[j][c]);
        }
      }
    }
  } else {
    const uint32_t wrows = EPI == kGemmSwiglu ? 2u * p.rows : p.rows;
    float *part = partials + static_cast<uint64_t>(slice) * kDTokCap * wrows;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t t = half * 256u + (th * 8 + c) * 16u + n;
      if (t < T) {
#pragma unroll
        for (int j = 0; j < TPW; ++j)
          *reinterpret_cast<float4 *>(part + static_cast<uint64_t>(t) * wrows + slot_row(TPW * rq + j) + q * 4u) =
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

// Blocks of 257..512 rows (gemm_deep_kernel): workgroups of 256 rows (a gate/up pair: 128 + 128) x 256 tokens, or
// of 192 rows (96 + 96) where the rows divide that way and the launch then fills the chip better.
inline uint32_t deep_wg_rows(int epilogue, int tpw) { return (epilogue == kGemmSwiglu ? 32u : 64u) * static_cast<uint32_t>(tpw); }

struct DeepPlan {
  int tpw;            // row tiles a wave: 4, 3, or 0 where the kernel does not take the shape
  uint32_t kslices;
};
// K slices as they would be chosen for `tpw` tiles a wave (0: the rows do not divide)
inline uint32_t deep_slices_for(int epilogue, uint32_t rows, uint32_t cols, int tpw, uint64_t workspace_bytes) {
  if (rows % deep_wg_rows(epilogue, tpw) != 0) return 0;
  const uint32_t wrows = epilogue == kGemmSwiglu ? 2u * rows : rows;
  const uint32_t groups = rows / deep_wg_rows(epilogue, tpw);
  uint32_t slices = 1;
  const int want = tuning(kTuneGemmBlockSlices);
  if (want > 0 && cols % (static_cast<uint32_t>(want) * 2u * kDK) == 0) {
    slices = static_cast<uint32_t>(want);
  } else {
    while (epilogue != kGemmSwiglu && groups * 2u * slices < 192u && slices < 8u && cols % (slices * 2u * 2u * kDK) == 0) slices *= 2u;
  }
  while (slices > 1 && static_cast<uint64_t>(slices) * kDTokCap * wrows * sizeof(float) > workspace_bytes) slices /= 2u;
  return slices;
}
// The tile height whose busiest CU has the least to do: rounds of 256 workgroups x rows a workgroup x columns a slice
inline DeepPlan deep_plan(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes) {
  DeepPlan best{0, 0};
  if (tokens <= kWTokCap || tokens > kDTokCap || cols % (2u * kDK) != 0) return best;
  uint64_t best_cost = ~uint64_t{0};
  for (int tpw = 4; tpw >= 3; --tpw) {
    const uint32_t slices = deep_slices_for(epilogue, rows, cols, tpw, workspace_bytes);
    if (slices == 0) continue;
    const uint64_t wgs = static_cast<uint64_t>(rows / deep_wg_rows(epilogue, tpw)) * 2u * slices;
    const uint64_t cost = (wgs + 255u) / 256u * deep_wg_rows(epilogue, tpw) * (cols / slices);
    if (cost < best_cost) {
      best_cost = cost;
      best = DeepPlan{tpw, slices};
    }
  }
  return best;
}

template <uint32_t DT, int EPI, int TPW>
hipError_t launch_deep_tpw(const GemmRowsParams &p, float *partials, uint32_t kslices, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t raised = hipSuccess;
  std::call_once(once, [] {
    raised = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_deep_kernel<DT, EPI, TPW>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(deep_lds_bytes(TPW)));
  });
  if (raised != hipSuccess) return raised;
  const uint32_t units = p.rows / deep_wg_rows(EPI, TPW) * kslices, halves = (p.tokens + 255u) / 256u;
  hipLaunchKernelGGL((gemm_deep_kernel<DT, EPI, TPW>), dim3((units + 7u) / 8u * 8u * halves), dim3(8 * kWave), deep_lds_bytes(TPW),
                     stream, p, partials, units, kslices);
  return hipGetLastError();
}

template <uint32_t DT, int EPI>
hipError_t launch_deep(const GemmRowsParams &p, float *partials, const DeepPlan &plan, hipStream_t stream) {
  const uint32_t kslices = plan.kslices;
  hipError_t err = plan.tpw == 3 ? launch_deep_tpw<DT, EPI, 3>(p, partials, kslices, stream)
                                 : launch_deep_tpw<DT, EPI, 4>(p, partials, kslices, stream);
  if (err == hipSuccess && kslices > 1) {
    if (EPI == kGemmResidual && p.norm_gamma != nullptr) {   // (the caller asked gemm_rows_fuses_norm first)
      hipLaunchKernelGGL((gemm_finish_norm_kernel<DT>), dim3(p.tokens), dim3(kFinNormThreads), 0, stream, p,
                         static_cast<const float *>(partials), kslices, kDTokCap);
    } else {
      const uint32_t threads = p.rows / 4u * p.tokens;
      hipLaunchKernelGGL((gemm_block_finish_kernel<DT, EPI>), dim3((threads + 255u) / 256u), dim3(256), 0, stream, p,
                         static_cast<const float *>(partials), kslices, kDTokCap);
    }
    err = hipGetLastError();
  }
  return err;
}

template <uint32_t DT>
hipError_t launch_deep_dt(int epilogue, const GemmRowsParams &p, const DeepPlan &plan, hipStream_t stream) {
  float *partials = static_cast<float *>(p.workspace);
  switch (epilogue) {
    case kGemmF32: return launch_deep<DT, kGemmF32>(p, partials, plan, stream);
    case kGemmResidual: return launch_deep<DT, kGemmResidual>(p, partials, plan, stream);
    case kGemmSwiglu: return launch_deep<DT, kGemmSwiglu>(p, partials, plan, stream);
    default: return hipErrorInvalidValue;
  }
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
      return plan.row_tiles == 2 ? launch_block_nr<DT, kGemmF32, 2>(p, partials, plan.kslices, plan.waves, stream)
                                 : launch_block_nr<DT, kGemmF32, 1>(p, partials, plan.kslices, plan.waves, stream);
    case kGemmResidual:
      return plan.row_tiles == 2 ? launch_block_nr<DT, kGemmResidual, 2>(p, partials, plan.kslices, plan.waves, stream)
                                 : launch_block_nr<DT, kGemmResidual, 1>(p, partials, plan.kslices, plan.waves, stream);
    case kGemmSwiglu: return launch_block_nr<DT, kGemmSwiglu, 2>(p, partials, plan.kslices, plan.waves, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

GemmBlockPlan gemm_block_plan(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes) {
  GemmBlockPlan plan{};
  const int mode = tuning(kTuneGemmBlockOff) == 1 ? 0 : 1;   // "gemm_block_off" override: never the shared-X kernel
  const int want_slices = tuning(kTuneGemmBlockSlices);
  const int want_tiles = tuning(kTuneGemmBlockRowTiles);
  const uint32_t min_tokens = tuning(kTuneGemmBlockMinTokens) > 0 ? static_cast<uint32_t>(tuning(kTuneGemmBlockMinTokens)) : 2u;
  // Waves per workgroup: four, or three for a gate/up pair of a small block where that gives every CU a workgroup
  // (rounds of 256 workgroups x rows a workgroup: 12288 pairs are 192 workgroups of 64 + 64 rows or 256 of 48 + 48).
  uint32_t waves = kBW;
  if (epilogue == kGemmSwiglu && tokens <= 64u && rows % 48u == 0 && tuning(kTuneGemmBlockWaves) != 4) {
    const uint32_t four = rows % 64u == 0 ? (rows / 64u + 255u) / 256u * 64u : ~0u, three = (rows / 48u + 255u) / 256u * 48u;
    if (three < four) waves = 3;
  }
  if (mode == 0 || tokens < min_tokens || tokens > kBTokCap || rows % (16u * waves) != 0 || cols % (kBRing * kBK) != 0) return plan;
  const uint32_t wrows = epilogue == kGemmSwiglu ? 2u * rows : rows;
  // Row tiles per wave: two where that still leaves a workgroup for most CUs.
  uint32_t tiles = epilogue == kGemmSwiglu ? 2u : (rows / (16u * kBW * 2u) >= 96u && rows % (16u * kBW * 2u) == 0 ? 2u : 1u);
  if (epilogue != kGemmSwiglu && (want_tiles == 1 || (want_tiles == 2 && rows % (16u * kBW * 2u) == 0))) tiles = want_tiles;
  const uint32_t groups = rows / (epilogue == kGemmSwiglu ? 16u * waves : 16u * kBW * tiles);
  // K slices: enough workgroups for three quarters of the CUs, each slice a whole number of rings of K-blocks.
  // More cost more than they bring - every slice writes its partial sums and the launch that adds them reads
  // them: qkv (6144 x 4096) in 2 / 4 / 8 slices 14.6 / 15.7 / 17.0 us at 32 rows and 21.8 / 24.6 / 25.9 at 128,
  // down (4096 x 12288) in 4 / 8 / 12 slices 21.4 / 23.0 / 25.1 and 31.2 / 34.2 / 36.8, o (4096 x 4096) in 2 / 4 / 8
  // slices 13.6 / 11.1 / 13.1 at 32 rows.
  // (A sliced gate/up pair would write and re-read 12.6 MB of partial sums per slice: measured no faster.)
  uint32_t slices = 1;
  while (epilogue != kGemmSwiglu && groups * slices < 192u && cols % (slices * 2u * kBRing * kBK) == 0) slices *= 2u;
  // A projection that would need eight or more slices of four K-blocks each stays with gemm_rows_kernel: pipelines
  // that short plus the second launch measured 12.6 / 15.9 / 20.0 us against 10.4 / 13.9 / 19.5 at 32 / 64 / 128
  // rows for a 4096 x 4096 projection in eight slices.
  if (want_slices == 0 && slices >= 8 && cols / slices <= 4u * kBK) return plan;
  if (want_slices > 0 && cols % (static_cast<uint32_t>(want_slices) * kBRing * kBK) == 0) slices = want_slices;
  if (slices > 1 && static_cast<uint64_t>(slices) * kBTokCap * wrows * sizeof(float) > workspace_bytes) {
    // not enough room for the partial sums: as many slices as fit (a power of two), or none
    while (slices > 1 && static_cast<uint64_t>(slices) * kBTokCap * wrows * sizeof(float) > workspace_bytes) slices /= 2u;
  }
  plan.row_tiles = tiles;
  plan.kslices = slices;
  plan.waves = waves;
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

// Blocks of 257..512 rows: K slices of gemm_deep_kernel, or 0 where it does not take the shape (rows a multiple of 256
// or 192; a gate/up pair: of 128 or 96). Enough workgroups (row groups x 2 token halves x slices) for three quarters
// of the CUs, each slice an even number of K-blocks, the partial sums within the workspace.
uint32_t gemm_deep_slices(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes) {
  return deep_plan(epilogue, rows, cols, tokens, workspace_bytes).kslices;
}

uint32_t gemm_rows_partial_slices(uint32_t rows, uint32_t cols, uint32_t tokens, uint32_t x_packed, uint64_t workspace_bytes,
                                  uint32_t *slice_stride) {
  if (x_packed == 0 || tokens > kBTokCap) return 0;
  const uint32_t slices = gemm_block_plan(kGemmF32, rows, cols, tokens, workspace_bytes).kslices;
  if (slice_stride != nullptr) *slice_stride = kBTokCap * rows;
  return slices >= 2 && slices <= 4 ? slices : 0;
}

bool gemm_rows_fuses_norm(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint32_t x_packed, uint64_t workspace_bytes) {
  if (epilogue != kGemmResidual || x_packed == 0 || rows % 4 != 0 ||
      rows > static_cast<uint32_t>(kFinNormThreads * kFinNormPerLane * 4))
    return false;
  // wherever a launch of its own adds the K slices: the deep or the wide kernel's, or the shared-X kernel's for smaller blocks
  if (tokens > kWTokCap) return gemm_deep_slices(epilogue, rows, cols, tokens, workspace_bytes) > 1;
  if (tokens > kBTokCap) return gemm_wide_slices(epilogue, rows, cols, tokens, workspace_bytes) > 1;
  return gemm_block_plan(epilogue, rows, cols, tokens, workspace_bytes).kslices > 1;
}

uint64_t gemm_block_workspace_bytes(uint32_t rows_max) {
  // room for 8 slices of the widest plain projection (or 2 of a gate/up pair of that width) at the deep kernel's
  // token stride
  return static_cast<uint64_t>(8) * kDTokCap * rows_max * sizeof(float);
}

hipError_t launch_gemm_wide(uint32_t dtype, int epilogue, const GemmRowsParams &p, uint32_t kslices, hipStream_t stream) {
  if (kslices == 0 || p.x_packed != static_cast<uint32_t>(kWTiles) || p.tokens <= kBTokCap || p.tokens > kWTokCap)
    return hipErrorInvalidValue;
  if (kslices > 1 && p.workspace == nullptr) return hipErrorInvalidValue;
  if (dtype == kBF16) return launch_wide_dt<kBF16>(epilogue, p, kslices, stream);
  if (dtype == kF16) return launch_wide_dt<kF16>(epilogue, p, kslices, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_gemm_deep(uint32_t dtype, int epilogue, const GemmRowsParams &p, uint32_t kslices, hipStream_t stream) {
  const DeepPlan plan = deep_plan(epilogue, p.rows, p.cols, p.tokens, p.workspace != nullptr ? p.workspace_bytes : 0);
  if (kslices == 0 || plan.kslices != kslices || p.x_packed != gemm_packed_tiles(p.tokens)) return hipErrorInvalidValue;
  if (kslices > 1 && p.workspace == nullptr) return hipErrorInvalidValue;
  if (dtype == kBF16) return launch_deep_dt<kBF16>(epilogue, p, plan, stream);
  if (dtype == kF16) return launch_deep_dt<kF16>(epilogue, p, plan, stream);
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
