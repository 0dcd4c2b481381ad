// Multi-row projection on the matrix cores: Y[t][r] = sum_c W[r][c] * X[t][c] for a block of
// T <= 128 token rows, streaming the weight matrix once for all of them. This is what a chunk of
// prompt tokens (and a small batch of sequences) needs: the weight bytes are the same as for one
// token, so the kernel is HBM-bound like the GEMV and T tokens cost about one.
// Reference: the cuBLAS GEMM calls of the chunked prefill and of the projection batch
// (native/cuda/hf_decode_sequence/projection.cu:99-106, 297-300; session_decode_prefill.inc.cu:
// 1879-2243); arithmetic as mat_vec_encoded_row_major per token (precision/block/ops.rs:75-91).
//
// gfx950 mapping: a workgroup owns 16 weight rows (for SwiGLU: 16 gate rows and their 16 up
// rows) over the full K; its 8 waves split K. A wave walks its K range in blocks of 256 columns:
// the block of W is requested with coalesced loads (512 contiguous bytes per row and
// instruction, like the GEMV), parked in a wave-private LDS tile and read back in matrix-operand
// order; the X operand comes straight from global memory (L2), one 16-byte piece per lane, token
// and K-step. v_mfma_f32_16x16x32 accumulates D[weight row][token] in f32, two token tiles per
// wave; the waves' partial sums meet in LDS and are added in wave order (deterministic), then
// the epilogue runs once per output element.
// Blocks of more than 64 rows with X in operand order take another kernel (gemm_block.hip) in which the
// waves of a workgroup split the rows instead and share each K-block of X through LDS.
#pragma once

#include "nv_common.cuh"

namespace nv {

constexpr uint32_t kGemmMaxTokens = 128;       // token rows of a block in any layout
constexpr uint32_t kGemmWideMaxTokens = 256;   // token rows of a block in operand order, where gemm_wide_slices takes the shape
constexpr uint32_t kGemmDeepMaxTokens = 512;   // ... where gemm_deep_slices takes the shape

// Operand order of a block of token rows X[t][k] (16-bit), the layout the multi-row GEMM reads fastest:
// for every K-step of 32 columns and every tile of 16 tokens the 64 lanes' 16-byte pieces in lane order,
// lane = (k % 32 / 8) * 16 + t % 16 holding columns k - k % 8 .. + 7 of token t. `tiles` token tiles per
// K-step; a buffer holds tiles * 16 token slots (slots past the block's tokens are never looked at).
__host__ __device__ __forceinline__ uint64_t gemm_x_packed_index(uint32_t tiles, uint32_t t, uint32_t k) {
  return (static_cast<uint64_t>(k / 32u) * tiles + t / 16u) * 512u + (((k % 32u) / 8u) * 16u + t % 16u) * 8u + k % 8u;
}
// Token tiles the GEMM works with for a block of `tokens` rows (its X buffer in operand order has as many).
__host__ __device__ __forceinline__ uint32_t gemm_packed_tiles(uint32_t tokens) {
  return tokens > 256u ? 32u : tokens > 128u ? 16u : tokens > 64u ? 8u : tokens > 32u ? 4u : 2u;
}
enum : int { kGemmF32 = 0, kGemmResidual = 1, kGemmSwiglu = 2 };

struct GemmRowsParams {
  const uint16_t *w;         // [rows][cols] row-major 16-bit (SwiGLU: [2*rows][cols], gate rows first)
  const uint16_t *x16;       // [tokens][cols] 16-bit inputs
  const uint16_t *bias;      // optional [rows] (SwiGLU: [2*rows])
  const float *residual;     // kGemmResidual: [tokens][rows]
  float *out_f32;            // kGemmF32 / kGemmResidual: [tokens][rows]
  uint16_t *out16;           // kGemmSwiglu: [tokens][rows] = round16(silu(gate) * up)
  uint32_t rows, cols, tokens;
  uint32_t pair_gap;         // kGemmSwiglu: elements left unused between the last gate row and the first up row
  uint32_t round_out;        // kGemmResidual: round the sum to 16 bit
  uint32_t x_packed;         // != 0: x16 is in matrix-operand order (gemm_x_packed_index) instead of [tokens][cols];
                             // the value is its token-tile count and must be gemm_packed_tiles(tokens)
  uint32_t out_packed_tiles; // kGemmSwiglu: != 0 writes out16 in operand order with this many token tiles
  uint32_t keep_partials;    // kGemmF32, only where gemm_rows_partial_slices() says so: the K slices' partial sums stay in
                             // the workspace ([slice][128 tokens][rows] f32) for a reader that adds them; out_f32 is not written
  void *workspace;           // optional: room for the f32 partial sums of the shared-X kernel's K slices
  uint64_t workspace_bytes;  // (gemm_block_workspace_bytes; without it that kernel runs unsliced or not at all)
  // kGemmResidual, optional, only where gemm_rows_fuses_norm() says so: the launch that adds the K slices also
  // writes the RMSNorm of every output row - norm_out16[t] = round16(y[t] * rsqrt(mean(y[t]^2) + norm_eps) *
  // norm_gamma), bit for bit what launch_rmsnorm_rows gives on out_f32 - in operand order when
  // norm_packed_tiles != 0.
  const uint16_t *norm_gamma;
  uint16_t *norm_out16;
  float norm_eps;
  uint32_t norm_packed_tiles;
};

// rows >= 16 (any count: the last workgroup overlaps its neighbour, so with a row count that is no
// multiple of 16 a residual must not be added in place), cols % 2048 == 0 (each of the 8 waves walks
// whole 256-column blocks), 1 <= tokens <= kGemmMaxTokens, 16-byte aligned w and x16.
bool gemm_rows_supported(uint32_t rows, uint32_t cols, uint32_t tokens);
hipError_t launch_gemm_rows(uint32_t dtype, int epilogue, const GemmRowsParams &p, hipStream_t stream);

// Blocks of more than 64 token rows with X in operand order: the kernel that shares the X operand through
// LDS (gemm_block.hip). The plan says whether it takes a shape (kslices != 0) and how: row tiles per wave
// and K slices (more than one needs slices x 128 x W rows f32 of workspace). launch_gemm_rows uses it by
// itself where the plan allows.
struct GemmBlockPlan {
  uint32_t row_tiles, kslices, waves;
};
GemmBlockPlan gemm_block_plan(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes);
// K slices (2..4) whose partial sums a plain projection of this shape can leave to its reader (keep_partials), with
// their stride in f32 elements; 0 where the launch has no slices, or more than a reader takes.
uint32_t gemm_rows_partial_slices(uint32_t rows, uint32_t cols, uint32_t tokens, uint32_t x_packed, uint64_t workspace_bytes,
                                  uint32_t *slice_stride);
// Workspace that lets every projection of up to `rows_max` output rows (a gate/up pair counts twice) use its plan.
uint64_t gemm_block_workspace_bytes(uint32_t rows_max);
hipError_t launch_gemm_block(uint32_t dtype, int epilogue, const GemmRowsParams &p, const GemmBlockPlan &plan,
                             hipStream_t stream);
// Blocks of 129..kGemmWideMaxTokens rows in operand order (16 token tiles): K slices the kernel for them
// would use for a shape (more than one needs slices x 256 x W rows f32 of workspace), 0 = shape not taken
// (rows a multiple of 128, gate/up pairs of 64; cols a multiple of 512 per slice). launch_gemm_rows uses it by itself.
uint32_t gemm_wide_slices(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes);
hipError_t launch_gemm_wide(uint32_t dtype, int epilogue, const GemmRowsParams &p, uint32_t kslices, hipStream_t stream);
// Blocks of 257..kGemmDeepMaxTokens rows in operand order (32 token tiles): the same for the kernel that takes
// 256 or 192 rows x 256 tokens per workgroup (rows a multiple of 192 or 256, a gate/up pair of 96 or 128, cols of 128).
uint32_t gemm_deep_slices(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint64_t workspace_bytes);
hipError_t launch_gemm_deep(uint32_t dtype, int epilogue, const GemmRowsParams &p, uint32_t kslices, hipStream_t stream);
// Whether launch_gemm_rows honours GemmRowsParams::norm_gamma for this shape (a K-sliced residual projection of a
// wide block, rows a multiple of 4 and at most 16384); otherwise the caller normalises with launch_rmsnorm_rows.
bool gemm_rows_fuses_norm(int epilogue, uint32_t rows, uint32_t cols, uint32_t tokens, uint32_t x_packed, uint64_t workspace_bytes);

// x16[t] = round16(x[t] * rsqrt(mean(x[t]^2) + eps) * gamma) for `tokens` rows of `cols` f32 values.
// packed_tiles != 0: out16 in operand order (gemm_x_packed_index) with that many token tiles.
hipError_t launch_rmsnorm_rows(uint32_t dtype, const float *x, const uint16_t *gamma, float eps, uint32_t tokens,
                               uint32_t cols, uint16_t *out16, hipStream_t stream, uint32_t packed_tiles = 0);

}  // namespace nv
