// Shared device helpers: 16-bit / fp8 codecs, wave64 reductions, error plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nv {

constexpr uint32_t kF16 = 0;
constexpr uint32_t kBF16 = 1;
constexpr int kWave = 64;          // CDNA wavefront
constexpr int kBlock = 256;        // 4 waves per workgroup everywhere in this library
constexpr int kWavesPerBlock = kBlock / kWave;

// ---- 16-bit codecs -------------------------------------------------------
// bf16: widen = shift; narrow = round-to-nearest-even on the dropped 16 bits
// (reference: precision/bits.rs:4-18, device_ops.cuh:9-31).
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
  const uint32_t bits = __float_as_uint(v);
  // both results are computed and one is selected: no branch in the hot epilogues
  const uint32_t rounded = (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
  const uint32_t nan = (bits >> 16) | 1u;
  return static_cast<uint16_t>((bits & 0x7fffffffu) > 0x7f800000u ? nan : rounded);
}
__device__ __forceinline__ float f16_to_f32(uint16_t b) {
  return static_cast<float>(__builtin_bit_cast(_Float16, b));
}
__device__ __forceinline__ uint16_t f32_to_f16(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));  // v_cvt_f16_f32: RNE
}

template <uint32_t DT>
__device__ __forceinline__ float dec16(uint16_t b) {
  if constexpr (DT == kBF16) return bf16_to_f32(b);
  else return f16_to_f32(b);
}
template <uint32_t DT>
__device__ __forceinline__ uint16_t enc16(float v) {
  if constexpr (DT == kBF16) return f32_to_bf16(v);
  else return f32_to_f16(v);
}
template <uint32_t DT>
__device__ __forceinline__ float round16(float v) {
  return dec16<DT>(enc16<DT>(v));
}
// One dword = two packed 16-bit values (little endian: low half first).
template <uint32_t DT>
__device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi) {
  if constexpr (DT == kBF16) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  } else {
    lo = f16_to_f32(static_cast<uint16_t>(w & 0xffffu));
    hi = f16_to_f32(static_cast<uint16_t>(w >> 16));
  }
}

// ---- wave64 / block reductions -------------------------------------------
// Through the lane-crossing modifiers of the vector ALU (DPP), not through the LDS crossbar that __shfl_xor
// compiles to: a row of 16 lanes folds in four steps (neighbour, pair, the mirrored half, the mirrored row:
// afterwards every lane of a row holds the row's result), and the four rows meet through four lane reads. The
// crossbar route was six dependent ds_bpermute round trips - about 0.25 us behind the last data of every row
// of a GEMV (the down projection 16.95 -> 16.7 us with the reduction taken out altogether). Every lane gets
// the result; the fold order is fixed, so results are deterministic.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppQuadSwap1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<kDppQuadSwap1>(v);
  v += dpp_move<kDppQuadSwap2>(v);
  v += dpp_move<kDppRowHalfMirror>(v);
  v += dpp_move<kDppRowMirror>(v);
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<kDppQuadSwap1>(v));
  v = fmaxf(v, dpp_move<kDppQuadSwap2>(v));
  v = fmaxf(v, dpp_move<kDppRowHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppRowMirror>(v));
  return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}
// Sum over a 256-thread block; every thread gets the result. `scratch` is
// kWavesPerBlock floats of LDS. Fixed combination order -> deterministic.
__device__ __forceinline__ float block_sum(float v, float *scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) total += scratch[w];
  return total;
}

// The same for a workgroup of WG waves (`scratch`: WG floats).
template <int WG>
__device__ __forceinline__ float block_sum_n(float v, float *scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < WG; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// (value desc, index asc) among finite candidates; `has` false = no candidate yet
// (reference: sampler.cu:35-40).
struct Best {
  float value;
  uint32_t index;
  uint32_t has;
};
__device__ __forceinline__ bool better(const Best &a, const Best &b) {
  if (!a.has) return false;
  if (!b.has) return true;
  return a.value > b.value || (a.value == b.value && a.index < b.index);
}
__device__ __forceinline__ Best wave_best(Best b) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Best other;
    other.value = __shfl_xor(b.value, o, kWave);
    other.index = __shfl_xor(b.index, o, kWave);
    other.has = __shfl_xor(b.has, o, kWave);
    if (better(other, b)) b = other;
  }
  return b;
}

// Launch-shape overrides for measurements and tests, set through nerva_hip_test_set_tuning (0 = the
// built-in choice). The product path never reads the environment for these.
enum TuningKnob : int {
  kTuneAttnSplits = 0,       // split-KV factor of a session's decode attention (read at session create)
  kTuneBatchSplits,          // split factor of the batch step's attention
  kTunePromptSplits,         // split factor of the prompt-block attention
  kTuneGemmRowTiles,         // multi-row GEMM: 1 or 2 row tiles per wave for every plain projection
  kTuneGemmKWaves,           // multi-row GEMM: 8 or 4 waves along K
  kTuneGemmBlockSlices,      // shared-X GEMM: K slices for every projection
  kTuneGemmBlockRowTiles,    // shared-X GEMM: 1 or 2 row tiles per wave
  kTuneGemmBlockMinTokens,   // shared-X GEMM: smallest token block it takes
  kTuneGemvExactStart,       // lean GEMV: 1 = exact start-up waits wherever they can run, 2 = nowhere
  kTuneMoeDownSharedFirst,   // lean MoE down: 2 = walk the shared expert last, as the caller orders the slots
  kTuneGemvWorkgroupWaves,   // lean GEMV: waves per workgroup for every launch (4 or 16)
  kTuneGemvXRegisters,       // lean GEMV: 2 = never keep the input vector in registers
  kTunePrefillBlockTokens,   // prompt blocks of a session: 128 = never the 256-token blocks (read at session create)
  kTuneGemvRotatedWalk,      // lean GEMV: 2 = never the rotated walk
  kTuneAttnMergeSpinLimit,   // decode attention: polls after which a split merge gives up (tests of the error path)
  kTuneAttnWithholdSplit,    // decode attention: 1 + a split that keeps its partial to itself (tests of the error path)
  kTuneBlockLayout,          // token blocks: 1 = [token][column] rows, 2 = matrix-operand order, whatever their size
  kTunePrefillAttentionRows, // prompt blocks: 1 = one attention workgroup set per token instead of the shared-tile kernel
  kTunePrefillWalk,          // 1 = start() walks the prompt token by token (read at session create)
  kTuneGemmBlockOff,         // 1 = blocks of up to 128 rows use gemm_rows_kernel, never the shared-X kernel
  kTuneGemmBlockWaves,       // shared-X GEMM, gate/up pairs of up to 64 token rows: 4 = never three-wave workgroups
  kTuneGemmBlockRotate,      // shared-X GEMM: 1 + the K-blocks between the starts of consecutive row groups (1: a common start)
  kTuneKnobs
};
int tuning(TuningKnob knob);

// 16-byte streaming load that does not pollute the caches with single-use weights.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream(const void *p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

}  // namespace nv
