// Counter-based synthetic tensor generator, device side. Integer hash + one
// exact int->float conversion + one f32 multiply + one f32 add, so a host
// implementation of the same recipe produces bit-identical values.
//   sum  = twelve 16-bit fields of three splitmix64 outputs (Irwin-Hall, n = 12)
//   val  = mean + float(2*sum - 786420) * (std / 131072)
#pragma once

#include "nv_common.cuh"

namespace nv {

__host__ __device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
__host__ __device__ __forceinline__ uint64_t synth_key(uint64_t seed, uint64_t tensor_id) {
  return splitmix64(seed ^ (tensor_id * 0xD6E8FEB86659FD93ull));
}
__device__ __forceinline__ float synth_value(uint64_t key, uint64_t index, float mean, float scale) {
  // the multiply and the add must round separately (a fused multiply-add would differ from the host)
#pragma clang fp contract(off)
  uint32_t sum = 0;
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const uint64_t h = splitmix64(key + (3 * index + static_cast<uint64_t>(j)) * 0x9E3779B97F4A7C15ull);
    sum += static_cast<uint32_t>(h & 0xffff) + static_cast<uint32_t>((h >> 16) & 0xffff) +
           static_cast<uint32_t>((h >> 32) & 0xffff) + static_cast<uint32_t>(h >> 48);
  }
  const int32_t centered = static_cast<int32_t>(2 * sum) - 786420;
  const float scaled = static_cast<float>(centered) * scale;
  return mean + scaled;
}

hipError_t launch_synth_16(void *dst, uint32_t dtype, uint64_t seed, uint64_t tensor_id,
                           uint64_t count, float mean, float std, hipStream_t stream);
hipError_t launch_synth_f32(void *dst, uint64_t seed, uint64_t tensor_id, uint64_t count, float mean,
                            float std, hipStream_t stream);
hipError_t launch_synth_fp8_block(void *weights, void *scales, uint64_t seed, uint64_t tensor_id,
                                  uint64_t rows, uint64_t cols, uint64_t block, float std,
                                  hipStream_t stream);
hipError_t launch_synth_tokens(uint32_t *dst, uint64_t seed, uint64_t tensor_id, uint64_t count,
                               uint32_t vocab, hipStream_t stream);

}  // namespace nv
