// Device-side synthetic tensor fills (see synth_fill.cuh for the recipe).
#include "synth_fill.cuh"

#include "fp8_codec.cuh"

namespace nv {

namespace {

template <uint32_t DT>
__global__ __launch_bounds__(kBlock) void synth16_kernel(uint16_t *dst, uint64_t key, uint64_t count,
                                                         float mean, float scale) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kBlock;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < count; i += stride)
    dst[i] = enc16<DT>(synth_value(key, i, mean, scale));
}

__global__ __launch_bounds__(kBlock) void synth32_kernel(float *dst, uint64_t key, uint64_t count,
                                                         float mean, float scale) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kBlock;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < count; i += stride)
    dst[i] = synth_value(key, i, mean, scale);
}

__global__ __launch_bounds__(kBlock) void synth_tokens_kernel(uint32_t *dst, uint64_t key,
                                                              uint64_t count, uint32_t vocab) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kBlock;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < count; i += stride)
    dst[i] = static_cast<uint32_t>(splitmix64(key + i * 0x9E3779B97F4A7C15ull) % vocab);
}

// One workgroup per (block_row, block_col) tile: amax -> S = amax/448 -> q = e4m3(w/S).
__global__ __launch_bounds__(kBlock) void synth_fp8_kernel(uint8_t *w, float *scales, uint64_t key,
                                                           uint64_t rows, uint64_t cols,
                                                           uint64_t block, float scale) {
  __shared__ float red[kWavesPerBlock];
  const uint64_t sc = (cols + block - 1) / block;
  const uint64_t br = blockIdx.x / sc, bc = blockIdx.x % sc;
  const uint64_t r0 = br * block, c0 = bc * block;
  const uint64_t r1 = min(rows, r0 + block), c1 = min(cols, c0 + block);
  const uint64_t tile_cols = c1 - c0, n = (r1 - r0) * tile_cols;
  float amax = 0.0f;
  for (uint64_t i = threadIdx.x; i < n; i += kBlock) {
    const uint64_t r = r0 + i / tile_cols, c = c0 + i % tile_cols;
    amax = fmaxf(amax, fabsf(synth_value(key, r * cols + c, 0.0f, scale)));
  }
  amax = wave_max(amax);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = amax > 0.0f ? __fdiv_rn(amax, 448.0f) : 1.0f;
  if (threadIdx.x == 0) scales[br * sc + bc] = s;
  for (uint64_t i = threadIdx.x; i < n; i += kBlock) {
    const uint64_t r = r0 + i / tile_cols, c = c0 + i % tile_cols;
    w[r * cols + c] = f32_to_fp8_e4m3fn(__fdiv_rn(synth_value(key, r * cols + c, 0.0f, scale), s));
  }
}

uint32_t fill_grid(uint64_t count) {
  uint64_t blocks = (count + kBlock - 1) / kBlock;
  if (blocks > 256u * 16u) blocks = 256u * 16u;
  return blocks == 0 ? 1u : static_cast<uint32_t>(blocks);
}

}  // namespace

hipError_t launch_synth_16(void *dst, uint32_t dtype, uint64_t seed, uint64_t tensor_id,
                           uint64_t count, float mean, float std, hipStream_t stream) {
  if (dst == nullptr || dtype > kBF16) return hipErrorInvalidValue;
  if (count == 0) return hipSuccess;
  const uint64_t key = synth_key(seed, tensor_id);
  const float scale = std / 131072.0f;
  if (dtype == kBF16)
    hipLaunchKernelGGL(synth16_kernel<kBF16>, dim3(fill_grid(count)), dim3(kBlock), 0, stream,
                       static_cast<uint16_t *>(dst), key, count, mean, scale);
  else
    hipLaunchKernelGGL(synth16_kernel<kF16>, dim3(fill_grid(count)), dim3(kBlock), 0, stream,
                       static_cast<uint16_t *>(dst), key, count, mean, scale);
  return hipGetLastError();
}

hipError_t launch_synth_f32(void *dst, uint64_t seed, uint64_t tensor_id, uint64_t count, float mean,
                            float std, hipStream_t stream) {
  if (dst == nullptr) return hipErrorInvalidValue;
  if (count == 0) return hipSuccess;
  hipLaunchKernelGGL(synth32_kernel, dim3(fill_grid(count)), dim3(kBlock), 0, stream,
                     static_cast<float *>(dst), synth_key(seed, tensor_id), count, mean,
                     std / 131072.0f);
  return hipGetLastError();
}

hipError_t launch_synth_tokens(uint32_t *dst, uint64_t seed, uint64_t tensor_id, uint64_t count,
                               uint32_t vocab, hipStream_t stream) {
  if (dst == nullptr || vocab == 0) return hipErrorInvalidValue;
  if (count == 0) return hipSuccess;
  hipLaunchKernelGGL(synth_tokens_kernel, dim3(fill_grid(count)), dim3(kBlock), 0, stream, dst,
                     synth_key(seed, tensor_id), count, vocab);
  return hipGetLastError();
}

hipError_t launch_synth_fp8_block(void *weights, void *scales, uint64_t seed, uint64_t tensor_id,
                                  uint64_t rows, uint64_t cols, uint64_t block, float std,
                                  hipStream_t stream) {
  if (weights == nullptr || scales == nullptr || rows == 0 || cols == 0 || block == 0)
    return hipErrorInvalidValue;
  const uint64_t tiles = ((rows + block - 1) / block) * ((cols + block - 1) / block);
  if (tiles > 0x7fffffffull) return hipErrorInvalidValue;
  hipLaunchKernelGGL(synth_fp8_kernel, dim3(static_cast<uint32_t>(tiles)), dim3(kBlock), 0, stream,
                     static_cast<uint8_t *>(weights), static_cast<float *>(scales),
                     synth_key(seed, tensor_id), rows, cols, block, std / 131072.0f);
  return hipGetLastError();
}

}  // namespace nv
