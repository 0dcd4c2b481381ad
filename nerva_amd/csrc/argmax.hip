// Stand-alone device argmax over a logits vector (the decode step itself fuses
// this into the LM-head GEMV epilogue). First maximum among finite values, ties
// to the lowest index (sampler.cu:35-40,89-119; common/token.rs:33-58).
#include "argmax.cuh"

#include "gemv_stream.cuh"

namespace nv {

namespace {

__global__ __launch_bounds__(kBlock) void argmax_kernel(const float *logits, uint32_t count,
                                                        SampleParams s) {
  __shared__ float red[kWavesPerBlock];
  __shared__ uint32_t red_i[kWavesPerBlock];
  __shared__ uint32_t red_h[kWavesPerBlock];
  Best b{0.0f, 0u, 0u};
  for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < count; i += gridDim.x * kBlock) {
    const float v = logits[i];
    Best c{v, i, isfinite(v) ? 1u : 0u};
    if (better(c, b)) b = c;
  }
  b = wave_best(b);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    red[wave] = b.value;
    red_i[wave] = b.index;
    red_h[wave] = b.has;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    Best block_best{red[0], red_i[0], red_h[0]};
    for (int w = 1; w < kWavesPerBlock; ++w) {
      Best o{red[w], red_i[w], red_h[w]};
      if (better(o, block_best)) block_best = o;
    }
    s.part_value[blockIdx.x] = block_best.value;
    s.part_index[blockIdx.x] = block_best.index;
    s.part_has[blockIdx.x] = block_best.has;
  }
}

}  // namespace

uint64_t sample_workspace_bytes() { return 3ull * kSampleMaxBlocks * sizeof(uint32_t); }

void sample_bind_workspace(SampleParams &s, void *workspace) {
  uint32_t *base = static_cast<uint32_t *>(workspace);
  s.part_value = reinterpret_cast<float *>(base);
  s.part_index = base + kSampleMaxBlocks;
  s.part_has = base + 2 * kSampleMaxBlocks;
}

hipError_t launch_argmax(const float *logits, uint32_t count, const SampleParams &s,
                         hipStream_t stream) {
  if (logits == nullptr || count == 0 || s.part_value == nullptr) return hipErrorInvalidValue;
  uint32_t blocks = (count + kBlock * 8 - 1) / (kBlock * 8);
  if (blocks > 512) blocks = 512;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(argmax_kernel, dim3(blocks), dim3(kBlock), 0, stream, logits, count, s);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  return launch_sample_finish(s, blocks, nullptr, 0, stream);
}

}  // namespace nv
