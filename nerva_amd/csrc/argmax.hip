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
  Best block_best{red[0], red_i[0], red_h[0]};
  for (int w = 1; w < kWavesPerBlock; ++w) {
    Best o{red[w], red_i[w], red_h[w]};
    if (better(o, block_best)) block_best = o;
  }
  __syncthreads();
  sample_finish(s, block_best, red, red_i, red_h);
}

}  // namespace

uint64_t sample_workspace_bytes() { return (3ull * kSampleMaxBlocks + 64) * sizeof(uint32_t); }

void sample_bind_workspace(SampleParams &s, void *workspace) {
  uint32_t *base = static_cast<uint32_t *>(workspace);
  s.counter = base;  // first 64 words: counter + padding
  s.part_value = reinterpret_cast<float *>(base + 64);
  s.part_index = base + 64 + kSampleMaxBlocks;
  s.part_has = base + 64 + 2 * kSampleMaxBlocks;
}

hipError_t launch_argmax(const float *logits, uint32_t count, const SampleParams &s,
                         hipStream_t stream) {
  if (logits == nullptr || count == 0 || s.counter == nullptr) return hipErrorInvalidValue;
  uint32_t blocks = (count + kBlock * 8 - 1) / (kBlock * 8);
  if (blocks > 512) blocks = 512;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(argmax_kernel, dim3(blocks), dim3(kBlock), 0, stream, logits, count, s);
  return hipGetLastError();
}

}  // namespace nv
