// Stand-alone device argmax over a logits vector (the decode step itself fuses
// this into the LM-head GEMV epilogue). First maximum among finite values, ties
// to the lowest index (sampler.cu:35-40,89-119; common/token.rs:33-58).
#include "argmax.cuh"

#include <mutex>

#include "gemv_stream.cuh"
#include "runtime_state.hpp"

namespace nv {

namespace {

// Candidate storage of nerva_hip_argmax_static: one (value, index, has) triple per workgroup of the
// first launch, kept in the library's own device image so the call never allocates. Every GPU holds
// its own copy at its own address; host code only ever uses the address that hipGetSymbolAddress
// returned for the current device (static_scratch), never the array's name.
constexpr uint32_t kArgmaxBlocks = 512;  // workgroups of the first launch (they loop over the logits)
static __device__ __align__(256) uint32_t scratch[3 * kArgmaxBlocks];

constexpr int kMaxDevices = 16;
std::mutex g_scratch_mutex;
uint32_t *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device. `resolve` (set-up calls only): ask the runtime for it if
// this device has none yet; without it an unresolved device is hipErrorNotInitialized - the entry point itself
// neither takes the mutex's slow path nor calls into the runtime's symbol tables (neither is safe under stream
// capture).
hipError_t static_scratch(uint32_t **out, bool resolve) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return err;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    if (!resolve) return hipErrorNotInitialized;
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (ptr == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = static_cast<uint32_t *>(ptr);
  }
  *out = g_scratch_ptr[device];
  return hipSuccess;
}

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
  if (blocks > kArgmaxBlocks) blocks = kArgmaxBlocks;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(argmax_kernel, dim3(blocks), dim3(kBlock), 0, stream, logits, count, s);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  return launch_sample_finish(s, blocks, nullptr, 0, stream);
}

hipError_t argmax_static_setup() {
  uint32_t *ptr = nullptr;
  return static_scratch(&ptr, true);
}

}  // namespace nv

extern "C" {

int nerva_hip_argmax_static(const float *logits, uint32_t count, uint32_t *token, void *stream,
                            int32_t *hip_error) {
  using namespace nv;
  auto done = [&](hipError_t err) {
    if (hip_error) *hip_error = static_cast<int32_t>(err);
    return err == hipSuccess ? 0 : -1;
  };
  if (hip_error) *hip_error = 0;
  if (logits == nullptr || token == nullptr || count == 0 || count > NERVA_HIP_ARGMAX_STATIC_MAX_COUNT)
    return done(hipErrorInvalidValue);
  // Nothing is created or resolved here: the library's stream (when the caller passes none) and the scratch
  // address of the current device come from nerva_hip_device_smoke, which has to have run on this device.
  hipStream_t s = stream != nullptr ? static_cast<hipStream_t>(stream) : library_stream_if_created();
  if (s == nullptr) return done(hipErrorNotInitialized);
  uint32_t *base = nullptr;
  hipError_t err = static_scratch(&base, false);
  if (err != hipSuccess) return done(err);
  SampleParams p{};
  p.part_value = reinterpret_cast<float *>(base);
  p.part_index = base + kArgmaxBlocks;
  p.part_has = base + 2 * kArgmaxBlocks;
  p.token_out = token;
  // Both launches write every candidate they later read, so nothing has to be cleared between calls.
  return done(launch_argmax(logits, count, p, s));
}

}  // extern "C"
