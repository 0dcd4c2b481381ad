// Host launcher for the weight-streaming GEMV kernels (gemv_stream.cuh).
#include "gemv_stream.cuh"

namespace nv {

namespace {

// Defaults chosen from on-device sweeps (rows per wave, loads in flight, dot2).
constexpr int kDefaultNR = 2;
constexpr int kDefaultU = 8;
constexpr bool kDefaultDot2 = false;
constexpr uint32_t kDefaultMaxBlocks = 256u * 8u;  // 8 workgroups per CU

template <uint32_t DT, int PRO, int EPI, int MODE>
hipError_t launch_one(const GemvParams &p, uint32_t blocks, size_t lds, hipStream_t stream) {
  if constexpr (MODE == kVecFull) {
    hipLaunchKernelGGL((gemv_kernel<DT, PRO, EPI, kDefaultNR, kDefaultU, kVecFull, kDefaultDot2>),
                       dim3(blocks), dim3(kBlock), lds, stream, p);
  } else if constexpr (MODE == kVecGuarded) {
    hipLaunchKernelGGL((gemv_kernel<DT, PRO, EPI, kDefaultNR, 4, kVecGuarded, false>), dim3(blocks),
                       dim3(kBlock), lds, stream, p);
  } else {
    hipLaunchKernelGGL((gemv_kernel<DT, PRO, EPI, kDefaultNR, 1, kScalar, false>), dim3(blocks),
                       dim3(kBlock), lds, stream, p);
  }
  return hipGetLastError();
}

template <uint32_t DT, int PRO, int MODE>
hipError_t launch_epi(int epilogue, const GemvParams &p, uint32_t blocks, size_t lds,
                      hipStream_t stream) {
  switch (epilogue) {
    case kEpiF32: return launch_one<DT, PRO, kEpiF32, MODE>(p, blocks, lds, stream);
    case kEpiResidual: return launch_one<DT, PRO, kEpiResidual, MODE>(p, blocks, lds, stream);
    case kEpiSwiglu: return launch_one<DT, PRO, kEpiSwiglu, MODE>(p, blocks, lds, stream);
    case kEpiOut16: return launch_one<DT, PRO, kEpiOut16, MODE>(p, blocks, lds, stream);
    case kEpiArgmax: return launch_one<DT, PRO, kEpiArgmax, MODE>(p, blocks, lds, stream);
    default: return hipErrorInvalidValue;
  }
}

template <uint32_t DT, int MODE>
hipError_t launch_pro(int prologue, int epilogue, const GemvParams &p, uint32_t blocks, size_t lds,
                      hipStream_t stream) {
  if (prologue == kProX16) return launch_epi<DT, kProX16, MODE>(epilogue, p, blocks, lds, stream);
  if (prologue == kProRmsNorm) return launch_epi<DT, kProRmsNorm, MODE>(epilogue, p, blocks, lds, stream);
  return hipErrorInvalidValue;
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

uint32_t gemv_grid_blocks(int epilogue, uint32_t rows, int rows_per_wave, int max_blocks) {
  const uint32_t units = epilogue == kEpiSwiglu ? rows : (rows + rows_per_wave - 1) / rows_per_wave;
  uint32_t blocks = (units + kWavesPerBlock - 1) / kWavesPerBlock;
  uint32_t cap = max_blocks > 0 ? static_cast<uint32_t>(max_blocks) : kDefaultMaxBlocks;
  if (epilogue == kEpiArgmax && cap > kSampleMaxBlocks) cap = kSampleMaxBlocks;
  if (blocks > cap) blocks = cap;
  return blocks == 0 ? 1 : blocks;
}

hipError_t launch_gemv(uint32_t dtype, int prologue, int epilogue, const GemvParams &p,
                       hipStream_t stream, const GemvTuning *tuning) {
  if (p.w == nullptr || p.rows == 0 || p.cols == 0) return hipErrorInvalidValue;
  if (prologue == kProX16 && p.x16 == nullptr) return hipErrorInvalidValue;
  if (prologue == kProRmsNorm && (p.xf == nullptr || p.gamma == nullptr)) return hipErrorInvalidValue;
  if ((epilogue == kEpiF32 || epilogue == kEpiResidual || epilogue == kEpiArgmax) && p.out_f32 == nullptr)
    return hipErrorInvalidValue;
  if ((epilogue == kEpiSwiglu || epilogue == kEpiOut16) && p.out16 == nullptr) return hipErrorInvalidValue;
  if (epilogue == kEpiResidual && p.residual == nullptr) return hipErrorInvalidValue;
  if (epilogue == kEpiArgmax &&
      (p.sample.part_value == nullptr || p.sample.part_index == nullptr ||
       p.sample.part_has == nullptr || p.sample.counter == nullptr))
    return hipErrorInvalidValue;
  if (dtype != kF16 && dtype != kBF16) return hipErrorInvalidValue;

  const bool vec = (p.cols % 8 == 0) && aligned16(p.w) &&
                   (prologue == kProX16 ? aligned16(p.x16) : aligned16(p.xf));
  const size_t lds = static_cast<size_t>((p.cols + 7) / 8 * 8) * sizeof(uint16_t);
  if (lds > 60 * 1024) return hipErrorInvalidValue;  // K up to 30720 fits one workgroup's LDS
  const uint32_t blocks = gemv_grid_blocks(epilogue, p.rows, kDefaultNR, tuning ? tuning->max_blocks : 0);

  const int mode = !vec ? kScalar : (p.cols % (kWave * 8) == 0 ? kVecFull : kVecGuarded);
  if (dtype == kBF16) {
    if (mode == kVecFull) return launch_pro<kBF16, kVecFull>(prologue, epilogue, p, blocks, lds, stream);
    if (mode == kVecGuarded) return launch_pro<kBF16, kVecGuarded>(prologue, epilogue, p, blocks, lds, stream);
    return launch_pro<kBF16, kScalar>(prologue, epilogue, p, blocks, lds, stream);
  }
  if (mode == kVecFull) return launch_pro<kF16, kVecFull>(prologue, epilogue, p, blocks, lds, stream);
  if (mode == kVecGuarded) return launch_pro<kF16, kVecGuarded>(prologue, epilogue, p, blocks, lds, stream);
  return launch_pro<kF16, kScalar>(prologue, epilogue, p, blocks, lds, stream);
}

}  // namespace nv
