// Host launcher for the weight-streaming GEMV kernels (gemv_stream.cuh).
#include <algorithm>

#include "gemv_stream.cuh"

namespace nv {

namespace {

// Defaults chosen from on-device sweeps over rows per wave, loads in flight, dot2
// and grid caps: all variants land within 3% of each other at ~7 TB/s + ~3 us per
// launch; one row per wave with the whole 4096-wide row (8 KiB) in flight and an
// uncapped grid is the best or tied-best on every decode shape.
constexpr int kDefaultNR = 1;
#ifndef NV_GEMV_U
#define NV_GEMV_U 8
#endif
constexpr int kDefaultU = NV_GEMV_U;  // chunks of 1 KiB in flight per wave per request batch
constexpr bool kDefaultDot2 = false;
constexpr uint32_t kCus = 256;                     // gfx950: 8 XCDs x 32 CUs
constexpr uint32_t kDefaultMaxBlocks = kCus * 6u;  // generic kernels: 6 workgroups per CU

// One workgroup: reduce the per-workgroup candidates, publish the token.
__global__ __launch_bounds__(1024) void sample_finish_kernel(SampleParams s, uint32_t count,
                                                             const uint32_t *cursor, uint32_t max_steps) {
  __shared__ float red_v[16];
  __shared__ uint32_t red_i[16];
  __shared__ uint32_t red_h[16];
  if (cursor != nullptr && *cursor >= max_steps) return;
  Best b{0.0f, 0u, 0u};
  for (uint32_t i = threadIdx.x; i < count; i += 1024) {
    Best o{s.part_value[i], s.part_index[i], s.part_has[i]};
    if (better(o, b)) b = o;
  }
  b = wave_best(b);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    red_v[wave] = b.value;
    red_i[wave] = b.index;
    red_h[wave] = b.has;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    Best t{red_v[0], red_i[0], red_h[0]};
    for (int w = 1; w < 16; ++w) {
      Best o{red_v[w], red_i[w], red_h[w]};
      if (better(o, t)) t = o;
    }
    publish_token(s, t.has ? t.index : 0u);
  }
}

template <uint32_t DT, int PRO, int EPI, int MODE>
hipError_t launch_one(const GemvParams &p, const GemvPlan &plan, size_t lds, hipStream_t stream) {
  constexpr int NR = EPI == kEpiSwiglu ? 2 : kDefaultNR;  // swiglu: the gate row and the up row
  const uint32_t blocks = plan.blocks;
  const int wg = plan.wg_waves;
  if constexpr (MODE == kFast) {
    // Launches whose waves own one or two rows of exactly two batches each (the step's o projection at
    // 4096 columns) take the variant with exact start-up waits: o 7.5 -> 7.2 us in the step.
    // It needs two batches per row at least. Measured with it forced on elsewhere ("gemv_exact_start" override:
    // 1 = wherever it can run, 2 = nowhere): down (six batches a row) 17.1 -> 17.6 us; the gate/up pair and the
    // LM head do not move, so only the plain and residual epilogues have the variant.
    constexpr bool kShortShapes = EPI == kEpiF32 || EPI == kEpiResidual;
    constexpr uint32_t kBatchCols = kWave * 8u * (4 / NR);
    const uint32_t units_per_wave = (p.rows + blocks * kWavesPerBlock - 1) / (blocks * kWavesPerBlock);
    const int forced = tuning(kTuneGemvExactStart);
    const bool can = kShortShapes && p.cols >= 2u * kBatchCols;
    const bool want = forced == 1 || (forced == 0 && units_per_wave <= 2 && p.cols == 2u * kBatchCols);
    // Waves per workgroup: the same waves in fewer workgroups (see the kernel).
    const uint32_t waves = blocks * kWavesPerBlock;
    // The input vector in registers (see the kernel): measured o 7.25 -> 7.05 us; qkv unchanged, gate_up
    // 31.8 -> 33.5 us, LM head 187 -> 189 us (one wave per SIMD less) - so only the short launches with a
    // 16-bit input take it.
    const bool xreg = PRO == kProX16 && p.cols == 4096u && tuning(kTuneGemvXRegisters) != 2;
#define NV_GEMV_LAUNCH(BB, EX, W, XR, RT)                                                                      \
  hipLaunchKernelGGL((gemv_fast_kernel<DT, PRO, EPI, NR, BB, EX, W, XR, RT>), dim3((waves + W - 1) / W),        \
                     dim3(W * kWave), lds, stream, p)
    if (plan.rotated) {
      // (which launches walk rotated, and with how many chunks a batch, is the plan's choice)
      if constexpr (EPI == kEpiSwiglu) {
        if (wg == 16) NV_GEMV_LAUNCH(2, false, 16, false, true);
        else NV_GEMV_LAUNCH(2, false, 4, false, true);
      } else if constexpr (PRO == kProRmsNorm && EPI == kEpiArgmax) {
        NV_GEMV_LAUNCH(1, false, 16, false, true);
      } else if constexpr (PRO == kProRmsNorm && EPI == kEpiF32) {
        NV_GEMV_LAUNCH(2, false, 4, false, true);
      } else {
        return hipErrorInvalidValue;
      }
    } else if (plan.chunks == 2 && NR == 1) {
      // rows that are whole batches of 1024 columns but not of 2048 (hidden 5120, MLP width 25600): two chunks a batch
      if (wg == 16) NV_GEMV_LAUNCH(2, false, 16, false, false);
      else NV_GEMV_LAUNCH(2, false, 4, false, false);
    } else if (can && want) {
      if constexpr (kShortShapes) {
        if (wg == 16) NV_GEMV_LAUNCH(4 / NR, true, 16, false, false);
        else if constexpr (PRO == kProX16) {
          if (xreg) NV_GEMV_LAUNCH(4 / NR, true, 4, true, false);
          else NV_GEMV_LAUNCH(4 / NR, true, 4, false, false);
        } else NV_GEMV_LAUNCH(4 / NR, true, 4, false, false);
      }
    } else {
      if (wg == 16) NV_GEMV_LAUNCH(4 / NR, false, 16, false, false);
      else NV_GEMV_LAUNCH(4 / NR, false, 4, false, false);
    }
#undef NV_GEMV_LAUNCH
  } else if constexpr (MODE == kVecFull) {
    hipLaunchKernelGGL((gemv_kernel<DT, PRO, EPI, NR, kDefaultU / NR, kVecFull, kDefaultDot2>),
                       dim3(plan.blocks), dim3(kBlock), lds, stream, p);
  } else if constexpr (MODE == kVecGuarded) {
    hipLaunchKernelGGL((gemv_kernel<DT, PRO, EPI, NR, 4, kVecGuarded, false>), dim3(plan.blocks),
                       dim3(kBlock), lds, stream, p);
  } else {
    hipLaunchKernelGGL((gemv_kernel<DT, PRO, EPI, NR, 1, kScalar, false>), dim3(plan.blocks),
                       dim3(kBlock), lds, stream, p);
  }
  return hipGetLastError();
}

template <uint32_t DT, int PRO, int MODE>
hipError_t launch_epi(int epilogue, const GemvParams &p, const GemvPlan &plan, size_t lds, hipStream_t stream) {
  switch (epilogue) {
    case kEpiF32: return launch_one<DT, PRO, kEpiF32, MODE>(p, plan, lds, stream);
    case kEpiResidual: return launch_one<DT, PRO, kEpiResidual, MODE>(p, plan, lds, stream);
    case kEpiSwiglu: return launch_one<DT, PRO, kEpiSwiglu, MODE>(p, plan, lds, stream);
    case kEpiOut16: return launch_one<DT, PRO, kEpiOut16, MODE>(p, plan, lds, stream);
    case kEpiArgmax: return launch_one<DT, PRO, kEpiArgmax, MODE>(p, plan, lds, stream);
    default: return hipErrorInvalidValue;
  }
}

template <uint32_t DT, int MODE>
hipError_t launch_pro(int prologue, int epilogue, const GemvParams &p, const GemvPlan &plan, size_t lds,
                      hipStream_t stream) {
  if (prologue == kProX16) return launch_epi<DT, kProX16, MODE>(epilogue, p, plan, lds, stream);
  if (prologue == kProRmsNorm) return launch_epi<DT, kProRmsNorm, MODE>(epilogue, p, plan, lds, stream);
  return hipErrorInvalidValue;
}

bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

// Waves per workgroup the lean kernel is launched with (4 or 16), per shape. Every workgroup fetches the input
// vector and the norm weights for itself (24 KiB at 4096 columns); the LM head's 2048 looping workgroups move
// 49 MB of that ahead of their weights, as 512 workgroups of 16 waves 12 MB: 197 -> 190 us. The step's other
// launches measured the same (qkv, o, down: within 0.1 us) or worse (gate_up 32.8 -> 34.6 us: one workgroup of
// 16 waves per CU instead of five of 4) with 16.
int fast_workgroup_waves(int prologue, int epilogue, uint32_t rows, uint32_t cols) {
  (void)cols;
  return prologue == kProRmsNorm && epilogue == kEpiArgmax && rows >= 65536u ? 16 : kWavesPerBlock;
}

}  // namespace

// kFast needs cols % 1024 == 0 and cols <= kFastMaxCols (kFastMaxColsLoop with a 16-bit input).
GemvPlan gemv_plan(int prologue, int epilogue, uint32_t rows, uint32_t cols, bool vec16,
                   const GemvTuning *tuning) {
  GemvPlan plan;
  const bool vec = vec16 && cols % 8 == 0;
  plan.mode = !vec ? kScalar : (cols % (kWave * 8) == 0 ? kVecFull : kVecGuarded);
  const uint32_t fast_cols = kWave * 8 * 2;
  const uint32_t max_cols = prologue == kProX16 ? kFastMaxColsLoop : kFastMaxCols;
  if (plan.mode == kVecFull && cols % fast_cols == 0 && cols <= max_cols && !(tuning && tuning->force_generic))
    plan.mode = kFast;
  // one wave per unit (a row, or a gate/up pair)
  const uint32_t want = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
  uint32_t blocks = want;
  if (tuning && tuning->max_blocks > 0) {
    blocks = std::min<uint32_t>(want, static_cast<uint32_t>(tuning->max_blocks));
  } else if (plan.mode == kFast) {
    // Workgroups that fit the machine at once: register budget, and the LDS copy of x.
    const uint32_t by_lds = (160u * 1024u) / (cols * 2u + 1024u);
    const uint32_t resident =
        kCus * std::min<uint32_t>(static_cast<uint32_t>(fast_waves_per_simd(prologue)), std::max(by_lds, 1u));
    if (want <= resident) {
      blocks = want;                       // everything is on the machine at once, one unit per wave
    } else if (want <= 2 * resident) {
      blocks = (want + 1) / 2;             // exactly two units per wave, pipelined in one round
    } else {
      blocks = std::min(want, kCus * 8u);  // long launches: oversubscribe, the dispatcher evens the tail
    }
  } else {
    blocks = std::min(want, kDefaultMaxBlocks);
  }
  if (epilogue == kEpiArgmax && blocks > kSampleMaxBlocks) blocks = kSampleMaxBlocks;
  plan.blocks = blocks == 0 ? 1 : blocks;
  plan.wg_waves = kWavesPerBlock;
  plan.rotated = false;
  plan.chunks = epilogue == kEpiSwiglu ? 2 : 4;
  if (plan.mode == kFast) {
    plan.wg_waves = nv::tuning(kTuneGemvWorkgroupWaves);
    if (plan.wg_waves != 4 && plan.wg_waves != 16) plan.wg_waves = fast_workgroup_waves(prologue, epilogue, rows, cols);
    if (epilogue != kEpiSwiglu && cols % (kWave * 8 * 4) != 0) plan.chunks = 2;
    // The rotated walk (see the kernel), where it measured faster; "gemv_rotated_walk" = 2 keeps the plain walk.
    const bool auto_grid = !(tuning && tuning->max_blocks > 0);
    if (nv::tuning(kTuneGemvRotatedWalk) != 2) {
      if (epilogue == kEpiSwiglu) {
        plan.rotated = true;                                  // gate/up pair: 2 KiB of each row a batch
      } else if (prologue == kProRmsNorm && epilogue == kEpiArgmax && plan.wg_waves == 16 && plan.chunks == 4) {
        plan.rotated = true;                                  // LM head: 1 KiB a batch
        plan.chunks = 1;
      } else if (prologue == kProRmsNorm && epilogue == kEpiF32 && plan.wg_waves == 4 && cols == 4096u && auto_grid &&
                 want > kCus * 4u && want <= kCus * 8u) {
        // a step's qkv projection (6144 rows): 2 KiB a batch on four workgroups a CU - 10.05 -> 9.65 us; three a CU
        // (every wave two rows) have too few requests in flight at this batch size, five leave a fifth of the waves
        // with twice the work of the others
        plan.rotated = true;
        plan.chunks = 2;
        plan.blocks = kCus * 4u;
      }
    }
  }
  plan.grid = (plan.blocks * kWavesPerBlock + plan.wg_waves - 1) / plan.wg_waves;
  return plan;
}

hipError_t launch_gemv(uint32_t dtype, int prologue, int epilogue, const GemvParams &p,
                       hipStream_t stream, const GemvTuning *tuning, uint32_t *blocks_used) {
  if (blocks_used) *blocks_used = 0;
  if (p.w == nullptr || p.rows == 0 || p.cols == 0) return hipErrorInvalidValue;
  if (prologue == kProX16 && p.x16 == nullptr) return hipErrorInvalidValue;
  if (prologue == kProRmsNorm && (p.xf == nullptr || p.gamma == nullptr)) return hipErrorInvalidValue;
  if ((epilogue == kEpiF32 || epilogue == kEpiResidual || epilogue == kEpiArgmax) && p.out_f32 == nullptr)
    return hipErrorInvalidValue;
  if ((epilogue == kEpiSwiglu || epilogue == kEpiOut16) && p.out16 == nullptr) return hipErrorInvalidValue;
  if (epilogue == kEpiResidual && p.residual == nullptr) return hipErrorInvalidValue;
  if (epilogue == kEpiArgmax && (p.sample.part_value == nullptr || p.sample.part_index == nullptr ||
                                 p.sample.part_has == nullptr))
    return hipErrorInvalidValue;
  if (dtype != kF16 && dtype != kBF16) return hipErrorInvalidValue;

  const bool vec16 = aligned16(p.w) && (prologue == kProX16 ? aligned16(p.x16)
                                                             : (aligned16(p.xf) && aligned16(p.gamma)));
  const size_t lds = static_cast<size_t>((p.cols + 7) / 8 * 8) * sizeof(uint16_t);
  if (lds > 60 * 1024) return hipErrorInvalidValue;  // K up to 30720 fits one workgroup's LDS
  const GemvPlan plan = gemv_plan(prologue, epilogue, p.rows, p.cols, vec16, tuning);
  const int mode = plan.mode;
  // (the plan counts four-wave workgroups; the lean kernel may launch the same waves as fewer, larger ones)
  if (blocks_used) *blocks_used = plan.grid;
  if (dtype == kBF16) {
    if (mode == kFast) return launch_pro<kBF16, kFast>(prologue, epilogue, p, plan, lds, stream);
    if (mode == kVecFull) return launch_pro<kBF16, kVecFull>(prologue, epilogue, p, plan, lds, stream);
    if (mode == kVecGuarded) return launch_pro<kBF16, kVecGuarded>(prologue, epilogue, p, plan, lds, stream);
    return launch_pro<kBF16, kScalar>(prologue, epilogue, p, plan, lds, stream);
  }
  if (mode == kFast) return launch_pro<kF16, kFast>(prologue, epilogue, p, plan, lds, stream);
  if (mode == kVecFull) return launch_pro<kF16, kVecFull>(prologue, epilogue, p, plan, lds, stream);
  if (mode == kVecGuarded) return launch_pro<kF16, kVecGuarded>(prologue, epilogue, p, plan, lds, stream);
  return launch_pro<kF16, kScalar>(prologue, epilogue, p, plan, lds, stream);
}

hipError_t launch_sample_finish(const SampleParams &s, uint32_t count, const uint32_t *cursor,
                                uint32_t max_steps, hipStream_t stream) {
  if (s.part_value == nullptr || s.part_index == nullptr || s.part_has == nullptr || count == 0 ||
      count > kSampleMaxBlocks)
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_finish_kernel, dim3(1), dim3(1024), 0, stream, s, count, cursor, max_steps);
  return hipGetLastError();
}

}  // namespace nv
