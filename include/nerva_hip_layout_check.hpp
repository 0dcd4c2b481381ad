// Compile-time layout checks for the structs of nerva_hip_api.h that mirror a
// reference struct. The expected numbers are sizeof/offsetof of the NervaCuda...
// originals (native/cuda/nerva_cuda_api.h) under the x86-64 SysV ABI, which is
// what the Rust #[repr(C)] mirrors in crates/nerva-cuda/src/**/ffi.rs assume.
#pragma once
#include <cstddef>

#include "nerva_hip_api.h"

#define NERVA_HIP_SIZE(T, N) static_assert(sizeof(T) == (N), #T " size differs from the reference ABI")
#define NERVA_HIP_OFF(T, F, N) \
  static_assert(offsetof(T, F) == (N), #T "." #F " offset differs from the reference ABI")

NERVA_HIP_SIZE(NervaHipDeviceSmokeResult, 232);
NERVA_HIP_SIZE(NervaHipSyntheticTokenSlot, 40);
NERVA_HIP_SIZE(NervaHipHfDecodeChainLayer, 440);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceWeightBlock, 72);
NERVA_HIP_SIZE(NervaHipHfDecodeSamplerConfig, 24);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceRequest, 208);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceResult, 528);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceSessionCreateRequest, 176);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceSessionCreateResult, 272);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceSessionRunRequest, 80);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceSessionStartRequest, 56);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceSessionAdvanceRequest, 32);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest, 16);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceBatchAdvanceRequest, 40);
NERVA_HIP_SIZE(NervaHipHfDecodeSequenceBatchAdvanceResult, 184);
NERVA_HIP_SIZE(NervaHipDeepSeekQuantDequantResult, 96);
NERVA_HIP_SIZE(NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest, 56);
NERVA_HIP_SIZE(NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest, 56);
NERVA_HIP_SIZE(NervaHipProjectionBenchRequest, 24);
NERVA_HIP_SIZE(NervaHipProjectionBenchResult, 408);
NERVA_HIP_SIZE(NervaHipDeepSeekMoeForwardRequest, 80);
NERVA_HIP_SIZE(NervaHipDeepSeekMoeForwardResult, 104);

NERVA_HIP_OFF(NervaHipSyntheticTokenSlot, version, 24);
NERVA_HIP_OFF(NervaHipHfDecodeChainLayer, w_linear_conv, 208);
NERVA_HIP_OFF(NervaHipHfDecodeChainLayer, mlp_kind, 280);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceRequest, sampler, 184);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceResult, observed_token_hash, 64);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceResult, graph_replays, 224);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceResult, hot_path_allocations, 400);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceSessionCreateRequest, embeddings, 48);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceSessionCreateRequest, detailed_profile, 144);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceSessionCreateResult, device_memory_bandwidth_bps, 264);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceSessionStartRequest, sampler, 32);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceBatchAdvanceRequest, output_tokens, 24);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceBatchAdvanceResult, observed_token_hash, 56);
NERVA_HIP_OFF(NervaHipHfDecodeSequenceBatchAdvanceResult, hot_path_allocations, 176);
