// Launch interface of the FP8 block-scaled GEMV and MoE expert kernels (fp8_gemv.hip).
#pragma once

#include "nv_common.cuh"

namespace nv {

struct Fp8GemvParams {
  const uint8_t *w;       // [rows x cols] e4m3fn
  const float *scales;    // [ceil(rows/block_rows) x ceil(cols/block_cols)]
  const uint16_t *x16;    // [tokens x cols] or null
  const float *xf;        // [tokens x cols] when x16 is null
  float *out;             // [tokens x rows]
  uint32_t rows, cols, block_rows, block_cols, tokens, input_dtype;
  uint32_t x_first = 1;  // set by the launcher (lean one-token kernel: activations requested ahead of the weights)
};

struct MoeFp8Params {
  const uint16_t *x16;
  const uint32_t *expert_ids;
  const float *expert_weights;
  const uint8_t *w_gate, *w_up, *w_down;
  const float *s_gate, *s_up, *s_down;
  float *act;   // [(top_k + shared) x inter]
  float *out;   // [hidden]
  uint32_t hidden, inter, num_experts, top_k, block, input_dtype;
  int32_t shared_index;
  uint32_t phases;   // 0: both launches; 1: gate/up only; 2: down only (act holds an earlier gate/up result)
  uint32_t shared_last;  // set by the launcher: lean down kernel walks the shared expert last (measurements)
};

struct MoeRouteParams {
  const float *logits;
  uint32_t *expert_ids;
  float *expert_weights;
  uint32_t num_experts, top_k, normalize;
};

hipError_t launch_fp8_gemv(const Fp8GemvParams &p, hipStream_t stream);
hipError_t launch_moe_fp8(const MoeFp8Params &p, hipStream_t stream);
hipError_t launch_moe_route(const MoeRouteParams &p, hipStream_t stream);

}  // namespace nv
