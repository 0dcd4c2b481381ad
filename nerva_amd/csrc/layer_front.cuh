// Fused "layer front" of the decode step: qkv projection (+RMSNorm), decode attention and the
// o projection (+bias, +residual) of one layer as three roles of ONE launch.
//
// Why one launch: the three pieces are a dependency chain, but most of their memory traffic is
// not. The o projection's weights, the attention's KV tiles and the qkv projection's weights
// can all be requested up front; only the small vectors between them (q/k/v rows, the
// attention output) have to wait. Roles are assigned by workgroup index in producer order -
// qkv rows first, then attention splits, then o rows - so a workgroup only ever waits for
// workgroups that were dispatched before it, and each role requests all of its weights / tiles
// into registers before it waits. A value handed from one role to another travels as an
// 8-byte (f32 value, epoch) word written and polled with device-coherent accesses: a matching
// epoch proves the value, so there are no flags to order against, no cache flushes and no
// read-modify-writes. Every wait is bounded; a wait that runs out raises abort_flag and the step
// is reported as failed by the host.
// Reference step order: launch_cublas_layer_session_step
// (native/cuda/hf_decode_sequence/session_decode_prefill.inc.cu:74-372).
#pragma once

#include "attn_decode.cuh"

namespace nv {

constexpr uint32_t kFrontThreads = 512;      // 8 waves per workgroup in every role
constexpr uint32_t kFrontRowsPerWg = 16;     // GEMV roles: two rows per wave
constexpr uint32_t kFrontFlagStride = 16;    // u32 words of one o workgroup's hint line (64 B): one word per kv head
constexpr uint32_t kFrontMaxOWgs = 256;      // hidden <= 4096

struct FrontParams {
  AttnParams attn;         // attention role (attn.qkv is what the qkv role writes)
  const uint16_t *wqkv;    // [A + 2 KV][hidden], or null: q/k/v were projected by an earlier launch
  const uint16_t *rms_attn;
  const float *x;          // [hidden] layer input: RMSNorm source and the residual of the o projection
  const uint16_t *wo;      // [hidden][A]
  const uint16_t *o_bias;  // optional [hidden]
  float *r;                // [hidden] x + o projection (+ bias)
  uint32_t hidden;
  float rms_eps;
  // hand-over storage (front_bind_workspace): tagged words, zero before the first launch
  uint64_t *qkv_tagged;    // [A + 2 KV] q|k|v from the qkv role to the attention role
  uint64_t *part_tagged;   // [heads][kAttnMaxSplits][130] split partials
  uint64_t *out_tagged;    // [A / 2] attention output (pairs of 16-bit values) from the attention role to the o role
  uint32_t *head_hints;    // [o workgroups][kFrontFlagStride] "kv head's output is about to appear", a line per consumer
  uint32_t *split_hints;   // [kv_heads][kAttnMaxSplits] "this split's partial has been stored"
  uint32_t *abort_flag;
  const uint32_t *step_counter;  // device word that grows by one per step; epochs derive from it
  uint32_t layer, layers;
  uint64_t *trace;         // optional [32] device timestamps of selected workgroups (tuning aid), or null
};

// Bytes of hand-over storage a caller provides (zeroed once; epochs never repeat afterwards).
uint64_t front_workspace_bytes(uint32_t heads, uint32_t kv_heads);
// Carves the hand-over buffers out of a workspace of front_workspace_bytes() (needs p.attn dims).
void front_bind_workspace(FrontParams &p, void *workspace);
// True when the shapes fit the fused kernel (otherwise: one launch per piece).
bool front_supported(uint32_t hidden, uint32_t heads, uint32_t kv_heads, uint32_t head_dim);
// Number of workgroups of each role for these parameters.
void front_grid(const FrontParams &p, uint32_t *q_wgs, uint32_t *a_wgs, uint32_t *o_wgs);
hipError_t launch_layer_front(uint32_t dtype, const FrontParams &p, hipStream_t stream);

}  // namespace nv
