// Fused "layer front" of the decode step: qkv projection (+RMSNorm), decode attention and the
// o projection (+bias, +residual) of one layer as three roles of ONE launch.
//
// Why one launch: the three pieces are a dependency chain, but most of their memory traffic is
// not. The o projection's weights, the attention's KV tiles and the qkv projection's weights
// can all be requested up front; only the small vectors between them (q/k/v rows, the
// attention output) have to wait. Roles are assigned by workgroup index in producer order -
// qkv rows first, then attention splits, then o rows - so a workgroup only ever waits for
// workgroups that were dispatched before it, and each role requests all of its weights / tiles
// into registers before it waits. Hand-over between roles uses device-coherent stores and
// loads plus epoch flags (no cache flush, no read-modify-write on the consumer side).
// Every wait is bounded; a wait that runs out raises abort_flag and the step is reported as
// failed by the host.
// Reference step order: launch_cublas_layer_session_step
// (native/cuda/hf_decode_sequence/session_decode_prefill.inc.cu:74-372).
#pragma once

#include "attn_decode.cuh"

namespace nv {

constexpr uint32_t kFrontThreads = 512;      // 8 waves per workgroup in every role
constexpr uint32_t kFrontRowsPerWg = 16;     // GEMV roles: two rows per wave
constexpr uint32_t kFrontFlagStride = 16;    // u32 words between the per-kv-head flags (64 B)

struct FrontParams {
  AttnParams attn;         // attention role (attn.qkv is what the qkv role writes)
  const uint16_t *wqkv;    // [A + 2 KV][hidden], or null: q/k/v were projected by an earlier launch
  const uint16_t *rms_attn;
  const float *x;          // [hidden] layer input: RMSNorm source and the residual of the o projection
  const uint16_t *wo;      // [hidden][A]
  const uint16_t *o_bias;  // optional [hidden]
  float *attn_f32;         // [A] attention output handed from the attention role to the o role
  float *r;                // [hidden] x + o projection (+ bias)
  uint32_t hidden;
  float rms_eps;
  uint32_t *head_flags;    // [kv_heads * kFrontFlagStride] attention output of a kv head is visible
  uint32_t *row_flags;     // [qkv workgroups] q/k/v rows of a workgroup are visible
  uint32_t *abort_flag;
  const uint32_t *step_counter;  // device word that grows by one per step; epochs derive from it
  uint32_t layer, layers;
  uint64_t *trace;         // optional [32] device timestamps of selected workgroups (tuning aid), or null
};

// Bytes of flag storage a caller provides (zeroed once; epochs only grow afterwards).
uint64_t front_flag_bytes(uint32_t heads, uint32_t kv_heads);
// Carves head_flags / row_flags out of a buffer of front_flag_bytes().
void front_bind_flags(FrontParams &p, void *flags);
// True when the shapes fit the fused kernel (otherwise: one launch per piece).
bool front_supported(uint32_t hidden, uint32_t heads, uint32_t kv_heads, uint32_t head_dim);
// Number of workgroups of each role for these parameters.
void front_grid(const FrontParams &p, uint32_t *q_wgs, uint32_t *a_wgs, uint32_t *o_wgs);
hipError_t launch_layer_front(uint32_t dtype, const FrontParams &p, hipStream_t stream);

}  // namespace nv
