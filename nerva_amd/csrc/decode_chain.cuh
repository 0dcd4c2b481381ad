// Persistent "layer chain" kernel of the decode step: the four weight-streaming GEMVs between
// two attention launches - o projection (+residual), gate/up (+RMSNorm, SwiGLU), down
// (+residual) and the next layer's qkv projection (+RMSNorm) - run as phases of ONE launch on
// 256 co-resident workgroups, separated by in-kernel grid barriers instead of kernel
// boundaries. Weight requests do not depend on activations, so every wave keeps its request
// ring running across the barriers: HBM stays busy while the producers' results are
// exchanged, which a chain of separate launches cannot do.
// Reference step order: launch_cublas_layer_session_step
// (native/cuda/hf_decode_sequence/session_decode_prefill.inc.cu:74-372).
#pragma once

#include "nv_common.cuh"

namespace nv {

constexpr uint32_t kChainGrid = 256;           // workgroups = CUs of the device, one per CU
constexpr int kChainWaves = 8;                 // weight-streaming waves per workgroup
constexpr int kChainThreads = (kChainWaves + 1) * kWave;  // + one wave that moves activations
constexpr uint32_t kChainFlagStride = 16;      // u32 words between arrival flags (64 B)
constexpr uint32_t kChainMaxBarriers = 3;      // barriers inside one launch

struct ChainParams {
  // weights of layer l, and of the layer whose qkv projection follows (null for the last layer)
  const uint16_t *wo, *o_bias, *rms_mlp, *wgu, *wdown, *rms_next, *wqkv_next;
  const uint16_t *attn16;   // [attn_dim] 16-bit attention output (input of the o projection)
  float *x;                 // [hidden] residual stream: read (o residual), rewritten by down
  float *r;                 // [hidden] x + o projection
  uint16_t *ff16;           // [inter] SwiGLU activations
  float *qkv;               // [qkv_rows] next layer's raw q|k|v
  uint32_t hidden, attn_dim, inter, qkv_rows;
  float eps;
  uint32_t round_out;       // prompt steps round the layer output to 16 bit
  uint32_t *flags;          // [kChainGrid * kChainFlagStride] arrival epochs, monotonic per sequence
  uint32_t *abort_flag;     // set when a bounded wait ran out; the step's results are then invalid
  const uint32_t *cursor;   // device position (epochs derive from it)
  uint32_t max_steps;
  uint32_t barrier_base;    // index of this launch's first barrier within the step
  uint32_t barriers_per_step;
  uint64_t *trace;          // optional [32] device timestamps of workgroup 0 (tuning aid), or null
};

// Bytes of the flag array a session must provide (zeroed whenever the position restarts).
constexpr uint64_t chain_flag_bytes() { return static_cast<uint64_t>(kChainGrid) * kChainFlagStride * 4; }
// True when the shapes fit the kernel (otherwise the step uses one launch per GEMV).
bool chain_supported(uint32_t hidden, uint32_t attn_dim, uint32_t inter, uint32_t qkv_rows);
// Raises the kernel's LDS limit (called once per session, outside any stream capture).
hipError_t chain_prepare(uint32_t dtype);
hipError_t launch_decode_chain(uint32_t dtype, const ChainParams &p, hipStream_t stream);

}  // namespace nv
