// C++17 host-side mirror of the reference's safe wrappers over the decode-session ABI
// (crates/nerva-cuda/src/decode/hf_sequence/session/{request,stateful,helpers,summary}.rs and
// smoke/status.rs): the same types under Hip names, the same validation before the call, the
// same mapping from (return code, result struct) to a summary. Header only; link libnerva_hip.
//
//   HipHfDecodeSequenceSessionConfig cfg{...};      // borrowed 16-bit weight spans
//   auto created = cfg.create();                     // {summary, optional session}
//   auto loop = HipHfDecodeSequenceLoop::start(*created.session, prompt, eos);
//   auto step = loop.loop_state->advance(16);        // summary.tokens holds the new tokens
#pragma once

#include <cstdint>
#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "nerva_hip_api.h"

namespace nerva::hip {

// smoke/status.rs:2-6
enum class SmokeStatus { Ok, Unavailable, Failed };

inline SmokeStatus status_from(int return_code, int32_t status, int32_t hip_error) {
  if (return_code == 0 && status == 0) return SmokeStatus::Ok;
  if (hip_error == NERVA_HIP_ERROR_NO_DEVICE) return SmokeStatus::Unavailable;
  return SmokeStatus::Failed;
}

// A borrowed contiguous range (the reference takes &[u16] / &[u32]).
template <typename T>
struct Span {
  const T *data = nullptr;
  size_t size = 0;
  Span() = default;
  Span(const T *d, size_t n) : data(d), size(n) {}
  Span(const std::vector<T> &v) : data(v.data()), size(v.size()) {}  // NOLINT: implicit on purpose
  bool empty() const { return size == 0; }
};

struct HipDeviceSmokeSummary {
  SmokeStatus status = SmokeStatus::Failed;
  int32_t device_count = 0;
  std::string gpu_name;
  uint64_t total_global_mem = 0;
};

inline HipDeviceSmokeSummary device_smoke() {
  NervaHipDeviceSmokeResult out{};
  const int rc = nerva_hip_device_smoke(&out);
  HipDeviceSmokeSummary s;
  s.status = status_from(rc, out.status, out.hip_error);
  s.device_count = out.device_count;
  s.gpu_name = std::string(out.gpu_name, strnlen(out.gpu_name, sizeof(out.gpu_name)));
  s.total_global_mem = out.total_global_mem;
  return s;
}

// request.rs: CudaHfDecodeSamplerConfig
struct HipHfDecodeSamplerConfig {
  float temperature = 0.0f, top_p = 1.0f;
  uint32_t top_k = 0;
  uint64_t seed = 0;
  static HipHfDecodeSamplerConfig greedy() { return {}; }
  std::optional<std::string> validate() const {
    if (!(temperature >= 0.0f)) return "HIP HF decode sampler temperature must be non-negative";
    if (!(top_p > 0.0f && top_p <= 1.0f)) return "HIP HF decode sampler top_p must be in (0, 1]";
    return std::nullopt;
  }
  NervaHipHfDecodeSamplerConfig to_ffi() const { return {temperature, top_p, top_k, 0u, seed}; }
};

// hf_chain: CudaHfDecodeChainLayer (dense full-attention subset)
struct HipHfDecodeChainLayer {
  Span<uint16_t> rms_attn_weight, rms_mlp_weight, w_q, w_k, w_v, w_o, w_gate, w_up, w_down;
  Span<uint16_t> q_norm_weight, k_norm_weight, q_bias, k_bias, v_bias, o_bias;  // optional
  NervaHipHfDecodeChainLayer to_ffi() const {
    NervaHipHfDecodeChainLayer l{};
    l.rms_attn_weight = rms_attn_weight.data;
    l.rms_mlp_weight = rms_mlp_weight.data;
    l.w_q = w_q.data;
    l.w_k = w_k.data;
    l.w_v = w_v.data;
    l.w_o = w_o.data;
    l.w_gate = w_gate.data;
    l.w_up = w_up.data;
    l.w_down = w_down.data;
    l.q_norm_weight = q_norm_weight.data;
    l.k_norm_weight = k_norm_weight.data;
    l.q_bias = q_bias.data;
    l.k_bias = k_bias.data;
    l.v_bias = v_bias.data;
    l.o_bias = o_bias.data;
    return l;
  }
  // hf_chain/layer.rs:352-399: with a declared weight plan the descriptors carry the data; the request
  // only says which optional tensors exist
  NervaHipHfDecodeChainLayer to_descriptor_layout_ffi() const {
    NervaHipHfDecodeChainLayer l{};
    l.q_norm_weight = q_norm_weight.data;
    l.k_norm_weight = k_norm_weight.data;
    l.q_bias = q_bias.data;
    l.k_bias = k_bias.data;
    l.v_bias = v_bias.data;
    l.o_bias = o_bias.data;
    return l;
  }
};

// weight_plan.rs:3-4
constexpr uint32_t HIP_HF_WEIGHT_STRATEGY_GPU_RESIDENT = 1, HIP_HF_WEIGHT_STRATEGY_GPU_STAGED = 2;
using HipHfDecodeSequenceWeightBlock = NervaHipHfDecodeSequenceWeightBlock;   // weight_plan.rs:9-22

// weight_plan.rs:102-126: FNV-1a-64 over (block_id, block_version, offset_bytes, bytes: u64; strategy:
// u32), little endian, block after block
inline uint64_t hash_weight_blocks(Span<HipHfDecodeSequenceWeightBlock> descriptors) {
  uint64_t hash = 0xcbf29ce484222325ull;
  auto mix = [&hash](uint64_t value, int bytes) {
    for (int i = 0; i < bytes; ++i) {
      hash ^= (value >> (8 * i)) & 0xffu;
      hash *= 0x00000100000001b3ull;
    }
  };
  for (size_t i = 0; i < descriptors.size; ++i) {
    const HipHfDecodeSequenceWeightBlock &d = descriptors.data[i];
    mix(d.block_id, 8);
    mix(d.block_version, 8);
    mix(d.offset_bytes, 8);
    mix(d.bytes, 8);
    mix(d.strategy, 4);
  }
  return hash;
}

// weight_plan.rs:24-100 CudaHfDecodeSequenceWeightPlan
struct HipHfDecodeSequenceWeightPlan {
  uint32_t blocks = 0, gpu_resident_blocks = 0, gpu_staged_blocks = 0;
  uint64_t weight_bytes = 0, gpu_resident_weight_bytes = 0, gpu_staged_weight_bytes = 0, descriptor_hash = 0;
  bool is_declared() const { return blocks != 0 || weight_bytes != 0; }
  std::optional<std::string> validate() const {
    if (!is_declared()) return std::nullopt;
    if (blocks == 0 || weight_bytes == 0 || descriptor_hash == 0) return "HIP HF decode sequence weight plan is incomplete";
    if (gpu_resident_blocks > blocks || gpu_staged_blocks > blocks - gpu_resident_blocks)
      return "HIP HF decode sequence weight block counts are invalid";
    if (gpu_resident_weight_bytes > weight_bytes || gpu_staged_weight_bytes > weight_bytes - gpu_resident_weight_bytes)
      return "HIP HF decode sequence weight byte counts are invalid";
    return std::nullopt;
  }
  std::optional<std::string> validate_descriptors(Span<HipHfDecodeSequenceWeightBlock> descriptors) const {
    if (!is_declared()) return std::nullopt;
    if (descriptors.size != blocks) return "HIP HF decode sequence weight descriptor count is invalid";
    for (size_t i = 0; i < descriptors.size; ++i) {
      const HipHfDecodeSequenceWeightBlock &d = descriptors.data[i];
      if ((d.host_source == nullptr && (d.source_file == nullptr || d.source_file_len == 0)) || d.offset_bytes % 2 != 0 ||
          d.bytes % 2 != 0)
        return "HIP HF decode sequence weight descriptor source is invalid";
    }
    if (hash_weight_blocks(descriptors) != descriptor_hash) return "HIP HF decode sequence weight descriptor hash is invalid";
    return std::nullopt;
  }
};

// session/summary.rs: CudaHfDecodeSequenceSessionCreateSummary (fields this backend fills)
struct HipHfDecodeSequenceSessionCreateSummary {
  SmokeStatus status = SmokeStatus::Failed;
  int32_t failure_stage = 0, hip_error = 0;
  uint32_t dtype = 0, hidden = 0, heads = 0, kv_heads = 0, head_dim = 0, intermediate = 0, vocab_size = 0,
           layer_count = 0, max_context_tokens = 0;
  uint64_t resident_weight_bytes = 0, resident_kv_bytes = 0, device_arena_bytes = 0, pinned_host_bytes = 0,
           h2d_bytes = 0, sync_calls = 0, hot_path_allocations = 0, device_memory_bandwidth_bps = 0;
  std::optional<std::string> error;
};

// summary.rs: CudaHfDecodeSequenceSummary (fields this backend fills)
struct HipHfDecodeSequenceSummary {
  SmokeStatus status = SmokeStatus::Failed;
  int32_t hip_error = 0;
  uint32_t steps = 0, seed_token = 0, last_token = 0;
  std::vector<uint32_t> tokens;
  uint64_t observed_token_hash = 0, kv_tokens = 0, graph_replays = 0, graph_nodes = 0, graph_launches = 0,
           graph_captures = 0, graph_cache_hits = 0, kernel_launches = 0, device_elapsed_ns = 0, sync_calls = 0,
           host_causality_edges = 0, hot_path_allocations = 0, h2d_bytes = 0, d2h_bytes = 0;
  std::optional<std::string> error;
};

namespace detail {
// helpers.rs: summary_from_run
inline HipHfDecodeSequenceSummary summary_from_run(int rc, const NervaHipHfDecodeSequenceResult &out,
                                                   std::vector<uint32_t> tokens) {
  HipHfDecodeSequenceSummary s;
  s.status = status_from(rc, out.status, out.hip_error);
  s.hip_error = out.hip_error;
  s.steps = out.steps;
  s.seed_token = out.seed_token;
  s.last_token = out.last_token;
  tokens.resize(s.status == SmokeStatus::Ok ? out.observed_tokens : 0);
  s.tokens = std::move(tokens);
  s.observed_token_hash = out.observed_token_hash;
  s.kv_tokens = out.kv_tokens;
  s.graph_replays = out.graph_replays;
  s.graph_nodes = out.graph_nodes;
  s.graph_launches = out.graph_launches;
  s.graph_captures = out.graph_captures;
  s.graph_cache_hits = out.graph_cache_hits;
  s.kernel_launches = out.kernel_launches;
  s.device_elapsed_ns = out.device_elapsed_ns;
  s.sync_calls = out.sync_calls;
  s.host_causality_edges = out.host_causality_edges;
  s.hot_path_allocations = out.hot_path_allocations;
  s.h2d_bytes = out.h2d_bytes;
  s.d2h_bytes = out.d2h_bytes;
  if (s.status == SmokeStatus::Unavailable) s.error = "HIP device unavailable";
  else if (s.status == SmokeStatus::Failed)
    s.error = out.hip_error == NERVA_HIP_ERROR_NOT_SUPPORTED
                  ? "HIP HF decode sequence request uses a feature this backend does not implement"
                  : "HIP HF decode sequence call failed (hip_error " + std::to_string(out.hip_error) + ")";
  return s;
}
// failures.rs: failed_run_summary
inline HipHfDecodeSequenceSummary failed_run_summary(std::string error) {
  HipHfDecodeSequenceSummary s;
  s.status = SmokeStatus::Failed;
  s.error = std::move(error);
  return s;
}
// stateful.rs:183-191 validate_loop_start
inline std::optional<std::string> validate_loop_start(Span<uint32_t> prompt, uint32_t vocab_size) {
  if (prompt.empty()) return "HIP HF decode sequence loop start requires prompt";
  for (size_t i = 0; i < prompt.size; ++i)
    if (prompt.data[i] >= vocab_size) return "HIP HF decode sequence loop prompt token is outside vocabulary";
  return std::nullopt;
}
}  // namespace detail

namespace detail {
// helpers.rs create_summary_from_result: (return code, result struct) -> summary
inline HipHfDecodeSequenceSessionCreateSummary create_summary_from_result(
    int rc, const NervaHipHfDecodeSequenceSessionCreateResult &out, const char *what) {
  HipHfDecodeSequenceSessionCreateSummary s;
  s.status = status_from(rc, out.status, out.hip_error);
  s.failure_stage = out.failure_stage;
  s.hip_error = out.hip_error;
  s.dtype = out.dtype;
  s.hidden = out.hidden;
  s.heads = out.heads;
  s.kv_heads = out.kv_heads;
  s.head_dim = out.head_dim;
  s.intermediate = out.intermediate;
  s.vocab_size = out.vocab_size;
  s.layer_count = out.layer_count;
  s.max_context_tokens = out.max_context_tokens;
  s.resident_weight_bytes = out.resident_weight_bytes;
  s.resident_kv_bytes = out.resident_kv_bytes;
  s.device_arena_bytes = out.device_arena_bytes;
  s.pinned_host_bytes = out.pinned_host_bytes;
  s.h2d_bytes = out.h2d_bytes;
  s.sync_calls = out.sync_calls;
  s.hot_path_allocations = out.hot_path_allocations;
  s.device_memory_bandwidth_bps = out.device_memory_bandwidth_bps;
  if (s.status == SmokeStatus::Unavailable) s.error = "HIP device unavailable";
  else if (s.status == SmokeStatus::Failed)
    s.error = std::string("HIP HF decode sequence session ") + what + " failed (hip_error " + std::to_string(out.hip_error) + ")";
  return s;
}

// request.rs:1290-1303 projection_batch_reason_name
inline const char *projection_batch_reason_name(uint32_t reason) {
  switch (reason) {
    case NERVA_HIP_BATCH_READY: return "ready";
    case NERVA_HIP_BATCH_INVALID_REQUEST: return "invalid_request";
    case NERVA_HIP_BATCH_NO_SESSIONS: return "no_sessions";
    case NERVA_HIP_BATCH_NO_READY_SESSIONS: return "no_ready_sessions";
    case NERVA_HIP_BATCH_SHARED_WEIGHTS_UNPROVEN: return "shared_weights_unproven";
    case NERVA_HIP_BATCH_INSUFFICIENT_COMPATIBLE_READY: return "insufficient_compatible_ready";
    default: return "unknown";
  }
}
}  // namespace detail

// request.rs:217-248 CudaHfDecodeSequenceBatchAdvanceSummary. tokens[i] belongs to sessions[i] of the
// call; UINT32_MAX marks a session that did not advance.
struct HipHfDecodeSequenceBatchAdvanceSummary {
  SmokeStatus status = SmokeStatus::Failed;
  std::string reason;
  bool exact = false;
  uint32_t requested_session_count = 0, eligible_session_count = 0, block_tokens = 0, target_block_tokens = 0,
           min_block_tokens = 0, dtype = 0, layer_count = 0, observed_tokens = 0, last_token = 0;
  uint64_t observed_token_hash = 0;
  std::vector<uint32_t> tokens;
  uint64_t d2h_bytes = 0, projection_elapsed_ns = 0, pack_kernel_launches = 0, projection_kernel_launches = 0,
           scatter_kernel_launches = 0, dependency_kernel_launches = 0, sampling_kernel_launches = 0, sync_calls = 0,
           hot_path_allocations = 0;
  int32_t hip_error = 0;
};

class HipHfDecodeSequenceSession;

struct HipHfDecodeSequenceSessionCreateOutput {
  HipHfDecodeSequenceSessionCreateSummary summary;
  std::unique_ptr<HipHfDecodeSequenceSession> session;  // null unless summary.status == Ok
};

// session/request.rs:105-108: owns the native handle; destroy on drop.
class HipHfDecodeSequenceSession {
 public:
  HipHfDecodeSequenceSession(NervaHipHfDecodeSequenceSession *handle, HipHfDecodeSequenceSessionCreateSummary summary)
      : handle_(handle), create_summary_(std::move(summary)) {}
  HipHfDecodeSequenceSession(const HipHfDecodeSequenceSession &) = delete;
  HipHfDecodeSequenceSession &operator=(const HipHfDecodeSequenceSession &) = delete;
  ~HipHfDecodeSequenceSession() {
    if (handle_ != nullptr) {
      NervaHipHfDecodeSequenceSessionCreateResult out{};
      (void)nerva_hip_hf_decode_sequence_session_destroy(handle_, &out);
    }
  }
  const HipHfDecodeSequenceSessionCreateSummary &create_summary() const { return create_summary_; }
  NervaHipHfDecodeSequenceSession *raw_handle() { return handle_; }

  // request.rs:380-407 fork_shared_weights: a second session on this one's resident weights; a
  // sequence that is under way is carried over to the child
  HipHfDecodeSequenceSessionCreateOutput fork_shared_weights(bool detailed_profile = false);

  // request.rs:575-597 batch_advance_one: one more token for every ready session of the same model
  static HipHfDecodeSequenceBatchAdvanceSummary batch_advance_one(const std::vector<HipHfDecodeSequenceSession *> &sessions,
                                                                  uint32_t target_block_tokens, uint32_t min_block_tokens) {
    std::vector<NervaHipHfDecodeSequenceSession *> handles;
    handles.reserve(sessions.size());
    for (HipHfDecodeSequenceSession *session : sessions) handles.push_back(session != nullptr ? session->raw_handle() : nullptr);
    std::vector<uint32_t> tokens(handles.size(), UINT32_MAX);
    NervaHipHfDecodeSequenceBatchAdvanceRequest rq{};
    rq.sessions = handles.data();
    rq.session_count = static_cast<uint32_t>(handles.size());
    rq.target_block_tokens = target_block_tokens;
    rq.min_block_tokens = min_block_tokens;
    rq.output_tokens = tokens.data();
    rq.output_token_capacity = static_cast<uint32_t>(tokens.size());
    NervaHipHfDecodeSequenceBatchAdvanceResult out{};
    const int rc = nerva_hip_hf_decode_sequence_batch_advance_one(&rq, &out);
    HipHfDecodeSequenceBatchAdvanceSummary s;
    s.status = rc == 0 && out.status == 0 ? SmokeStatus::Ok : SmokeStatus::Failed;   // request.rs:1251-1255
    s.reason = detail::projection_batch_reason_name(out.reason);
    s.exact = out.exact != 0;
    s.requested_session_count = out.requested_session_count;
    s.eligible_session_count = out.eligible_session_count;
    s.block_tokens = out.block_tokens;
    s.target_block_tokens = out.target_block_tokens;
    s.min_block_tokens = out.min_block_tokens;
    s.dtype = out.dtype;
    s.layer_count = out.layer_count;
    s.observed_tokens = out.observed_tokens;
    s.last_token = out.last_token;
    s.observed_token_hash = out.observed_token_hash;
    s.tokens = std::move(tokens);
    s.d2h_bytes = out.d2h_bytes;
    s.projection_elapsed_ns = out.projection_elapsed_ns;
    s.pack_kernel_launches = out.pack_kernel_launches;
    s.projection_kernel_launches = out.projection_kernel_launches;
    s.scatter_kernel_launches = out.scatter_kernel_launches;
    s.dependency_kernel_launches = out.dependency_kernel_launches;
    s.sampling_kernel_launches = out.sampling_kernel_launches;
    s.sync_calls = out.sync_calls;
    s.hot_path_allocations = out.hot_path_allocations;
    s.hip_error = out.hip_error;
    return s;
  }

  // request.rs:412-457 run / run_with_sampler: prompt walk + `steps` tokens in one call
  HipHfDecodeSequenceSummary run(Span<uint32_t> prompt, size_t steps, std::optional<uint32_t> eos_token = std::nullopt,
                                 HipHfDecodeSamplerConfig sampler = HipHfDecodeSamplerConfig::greedy()) {
    if (auto e = detail::validate_loop_start(prompt, create_summary_.vocab_size)) return detail::failed_run_summary(*e);
    if (auto e = sampler.validate()) return detail::failed_run_summary(*e);
    if (steps == 0) return detail::failed_run_summary("HIP HF decode sequence run requires steps");
    std::vector<uint32_t> tokens(steps);
    NervaHipHfDecodeSequenceSessionRunRequest rq{};
    rq.session = handle_;
    rq.steps = static_cast<uint32_t>(steps);
    rq.seed_token = prompt.data[prompt.size - 1];
    rq.prompt_tokens = prompt.data;
    rq.prompt_token_count = static_cast<uint32_t>(prompt.size);
    rq.has_eos_token = eos_token.has_value() ? 1u : 0u;
    rq.eos_token = eos_token.value_or(0);
    rq.output_tokens = tokens.data();
    rq.output_token_capacity = static_cast<uint32_t>(tokens.size());
    rq.sampler = sampler.to_ffi();
    NervaHipHfDecodeSequenceResult out{};
    const int rc = nerva_hip_hf_decode_sequence_session_run(&rq, &out);
    return detail::summary_from_run(rc, out, std::move(tokens));
  }

 private:
  NervaHipHfDecodeSequenceSession *handle_;
  HipHfDecodeSequenceSessionCreateSummary create_summary_;
};

// session/request.rs:84-103 CudaHfDecodeSequenceSessionConfig
struct HipHfDecodeSequenceSessionConfig {
  uint32_t dtype = NERVA_HIP_DTYPE_BF16;
  size_t hidden = 0, heads = 0, kv_heads = 0, head_dim = 0, intermediate = 0, vocab_size = 0, max_context_tokens = 0;
  float rms_eps = 1e-6f;
  std::optional<float> rope_theta;
  Span<uint16_t> embeddings;
  std::vector<HipHfDecodeChainLayer> layers;
  Span<uint16_t> final_norm_weight, lm_head;
  bool detailed_profile = false;
  // request.rs:99-100: a declared plan makes weight_blocks the source of the weights (the tensor spans
  // then only mark which optional tensors exist and may be empty otherwise). Sessions whose plans
  // have the same descriptor hash hold the same weights and may advance as one batch.
  std::optional<HipHfDecodeSequenceWeightPlan> weight_plan;
  Span<HipHfDecodeSequenceWeightBlock> weight_blocks;

  // validation.rs: every span must have exactly the size its shape implies
  std::optional<std::string> validate() const {
    if (hidden == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || intermediate == 0 || vocab_size == 0)
      return "HIP HF decode sequence session requires non-zero dimensions";
    if (heads % kv_heads != 0) return "HIP HF decode sequence session requires heads divisible by kv_heads";
    if (max_context_tokens == 0) return "HIP HF decode sequence session requires max_context_tokens";
    if (dtype != NERVA_HIP_DTYPE_F16 && dtype != NERVA_HIP_DTYPE_BF16) return "HIP HF decode sequence session dtype must be f16 or bf16";
    if (weight_plan.has_value()) {   // validation.rs:53-66: the plan and its descriptors, then no span lengths
      if (auto e = weight_plan->validate()) return e;
      if (auto e = weight_plan->validate_descriptors(weight_blocks)) return e;
      if (weight_plan->is_declared()) return std::nullopt;
    }
    const size_t a = heads * head_dim, kv = kv_heads * head_dim;
    if (embeddings.size != vocab_size * hidden) return "HIP HF decode sequence embeddings have the wrong size";
    if (lm_head.size != vocab_size * hidden) return "HIP HF decode sequence lm_head has the wrong size";
    if (final_norm_weight.size != hidden) return "HIP HF decode sequence final norm has the wrong size";
    for (const HipHfDecodeChainLayer &l : layers) {
      if (l.rms_attn_weight.size != hidden || l.rms_mlp_weight.size != hidden) return "HIP HF decode layer norm has the wrong size";
      if (l.w_q.size != a * hidden || l.w_k.size != kv * hidden || l.w_v.size != kv * hidden || l.w_o.size != hidden * a)
        return "HIP HF decode layer attention projection has the wrong size";
      if (l.w_gate.size != intermediate * hidden || l.w_up.size != intermediate * hidden || l.w_down.size != hidden * intermediate)
        return "HIP HF decode layer MLP projection has the wrong size";
      if ((!l.q_norm_weight.empty() && l.q_norm_weight.size != head_dim) || (!l.k_norm_weight.empty() && l.k_norm_weight.size != head_dim))
        return "HIP HF decode layer q/k norm has the wrong size";
      if ((!l.q_bias.empty() && l.q_bias.size != a) || (!l.k_bias.empty() && l.k_bias.size != kv) ||
          (!l.v_bias.empty() && l.v_bias.size != kv) || (!l.o_bias.empty() && l.o_bias.size != hidden))
        return "HIP HF decode layer bias has the wrong size";
    }
    return std::nullopt;
  }

  // request.rs:294-330 create
  HipHfDecodeSequenceSessionCreateOutput create() const {
    HipHfDecodeSequenceSessionCreateOutput result;
    if (auto e = validate()) {
      result.summary.status = SmokeStatus::Failed;
      result.summary.error = *e;
      return result;
    }
    std::vector<NervaHipHfDecodeChainLayer> ffi_layers;
    ffi_layers.reserve(layers.size());
    const HipHfDecodeSequenceWeightPlan plan = weight_plan.value_or(HipHfDecodeSequenceWeightPlan{});
    const bool use_descriptors = plan.is_declared();
    for (const HipHfDecodeChainLayer &l : layers) ffi_layers.push_back(use_descriptors ? l.to_descriptor_layout_ffi() : l.to_ffi());
    NervaHipHfDecodeSequenceSessionCreateRequest rq{};
    rq.dtype = dtype;
    rq.hidden = static_cast<uint32_t>(hidden);
    rq.heads = static_cast<uint32_t>(heads);
    rq.kv_heads = static_cast<uint32_t>(kv_heads);
    rq.head_dim = static_cast<uint32_t>(head_dim);
    rq.intermediate = static_cast<uint32_t>(intermediate);
    rq.vocab_size = static_cast<uint32_t>(vocab_size);
    rq.layer_count = static_cast<uint32_t>(layers.size());
    rq.max_context_tokens = static_cast<uint32_t>(max_context_tokens);
    rq.rms_eps = rms_eps;
    rq.rope_theta = rope_theta.value_or(0.0f);
    rq.embeddings = use_descriptors ? nullptr : embeddings.data;   // helpers.rs:13-19 planned_ptr
    rq.layers = ffi_layers.data();
    rq.final_norm_weight = use_descriptors ? nullptr : final_norm_weight.data;
    rq.lm_head = use_descriptors ? nullptr : lm_head.data;
    rq.detailed_profile = detailed_profile ? 1u : 0u;
    rq.planned_weight_blocks = plan.blocks;
    rq.planned_gpu_resident_blocks = plan.gpu_resident_blocks;
    rq.planned_gpu_staged_blocks = plan.gpu_staged_blocks;
    rq.planned_weight_bytes = plan.weight_bytes;
    rq.planned_gpu_resident_weight_bytes = plan.gpu_resident_weight_bytes;
    rq.planned_gpu_staged_weight_bytes = plan.gpu_staged_weight_bytes;
    rq.planned_weight_descriptors = weight_blocks.empty() ? nullptr : weight_blocks.data;
    rq.planned_weight_descriptor_count = static_cast<uint32_t>(weight_blocks.size);
    rq.planned_weight_descriptor_hash = plan.descriptor_hash;
    NervaHipHfDecodeSequenceSessionCreateResult out{};
    NervaHipHfDecodeSequenceSession *handle = nullptr;
    const int rc = nerva_hip_hf_decode_sequence_session_create(&rq, &out, &handle);
    result.summary = detail::create_summary_from_result(rc, out, "create");
    if (result.summary.status == SmokeStatus::Ok && handle != nullptr)
      result.session = std::make_unique<HipHfDecodeSequenceSession>(handle, result.summary);
    return result;
  }
};

inline HipHfDecodeSequenceSessionCreateOutput HipHfDecodeSequenceSession::fork_shared_weights(bool detailed_profile) {
  HipHfDecodeSequenceSessionCreateOutput result;
  NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest rq{};
  rq.parent = handle_;
  rq.detailed_profile = detailed_profile ? 1u : 0u;
  NervaHipHfDecodeSequenceSessionCreateResult out{};
  NervaHipHfDecodeSequenceSession *handle = nullptr;
  const int rc = nerva_hip_hf_decode_sequence_session_fork_shared_weights(&rq, &out, &handle);
  result.summary = detail::create_summary_from_result(rc, out, "fork");
  if (result.summary.status == SmokeStatus::Ok && handle != nullptr)
    result.session = std::make_unique<HipHfDecodeSequenceSession>(handle, result.summary);
  return result;
}

struct HipHfDecodeSequenceLoopStart;

// session/stateful.rs:20-181 CudaHfDecodeSequenceLoop
class HipHfDecodeSequenceLoop {
 public:
  static HipHfDecodeSequenceLoopStart start(HipHfDecodeSequenceSession &session, Span<uint32_t> prompt,
                                            std::optional<uint32_t> eos_token = std::nullopt);
  static HipHfDecodeSequenceLoopStart start_with_sampler(HipHfDecodeSequenceSession &session, Span<uint32_t> prompt,
                                                         std::optional<uint32_t> eos_token,
                                                         HipHfDecodeSamplerConfig sampler);
  static HipHfDecodeSequenceSummary start_session_with_sampler(HipHfDecodeSequenceSession &session,
                                                               Span<uint32_t> prompt, std::optional<uint32_t> eos_token,
                                                               HipHfDecodeSamplerConfig sampler) {
    if (auto e = detail::validate_loop_start(prompt, session.create_summary().vocab_size))
      return detail::failed_run_summary(*e);
    if (auto e = sampler.validate()) return detail::failed_run_summary(*e);
    NervaHipHfDecodeSequenceSessionStartRequest rq{};
    rq.session = session.raw_handle();
    rq.prompt_tokens = prompt.data;
    rq.prompt_token_count = static_cast<uint32_t>(prompt.size);
    rq.has_eos_token = eos_token.has_value() ? 1u : 0u;
    rq.eos_token = eos_token.value_or(0);
    rq.sampler = sampler.to_ffi();
    NervaHipHfDecodeSequenceResult out{};
    const int rc = nerva_hip_hf_decode_sequence_session_start(&rq, &out);
    return detail::summary_from_run(rc, out, {});
  }
  static HipHfDecodeSequenceLoop from_started(HipHfDecodeSequenceSession &session, std::optional<uint32_t> eos_token) {
    return HipHfDecodeSequenceLoop(session, eos_token);
  }
  // stateful.rs:121-151: tokens past a stop token are not produced; the loop is then finished
  HipHfDecodeSequenceSummary advance(size_t steps) {
    if (finished_) return detail::failed_run_summary("HIP HF decode sequence loop is finished");
    if (steps == 0) return detail::failed_run_summary("HIP HF decode sequence loop advance requires steps");
    std::vector<uint32_t> tokens(steps);
    NervaHipHfDecodeSequenceSessionAdvanceRequest rq{};
    rq.session = session_->raw_handle();
    rq.steps = static_cast<uint32_t>(steps);
    rq.output_tokens = tokens.data();
    rq.output_token_capacity = static_cast<uint32_t>(tokens.size());
    NervaHipHfDecodeSequenceResult out{};
    const int rc = nerva_hip_hf_decode_sequence_session_advance(&rq, &out);
    HipHfDecodeSequenceSummary s = detail::summary_from_run(rc, out, std::move(tokens));
    if (s.status == SmokeStatus::Ok && eos_token_.has_value() && !s.tokens.empty() && s.tokens.back() == *eos_token_)
      finished_ = true;
    return s;
  }
  bool finished() const { return finished_; }

  // stateful.rs:153-180: the sessions of these loops advance together; a loop whose new token is its
  // stop token is finished afterwards
  static HipHfDecodeSequenceBatchAdvanceSummary batch_advance_one(const std::vector<HipHfDecodeSequenceLoop *> &loops,
                                                                  uint32_t target_block_tokens, uint32_t min_block_tokens) {
    std::vector<HipHfDecodeSequenceSession *> sessions;
    sessions.reserve(loops.size());
    for (HipHfDecodeSequenceLoop *loop : loops) sessions.push_back(loop != nullptr ? loop->session_ : nullptr);
    HipHfDecodeSequenceBatchAdvanceSummary summary =
        HipHfDecodeSequenceSession::batch_advance_one(sessions, target_block_tokens, min_block_tokens);
    if (summary.status == SmokeStatus::Ok) {
      for (size_t i = 0; i < loops.size() && i < summary.tokens.size(); ++i) {
        const uint32_t token = summary.tokens[i];
        if (token != UINT32_MAX && loops[i] != nullptr)
          loops[i]->finished_ = loops[i]->eos_token_.has_value() && token == *loops[i]->eos_token_;
      }
    }
    return summary;
  }

 private:
  HipHfDecodeSequenceLoop(HipHfDecodeSequenceSession &session, std::optional<uint32_t> eos_token)
      : session_(&session), eos_token_(eos_token) {}
  HipHfDecodeSequenceSession *session_;
  std::optional<uint32_t> eos_token_;
  bool finished_ = false;
};

struct HipHfDecodeSequenceLoopStart {
  HipHfDecodeSequenceSummary summary;
  std::optional<HipHfDecodeSequenceLoop> loop_state;  // empty unless summary.status == Ok
};

inline HipHfDecodeSequenceLoopStart HipHfDecodeSequenceLoop::start(HipHfDecodeSequenceSession &session,
                                                                   Span<uint32_t> prompt,
                                                                   std::optional<uint32_t> eos_token) {
  return start_with_sampler(session, prompt, eos_token, HipHfDecodeSamplerConfig::greedy());
}

inline HipHfDecodeSequenceLoopStart HipHfDecodeSequenceLoop::start_with_sampler(
    HipHfDecodeSequenceSession &session, Span<uint32_t> prompt, std::optional<uint32_t> eos_token,
    HipHfDecodeSamplerConfig sampler) {
  HipHfDecodeSequenceLoopStart result;
  result.summary = start_session_with_sampler(session, prompt, eos_token, sampler);
  if (result.summary.status == SmokeStatus::Ok) result.loop_state = HipHfDecodeSequenceLoop(session, eos_token);
  return result;
}

}  // namespace nerva::hip
