/* nerva_hip_api.h - flat C ABI of libnerva_hip (MI355X / gfx950 decode backend).
 *
 * This is the boundary a `nerva-hip` host crate binds, the way `nerva-cuda`
 * binds native/cuda/nerva_cuda_api.h in the reference. Every struct marked
 * "mirrors" has the same field order, widths and enum values as the cited
 * NervaCuda... struct (the `cuda_error` slot carries a hipError_t and is named
 * `hip_error`), so the Rust #[repr(C)] mirrors only need their prefix changed.
 * include/nerva_hip_layout_check.hpp static_asserts the sizes and key offsets.
 *
 * Conventions (reference: nerva_cuda_api.h:2141-2310,
 * session_api_lifecycle.inc.cu:5-55,1117-1144, native_stubs.rs:5-33):
 *   - every call returns 0 on success and -1 on failure;
 *   - a null `out` returns -1; otherwise `out` is zeroed and status = -1 first;
 *   - no device present: status = -1, hip_error = 100 (hipErrorNoDevice);
 *   - nothing throws, aborts or logs across this boundary;
 *   - a session is driven by one host thread at a time; callers serialise.
 *
 * Citations are reference paths (relative to the reference checkout).
 */
#ifndef NERVA_HIP_API_H_
#define NERVA_HIP_API_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NERVA_HIP_DTYPE_F16 0u  /* types.cuh:9 */
#define NERVA_HIP_DTYPE_BF16 1u /* types.cuh:10 */
#define NERVA_HIP_MLP_DENSE 0u  /* types.cuh:12 */
#define NERVA_HIP_ATTENTION_FULL 0u /* types.cuh:14 */
#define NERVA_HIP_SLOT_REQUEST_ID 1u  /* types.cuh:34 */
#define NERVA_HIP_SLOT_SEQUENCE_ID 1u /* types.cuh:35 */
#define NERVA_HIP_SLOT_DEVICE_COMPLETE 1u /* types.cuh:36 */
/* No counterpart in the reference: the slot of a token whose step a device-side bounded wait gave up on (the
 * attention's split merge). The token is not valid; the call that reads the slot returns -1 with
 * hip_error = NERVA_HIP_ERROR_STEP_FAULT, and the sequence has to be started again. */
#define NERVA_HIP_SLOT_DEVICE_FAULT 2u
#define NERVA_HIP_ERROR_STEP_FAULT 719 /* hipErrorLaunchFailure */
#define NERVA_HIP_KV_BLOCK_TOKENS 16u /* types.cuh:64 */
#define NERVA_HIP_ERROR_NO_DEVICE 100 /* native_stubs.rs:5-16 */
#define NERVA_HIP_ERROR_NOT_SUPPORTED 801 /* hipErrorNotSupported */
#define NERVA_HIP_ERROR_INVALID_VALUE 1 /* hipErrorInvalidValue */

/* mirrors NervaCudaDeviceSmokeResult (nerva_cuda_api.h:9-27) */
typedef struct NervaHipDeviceSmokeResult {
  int32_t status, hip_error;
  uint32_t value;
  int32_t device_count, device_ordinal, driver_version, runtime_version,
      compute_capability_major, compute_capability_minor, posix_fd_handle_supported,
      vmm_posix_fd_export_verified, gpu_direct_rdma_supported,
      gpu_direct_rdma_with_cuda_vmm_supported;
  uint64_t total_global_mem, free_global_mem;
  char gpu_name[128], pci_bus_id[32];
} NervaHipDeviceSmokeResult;

/* mirrors NervaCudaSyntheticTokenSlot (nerva_cuda_api.h:29-37); 40 bytes.
 * The sampler writes {1, 1, pos, token, pos+1, 1, 0} (sampler.cu:394-407). */
typedef struct NervaHipSyntheticTokenSlot {
  uint32_t request_id, sequence_id;
  uint64_t token_index;
  uint32_t token;
  uint64_t version;
  uint32_t completion, host_copied;
} NervaHipSyntheticTokenSlot;

/* mirrors NervaCudaHfDecodeChainLayer (nerva_cuda_api.h:255-332). Host
 * pointers to row-major [out, in] 16-bit matrices, read only during create.
 * This backend runs dense full-attention layers: a non-zero mlp_kind,
 * attention_kind, linear_* or deepseek_* field, or a non-null w_q_gate /
 * router / expert / w_linear_* pointer, fails create with
 * hip_error = NERVA_HIP_ERROR_NOT_SUPPORTED. */
typedef struct NervaHipHfDecodeChainLayer {
  const uint16_t *rms_attn_weight, *rms_mlp_weight, *w_q, *w_q_gate, *w_k, *q_norm_weight,
      *k_norm_weight, *w_v, *w_o, *q_bias, *k_bias, *v_bias, *o_bias, *w_gate, *w_up, *w_down,
      *w_router, *w_expert_gate_up, *w_expert_down, *w_shared_expert_gate, *w_shared_expert_up,
      *w_shared_expert_down, *w_shared_expert_router;
  uint32_t linear_key_heads, linear_value_heads, linear_key_head_dim, linear_value_head_dim,
      linear_conv_kernel;
  const uint16_t *w_linear_conv, *w_linear_qkv, *w_linear_z, *w_linear_b, *w_linear_a,
      *w_linear_dt_bias;
  const float *w_linear_a_log;
  const uint16_t *w_linear_norm, *w_linear_out;
  uint32_t mlp_kind, moe_intermediate, shared_expert_intermediate, num_experts,
      experts_per_token, norm_topk_prob, attention_kind, deepseek_mode, deepseek_flags,
      deepseek_storage, deepseek_hc_mult, deepseek_hc_sinkhorn_iters, deepseek_q_lora_rank,
      deepseek_kv_lora_rank, deepseek_o_lora_rank, deepseek_o_groups, deepseek_qk_nope_head_dim,
      deepseek_qk_rope_head_dim, deepseek_v_head_dim, deepseek_compress_ratio,
      deepseek_index_topk, deepseek_index_n_heads, deepseek_index_head_dim,
      deepseek_router_num_groups, deepseek_router_topk_groups;
  float deepseek_routed_scaling_factor, deepseek_hc_eps, deepseek_hc_post_alpha;
  uint32_t deepseek_rope_scaling_type, deepseek_rope_original_max_position;
  float deepseek_rope_scaling_factor, deepseek_rope_extrapolation_factor,
      deepseek_rope_attn_factor, deepseek_rope_beta_fast, deepseek_rope_beta_slow,
      deepseek_rope_mscale, deepseek_rope_mscale_all_dim, deepseek_compress_rope_theta,
      deepseek_swiglu_limit;
} NervaHipHfDecodeChainLayer;

/* mirrors NervaCudaHfDecodeSequenceWeightBlock (nerva_cuda_api.h:380-391): one block of a declared
 * weight plan. The blocks tile the weight bytes [0, resident_weight_bytes) in the reference's arena
 * order - embeddings; per layer rms_attn, w_q, [q_norm], w_k, [k_norm], w_v, w_o, rms_mlp, w_gate,
 * w_up, w_down, [q_bias, k_bias, v_bias, o_bias]; final norm; LM head - and need not follow tensor
 * boundaries. Source: host memory (host_source) or `bytes` bytes of a file at file_offset_begin
 * (source_file, not NUL-terminated, source_file_len bytes). A request with planned_weight_blocks or
 * planned_weight_bytes != 0 declares a plan: it must then hold one descriptor per block and the
 * FNV-1a-64 hash over (block_id, block_version, offset_bytes, bytes: u64; strategy: u32) of all
 * of them, the descriptors are THE source of the weights (weights.cu:411-467, 797-908), and the tensor
 * pointers only mark which optional tensors exist (all others may be null). */
#define NERVA_HIP_WEIGHT_STRATEGY_GPU_RESIDENT 1u /* weight_plan.rs:3 */
#define NERVA_HIP_WEIGHT_STRATEGY_GPU_STAGED 2u   /* weight_plan.rs:4 */
typedef struct NervaHipHfDecodeSequenceWeightBlock {
  const uint16_t *host_source;
  const char *source_file;
  uint64_t source_file_len, file_offset_begin, block_id, block_version, offset_bytes, bytes;
  uint32_t strategy, reserved;
} NervaHipHfDecodeSequenceWeightBlock;

/* mirrors NervaCudaHfDecodeSamplerConfig (nerva_cuda_api.h:393-399).
 * Greedy <=> !(temperature > 0) || top_k == 1 (sampler.cu:89); otherwise Gumbel-max over the whole
 * vocabulary (top_k == 0 and top_p >= 0.999999) or top-k / top-p with the reference's hash random
 * numbers. Out-of-range values are normalised like sampler.cu:422-433. */
typedef struct NervaHipHfDecodeSamplerConfig {
  float temperature, top_p;
  uint32_t top_k, reserved;
  uint64_t seed;
} NervaHipHfDecodeSamplerConfig;

/* mirrors NervaCudaHfDecodeSequenceRequest (nerva_cuda_api.h:401-434) */
typedef struct NervaHipHfDecodeSequenceRequest {
  uint32_t dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab_size, layer_count,
      steps, seed_token;
  const uint32_t *prompt_tokens;
  uint32_t prompt_token_count, has_eos_token, eos_token;
  float rms_eps, rope_theta;
  const uint16_t *embeddings;
  const NervaHipHfDecodeChainLayer *layers;
  const uint16_t *final_norm_weight, *lm_head;
  uint32_t planned_weight_blocks, planned_gpu_resident_blocks, planned_gpu_staged_blocks;
  uint64_t planned_weight_bytes, planned_gpu_resident_weight_bytes,
      planned_gpu_staged_weight_bytes;
  const NervaHipHfDecodeSequenceWeightBlock *planned_weight_descriptors;
  uint32_t planned_weight_descriptor_count;
  uint64_t planned_weight_descriptor_hash;
  uint32_t *output_tokens;
  uint32_t output_token_capacity;
  NervaHipHfDecodeSamplerConfig sampler;
} NervaHipHfDecodeSequenceRequest;

/* mirrors NervaCudaHfDecodeSequenceResult (nerva_cuda_api.h:436-513) */
typedef struct NervaHipHfDecodeSequenceResult {
  int32_t status, hip_error, device_count;
  uint32_t dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab_size, layer_count,
      steps, seed_token, observed_tokens, last_token;
  uint64_t observed_token_hash, resident_weight_bytes;
  uint32_t planned_weight_blocks, planned_gpu_resident_blocks, planned_gpu_staged_blocks;
  uint64_t planned_weight_bytes, planned_gpu_resident_weight_bytes,
      planned_gpu_staged_weight_bytes, descriptor_gpu_resident_h2d_bytes,
      descriptor_gpu_staged_h2d_bytes;
  uint32_t planned_weight_descriptor_count;
  uint64_t planned_weight_descriptor_hash, resident_kv_bytes, deepseek_mhc_residual_bytes,
      deepseek_mhc_post_mix_bytes, deepseek_mhc_comb_mix_bytes, kv_tokens, device_arena_bytes,
      pinned_host_bytes, h2d_bytes, d2h_bytes, graph_replays, graph_nodes, graph_launches,
      graph_captures, graph_cache_hits, kernel_launches, experimental_rt_selector_launches;
  uint32_t experimental_rt_sparse_attention_active, experimental_rt_dense_attention_chunks,
      experimental_rt_attention_chunks, experimental_rt_reserved;
  uint64_t device_elapsed_ns, projection_ns, qkv_projection_ns, attention_output_projection_ns,
      gate_up_projection_ns, down_projection_ns, lm_head_projection_ns, attention_ns, mlp_ns,
      norm_ns, sampling_ns, sync_calls, host_causality_edges, hot_path_allocations,
      deepseek_compressor_state_writes, deepseek_compressed_kv_writes,
      deepseek_indexer_state_writes, deepseek_indexer_kv_writes,
      deepseek_compressed_kv_attention_reads, deepseek_compressed_kv_attention_slots_scanned,
      deepseek_sparse_topk_selections, deepseek_sparse_topk_slots_selected,
      deepseek_sparse_topk_candidates_scored, deepseek_sparse_topk_selection_hash,
      deepseek_v3_grouped_router_selections, deepseek_v4_bias_router_selections,
      deepseek_v4_hash_router_selections, deepseek_raw_attention_tokens_scanned,
      deepseek_sparse_attention_output_hash;
} NervaHipHfDecodeSequenceResult;

typedef struct NervaHipHfDecodeSequenceSession NervaHipHfDecodeSequenceSession;

/* mirrors NervaCudaHfDecodeSequenceSessionCreateRequest (nerva_cuda_api.h:606-638) */
typedef struct NervaHipHfDecodeSequenceSessionCreateRequest {
  uint32_t dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab_size, layer_count,
      max_context_tokens;
  float rms_eps, rope_theta;
  const uint16_t *embeddings;
  const NervaHipHfDecodeChainLayer *layers;
  const uint16_t *final_norm_weight, *lm_head;
  uint32_t planned_weight_blocks, planned_gpu_resident_blocks, planned_gpu_staged_blocks;
  uint64_t planned_weight_bytes, planned_gpu_resident_weight_bytes,
      planned_gpu_staged_weight_bytes;
  const NervaHipHfDecodeSequenceWeightBlock *planned_weight_descriptors;
  uint32_t planned_weight_descriptor_count;
  uint64_t planned_weight_descriptor_hash;
  uint32_t detailed_profile, experimental_rt_decode, experimental_rt_mode,
      experimental_rt_page_tokens, experimental_rt_pages, experimental_rt_local_window_tokens,
      experimental_rt_sink_tokens;
} NervaHipHfDecodeSequenceSessionCreateRequest;

/* mirrors NervaCudaHfDecodeSequenceSessionCreateResult (nerva_cuda_api.h:640-687) */
typedef struct NervaHipHfDecodeSequenceSessionCreateResult {
  int32_t status, hip_error, failure_stage, device_count;
  uint32_t dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab_size, layer_count,
      max_context_tokens, prefill_chunk_tokens, head_threads;
  uint64_t resident_weight_bytes;
  uint32_t planned_weight_blocks, planned_gpu_resident_blocks, planned_gpu_staged_blocks;
  uint64_t planned_weight_bytes, planned_gpu_resident_weight_bytes,
      planned_gpu_staged_weight_bytes, descriptor_gpu_resident_h2d_bytes,
      descriptor_gpu_staged_h2d_bytes;
  uint32_t planned_weight_descriptor_count;
  uint64_t planned_weight_descriptor_hash;
  uint32_t experimental_rt_decode_requested, experimental_rt_decode_enabled,
      experimental_rt_mode, experimental_rt_page_tokens, experimental_rt_pages,
      experimental_rt_local_window_tokens, experimental_rt_sink_tokens,
      deepseek_v4_attention_aux_streams, deepseek_v4_attention_events;
  uint64_t deepseek_v4_swa_kv_bytes, deepseek_mhc_residual_bytes, deepseek_mhc_post_mix_bytes,
      deepseek_mhc_comb_mix_bytes, resident_kv_bytes, device_arena_bytes, pinned_host_bytes,
      h2d_bytes, sync_calls, hot_path_allocations, device_memory_bandwidth_bps;
} NervaHipHfDecodeSequenceSessionCreateResult;

/* mirrors NervaCudaHfDecodeSequenceSessionRunRequest (nerva_cuda_api.h:694-705) */
typedef struct NervaHipHfDecodeSequenceSessionRunRequest {
  NervaHipHfDecodeSequenceSession *session;
  uint32_t steps, seed_token;
  const uint32_t *prompt_tokens;
  uint32_t prompt_token_count, has_eos_token, eos_token;
  uint32_t *output_tokens;
  uint32_t output_token_capacity;
  NervaHipHfDecodeSamplerConfig sampler;
} NervaHipHfDecodeSequenceSessionRunRequest;

/* mirrors NervaCudaHfDecodeSequenceSessionStartRequest (nerva_cuda_api.h:707-714) */
typedef struct NervaHipHfDecodeSequenceSessionStartRequest {
  NervaHipHfDecodeSequenceSession *session;
  const uint32_t *prompt_tokens;
  uint32_t prompt_token_count, has_eos_token, eos_token;
  NervaHipHfDecodeSamplerConfig sampler;
} NervaHipHfDecodeSequenceSessionStartRequest;

/* mirrors NervaCudaHfDecodeSequenceSessionAdvanceRequest (nerva_cuda_api.h:716-721) */
typedef struct NervaHipHfDecodeSequenceSessionAdvanceRequest {
  NervaHipHfDecodeSequenceSession *session;
  uint32_t steps;
  uint32_t *output_tokens;
  uint32_t output_token_capacity;
} NervaHipHfDecodeSequenceSessionAdvanceRequest;

/* mirrors NervaCudaHfDecodeSequenceSessionForkSharedWeightsRequest (nerva_cuda_api.h:689-692) */
typedef struct NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest {
  NervaHipHfDecodeSequenceSession *parent;
  uint32_t detailed_profile;
} NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest;

/* reasons of a batch step (session_prelude.inc.cu:56-64) */
#define NERVA_HIP_BATCH_READY 0u
#define NERVA_HIP_BATCH_INVALID_REQUEST 1u
#define NERVA_HIP_BATCH_NO_SESSIONS 2u
#define NERVA_HIP_BATCH_NO_READY_SESSIONS 3u
#define NERVA_HIP_BATCH_SHARED_WEIGHTS_UNPROVEN 4u
#define NERVA_HIP_BATCH_INSUFFICIENT_COMPATIBLE_READY 5u
#define NERVA_HIP_BATCH_MAX_BLOCK_TOKENS 32u /* types.cuh:63 */

/* mirrors NervaCudaHfDecodeSequenceBatchAdvanceRequest (nerva_cuda_api.h:936-943) */
typedef struct NervaHipHfDecodeSequenceBatchAdvanceRequest {
  NervaHipHfDecodeSequenceSession **sessions;
  uint32_t session_count, target_block_tokens, min_block_tokens;
  uint32_t *output_tokens; /* [session_count], written at the index of each session that advanced */
  uint32_t output_token_capacity;
} NervaHipHfDecodeSequenceBatchAdvanceRequest;

/* mirrors NervaCudaHfDecodeSequenceBatchAdvanceResult (nerva_cuda_api.h:945-976). The launch
 * counters count this library's launches: pack = embedding and RMSNorm rows, projection = the
 * multi-row GEMMs (or GEMVs), scatter = K/V rows into the caches, dependency = attention,
 * sampling = sampler launches. *_elapsed_ns stay 0 except projection_elapsed_ns, which is the
 * device time of the whole batch step (the projections are not timed apart from the rest). */
typedef struct NervaHipHfDecodeSequenceBatchAdvanceResult {
  int32_t status, hip_error, device_count;
  uint32_t reason, exact, requested_session_count, eligible_session_count, block_tokens,
      target_block_tokens, min_block_tokens, dtype, layer_count, observed_tokens, last_token;
  uint64_t observed_token_hash, d2h_bytes, projection_elapsed_ns, qkv_elapsed_ns,
      attention_output_elapsed_ns, gate_up_elapsed_ns, down_elapsed_ns, lm_head_elapsed_ns,
      pack_kernel_launches, projection_kernel_launches, scatter_kernel_launches,
      dependency_kernel_launches, experimental_rt_selector_launches, sampling_kernel_launches,
      sync_calls, hot_path_allocations;
} NervaHipHfDecodeSequenceBatchAdvanceResult;

/* mirrors NervaCudaDeepSeekQuantDequantResult (nerva_cuda_api.h:1338-1354) */
typedef struct NervaHipDeepSeekQuantDequantResult {
  int32_t status, hip_error, device_count;
  uint32_t rows, cols, block_rows, block_cols;
  uint64_t output_hash, device_arena_bytes, pinned_host_bytes, h2d_bytes, d2h_bytes,
      kernel_launches, sync_calls, hot_path_allocations;
} NervaHipDeepSeekQuantDequantResult;

/* mirrors NervaCudaDeepSeekQuantFp8F32ScaleEncodedMatvecRequest
 * (nerva_cuda_api.h:1367-1377). All pointers are HOST pointers. */
typedef struct NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest {
  uint32_t rows, cols, block_rows, block_cols, input_dtype;
  const uint8_t *weights;
  const float *scales;
  const uint16_t *input;
  float *output;
} NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest;

/* mirrors NervaCudaDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest
 * (nerva_cuda_api.h:1379-1390). input [tokens x cols], output [tokens x rows]. */
typedef struct NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest {
  uint32_t rows, cols, tokens, block_rows, block_cols, input_dtype;
  const uint8_t *weights;
  const float *scales;
  const uint16_t *input;
  float *output;
} NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest;

/* mirrors NervaCudaProjectionBenchRequest (nerva_cuda_api.h:1075-1082) */
typedef struct NervaHipProjectionBenchRequest {
  uint32_t dtype, rows, cols, iterations, warmup_iterations, block_tokens;
} NervaHipProjectionBenchRequest;

/* mirrors NervaCudaProjectionBenchResult (nerva_cuda_api.h:1084-1144). The
 * cublaslt_* slots stay zero (no vendor GEMV on this backend); custom_* is the
 * hand-written kernel. */
typedef struct NervaHipProjectionBenchResult {
  int32_t status, hip_error, device_count, device_ordinal, compute_capability_major,
      compute_capability_minor;
  uint32_t dtype, rows, cols, block_tokens, iterations, warmup_iterations;
  uint64_t matrix_bytes, input_bytes, output_bytes, cublaslt_total_ns, cublaslt_avg_ns,
      cublaslt_default_total_ns, cublaslt_default_avg_ns;
  uint32_t cublaslt_heuristic_count, cublaslt_best_heuristic_index;
  uint64_t cublaslt_best_heuristic_total_ns, cublaslt_best_heuristic_avg_ns, custom_total_ns,
      custom_avg_ns, cublaslt_graph_total_ns, cublaslt_graph_avg_ns,
      cublaslt_default_graph_total_ns, cublaslt_default_graph_avg_ns,
      cublaslt_best_heuristic_graph_total_ns, cublaslt_best_heuristic_graph_avg_ns,
      custom_graph_total_ns, custom_graph_avg_ns, cublaslt_graph_nodes, custom_graph_nodes,
      graph_replays, graph_captures;
  uint32_t selected_graph_strategy;
  uint64_t cublaslt_effective_bandwidth_bps, custom_effective_bandwidth_bps;
  uint32_t selected_strategy, mismatch_count;
  float max_abs_diff;
  uint64_t kernel_launches, sync_calls, device_allocations, device_frees, device_arena_bytes,
      hot_path_allocations, block_cublaslt_total_ns, block_cublaslt_avg_ns,
      block_cublaslt_per_token_ns, block_cublaslt_graph_total_ns, block_cublaslt_graph_avg_ns,
      block_cublaslt_graph_per_token_ns, block_cublaslt_graph_nodes,
      block_cublaslt_speedup_x1000, block_cublaslt_graph_speedup_x1000,
      block_cublaslt_effective_bandwidth_bps;
} NervaHipProjectionBenchResult;

/* mirrors NervaCudaDeepSeekMoeForwardRequest (nerva_cuda_api.h:2023-2037); host f32 pointers */
typedef struct NervaHipDeepSeekMoeForwardRequest {
  uint32_t hidden_size, intermediate_size, num_experts, top_k, clamp_swiglu;
  float swiglu_limit;
  const float *input;
  const uint32_t *expert_ids;
  const float *expert_weights, *w_gate, *w_up, *w_down;
  float *output;
} NervaHipDeepSeekMoeForwardRequest;

/* mirrors NervaCudaDeepSeekMoeForwardResult (nerva_cuda_api.h:2039-2058) */
typedef struct NervaHipDeepSeekMoeForwardResult {
  int32_t status, hip_error, device_count, moe_error;
  uint32_t hidden_size, intermediate_size, num_experts, top_k, clamp_swiglu;
  float swiglu_limit;
  uint64_t output_hash, device_arena_bytes, pinned_host_bytes, h2d_bytes, d2h_bytes,
      kernel_launches, sync_calls, hot_path_allocations;
} NervaHipDeepSeekMoeForwardResult;

/* ------------------------------------------------------------------------
 * Entry points that replace a reference entry point one for one.
 * ---------------------------------------------------------------------- */

/* replaces nerva_cuda_device_smoke (nerva_cuda_api.h:2141) */
int nerva_hip_device_smoke(NervaHipDeviceSmokeResult *out);

/* replaces nerva_cuda_hf_decode_sequence_u16 (nerva_cuda_api.h:2157-2159):
 * create + start + advance(steps) + destroy in one call. */
int nerva_hip_hf_decode_sequence_u16(const NervaHipHfDecodeSequenceRequest *request,
                                     NervaHipHfDecodeSequenceResult *out);

/* replaces nerva_cuda_hf_decode_sequence_session_create (nerva_cuda_api.h:2163-2166) */
int nerva_hip_hf_decode_sequence_session_create(
    const NervaHipHfDecodeSequenceSessionCreateRequest *request,
    NervaHipHfDecodeSequenceSessionCreateResult *out, NervaHipHfDecodeSequenceSession **session);

/* replaces nerva_cuda_hf_decode_sequence_session_run (nerva_cuda_api.h:2167-2169) */
int nerva_hip_hf_decode_sequence_session_run(const NervaHipHfDecodeSequenceSessionRunRequest *request,
                                             NervaHipHfDecodeSequenceResult *out);

/* replaces nerva_cuda_hf_decode_sequence_session_start (nerva_cuda_api.h:2170-2172):
 * prefills the whole prompt and samples token 0 into slots[prompt_count-1]. */
int nerva_hip_hf_decode_sequence_session_start(
    const NervaHipHfDecodeSequenceSessionStartRequest *request, NervaHipHfDecodeSequenceResult *out);

/* replaces nerva_cuda_hf_decode_sequence_session_advance (nerva_cuda_api.h:2173-2175):
 * the first advance(steps) returns `steps` tokens with steps-1 graph replays. */
int nerva_hip_hf_decode_sequence_session_advance(
    const NervaHipHfDecodeSequenceSessionAdvanceRequest *request,
    NervaHipHfDecodeSequenceResult *out);

/* replaces nerva_cuda_hf_decode_sequence_session_destroy (nerva_cuda_api.h:2216-2218) */
int nerva_hip_hf_decode_sequence_session_destroy(NervaHipHfDecodeSequenceSession *session,
                                                 NervaHipHfDecodeSequenceSessionCreateResult *out);

/* replaces nerva_cuda_hf_decode_sequence_session_fork_shared_weights (nerva_cuda_api.h:2212-2215):
 * a second session on the parent's resident weights with a KV cache, token slots and cursor of its
 * own. If the parent has a sequence under way (started, not finished), the child starts as a copy
 * of it - prompt, slots, cursor, cache, sampler - and both go on independently. The weights are
 * freed when the last session holding them is destroyed, in any order. */
int nerva_hip_hf_decode_sequence_session_fork_shared_weights(
    const NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest *request,
    NervaHipHfDecodeSequenceSessionCreateResult *out, NervaHipHfDecodeSequenceSession **session);

/* replaces nerva_cuda_hf_decode_sequence_batch_advance_one (nerva_cuda_api.h:2209-2211): one more
 * token for each of up to 32 ready sessions of the same model through ONE stream of the weights.
 * Ready = started, not finished, every token computed so far already handed out by advance
 * (prompt + observed == cursor + 1). Sessions count as the same model when their weight
 * descriptor hashes are non-zero and equal and their dimensions agree; the largest such group is
 * taken in request order (status 0 with a reason other than READY means nothing ran). Each
 * session samples with its own sampler and position. */
int nerva_hip_hf_decode_sequence_batch_advance_one(
    const NervaHipHfDecodeSequenceBatchAdvanceRequest *request,
    NervaHipHfDecodeSequenceBatchAdvanceResult *out);

/* replaces nerva_cuda_deepseek_quant_fp8_f32_scale_encoded_matvec (nerva_cuda_api.h:2245-2247) */
int nerva_hip_deepseek_quant_fp8_f32_scale_encoded_matvec(
    const NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest *request,
    NervaHipDeepSeekQuantDequantResult *out);

/* replaces nerva_cuda_deepseek_quant_fp8_f32_scale_encoded_gemm_tokens (nerva_cuda_api.h:2248-2250) */
int nerva_hip_deepseek_quant_fp8_f32_scale_encoded_gemm_tokens(
    const NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest *request,
    NervaHipDeepSeekQuantDequantResult *out);

/* replaces nerva_cuda_projection_bench (nerva_cuda_api.h:2227-2228). Unlike the
 * reference's loop, which re-reads one matrix, this one cycles through enough
 * distinct copies of the matrix to exceed 1 GiB so that the 256 MB last-level
 * cache cannot serve repeats (set NERVA_HIP_BENCH_RESIDENT=1 to re-read one copy). */
int nerva_hip_projection_bench(const NervaHipProjectionBenchRequest *request,
                               NervaHipProjectionBenchResult *out);

/* replaces nerva_cuda_deepseek_moe_forward (nerva_cuda_api.h:2302-2304): f32
 * routed experts with optional SwiGLU clamp, host pointers. */
int nerva_hip_deepseek_moe_forward(const NervaHipDeepSeekMoeForwardRequest *request,
                                   NervaHipDeepSeekMoeForwardResult *out);

/* ------------------------------------------------------------------------
 * Device-pointer operator entry points. The reference exposes these kernels
 * only inside its session (native/cuda/hf_decode_sequence/session_decode_prefill.inc.cu:74-372);
 * they are exported here so each one can be checked and timed on its own.
 * All pointers are DEVICE pointers obtained from nerva_hip_malloc; `stream`
 * is a hipStream_t or NULL for the library's own stream. Launch only: call
 * nerva_hip_stream_synchronize before reading results. Return 0 / -1 and
 * leave the hipError_t in *hip_error when it is non-null.
 * ---------------------------------------------------------------------- */

typedef struct NervaHipGemvRequest {
  uint32_t dtype;            /* NERVA_HIP_DTYPE_* of weights and 16-bit vectors */
  uint32_t rows, cols;       /* W is row-major [rows x cols] (for swiglu: [2*rows x cols], gate rows first) */
  uint32_t prologue;         /* 0: input16 is the 16-bit x;  1: x = round16(rmsnorm(input_f32, gamma, eps)) */
  uint32_t epilogue;         /* 0: f32 out; 1: f32 out = y + residual; 2: out16 = round16(silu(gate)*up);
                                3: out16 = round16(y) */
  uint32_t round_output;     /* epilogue 1: round the sum to 16 bits (prompt-token staging) */
  float rms_eps;
  uint32_t pair_gap;         /* epilogue 2: elements left unused between the last gate row and the first up row
                                (a multiple of 8; 0 = the up rows follow the gate rows directly) */
  const uint16_t *weights;
  const uint16_t *input16;   /* [cols] */
  const float *input_f32;    /* [cols] */
  const uint16_t *gamma;     /* [cols] */
  const uint16_t *bias;      /* optional [rows] */
  const float *residual;     /* [rows] */
  float *output_f32;         /* [rows] */
  uint16_t *output16;        /* [rows] */
} NervaHipGemvRequest;

/* y = W.x weight-streaming GEMV (mat_vec_encoded_row_major, precision/block/ops.rs:75-91;
 * device staging projection.cu:63-79) with the fused prologues/epilogues of the
 * decode step (device_ops.cuh:317-332, kernels.cu:577-612,651-668). */
int nerva_hip_gemv(const NervaHipGemvRequest *request, void *stream, int32_t *hip_error);

/* The launch shape nerva_hip_gemv (and the session's step) chooses for a request of these sizes with
 * 16-byte-aligned pointers: *kernel, low four bits = 0 scalar, 1 guarded vector, 2 full vector, 3 the lean
 * production-shape kernel; bit 4 = the lean kernel walks its rows from a rotated start; bits 8 and up = 1 KiB
 * chunks of a row per request batch; *workgroups = the grid. Host arithmetic only (no device is touched):
 * measurements taken for one launch shape (counter profiles) are keyed to it. No counterpart. */
int nerva_hip_gemv_launch_shape(uint32_t prologue, uint32_t epilogue, uint32_t rows, uint32_t cols,
                                uint32_t *kernel, uint32_t *workgroups);

typedef struct NervaHipFp8GemvRequest {
  uint32_t rows, cols, block_rows, block_cols;
  uint32_t input_dtype;      /* dtype of input16 */
  const uint8_t *weights;    /* e4m3fn [rows x cols] */
  const float *scales;       /* [ceil(rows/block_rows) x ceil(cols/block_cols)] */
  const uint16_t *input16;   /* [cols], or NULL */
  const float *input_f32;    /* [cols], used when input16 is NULL */
  float *output;             /* [rows] */
} NervaHipFp8GemvRequest;

/* y[r] = sum_c (e4m3(W[r,c]) * S[r/br, c/bc]) * x[c], dequantised in f32 registers
 * (reference contract: crates/nerva-cuda/src/tests/deepseek_quant.rs:689-713).
 * The activation vector lives in one workgroup's LDS: cols <= 15360, or <= 30720 for a 16-byte
 * aligned input16 with cols and block_cols multiples of 16 and 16-byte aligned weights (the 16-bit
 * values then stay 16 bit, and the launch takes the lean row-pair kernel whatever cols modulo 1024);
 * beyond that the call fails with hipErrorInvalidValue. */
int nerva_hip_fp8_gemv(const NervaHipFp8GemvRequest *request, void *stream, int32_t *hip_error);

typedef struct NervaHipPagedAttentionRequest {
  uint32_t dtype, heads, kv_heads, head_dim;
  uint32_t layer, block_count;  /* KV cache holds [layers][block_count] blocks of 16 tokens */
  uint32_t position;            /* index of the token being decoded; keys 0..position are attended */
  uint32_t append;              /* 1: qkv_f32 carries k,v of this token -> norm/RoPE/round/append first */
  float rms_eps, rope_theta;    /* rope_theta <= 0 disables RoPE */
  const float *qkv_f32;         /* [heads*hd | kv_heads*hd | kv_heads*hd] raw projections */
  const uint16_t *q_norm, *k_norm;        /* optional [head_dim] */
  const uint16_t *q_bias, *k_bias, *v_bias; /* optional */
  uint16_t *k_cache, *v_cache;  /* [layer][block][kv_head][16][head_dim], 16-bit */
  const uint32_t *block_table;  /* [block_count] logical -> physical */
  void *workspace;              /* nerva_hip_paged_attention_workspace_bytes() bytes, zero-initialised once */
  float *output_f32;            /* optional [heads*hd] */
  uint16_t *output16;           /* [heads*hd] rounded */
  uint32_t splits;              /* 0: the library's split-KV factor; 1..64: this one (tests). Refused with
                                   hipErrorInvalidValue, and nothing launched, when it exceeds block_count or when
                                   kv_heads * splits exceeds the device's compute units: the splits of a kv head
                                   merge inside the launch and have to be resident together */
} NervaHipPagedAttentionRequest;

/* Fused per-head RMSNorm + RoPE + KV append + paged GQA split-KV decode attention
 * (kernels.cu:287-555, attention_kernels.cu:263-760; exact_blockwise_attention_into,
 * attention/exact/run.rs:13-127). */
int nerva_hip_paged_gqa_decode(const NervaHipPagedAttentionRequest *request, void *stream,
                               int32_t *hip_error);
uint64_t nerva_hip_paged_attention_workspace_bytes(uint32_t heads, uint32_t head_dim);
/* The largest split factor nerva_hip_paged_gqa_decode accepts for this many kv heads on the current device. */
uint64_t nerva_hip_paged_attention_max_splits(uint32_t kv_heads);
/* No counterpart in the reference (its attention reduces in a second launch and has no in-launch wait).
 * Synchronises `stream` and reports whether a launch of nerva_hip_paged_gqa_decode on this workspace gave up
 * waiting for a split's partial since the last call: 0 = none did; -1 with hip_error =
 * NERVA_HIP_ERROR_STEP_FAULT = one did - its outputs are NaN - and the report is cleared, so that the
 * workspace serves the next launch as if nothing had happened (partials are tagged per launch: what a late
 * split still stores is never taken for a later launch's). */
int nerva_hip_paged_attention_status(void *workspace, uint32_t heads, uint32_t head_dim, void *stream, int32_t *hip_error);
/* Element offset of (layer, physical block, kv_head, token-in-block, dim) in the K (is_value 0)
 * or V (is_value 1) cache array. A (block, kv_head) tile of 16 tokens x head_dim elements is
 * contiguous; inside it the order is the library's own (matrix-core operand order at head_dim
 * 128, row-major otherwise), so hosts that fill or read a cache go through this function. */
uint64_t nerva_hip_kv_cache_offset(uint32_t block_count, uint32_t kv_heads, uint32_t head_dim,
                                   uint32_t layer, uint32_t physical_block, uint32_t kv_head,
                                   uint32_t token_in_block, uint32_t dim, uint32_t is_value);

typedef struct NervaHipArgmaxRequest {
  uint32_t count;
  const float *logits;
  uint32_t *token;           /* device u32 */
  void *workspace;           /* nerva_hip_argmax_workspace_bytes() bytes, zero-initialised once */
} NervaHipArgmaxRequest;

/* First maximum among finite logits, ties to the lowest index (sampler.cu:35-40,89-119;
 * greedy_argmax, common/token.rs:33-58). */
int nerva_hip_argmax(const NervaHipArgmaxRequest *request, void *stream, int32_t *hip_error);
uint64_t nerva_hip_argmax_workspace_bytes(void);

/* nerva_hip_argmax for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same rule and same
 * result as nerva_hip_argmax; the per-workgroup candidates live in a 6 KiB array inside the
 * library's device image instead of a caller workspace, and the call performs no hipMalloc, hipFree
 * or other allocating routine: two kernel launches on `stream` (pass the caller's stream; NULL
 * uses the library's stream). `logits` and `token` are device pointers. nerva_hip_device_smoke has to
 * have run on the device first: it resolves the array's address there and creates the library's
 * stream; before that the call fails with hipErrorNotInitialized (3) instead of setting either up
 * itself. count > NERVA_HIP_ARGMAX_STATIC_MAX_COUNT fails with hipErrorInvalidValue and launches
 * nothing. All calls on one GPU share the array: calls that overlap on one GPU (different streams,
 * or graphs replayed concurrently) race. */
#define NERVA_HIP_ARGMAX_STATIC_MAX_COUNT 16777216u
int nerva_hip_argmax_static(const float *logits, uint32_t count, uint32_t *token, void *stream,
                            int32_t *hip_error);

typedef struct NervaHipGemmRowsRequest {
  uint32_t dtype;            /* NERVA_HIP_DTYPE_* of weights and 16-bit vectors */
  uint32_t rows, cols;       /* W is row-major [rows x cols] (epilogue 2: [2*rows x cols], gate rows first) */
  uint32_t tokens;           /* 1..128 input rows */
  uint32_t epilogue;         /* 0: f32 out; 1: f32 out = y + bias + residual; 2: out16 = round16(silu(gate)*up) */
  uint32_t round_output;     /* epilogue 1: round the sum to 16 bits (prompt-token staging) */
  const uint16_t *weights;
  const uint16_t *input16;   /* [tokens][cols] */
  const uint16_t *bias;      /* optional [rows] ([2*rows] for epilogue 2) */
  const float *residual;     /* epilogue 1: [tokens][rows] */
  float *output_f32;         /* epilogues 0, 1: [tokens][rows] */
  uint16_t *output16;        /* epilogue 2: [tokens][rows] */
  /* != 0: input16 / output16 are in matrix-operand order instead of [tokens][cols] rows, the layout
   * the kernel reads with full cache lines: element (token t, column k) at index
   * nerva_hip_gemm_operand_index(tokens, t, k); the buffer holds 32 token slots for tokens <= 32, 64 for tokens <= 64, 128 for tokens
   * <= 128, 256 for tokens <= 256, 512 above (slots past `tokens` are never looked at). */
  uint32_t input_operand_order, output16_operand_order;
  /* Optional device scratch of nerva_hip_gemm_rows_workspace_bytes(rows) bytes (rows doubled for
   * epilogue 2). With more than 64 tokens in operand order the projections with few rows are split
   * along K across workgroups, which leave f32 partial sums here; without it they run unsplit. */
  void *workspace;
  uint64_t workspace_bytes;
} NervaHipGemmRowsRequest;

/* Projection of a block of up to 128 token rows (up to 256 with input_operand_order where rows is a multiple of
 * 96 or 128 - gate/up pairs: 48 or 64 - and cols of 512; up to 512 where rows is a multiple of 192
 * or 256 - gate/up pairs: 96 or 128 - and cols of 128) through one weight matrix on the matrix cores,
 * streaming the weights once: per token the arithmetic of mat_vec_encoded_row_major
 * (precision/block/ops.rs:75-91); the reference issues cuBLAS GEMMs for this in its chunked
 * prefill and projection batch (projection.cu:99-106, 297-300). rows >= 16 (with rows % 16 != 0 the residual must
 * not alias the output), cols % 2048 == 0. */
int nerva_hip_gemm_rows(const NervaHipGemmRowsRequest *request, void *stream, int32_t *hip_error);
uint64_t nerva_hip_gemm_rows_workspace_bytes(uint32_t rows);
/* Index of element (token, column) of a block of `tokens` rows in matrix-operand order: for every 32
 * columns and every 16 tokens, 64 pieces of 8 columns, piece (column % 32 / 8) * 16 + token % 16. */
uint64_t nerva_hip_gemm_operand_index(uint32_t tokens, uint32_t token, uint32_t column);
/* out16[t] = round16(rmsnorm(x[t]) * gamma) for `tokens` rows of `cols` f32 values
 * (rms_norm_encoded_into, ops.rs:31-50, once per row). */
int nerva_hip_rmsnorm_rows(uint32_t dtype, const float *x, const uint16_t *gamma, float eps, uint32_t tokens,
                           uint32_t cols, uint16_t *out16, void *stream, int32_t *hip_error);

typedef struct NervaHipSampleRequest {
  uint32_t vocab;
  uint32_t position;            /* sequence position of the sampled token: the random-number counter */
  const float *logits;          /* device [vocab] */
  NervaHipHfDecodeSamplerConfig sampler;
  uint32_t *token;              /* device u32 */
  void *workspace;              /* device, nerva_hip_sample_workspace_bytes(vocab) bytes */
} NervaHipSampleRequest;

/* One token from logits by the session's sampler (sampler.cu:66-392): greedy when
 * !(temperature > 0) or top_k == 1; Gumbel-max over the whole vocabulary when top_k == 0 and
 * top_p >= 0.999999; otherwise the k = (top_k == 0 ? 128 : min(top_k, 128)) best finite logits by
 * (value desc, index asc), softmax with temperature in that order, nucleus top_p, one draw. Random
 * numbers are a hash of (seed, position, index, salt), so equal inputs give equal tokens. The
 * configuration is normalised like the reference's ABI does (sampler.cu:422-433), never refused. */
int nerva_hip_sample(const NervaHipSampleRequest *request, void *stream, int32_t *hip_error);
uint64_t nerva_hip_sample_workspace_bytes(uint32_t vocab);

typedef struct NervaHipMoeFp8Request {
  uint32_t hidden, intermediate, num_experts, top_k, block, input_dtype;
  int32_t shared_index;         /* expert index of the always-on shared expert, or -1 */
  const uint16_t *input16;      /* [hidden] */
  const uint32_t *expert_ids;   /* device [top_k] */
  const float *expert_weights;  /* device [top_k] */
  const uint8_t *w_gate, *w_up; /* [E][intermediate][hidden] e4m3fn */
  const float *s_gate, *s_up;   /* [E][ceil(I/block)][ceil(H/block)] */
  const uint8_t *w_down;        /* [E][hidden][intermediate] */
  const float *s_down;          /* [E][ceil(H/block)][ceil(I/block)] */
  float *activation;            /* scratch f32 [(top_k+1) * intermediate] */
  float *output;                /* f32 [hidden] */
  uint32_t phases;              /* 0: the whole operator (two launches); 1: gate/up + SwiGLU only (fills
                                   `activation`); 2: down + combine only (reads `activation`) - timing */
} NervaHipMoeFp8Request;

/* out = sum_k w_k * Wd_e(swiglu(Wg_e x, Wu_e x)) + shared(x) with FP8 block-scaled
 * expert weights (reference/moe.rs:76-166, precision/block/moe.rs:744-859;
 * kernels_sparse_moe.inc.cu:323-397,787-946). The expert ids are device data, so the host cannot
 * refuse them: an id >= num_experts makes every output element NaN (no memory outside the bank is
 * read), never a plausible result from another expert. */
int nerva_hip_moe_fp8_experts(const NervaHipMoeFp8Request *request, void *stream, int32_t *hip_error);

typedef struct NervaHipMoeRouteRequest {
  uint32_t num_experts, top_k, normalize;
  const float *logits;       /* device [num_experts] */
  uint32_t *expert_ids;      /* device [top_k] */
  float *expert_weights;     /* device [top_k] */
} NervaHipMoeRouteRequest;

/* softmax -> top-k by (probability desc, index asc) -> optional renormalisation
 * (select_moe_route_for_logits Softmax arm, precision/block/moe.rs:1107-1155,1303-1326). */
int nerva_hip_moe_route_softmax(const NervaHipMoeRouteRequest *request, void *stream,
                                int32_t *hip_error);

/* ------------------------------------------------------------------------
 * Device memory / stream plumbing for hosts that have no HIP binding of their own.
 * ---------------------------------------------------------------------- */
int nerva_hip_malloc(void **device_ptr, uint64_t bytes);
int nerva_hip_free(void *device_ptr);
int nerva_hip_memcpy_h2d(void *device_dst, const void *host_src, uint64_t bytes);
int nerva_hip_memcpy_d2h(void *host_dst, const void *device_src, uint64_t bytes);
int nerva_hip_memset(void *device_dst, int value, uint64_t bytes);
int nerva_hip_stream_synchronize(void *stream);
/* Counts hipMalloc/hipHostMalloc calls made by the library since load (hot-path allocation audit). */
uint64_t nerva_hip_allocation_count(void);
/* Operator timing (no reference counterpart). Between begin and end, device-pointer operator
 * calls made with a null stream are recorded, not run; end turns them into one hipGraph, replays
 * it `warmup_replays` + `timed_replays` times and reports the average device time of a replay
 * (hipEvents on the library stream). Only launches may be issued in between: no copies, no
 * allocation, no synchronisation. One recording at a time, one host thread. */
int nerva_hip_timer_capture_begin(void);
int nerva_hip_timer_capture_end(uint32_t warmup_replays, uint32_t timed_replays, uint64_t *nodes,
                                double *avg_replay_ns);
/* The same, with the shortest and the median replay beside the average (every replay between two events of
 * its own). */
int nerva_hip_timer_capture_end_stats(uint32_t warmup_replays, uint32_t timed_replays, uint64_t *nodes,
                                      double *avg_replay_ns, double *min_replay_ns, double *median_replay_ns);
/* Plain device-to-device copy kernel (16-byte aligned pointers and size): moves exactly `bytes`
 * in and `bytes` out, the known-size transfer memory counters are calibrated against. */
int nerva_hip_copy_d2d(void *device_dst, const void *device_src, uint64_t bytes, void *stream);

/* Synthetic tensors generated on the device by the counter-based generator the
 * tests' CPU oracle also implements (values are bit-identical on both sides):
 * value = mean + float(2*sum12(u16) - 786420) * (std/131072), rounded to `dtype`. */
int nerva_hip_synth_fill_16(void *device_dst, uint32_t dtype, uint64_t seed, uint64_t tensor_id,
                            uint64_t count, float mean, float std);
int nerva_hip_synth_fill_f32(void *device_dst, uint64_t seed, uint64_t tensor_id, uint64_t count,
                             float mean, float std);
int nerva_hip_synth_fill_fp8_block(void *device_weights, void *device_scales, uint64_t seed,
                                   uint64_t tensor_id, uint64_t rows, uint64_t cols, uint64_t block,
                                   float std);

/* ------------------------------------------------------------------------
 * Benchmark helpers (no reference counterpart).
 * ---------------------------------------------------------------------- */

/* Same request as session_create but every weight pointer is ignored: weights
 * are generated on the device (N(0, weight_std), norms 1 + N(0, weight_std)) from
 * `seed`, so a 16 GB model never crosses PCIe. Tensor ids: 1 embeddings,
 * 2 final_norm, 3 lm_head, 16*(layer+1)+k for the k-th pointer of the layer in
 * struct order (rms_attn=0, rms_mlp=1, w_q=2, w_k=4, q_norm=5, k_norm=6, w_v=7,
 * w_o=8, w_gate=13, w_up=14, w_down=15). */
int nerva_hip_bench_session_create_synthetic(
    const NervaHipHfDecodeSequenceSessionCreateRequest *request, uint64_t seed, float weight_std,
    uint32_t with_qk_norm, NervaHipHfDecodeSequenceSessionCreateResult *out,
    NervaHipHfDecodeSequenceSession **session);

typedef struct NervaHipStepProfile {
  int32_t status, hip_error;
  uint32_t position, launches;
  /* average device ns per launch over `repeats` un-graphed steps, hipEvent pairs around each launch */
  uint64_t embed_ns, qkv_ns, attention_ns, o_ns, gate_up_ns, down_ns, lm_head_ns, total_ns;
  uint64_t qkv_bytes, attention_bytes, o_bytes, gate_up_bytes, down_bytes, lm_head_bytes;
  /* average device ns per launch when the `layers` launches of one kind run back to back
   * between a single hipEvent pair (no per-launch event gap): the kernel's own duration */
  uint64_t qkv_stream_ns, attention_stream_ns, o_stream_ns, gate_up_stream_ns, down_stream_ns;
} NervaHipStepProfile;

/* Runs `repeats` decode steps eagerly at the session's current cursor WITHOUT
 * advancing it or publishing tokens, bracketing each launch with hipEvents on
 * the session stream (the reference's detailed_profile pass:
 * session_profile.inc.cu:35-56, session_decode_prefill.inc.cu:374-809). */
int nerva_hip_session_profile_step(NervaHipHfDecodeSequenceSession *session, uint32_t repeats,
                                   NervaHipStepProfile *out);

/* Test and measurement hook (no counterpart): overrides one launch-shape choice for the whole process;
 * value 0 restores the built-in choice. Names: "attn_splits" (split-KV factor of a session's decode
 * attention, read when a session is created), "batch_splits", "prompt_splits" (the batch step's and the
 * prompt blocks' attention), "gemm_row_tiles" (1|2), "gemm_k_waves" (8|4), "gemm_block_slices",
 * "gemm_block_row_tiles" (1|2), "gemm_block_min_tokens" (the multi-row projections), "gemv_exact_start"
 * (1: the lean GEMV's exact start-up waits wherever they can run, 2: nowhere), "moe_down_shared_first" (2: the
 * MoE down launch walks the shared expert last instead of first), "gemv_workgroup_waves" (4|16: waves per
 * workgroup of every lean GEMV launch), "gemv_x_registers" (2: the lean GEMV never keeps the input vector in
 * registers), "prefill_block_tokens" (128 | 256: sessions created afterwards prefill in blocks of at most
 * that many tokens even where larger blocks apply), "gemv_rotated_walk" (2: the lean GEMV never walks its rows from a rotated
 * start), "attn_merge_spin_limit" and "attn_withhold_split" (the bounded wait of the decode attention's split
 * merge: polls before it gives up; 1 + the split that keeps its partial to itself), and the comparison modes
 * "block_layout" (1: token blocks as [token][column] rows, 2: in matrix-operand order, whatever their size),
 * "prefill_attention_rows" (1: prompt blocks with one attention workgroup set per token), "prefill_walk" (1:
 * sessions created afterwards walk their prompts token by token), "gemm_block_off" (1: token blocks of up to 128
 * rows never through the kernel that shares the X block through LDS), "gemm_block_waves" (4: the gate/up pair of a block of up to 64 rows
 * never in three-wave workgroups), "gemm_block_rotate" (1 + the K-blocks between the places where consecutive row
 * groups of that kernel start their walk; 1: a common start). Values a kernel
 * cannot take are ignored where they are read. -1 for an unknown name. A null name restores every built-in
 * choice. */
int nerva_hip_test_set_tuning(const char *name, int32_t value);

/* 1 when this process launches its steps kernel by kernel instead of replaying captured graphs:
 * NERVA_HIP_EAGER_STEPS=1, or the ROCm profiler's environment was found at the first call (a traced
 * process must not reach hipGraphLaunch on this stack). Decided once per process. */
int nerva_hip_steps_are_eager(void);

/* Reads back the f32 logits of the last sampled position (vocab_size floats) and
 * one KV row (kv_heads*head_dim 16-bit values each for K and V) for parity tests. */
/* 1 when a batch step led by this session streams the weights once for all its sequences (the
 * model's shapes fit the multi-row kernels: head_dim 128, GQA factor 1/2/4/8, K dimensions multiples
 * of 2048), 0 when every sequence of such a step runs its own decode step; -1 for a null session. */
int nerva_hip_session_shares_weight_stream(NervaHipHfDecodeSequenceSession *session);
int nerva_hip_session_read_logits(NervaHipHfDecodeSequenceSession *session, float *host_logits);
/* Test hook (no counterpart): copies `count` token slots, from slot `first`, out of the session's device memory
 * as the device wrote them (40 bytes each: nerva_cuda_api.h:29-37, sampler.cu:394-407). */
int nerva_hip_session_read_slots(NervaHipHfDecodeSequenceSession *session, uint32_t first, uint32_t count,
                                 NervaHipSyntheticTokenSlot *host_slots);
/* Test hook (no counterpart): arms a trace of the NEXT decode step the session launches (through
 * advance): that one step runs kernel by kernel instead of as a graph replay, and after each kernel
 * its output vector is copied into `device_buffer`, one 256-byte-aligned slot behind the other, in
 * this order: x after the embedding [hidden f32]; per layer the attention RMSNorm's output as the qkv
 * rows are multiplied with it [hidden 16-bit], qkv [(heads + 2 kv_heads) * head_dim f32], attention
 * output [heads * head_dim 16-bit], r after the o projection [hidden f32], the MLP RMSNorm's output
 * [hidden 16-bit], SwiGLU output [intermediate 16-bit], x after the down projection [hidden f32]; then
 * the final RMSNorm's output [hidden 16-bit] and the logits [vocab f32].
 * The step is otherwise the ordinary one (same kernels, same launch shapes, token slot, cursor).
 * Greedy sessions on the launch-per-piece step only; -1 otherwise or when the buffer is smaller than
 * nerva_hip_session_step_trace_bytes(). A NULL buffer disarms a trace that has not run yet. */
uint64_t nerva_hip_session_step_trace_bytes(NervaHipHfDecodeSequenceSession *session);
int nerva_hip_session_trace_next_step(NervaHipHfDecodeSequenceSession *session, void *device_buffer,
                                      uint64_t bytes);
int nerva_hip_session_read_kv(NervaHipHfDecodeSequenceSession *session, uint32_t layer, uint32_t token,
                              uint16_t *host_k, uint16_t *host_v);
/* Same for tokens [first_token, first_token + token_count): host_k / host_v receive
 * [token_count][kv_heads*head_dim] rows (the layout a contiguous CPU cache uses). */
int nerva_hip_session_read_kv_range(NervaHipHfDecodeSequenceSession *session, uint32_t layer,
                                    uint32_t first_token, uint32_t token_count, uint16_t *host_k,
                                    uint16_t *host_v);

#ifdef __cplusplus
}
#endif
#endif /* NERVA_HIP_API_H_ */
