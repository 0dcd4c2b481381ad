//! The C ABI of libnerva_hip as Rust sees it. GENERATED from include/nerva_hip_api.h by
//! generate_ffi.py - edit the header and regenerate; tests/test_rust_mirror_cpu.py fails when
//! this file and the header disagree.
#![allow(non_camel_case_types, non_snake_case, dead_code)]

use std::os::raw::{c_char, c_int, c_void};

/// Opaque to callers: created by session_create, released by session_destroy.
#[repr(C)]
pub struct NervaHipHfDecodeSequenceSession {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipDeviceSmokeResult {
    pub status: i32,
    pub hip_error: i32,
    pub value: u32,
    pub device_count: i32,
    pub device_ordinal: i32,
    pub driver_version: i32,
    pub runtime_version: i32,
    pub compute_capability_major: i32,
    pub compute_capability_minor: i32,
    pub posix_fd_handle_supported: i32,
    pub vmm_posix_fd_export_verified: i32,
    pub gpu_direct_rdma_supported: i32,
    pub gpu_direct_rdma_with_cuda_vmm_supported: i32,
    pub total_global_mem: u64,
    pub free_global_mem: u64,
    pub gpu_name: [c_char; 128],
    pub pci_bus_id: [c_char; 32],
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipSyntheticTokenSlot {
    pub request_id: u32,
    pub sequence_id: u32,
    pub token_index: u64,
    pub token: u32,
    pub version: u64,
    pub completion: u32,
    pub host_copied: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeChainLayer {
    pub rms_attn_weight: *const u16,
    pub rms_mlp_weight: *const u16,
    pub w_q: *const u16,
    pub w_q_gate: *const u16,
    pub w_k: *const u16,
    pub q_norm_weight: *const u16,
    pub k_norm_weight: *const u16,
    pub w_v: *const u16,
    pub w_o: *const u16,
    pub q_bias: *const u16,
    pub k_bias: *const u16,
    pub v_bias: *const u16,
    pub o_bias: *const u16,
    pub w_gate: *const u16,
    pub w_up: *const u16,
    pub w_down: *const u16,
    pub w_router: *const u16,
    pub w_expert_gate_up: *const u16,
    pub w_expert_down: *const u16,
    pub w_shared_expert_gate: *const u16,
    pub w_shared_expert_up: *const u16,
    pub w_shared_expert_down: *const u16,
    pub w_shared_expert_router: *const u16,
    pub linear_key_heads: u32,
    pub linear_value_heads: u32,
    pub linear_key_head_dim: u32,
    pub linear_value_head_dim: u32,
    pub linear_conv_kernel: u32,
    pub w_linear_conv: *const u16,
    pub w_linear_qkv: *const u16,
    pub w_linear_z: *const u16,
    pub w_linear_b: *const u16,
    pub w_linear_a: *const u16,
    pub w_linear_dt_bias: *const u16,
    pub w_linear_a_log: *const f32,
    pub w_linear_norm: *const u16,
    pub w_linear_out: *const u16,
    pub mlp_kind: u32,
    pub moe_intermediate: u32,
    pub shared_expert_intermediate: u32,
    pub num_experts: u32,
    pub experts_per_token: u32,
    pub norm_topk_prob: u32,
    pub attention_kind: u32,
    pub deepseek_mode: u32,
    pub deepseek_flags: u32,
    pub deepseek_storage: u32,
    pub deepseek_hc_mult: u32,
    pub deepseek_hc_sinkhorn_iters: u32,
    pub deepseek_q_lora_rank: u32,
    pub deepseek_kv_lora_rank: u32,
    pub deepseek_o_lora_rank: u32,
    pub deepseek_o_groups: u32,
    pub deepseek_qk_nope_head_dim: u32,
    pub deepseek_qk_rope_head_dim: u32,
    pub deepseek_v_head_dim: u32,
    pub deepseek_compress_ratio: u32,
    pub deepseek_index_topk: u32,
    pub deepseek_index_n_heads: u32,
    pub deepseek_index_head_dim: u32,
    pub deepseek_router_num_groups: u32,
    pub deepseek_router_topk_groups: u32,
    pub deepseek_routed_scaling_factor: f32,
    pub deepseek_hc_eps: f32,
    pub deepseek_hc_post_alpha: f32,
    pub deepseek_rope_scaling_type: u32,
    pub deepseek_rope_original_max_position: u32,
    pub deepseek_rope_scaling_factor: f32,
    pub deepseek_rope_extrapolation_factor: f32,
    pub deepseek_rope_attn_factor: f32,
    pub deepseek_rope_beta_fast: f32,
    pub deepseek_rope_beta_slow: f32,
    pub deepseek_rope_mscale: f32,
    pub deepseek_rope_mscale_all_dim: f32,
    pub deepseek_compress_rope_theta: f32,
    pub deepseek_swiglu_limit: f32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceWeightBlock {
    pub host_source: *const u16,
    pub source_file: *const c_char,
    pub source_file_len: u64,
    pub file_offset_begin: u64,
    pub block_id: u64,
    pub block_version: u64,
    pub offset_bytes: u64,
    pub bytes: u64,
    pub strategy: u32,
    pub reserved: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSamplerConfig {
    pub temperature: f32,
    pub top_p: f32,
    pub top_k: u32,
    pub reserved: u32,
    pub seed: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceRequest {
    pub dtype: u32,
    pub hidden: u32,
    pub heads: u32,
    pub kv_heads: u32,
    pub head_dim: u32,
    pub intermediate: u32,
    pub vocab_size: u32,
    pub layer_count: u32,
    pub steps: u32,
    pub seed_token: u32,
    pub prompt_tokens: *const u32,
    pub prompt_token_count: u32,
    pub has_eos_token: u32,
    pub eos_token: u32,
    pub rms_eps: f32,
    pub rope_theta: f32,
    pub embeddings: *const u16,
    pub layers: *const NervaHipHfDecodeChainLayer,
    pub final_norm_weight: *const u16,
    pub lm_head: *const u16,
    pub planned_weight_blocks: u32,
    pub planned_gpu_resident_blocks: u32,
    pub planned_gpu_staged_blocks: u32,
    pub planned_weight_bytes: u64,
    pub planned_gpu_resident_weight_bytes: u64,
    pub planned_gpu_staged_weight_bytes: u64,
    pub planned_weight_descriptors: *const NervaHipHfDecodeSequenceWeightBlock,
    pub planned_weight_descriptor_count: u32,
    pub planned_weight_descriptor_hash: u64,
    pub output_tokens: *mut u32,
    pub output_token_capacity: u32,
    pub sampler: NervaHipHfDecodeSamplerConfig,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceResult {
    pub status: i32,
    pub hip_error: i32,
    pub device_count: i32,
    pub dtype: u32,
    pub hidden: u32,
    pub heads: u32,
    pub kv_heads: u32,
    pub head_dim: u32,
    pub intermediate: u32,
    pub vocab_size: u32,
    pub layer_count: u32,
    pub steps: u32,
    pub seed_token: u32,
    pub observed_tokens: u32,
    pub last_token: u32,
    pub observed_token_hash: u64,
    pub resident_weight_bytes: u64,
    pub planned_weight_blocks: u32,
    pub planned_gpu_resident_blocks: u32,
    pub planned_gpu_staged_blocks: u32,
    pub planned_weight_bytes: u64,
    pub planned_gpu_resident_weight_bytes: u64,
    pub planned_gpu_staged_weight_bytes: u64,
    pub descriptor_gpu_resident_h2d_bytes: u64,
    pub descriptor_gpu_staged_h2d_bytes: u64,
    pub planned_weight_descriptor_count: u32,
    pub planned_weight_descriptor_hash: u64,
    pub resident_kv_bytes: u64,
    pub deepseek_mhc_residual_bytes: u64,
    pub deepseek_mhc_post_mix_bytes: u64,
    pub deepseek_mhc_comb_mix_bytes: u64,
    pub kv_tokens: u64,
    pub device_arena_bytes: u64,
    pub pinned_host_bytes: u64,
    pub h2d_bytes: u64,
    pub d2h_bytes: u64,
    pub graph_replays: u64,
    pub graph_nodes: u64,
    pub graph_launches: u64,
    pub graph_captures: u64,
    pub graph_cache_hits: u64,
    pub kernel_launches: u64,
    pub experimental_rt_selector_launches: u64,
    pub experimental_rt_sparse_attention_active: u32,
    pub experimental_rt_dense_attention_chunks: u32,
    pub experimental_rt_attention_chunks: u32,
    pub experimental_rt_reserved: u32,
    pub device_elapsed_ns: u64,
    pub projection_ns: u64,
    pub qkv_projection_ns: u64,
    pub attention_output_projection_ns: u64,
    pub gate_up_projection_ns: u64,
    pub down_projection_ns: u64,
    pub lm_head_projection_ns: u64,
    pub attention_ns: u64,
    pub mlp_ns: u64,
    pub norm_ns: u64,
    pub sampling_ns: u64,
    pub sync_calls: u64,
    pub host_causality_edges: u64,
    pub hot_path_allocations: u64,
    pub deepseek_compressor_state_writes: u64,
    pub deepseek_compressed_kv_writes: u64,
    pub deepseek_indexer_state_writes: u64,
    pub deepseek_indexer_kv_writes: u64,
    pub deepseek_compressed_kv_attention_reads: u64,
    pub deepseek_compressed_kv_attention_slots_scanned: u64,
    pub deepseek_sparse_topk_selections: u64,
    pub deepseek_sparse_topk_slots_selected: u64,
    pub deepseek_sparse_topk_candidates_scored: u64,
    pub deepseek_sparse_topk_selection_hash: u64,
    pub deepseek_v3_grouped_router_selections: u64,
    pub deepseek_v4_bias_router_selections: u64,
    pub deepseek_v4_hash_router_selections: u64,
    pub deepseek_raw_attention_tokens_scanned: u64,
    pub deepseek_sparse_attention_output_hash: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceSessionCreateRequest {
    pub dtype: u32,
    pub hidden: u32,
    pub heads: u32,
    pub kv_heads: u32,
    pub head_dim: u32,
    pub intermediate: u32,
    pub vocab_size: u32,
    pub layer_count: u32,
    pub max_context_tokens: u32,
    pub rms_eps: f32,
    pub rope_theta: f32,
    pub embeddings: *const u16,
    pub layers: *const NervaHipHfDecodeChainLayer,
    pub final_norm_weight: *const u16,
    pub lm_head: *const u16,
    pub planned_weight_blocks: u32,
    pub planned_gpu_resident_blocks: u32,
    pub planned_gpu_staged_blocks: u32,
    pub planned_weight_bytes: u64,
    pub planned_gpu_resident_weight_bytes: u64,
    pub planned_gpu_staged_weight_bytes: u64,
    pub planned_weight_descriptors: *const NervaHipHfDecodeSequenceWeightBlock,
    pub planned_weight_descriptor_count: u32,
    pub planned_weight_descriptor_hash: u64,
    pub detailed_profile: u32,
    pub experimental_rt_decode: u32,
    pub experimental_rt_mode: u32,
    pub experimental_rt_page_tokens: u32,
    pub experimental_rt_pages: u32,
    pub experimental_rt_local_window_tokens: u32,
    pub experimental_rt_sink_tokens: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceSessionCreateResult {
    pub status: i32,
    pub hip_error: i32,
    pub failure_stage: i32,
    pub device_count: i32,
    pub dtype: u32,
    pub hidden: u32,
    pub heads: u32,
    pub kv_heads: u32,
    pub head_dim: u32,
    pub intermediate: u32,
    pub vocab_size: u32,
    pub layer_count: u32,
    pub max_context_tokens: u32,
    pub prefill_chunk_tokens: u32,
    pub head_threads: u32,
    pub resident_weight_bytes: u64,
    pub planned_weight_blocks: u32,
    pub planned_gpu_resident_blocks: u32,
    pub planned_gpu_staged_blocks: u32,
    pub planned_weight_bytes: u64,
    pub planned_gpu_resident_weight_bytes: u64,
    pub planned_gpu_staged_weight_bytes: u64,
    pub descriptor_gpu_resident_h2d_bytes: u64,
    pub descriptor_gpu_staged_h2d_bytes: u64,
    pub planned_weight_descriptor_count: u32,
    pub planned_weight_descriptor_hash: u64,
    pub experimental_rt_decode_requested: u32,
    pub experimental_rt_decode_enabled: u32,
    pub experimental_rt_mode: u32,
    pub experimental_rt_page_tokens: u32,
    pub experimental_rt_pages: u32,
    pub experimental_rt_local_window_tokens: u32,
    pub experimental_rt_sink_tokens: u32,
    pub deepseek_v4_attention_aux_streams: u32,
    pub deepseek_v4_attention_events: u32,
    pub deepseek_v4_swa_kv_bytes: u64,
    pub deepseek_mhc_residual_bytes: u64,
    pub deepseek_mhc_post_mix_bytes: u64,
    pub deepseek_mhc_comb_mix_bytes: u64,
    pub resident_kv_bytes: u64,
    pub device_arena_bytes: u64,
    pub pinned_host_bytes: u64,
    pub h2d_bytes: u64,
    pub sync_calls: u64,
    pub hot_path_allocations: u64,
    pub device_memory_bandwidth_bps: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceSessionRunRequest {
    pub session: *mut NervaHipHfDecodeSequenceSession,
    pub steps: u32,
    pub seed_token: u32,
    pub prompt_tokens: *const u32,
    pub prompt_token_count: u32,
    pub has_eos_token: u32,
    pub eos_token: u32,
    pub output_tokens: *mut u32,
    pub output_token_capacity: u32,
    pub sampler: NervaHipHfDecodeSamplerConfig,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceSessionStartRequest {
    pub session: *mut NervaHipHfDecodeSequenceSession,
    pub prompt_tokens: *const u32,
    pub prompt_token_count: u32,
    pub has_eos_token: u32,
    pub eos_token: u32,
    pub sampler: NervaHipHfDecodeSamplerConfig,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceSessionAdvanceRequest {
    pub session: *mut NervaHipHfDecodeSequenceSession,
    pub steps: u32,
    pub output_tokens: *mut u32,
    pub output_token_capacity: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest {
    pub parent: *mut NervaHipHfDecodeSequenceSession,
    pub detailed_profile: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceBatchAdvanceRequest {
    pub sessions: *mut *mut NervaHipHfDecodeSequenceSession,
    pub session_count: u32,
    pub target_block_tokens: u32,
    pub min_block_tokens: u32,
    pub output_tokens: *mut u32,
    pub output_token_capacity: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipHfDecodeSequenceBatchAdvanceResult {
    pub status: i32,
    pub hip_error: i32,
    pub device_count: i32,
    pub reason: u32,
    pub exact: u32,
    pub requested_session_count: u32,
    pub eligible_session_count: u32,
    pub block_tokens: u32,
    pub target_block_tokens: u32,
    pub min_block_tokens: u32,
    pub dtype: u32,
    pub layer_count: u32,
    pub observed_tokens: u32,
    pub last_token: u32,
    pub observed_token_hash: u64,
    pub d2h_bytes: u64,
    pub projection_elapsed_ns: u64,
    pub qkv_elapsed_ns: u64,
    pub attention_output_elapsed_ns: u64,
    pub gate_up_elapsed_ns: u64,
    pub down_elapsed_ns: u64,
    pub lm_head_elapsed_ns: u64,
    pub pack_kernel_launches: u64,
    pub projection_kernel_launches: u64,
    pub scatter_kernel_launches: u64,
    pub dependency_kernel_launches: u64,
    pub experimental_rt_selector_launches: u64,
    pub sampling_kernel_launches: u64,
    pub sync_calls: u64,
    pub hot_path_allocations: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipDeepSeekQuantDequantResult {
    pub status: i32,
    pub hip_error: i32,
    pub device_count: i32,
    pub rows: u32,
    pub cols: u32,
    pub block_rows: u32,
    pub block_cols: u32,
    pub output_hash: u64,
    pub device_arena_bytes: u64,
    pub pinned_host_bytes: u64,
    pub h2d_bytes: u64,
    pub d2h_bytes: u64,
    pub kernel_launches: u64,
    pub sync_calls: u64,
    pub hot_path_allocations: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest {
    pub rows: u32,
    pub cols: u32,
    pub block_rows: u32,
    pub block_cols: u32,
    pub input_dtype: u32,
    pub weights: *const u8,
    pub scales: *const f32,
    pub input: *const u16,
    pub output: *mut f32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest {
    pub rows: u32,
    pub cols: u32,
    pub tokens: u32,
    pub block_rows: u32,
    pub block_cols: u32,
    pub input_dtype: u32,
    pub weights: *const u8,
    pub scales: *const f32,
    pub input: *const u16,
    pub output: *mut f32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipProjectionBenchRequest {
    pub dtype: u32,
    pub rows: u32,
    pub cols: u32,
    pub iterations: u32,
    pub warmup_iterations: u32,
    pub block_tokens: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipProjectionBenchResult {
    pub status: i32,
    pub hip_error: i32,
    pub device_count: i32,
    pub device_ordinal: i32,
    pub compute_capability_major: i32,
    pub compute_capability_minor: i32,
    pub dtype: u32,
    pub rows: u32,
    pub cols: u32,
    pub block_tokens: u32,
    pub iterations: u32,
    pub warmup_iterations: u32,
    pub matrix_bytes: u64,
    pub input_bytes: u64,
    pub output_bytes: u64,
    pub cublaslt_total_ns: u64,
    pub cublaslt_avg_ns: u64,
    pub cublaslt_default_total_ns: u64,
    pub cublaslt_default_avg_ns: u64,
    pub cublaslt_heuristic_count: u32,
    pub cublaslt_best_heuristic_index: u32,
    pub cublaslt_best_heuristic_total_ns: u64,
    pub cublaslt_best_heuristic_avg_ns: u64,
    pub custom_total_ns: u64,
    pub custom_avg_ns: u64,
    pub cublaslt_graph_total_ns: u64,
    pub cublaslt_graph_avg_ns: u64,
    pub cublaslt_default_graph_total_ns: u64,
    pub cublaslt_default_graph_avg_ns: u64,
    pub cublaslt_best_heuristic_graph_total_ns: u64,
    pub cublaslt_best_heuristic_graph_avg_ns: u64,
    pub custom_graph_total_ns: u64,
    pub custom_graph_avg_ns: u64,
    pub cublaslt_graph_nodes: u64,
    pub custom_graph_nodes: u64,
    pub graph_replays: u64,
    pub graph_captures: u64,
    pub selected_graph_strategy: u32,
    pub cublaslt_effective_bandwidth_bps: u64,
    pub custom_effective_bandwidth_bps: u64,
    pub selected_strategy: u32,
    pub mismatch_count: u32,
    pub max_abs_diff: f32,
    pub kernel_launches: u64,
    pub sync_calls: u64,
    pub device_allocations: u64,
    pub device_frees: u64,
    pub device_arena_bytes: u64,
    pub hot_path_allocations: u64,
    pub block_cublaslt_total_ns: u64,
    pub block_cublaslt_avg_ns: u64,
    pub block_cublaslt_per_token_ns: u64,
    pub block_cublaslt_graph_total_ns: u64,
    pub block_cublaslt_graph_avg_ns: u64,
    pub block_cublaslt_graph_per_token_ns: u64,
    pub block_cublaslt_graph_nodes: u64,
    pub block_cublaslt_speedup_x1000: u64,
    pub block_cublaslt_graph_speedup_x1000: u64,
    pub block_cublaslt_effective_bandwidth_bps: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipDeepSeekMoeForwardRequest {
    pub hidden_size: u32,
    pub intermediate_size: u32,
    pub num_experts: u32,
    pub top_k: u32,
    pub clamp_swiglu: u32,
    pub swiglu_limit: f32,
    pub input: *const f32,
    pub expert_ids: *const u32,
    pub expert_weights: *const f32,
    pub w_gate: *const f32,
    pub w_up: *const f32,
    pub w_down: *const f32,
    pub output: *mut f32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipDeepSeekMoeForwardResult {
    pub status: i32,
    pub hip_error: i32,
    pub device_count: i32,
    pub moe_error: i32,
    pub hidden_size: u32,
    pub intermediate_size: u32,
    pub num_experts: u32,
    pub top_k: u32,
    pub clamp_swiglu: u32,
    pub swiglu_limit: f32,
    pub output_hash: u64,
    pub device_arena_bytes: u64,
    pub pinned_host_bytes: u64,
    pub h2d_bytes: u64,
    pub d2h_bytes: u64,
    pub kernel_launches: u64,
    pub sync_calls: u64,
    pub hot_path_allocations: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipGemvRequest {
    pub dtype: u32,
    pub rows: u32,
    pub cols: u32,
    pub prologue: u32,
    pub epilogue: u32,
    pub round_output: u32,
    pub rms_eps: f32,
    pub pair_gap: u32,
    pub weights: *const u16,
    pub input16: *const u16,
    pub input_f32: *const f32,
    pub gamma: *const u16,
    pub bias: *const u16,
    pub residual: *const f32,
    pub output_f32: *mut f32,
    pub output16: *mut u16,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipFp8GemvRequest {
    pub rows: u32,
    pub cols: u32,
    pub block_rows: u32,
    pub block_cols: u32,
    pub input_dtype: u32,
    pub weights: *const u8,
    pub scales: *const f32,
    pub input16: *const u16,
    pub input_f32: *const f32,
    pub output: *mut f32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipPagedAttentionRequest {
    pub dtype: u32,
    pub heads: u32,
    pub kv_heads: u32,
    pub head_dim: u32,
    pub layer: u32,
    pub block_count: u32,
    pub position: u32,
    pub append: u32,
    pub rms_eps: f32,
    pub rope_theta: f32,
    pub qkv_f32: *const f32,
    pub q_norm: *const u16,
    pub k_norm: *const u16,
    pub q_bias: *const u16,
    pub k_bias: *const u16,
    pub v_bias: *const u16,
    pub k_cache: *mut u16,
    pub v_cache: *mut u16,
    pub block_table: *const u32,
    pub workspace: *mut c_void,
    pub output_f32: *mut f32,
    pub output16: *mut u16,
    pub splits: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipArgmaxRequest {
    pub count: u32,
    pub logits: *const f32,
    pub token: *mut u32,
    pub workspace: *mut c_void,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipGemmRowsRequest {
    pub dtype: u32,
    pub rows: u32,
    pub cols: u32,
    pub tokens: u32,
    pub epilogue: u32,
    pub round_output: u32,
    pub weights: *const u16,
    pub input16: *const u16,
    pub bias: *const u16,
    pub residual: *const f32,
    pub output_f32: *mut f32,
    pub output16: *mut u16,
    pub input_operand_order: u32,
    pub output16_operand_order: u32,
    pub workspace: *mut c_void,
    pub workspace_bytes: u64,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipSampleRequest {
    pub vocab: u32,
    pub position: u32,
    pub logits: *const f32,
    pub sampler: NervaHipHfDecodeSamplerConfig,
    pub token: *mut u32,
    pub workspace: *mut c_void,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipMoeFp8Request {
    pub hidden: u32,
    pub intermediate: u32,
    pub num_experts: u32,
    pub top_k: u32,
    pub block: u32,
    pub input_dtype: u32,
    pub shared_index: i32,
    pub input16: *const u16,
    pub expert_ids: *const u32,
    pub expert_weights: *const f32,
    pub w_gate: *const u8,
    pub w_up: *const u8,
    pub s_gate: *const f32,
    pub s_up: *const f32,
    pub w_down: *const u8,
    pub s_down: *const f32,
    pub activation: *mut f32,
    pub output: *mut f32,
    pub phases: u32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipMoeRouteRequest {
    pub num_experts: u32,
    pub top_k: u32,
    pub normalize: u32,
    pub logits: *const f32,
    pub expert_ids: *mut u32,
    pub expert_weights: *mut f32,
}

#[repr(C)]
#[derive(Copy, Clone)]
pub struct NervaHipStepProfile {
    pub status: i32,
    pub hip_error: i32,
    pub position: u32,
    pub launches: u32,
    pub embed_ns: u64,
    pub qkv_ns: u64,
    pub attention_ns: u64,
    pub o_ns: u64,
    pub gate_up_ns: u64,
    pub down_ns: u64,
    pub lm_head_ns: u64,
    pub total_ns: u64,
    pub qkv_bytes: u64,
    pub attention_bytes: u64,
    pub o_bytes: u64,
    pub gate_up_bytes: u64,
    pub down_bytes: u64,
    pub lm_head_bytes: u64,
    pub qkv_stream_ns: u64,
    pub attention_stream_ns: u64,
    pub o_stream_ns: u64,
    pub gate_up_stream_ns: u64,
    pub down_stream_ns: u64,
}

unsafe extern "C" {
    pub fn nerva_hip_device_smoke(out: *mut NervaHipDeviceSmokeResult) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_u16(request: *const NervaHipHfDecodeSequenceRequest, out: *mut NervaHipHfDecodeSequenceResult) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_session_create(request: *const NervaHipHfDecodeSequenceSessionCreateRequest, out: *mut NervaHipHfDecodeSequenceSessionCreateResult, session: *mut *mut NervaHipHfDecodeSequenceSession) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_session_run(request: *const NervaHipHfDecodeSequenceSessionRunRequest, out: *mut NervaHipHfDecodeSequenceResult) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_session_start(request: *const NervaHipHfDecodeSequenceSessionStartRequest, out: *mut NervaHipHfDecodeSequenceResult) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_session_advance(request: *const NervaHipHfDecodeSequenceSessionAdvanceRequest, out: *mut NervaHipHfDecodeSequenceResult) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_session_destroy(session: *mut NervaHipHfDecodeSequenceSession, out: *mut NervaHipHfDecodeSequenceSessionCreateResult) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_session_fork_shared_weights(request: *const NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest, out: *mut NervaHipHfDecodeSequenceSessionCreateResult, session: *mut *mut NervaHipHfDecodeSequenceSession) -> c_int;
    pub fn nerva_hip_hf_decode_sequence_batch_advance_one(request: *const NervaHipHfDecodeSequenceBatchAdvanceRequest, out: *mut NervaHipHfDecodeSequenceBatchAdvanceResult) -> c_int;
    pub fn nerva_hip_deepseek_quant_fp8_f32_scale_encoded_matvec(request: *const NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest, out: *mut NervaHipDeepSeekQuantDequantResult) -> c_int;
    pub fn nerva_hip_deepseek_quant_fp8_f32_scale_encoded_gemm_tokens(request: *const NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest, out: *mut NervaHipDeepSeekQuantDequantResult) -> c_int;
    pub fn nerva_hip_projection_bench(request: *const NervaHipProjectionBenchRequest, out: *mut NervaHipProjectionBenchResult) -> c_int;
    pub fn nerva_hip_deepseek_moe_forward(request: *const NervaHipDeepSeekMoeForwardRequest, out: *mut NervaHipDeepSeekMoeForwardResult) -> c_int;
    pub fn nerva_hip_gemv(request: *const NervaHipGemvRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_gemv_launch_shape(prologue: u32, epilogue: u32, rows: u32, cols: u32, kernel: *mut u32, workgroups: *mut u32) -> c_int;
    pub fn nerva_hip_fp8_gemv(request: *const NervaHipFp8GemvRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_paged_gqa_decode(request: *const NervaHipPagedAttentionRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_paged_attention_workspace_bytes(heads: u32, head_dim: u32) -> u64;
    pub fn nerva_hip_paged_attention_max_splits(kv_heads: u32) -> u64;
    pub fn nerva_hip_paged_attention_status(workspace: *mut c_void, heads: u32, head_dim: u32, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_kv_cache_offset(block_count: u32, kv_heads: u32, head_dim: u32, layer: u32, physical_block: u32, kv_head: u32, token_in_block: u32, dim: u32, is_value: u32) -> u64;
    pub fn nerva_hip_argmax(request: *const NervaHipArgmaxRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_argmax_workspace_bytes() -> u64;
    pub fn nerva_hip_argmax_static(logits: *const f32, count: u32, token: *mut u32, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_gemm_rows(request: *const NervaHipGemmRowsRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_gemm_rows_workspace_bytes(rows: u32) -> u64;
    pub fn nerva_hip_gemm_operand_index(tokens: u32, token: u32, column: u32) -> u64;
    pub fn nerva_hip_rmsnorm_rows(dtype: u32, x: *const f32, gamma: *const u16, eps: f32, tokens: u32, cols: u32, out16: *mut u16, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_sample(request: *const NervaHipSampleRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_sample_workspace_bytes(vocab: u32) -> u64;
    pub fn nerva_hip_moe_fp8_experts(request: *const NervaHipMoeFp8Request, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_moe_route_softmax(request: *const NervaHipMoeRouteRequest, stream: *mut c_void, hip_error: *mut i32) -> c_int;
    pub fn nerva_hip_malloc(device_ptr: *mut *mut c_void, bytes: u64) -> c_int;
    pub fn nerva_hip_free(device_ptr: *mut c_void) -> c_int;
    pub fn nerva_hip_memcpy_h2d(device_dst: *mut c_void, host_src: *const c_void, bytes: u64) -> c_int;
    pub fn nerva_hip_memcpy_d2h(host_dst: *mut c_void, device_src: *const c_void, bytes: u64) -> c_int;
    pub fn nerva_hip_memset(device_dst: *mut c_void, value: c_int, bytes: u64) -> c_int;
    pub fn nerva_hip_stream_synchronize(stream: *mut c_void) -> c_int;
    pub fn nerva_hip_allocation_count() -> u64;
    pub fn nerva_hip_timer_capture_begin() -> c_int;
    pub fn nerva_hip_timer_capture_end(warmup_replays: u32, timed_replays: u32, nodes: *mut u64, avg_replay_ns: *mut f64) -> c_int;
    pub fn nerva_hip_timer_capture_end_stats(warmup_replays: u32, timed_replays: u32, nodes: *mut u64, avg_replay_ns: *mut f64, min_replay_ns: *mut f64, median_replay_ns: *mut f64) -> c_int;
    pub fn nerva_hip_copy_d2d(device_dst: *mut c_void, device_src: *const c_void, bytes: u64, stream: *mut c_void) -> c_int;
    pub fn nerva_hip_synth_fill_16(device_dst: *mut c_void, dtype: u32, seed: u64, tensor_id: u64, count: u64, mean: f32, std: f32) -> c_int;
    pub fn nerva_hip_synth_fill_f32(device_dst: *mut c_void, seed: u64, tensor_id: u64, count: u64, mean: f32, std: f32) -> c_int;
    pub fn nerva_hip_synth_fill_fp8_block(device_weights: *mut c_void, device_scales: *mut c_void, seed: u64, tensor_id: u64, rows: u64, cols: u64, block: u64, std: f32) -> c_int;
    pub fn nerva_hip_bench_session_create_synthetic(request: *const NervaHipHfDecodeSequenceSessionCreateRequest, seed: u64, weight_std: f32, with_qk_norm: u32, out: *mut NervaHipHfDecodeSequenceSessionCreateResult, session: *mut *mut NervaHipHfDecodeSequenceSession) -> c_int;
    pub fn nerva_hip_session_profile_step(session: *mut NervaHipHfDecodeSequenceSession, repeats: u32, out: *mut NervaHipStepProfile) -> c_int;
    pub fn nerva_hip_test_set_tuning(name: *const c_char, value: i32) -> c_int;
    pub fn nerva_hip_steps_are_eager() -> c_int;
    pub fn nerva_hip_session_shares_weight_stream(session: *mut NervaHipHfDecodeSequenceSession) -> c_int;
    pub fn nerva_hip_session_read_logits(session: *mut NervaHipHfDecodeSequenceSession, host_logits: *mut f32) -> c_int;
    pub fn nerva_hip_session_read_slots(session: *mut NervaHipHfDecodeSequenceSession, first: u32, count: u32, host_slots: *mut NervaHipSyntheticTokenSlot) -> c_int;
    pub fn nerva_hip_session_step_trace_bytes(session: *mut NervaHipHfDecodeSequenceSession) -> u64;
    pub fn nerva_hip_session_trace_next_step(session: *mut NervaHipHfDecodeSequenceSession, device_buffer: *mut c_void, bytes: u64) -> c_int;
    pub fn nerva_hip_session_read_kv(session: *mut NervaHipHfDecodeSequenceSession, layer: u32, token: u32, host_k: *mut u16, host_v: *mut u16) -> c_int;
    pub fn nerva_hip_session_read_kv_range(session: *mut NervaHipHfDecodeSequenceSession, layer: u32, first_token: u32, token_count: u32, host_k: *mut u16, host_v: *mut u16) -> c_int;
}
