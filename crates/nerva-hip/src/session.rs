//! Safe wrappers over the decode-session entry points, with the shapes of nerva-cuda's
//! (crates/nerva-cuda/src/decode/hf_sequence/session/{request,stateful,summary}.rs): a config that
//! borrows the host weights and creates a session, a session that owns the device state and releases
//! it on drop, and a loop that starts a prompt and advances token by token. Failures never panic:
//! every call returns a summary whose `status` says Ok / Unavailable / Failed.
use std::ptr;

use crate::ffi::*;

pub const HIP_ERROR_NO_DEVICE: i32 = 100;
pub const DTYPE_F16: u32 = 0;
pub const DTYPE_BF16: u32 = 1;

/// crates/nerva-cuda/src/smoke/status.rs
#[derive(Copy, Clone, Debug, Eq, PartialEq)]
pub enum SmokeStatus {
    Ok,
    Unavailable,
    Failed,
}

impl SmokeStatus {
    pub fn from_native(status: i32, hip_error: i32) -> Self {
        if status == 0 {
            SmokeStatus::Ok
        } else if hip_error == HIP_ERROR_NO_DEVICE {
            SmokeStatus::Unavailable
        } else {
            SmokeStatus::Failed
        }
    }
}

pub fn device_smoke() -> (SmokeStatus, NervaHipDeviceSmokeResult) {
    let mut out: NervaHipDeviceSmokeResult = unsafe { std::mem::zeroed() };
    unsafe { nerva_hip_device_smoke(&mut out) };
    (SmokeStatus::from_native(out.status, out.hip_error), out)
}

/// Host weights of one dense decoder layer, row-major [out, in] 16-bit as a checkpoint stores them.
#[derive(Copy, Clone)]
pub struct HipHfDecodeChainLayer<'a> {
    pub rms_attn_weight: &'a [u16],
    pub rms_mlp_weight: &'a [u16],
    pub w_q: &'a [u16],
    pub w_k: &'a [u16],
    pub w_v: &'a [u16],
    pub w_o: &'a [u16],
    pub q_norm_weight: Option<&'a [u16]>,
    pub k_norm_weight: Option<&'a [u16]>,
    pub q_bias: Option<&'a [u16]>,
    pub k_bias: Option<&'a [u16]>,
    pub v_bias: Option<&'a [u16]>,
    pub o_bias: Option<&'a [u16]>,
    pub w_gate: &'a [u16],
    pub w_up: &'a [u16],
    pub w_down: &'a [u16],
}

fn opt_ptr(slice: Option<&[u16]>) -> *const u16 {
    slice.map_or(ptr::null(), <[u16]>::as_ptr)
}

impl HipHfDecodeChainLayer<'_> {
    fn native(&self) -> NervaHipHfDecodeChainLayer {
        let mut layer: NervaHipHfDecodeChainLayer = unsafe { std::mem::zeroed() };
        layer.rms_attn_weight = self.rms_attn_weight.as_ptr();
        layer.rms_mlp_weight = self.rms_mlp_weight.as_ptr();
        layer.w_q = self.w_q.as_ptr();
        layer.w_k = self.w_k.as_ptr();
        layer.w_v = self.w_v.as_ptr();
        layer.w_o = self.w_o.as_ptr();
        layer.q_norm_weight = opt_ptr(self.q_norm_weight);
        layer.k_norm_weight = opt_ptr(self.k_norm_weight);
        layer.q_bias = opt_ptr(self.q_bias);
        layer.k_bias = opt_ptr(self.k_bias);
        layer.v_bias = opt_ptr(self.v_bias);
        layer.o_bias = opt_ptr(self.o_bias);
        layer.w_gate = self.w_gate.as_ptr();
        layer.w_up = self.w_up.as_ptr();
        layer.w_down = self.w_down.as_ptr();
        layer
    }
}

pub struct HipHfDecodeSequenceSessionConfig<'a> {
    pub dtype: u32,
    pub hidden: usize,
    pub heads: usize,
    pub kv_heads: usize,
    pub head_dim: usize,
    pub intermediate: usize,
    pub vocab_size: usize,
    pub max_context_tokens: usize,
    pub rms_eps: f32,
    pub rope_theta: Option<f32>,
    pub embeddings: &'a [u16],
    pub layers: &'a [HipHfDecodeChainLayer<'a>],
    pub final_norm_weight: &'a [u16],
    pub lm_head: &'a [u16],
}

#[derive(Clone, Debug)]
pub struct HipHfDecodeSequenceSessionCreateSummary {
    pub status: SmokeStatus,
    pub hip_error: i32,
    pub failure_stage: i32,
    pub vocab_size: usize,
    pub max_context_tokens: usize,
    pub resident_weight_bytes: u64,
    pub resident_kv_bytes: u64,
    pub device_arena_bytes: u64,
    pub error: Option<&'static str>,
}

pub struct HipHfDecodeSequenceSessionCreateOutput {
    pub summary: HipHfDecodeSequenceSessionCreateSummary,
    pub session: Option<HipHfDecodeSequenceSession>,
}

impl HipHfDecodeSequenceSessionConfig<'_> {
    /// The argument checks nerva-cuda makes before it calls into native code (session/config.rs).
    pub fn validate(&self) -> Option<&'static str> {
        if self.dtype != DTYPE_F16 && self.dtype != DTYPE_BF16 {
            return Some("dtype must be f16 or bf16");
        }
        if self.hidden == 0 || self.heads == 0 || self.kv_heads == 0 || self.head_dim == 0 {
            return Some("model dimensions must be non-zero");
        }
        if self.intermediate == 0 || self.vocab_size == 0 || self.max_context_tokens == 0 || self.layers.is_empty() {
            return Some("model dimensions must be non-zero");
        }
        if self.heads % self.kv_heads != 0 {
            return Some("heads must be a multiple of kv_heads");
        }
        if self.embeddings.len() != self.vocab_size * self.hidden || self.lm_head.len() != self.vocab_size * self.hidden {
            return Some("embedding / lm_head size does not match vocab_size x hidden");
        }
        if self.final_norm_weight.len() != self.hidden {
            return Some("final norm size does not match hidden");
        }
        // every size crosses the boundary as u32, and the products below must not wrap either
        for value in [self.hidden, self.heads, self.kv_heads, self.head_dim, self.intermediate, self.vocab_size,
                      self.max_context_tokens, self.layers.len()] {
            if u32::try_from(value).is_err() {
                return Some("a model dimension does not fit 32 bits");
            }
        }
        let (Some(attention), Some(kv_hidden)) = (self.heads.checked_mul(self.head_dim), self.kv_heads.checked_mul(self.head_dim))
        else {
            return Some("heads x head_dim overflows");
        };
        // Native code reads every layer tensor at the size the dimensions imply, so each slice is checked here
        // (crates/nerva-cuda/src/decode/hf_chain/layer.rs:582,710-721, hf_step/request.rs:133-139): a short slice
        // must never reach the pointer cast.
        let size = |rows: usize, cols: usize| rows.checked_mul(cols);
        for layer in self.layers {
            let matrices = [(layer.w_q, size(attention, self.hidden)), (layer.w_k, size(kv_hidden, self.hidden)),
                            (layer.w_v, size(kv_hidden, self.hidden)), (layer.w_o, size(self.hidden, attention)),
                            (layer.w_gate, size(self.intermediate, self.hidden)),
                            (layer.w_up, size(self.intermediate, self.hidden)),
                            (layer.w_down, size(self.hidden, self.intermediate))];
            for (slice, want) in matrices {
                if want.map_or(true, |n| slice.len() != n) {
                    return Some("a layer matrix does not match the model dimensions");
                }
            }
            if layer.rms_attn_weight.len() != self.hidden || layer.rms_mlp_weight.len() != self.hidden {
                return Some("a layer norm weight does not match hidden");
            }
            let optional = [(layer.q_norm_weight, self.head_dim), (layer.k_norm_weight, self.head_dim),
                            (layer.q_bias, attention), (layer.k_bias, kv_hidden), (layer.v_bias, kv_hidden),
                            (layer.o_bias, self.hidden)];
            for (slice, want) in optional {
                if slice.map_or(false, |s| s.len() != want) {
                    return Some("an optional layer tensor does not match the model dimensions");
                }
            }
        }
        None
    }

    pub fn create(&self) -> HipHfDecodeSequenceSessionCreateOutput {
        let failed = |status: SmokeStatus, hip_error: i32, stage: i32, error: Option<&'static str>| {
            HipHfDecodeSequenceSessionCreateOutput {
                summary: HipHfDecodeSequenceSessionCreateSummary {
                    status,
                    hip_error,
                    failure_stage: stage,
                    vocab_size: self.vocab_size,
                    max_context_tokens: self.max_context_tokens,
                    resident_weight_bytes: 0,
                    resident_kv_bytes: 0,
                    device_arena_bytes: 0,
                    error,
                },
                session: None,
            }
        };
        if let Some(error) = self.validate() {
            return failed(SmokeStatus::Failed, 0, 0, Some(error));
        }
        let native_layers: Vec<NervaHipHfDecodeChainLayer> = self.layers.iter().map(|l| l.native()).collect();
        let mut request: NervaHipHfDecodeSequenceSessionCreateRequest = unsafe { std::mem::zeroed() };
        request.dtype = self.dtype;
        request.hidden = u32::try_from(self.hidden).unwrap_or(0); // validate() has checked the range
        request.heads = u32::try_from(self.heads).unwrap_or(0); // validate() has checked the range
        request.kv_heads = u32::try_from(self.kv_heads).unwrap_or(0); // validate() has checked the range
        request.head_dim = u32::try_from(self.head_dim).unwrap_or(0); // validate() has checked the range
        request.intermediate = u32::try_from(self.intermediate).unwrap_or(0); // validate() has checked the range
        request.vocab_size = u32::try_from(self.vocab_size).unwrap_or(0); // validate() has checked the range
        request.layer_count = u32::try_from(native_layers.len()).unwrap_or(0);
        request.max_context_tokens = u32::try_from(self.max_context_tokens).unwrap_or(0); // validate() has checked the range
        request.rms_eps = self.rms_eps;
        request.rope_theta = self.rope_theta.unwrap_or(0.0);
        request.embeddings = self.embeddings.as_ptr();
        request.layers = native_layers.as_ptr();
        request.final_norm_weight = self.final_norm_weight.as_ptr();
        request.lm_head = self.lm_head.as_ptr();
        let mut out: NervaHipHfDecodeSequenceSessionCreateResult = unsafe { std::mem::zeroed() };
        let mut handle: *mut NervaHipHfDecodeSequenceSession = ptr::null_mut();
        let rc = unsafe { nerva_hip_hf_decode_sequence_session_create(&request, &mut out, &mut handle) };
        let status = SmokeStatus::from_native(out.status, out.hip_error);
        if rc != 0 || status != SmokeStatus::Ok || handle.is_null() {
            return failed(if status == SmokeStatus::Ok { SmokeStatus::Failed } else { status }, out.hip_error, out.failure_stage, None);
        }
        let summary = HipHfDecodeSequenceSessionCreateSummary {
            status,
            hip_error: out.hip_error,
            failure_stage: out.failure_stage,
            vocab_size: out.vocab_size as usize,
            max_context_tokens: out.max_context_tokens as usize,
            resident_weight_bytes: out.resident_weight_bytes,
            resident_kv_bytes: out.resident_kv_bytes,
            device_arena_bytes: out.device_arena_bytes,
            error: None,
        };
        HipHfDecodeSequenceSessionCreateOutput {
            summary: summary.clone(),
            session: Some(HipHfDecodeSequenceSession { handle, create_summary: summary }),
        }
    }
}

/// Owns the device side of a session (weights, KV cache, captured step). Not `Send`: one host
/// thread drives a session, as with nerva-cuda's.
pub struct HipHfDecodeSequenceSession {
    handle: *mut NervaHipHfDecodeSequenceSession,
    create_summary: HipHfDecodeSequenceSessionCreateSummary,
}

impl HipHfDecodeSequenceSession {
    pub fn create_summary(&self) -> &HipHfDecodeSequenceSessionCreateSummary {
        &self.create_summary
    }
}

impl Drop for HipHfDecodeSequenceSession {
    fn drop(&mut self) {
        if !self.handle.is_null() {
            let mut out: NervaHipHfDecodeSequenceSessionCreateResult = unsafe { std::mem::zeroed() };
            unsafe { nerva_hip_hf_decode_sequence_session_destroy(self.handle, &mut out) };
            self.handle = ptr::null_mut();
        }
    }
}

#[derive(Clone, Debug)]
pub struct HipHfDecodeSequenceSummary {
    pub status: SmokeStatus,
    pub hip_error: i32,
    pub tokens: Vec<u32>,
    pub observed_token_hash: u64,
    pub kv_tokens: u64,
    pub graph_replays: u64,
    pub graph_nodes: u64,
    pub kernel_launches: u64,
    pub sync_calls: u64,
    pub host_causality_edges: u64,
    pub hot_path_allocations: u64,
    pub device_elapsed_ns: u64,
    pub error: Option<&'static str>,
}

fn summary_from(out: &NervaHipHfDecodeSequenceResult, tokens: Vec<u32>, error: Option<&'static str>) -> HipHfDecodeSequenceSummary {
    HipHfDecodeSequenceSummary {
        status: if error.is_some() { SmokeStatus::Failed } else { SmokeStatus::from_native(out.status, out.hip_error) },
        hip_error: out.hip_error,
        tokens,
        observed_token_hash: out.observed_token_hash,
        kv_tokens: out.kv_tokens,
        graph_replays: out.graph_replays,
        graph_nodes: out.graph_nodes,
        kernel_launches: out.kernel_launches,
        sync_calls: out.sync_calls,
        host_causality_edges: out.host_causality_edges,
        hot_path_allocations: out.hot_path_allocations,
        device_elapsed_ns: out.device_elapsed_ns,
        error,
    }
}

/// A prompt under way on a session: `start` prefills the prompt and samples the first token,
/// `advance` hands out the next tokens (crates/nerva-cuda/.../session/stateful.rs:27-153).
pub struct HipHfDecodeSequenceLoop<'a> {
    session: &'a mut HipHfDecodeSequenceSession,
    eos_token: Option<u32>,
    finished: bool,
}

impl<'a> HipHfDecodeSequenceLoop<'a> {
    /// Greedy sampling (an all-zero sampler configuration is greedy: sampler.cu:89, 422-433).
    pub fn start(
        session: &'a mut HipHfDecodeSequenceSession,
        prompt_tokens: &[u32],
        eos_token: Option<u32>,
    ) -> (HipHfDecodeSequenceSummary, Option<HipHfDecodeSequenceLoop<'a>>) {
        let empty: NervaHipHfDecodeSequenceResult = unsafe { std::mem::zeroed() };
        if prompt_tokens.is_empty() {
            return (summary_from(&empty, Vec::new(), Some("prompt must not be empty")), None);
        }
        let vocab = session.create_summary.vocab_size;
        if prompt_tokens.iter().any(|&t| t as usize >= vocab) {
            return (summary_from(&empty, Vec::new(), Some("prompt token outside the vocabulary")), None);
        }
        let Ok(prompt_token_count) = u32::try_from(prompt_tokens.len()) else {
            return (summary_from(&empty, Vec::new(), Some("prompt longer than 32 bits count")), None);
        };
        let mut request: NervaHipHfDecodeSequenceSessionStartRequest = unsafe { std::mem::zeroed() };
        request.session = session.handle;
        request.prompt_tokens = prompt_tokens.as_ptr();
        request.prompt_token_count = prompt_token_count;
        request.has_eos_token = eos_token.is_some() as u32;
        request.eos_token = eos_token.unwrap_or(0);
        let mut out: NervaHipHfDecodeSequenceResult = unsafe { std::mem::zeroed() };
        unsafe { nerva_hip_hf_decode_sequence_session_start(&request, &mut out) };
        let summary = summary_from(&out, Vec::new(), None);
        let loop_state = (summary.status == SmokeStatus::Ok).then_some(HipHfDecodeSequenceLoop {
            session,
            eos_token,
            finished: false,
        });
        (summary, loop_state)
    }

    pub fn finished(&self) -> bool {
        self.finished
    }

    /// Up to `steps` more tokens; fewer when the stop token shows up. Fails (status Failed, no
    /// tokens) past the session's context, like the native call.
    pub fn advance(&mut self, steps: usize) -> HipHfDecodeSequenceSummary {
        let empty: NervaHipHfDecodeSequenceResult = unsafe { std::mem::zeroed() };
        if self.finished {
            return summary_from(&empty, Vec::new(), Some("sequence already finished"));
        }
        if steps == 0 {
            return summary_from(&empty, Vec::new(), Some("steps must be non-zero"));
        }
        let Ok(step_count) = u32::try_from(steps) else {
            return summary_from(&empty, Vec::new(), Some("steps do not fit 32 bits"));
        };
        let mut tokens = vec![0u32; steps];
        let mut request: NervaHipHfDecodeSequenceSessionAdvanceRequest = unsafe { std::mem::zeroed() };
        request.session = self.session.handle;
        request.steps = step_count;
        request.output_tokens = tokens.as_mut_ptr();
        request.output_token_capacity = step_count;
        let mut out: NervaHipHfDecodeSequenceResult = unsafe { std::mem::zeroed() };
        unsafe { nerva_hip_hf_decode_sequence_session_advance(&request, &mut out) };
        tokens.truncate(out.observed_tokens as usize);
        let stopped = self.eos_token.is_some_and(|eos| tokens.last() == Some(&eos));
        let summary = summary_from(&out, tokens, None);
        self.finished = summary.status != SmokeStatus::Ok || stopped || (summary.tokens.len() < steps);
        summary
    }
}
