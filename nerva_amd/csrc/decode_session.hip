// Decode session: one static device arena, weights resident, paged KV cache,
// the whole decode step captured once as a hipGraph and replayed per token.
// Replaces the reference's session object and lifecycle entry points
// (native/cuda/hf_decode_sequence/session_api_lifecycle.inc.cu:1-1311,
// session_decode_prefill.inc.cu:74-372, session_graph_result.inc.cu:87-209).
//
// One decode step is 3 + 5*layers launches, with no host round trip:
//   embed               x = f32(emb[token]); token = prompt[pos] or slots[pos-1].token
//   per layer
//     qkv   GEMV  [rmsnorm(x, g_attn) prologue]                  -> qkv f32
//     attn  q/k norm + RoPE + KV append + split-KV attention      -> attn 16-bit
//     o     GEMV  [+ o_bias + x epilogue]                         -> r f32
//     gate_up GEMV [rmsnorm(r, g_mlp) prologue, silu(g)*u epilogue] -> ff 16-bit
//     down  GEMV  [+ r epilogue]                                  -> x f32
//   lm_head GEMV [rmsnorm(x, g_final) prologue, per-workgroup argmax epilogue]
//   sample finish (one workgroup)                                  -> slot[pos], cursor = pos+1
// Every kernel reads the position from device memory, so one captured graph
// serves every position and every prompt length.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <unistd.h>

#include <algorithm>
#include <string>
#include <atomic>
#include <vector>

#include "argmax.cuh"
#include "attn_decode.cuh"
#include "gemm_rows.cuh"
#include "sampler.cuh"
#include "gemv_stream.cuh"
#include "runtime_state.hpp"
#include "synth_fill.cuh"

using namespace nv;

namespace {

using Slot = NervaHipSyntheticTokenSlot;

struct LayerDev {
  const uint16_t *rms_attn, *rms_mlp, *wqkv, *q_norm, *k_norm, *q_bias, *k_bias, *v_bias, *wo, *o_bias,
      *wgu, *wdown;
};

enum StepMode { kDecodeStep = 0, kPromptStep = 1, kPromptHeadStep = 2 };
enum LaunchKind { kLEmbed = 0, kLQkv, kLAttn, kLO, kLGateUp, kLDown, kLHead, kLAdvance, kLKinds };

// The weight arena of a session and of every session forked from it (one stream of the weights can
// then serve a token row of each of them); freed by the last of them to go.
struct SharedWeights {
  char *origin = nullptr;  // what the allocator returned (and takes back)
  char *base = nullptr;    // the first kMatrixAlign boundary in it: offsets of the weight layout count from here
  uint64_t bytes = 0;
  std::atomic<uint32_t> refs{1};
};

// What a batch step needs to know of each of its sequences, in device memory: the cache and position
// for the attention launches, the token slots for the embedding.
struct BatchTable {
  AttnSeq seq[kGemmMaxTokens];
  const Slot *slots[kGemmMaxTokens];
  SamplerParams sample[kGemmMaxTokens];
};

struct StepProfiler {
  hipStream_t stream;
  std::vector<hipEvent_t> events;  // pairs
  std::vector<int> kinds;
  size_t used = 0;
  hipError_t before(int kind) {
    if (used + 2 > events.size()) {
      for (int i = 0; i < 2; ++i) {
        hipEvent_t e;
        hipError_t err = hipEventCreate(&e);
        if (err != hipSuccess) return err;
        events.push_back(e);
      }
    }
    kinds.push_back(kind);
    return hipEventRecord(events[used], stream);
  }
  hipError_t after() {
    hipError_t err = hipEventRecord(events[used + 1], stream);
    used += 2;
    return err;
  }
  ~StepProfiler() {
    for (hipEvent_t e : events) (void)hipEventDestroy(e);
  }
};

}  // namespace

struct NervaHipHfDecodeSequenceSession {
  uint32_t dtype = 0, hidden = 0, heads = 0, kv_heads = 0, head_dim = 0, intermediate = 0, vocab = 0,
           layers = 0, max_ctx = 0;
  float eps = 0.0f, theta = 0.0f;
  hipStream_t stream = nullptr;
  SharedWeights *weights = nullptr;  // shared with forks
  char *arena = nullptr;             // everything but the weights: KV cache, sequence state, activations, workspaces
  uint32_t pair_gap = 0;             // elements between a layer's gate rows and its up rows (see kPairGapElems)
  bool arena_in_weights = false;     // `arena` lies behind the weights in their allocation (the creating session)
  uint64_t state_bytes = 0;          // size of `arena`
  uint64_t arena_bytes = 0;          // weights + state, as reported to the caller
  char *pinned = nullptr;
  uint64_t pinned_bytes = 0;
  std::vector<LayerDev> layer;
  const uint16_t *emb = nullptr, *final_norm = nullptr, *lm_head = nullptr;
  uint16_t *kc = nullptr, *vc = nullptr;
  uint32_t block_count = 0;
  uint32_t *table = nullptr, *prompt = nullptr;
  uint32_t *state = nullptr;  // state[0] cursor, state[1] prompt count, state[2] steps executed so far,
                              // state[3] fault word (set by a kernel whose bounded wait gave up; cleared by start)
  Slot *slots = nullptr;
  float *x = nullptr, *r = nullptr, *qkv = nullptr, *logits = nullptr, *rope_freq = nullptr, *rope_cs = nullptr;
  uint16_t *attn16 = nullptr, *ff16 = nullptr;
  void *attn_ws = nullptr, *sample_ws = nullptr;
  uint32_t attn_splits = 1;
  uint32_t attn_single_blocks = 0;   // contexts of up to this many blocks go to one split (0 with a forced split factor)
  uint64_t *attn_tagged = nullptr;   // tagged split partials of the decode step kernel
  uint32_t *attn_plan = nullptr;     // this step's split plan of the decode attention (attn_plan_fill), or null
  uint64_t *attn_trace = nullptr;  // NERVA_HIP_ATTN_TRACE=1: per-layer stage timestamps of selected attention workgroups
  Slot *host_slots = nullptr;
  uint32_t *host_prompt = nullptr;
  uint32_t *host_state = nullptr;
  // captured steps: 0 decode step with the greedy finish, 1 prompt step, 2 decode step with the
  // temperature / top-k / top-p sampler (its parameters live in device memory, so one capture
  // serves every such configuration)
  hipGraph_t graph[3] = {nullptr, nullptr, nullptr};
  hipGraphExec_t exec[3] = {nullptr, nullptr, nullptr};
  uint64_t graph_nodes[3] = {0, 0, 0};
  // prompt blocks: up to prefill_block_tokens prompt tokens per pass through the layers (weights streamed
  // once per block on the matrix cores); false = one prompt step per token
  bool block_prefill = false;
  // the multi-row kernels take this model's shapes (prompt blocks and batch steps need it)
  bool rows_ready = false;
  float *blogits = nullptr;          // [NERVA_HIP_BATCH_MAX_BLOCK_TOKENS][vocab] logits of a batch step
  BatchTable *btable = nullptr, *host_btable = nullptr;
  Slot *bslots = nullptr, *host_bslots = nullptr;   // a batch step's published slots, gathered for one copy
  float *px = nullptr, *pr = nullptr, *pqkv = nullptr, *prope = nullptr;
  uint16_t *pxn16 = nullptr, *pattn16 = nullptr, *pff16 = nullptr;
  char *pattn_ws = nullptr;
  uint64_t pattn_ws_stride = 0;
  char *pgemm_ws = nullptr;        // partial sums of the K-sliced projections of a prompt block
  uint64_t pgemm_ws_bytes = 0;
  uint32_t prefill_block_tokens = kGemmMaxTokens;   // tokens per prompt block: 512 or 256 where every projection has the kernel for it
  SamplerDev sampler{};            // normalised configuration of the active sequence
  SamplerDev *sampler_dev = nullptr;
  uint64_t *sampler_keys = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  // test hook: the next decode step is launched kernel by kernel and every intermediate vector is
  // copied behind the previous one into this caller-owned device buffer (step_trace_bytes)
  char *trace_buf = nullptr;
  uint64_t trace_used = 0;
  // echo of the caller's weight plan
  uint32_t planned_weight_blocks = 0, planned_gpu_resident_blocks = 0, planned_gpu_staged_blocks = 0,
           planned_weight_descriptor_count = 0;
  uint64_t planned_weight_bytes = 0, planned_gpu_resident_weight_bytes = 0,
           planned_gpu_staged_weight_bytes = 0, planned_weight_descriptor_hash = 0;
  uint64_t resident_weight_bytes = 0, kv_bytes = 0;
  // active sequence
  bool started = false, finished = false;
  uint32_t prompt_count = 0, observed = 0, cursor = 0, seed_token = 0, has_eos = 0, eos = 0;
};

using Session = NervaHipHfDecodeSequenceSession;

namespace {

template <uint32_t DT>
__global__ __launch_bounds__(kBlock) void embed_kernel(const uint16_t *emb, const uint32_t *prompt,
                                                       const Slot *slots, uint32_t *state,
                                                       uint32_t max_steps, uint32_t hidden,
                                                       uint32_t vocab, float *x, const float *rope_freq,
                                                       float *rope_cs, uint32_t half_dim, uint32_t *attn_plan,
                                                       const uint32_t *table, uint32_t attn_splits,
                                                       uint32_t attn_single_blocks) {
  const uint32_t pos = state[0];
  // the position goes into the attention plan even past the last step: the attention launches take
  // their step guard from there
  if (attn_plan != nullptr && blockIdx.x == 0 && threadIdx.x == 0) attn_plan[0] = pos;
  if (pos >= max_steps) return;
  // this step's split plan of the decode attention, once for all layers
  if (attn_plan != nullptr && blockIdx.x == 0)
    for (uint32_t e = threadIdx.x; e < attn_splits * kAttnPlanWaves; e += kBlock)
      attn_plan_fill(attn_plan, table, pos, attn_splits, attn_single_blocks, e, state[2] + 1u);  // (entry 0 = the thread that counts)
  // steps executed so far: the tags of the attention's split partials derive from it (through the plan; nobody
  // else reads it in this launch, and only the thread that writes it uses what it read above)
  if (blockIdx.x == 0 && threadIdx.x == 0) state[2] = state[2] + 1u;
  // this step's RoPE angles, once: cos at [i], sin at [half_dim + i] (f32 angle = pos / theta^(2i/d))
  if (rope_freq != nullptr && blockIdx.x == 0) {
    for (uint32_t i = threadIdx.x; i < half_dim; i += kBlock) {
      float sn, cs;
      sincosf(static_cast<float>(pos) / rope_freq[i], &sn, &cs);
      rope_cs[i] = cs;
      rope_cs[half_dim + i] = sn;
    }
  }
  uint32_t token = pos < state[1] ? prompt[pos] : slots[pos - 1].token;
  if (token >= vocab) token = 0;  // prompts are validated on the host; sampled ids are < vocab
  const uint16_t *row = emb + static_cast<uint64_t>(token) * hidden;
  for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < hidden; i += gridDim.x * kBlock)
    x[i] = dec16<DT>(row[i]);
}

// Prompt block: embedding rows and rotation tables of positions first .. first + gridDim.x - 1.
template <uint32_t DT>
__global__ __launch_bounds__(kBlock) void embed_rows_kernel(const uint16_t *emb, const uint32_t *prompt, uint32_t first,
                                                            uint32_t hidden, uint32_t vocab, float *x,
                                                            const float *rope_freq, float *rope_cs, uint32_t half_dim) {
  const uint32_t t = blockIdx.x, pos = first + t;
  if (rope_freq != nullptr) {
    for (uint32_t i = threadIdx.x; i < half_dim; i += kBlock) {
      float sn, cs;
      sincosf(static_cast<float>(pos) / rope_freq[i], &sn, &cs);
      rope_cs[static_cast<uint64_t>(t) * 2 * half_dim + i] = cs;
      rope_cs[static_cast<uint64_t>(t) * 2 * half_dim + half_dim + i] = sn;
    }
  }
  uint32_t token = prompt[pos];
  if (token >= vocab) token = 0;  // prompts are validated on the host
  const uint16_t *row = emb + static_cast<uint64_t>(token) * hidden;
  for (uint32_t i = threadIdx.x; i < hidden; i += kBlock) x[static_cast<uint64_t>(t) * hidden + i] = dec16<DT>(row[i]);
}

// Batch step: row t is the embedding of the token sequence t produced last (slot[position - 1]), and
// the rotation table of its position.
template <uint32_t DT>
__global__ __launch_bounds__(kBlock) void embed_batch_kernel(const uint16_t *emb, const BatchTable *table, uint32_t hidden,
                                                             uint32_t vocab, float *x, const float *rope_freq,
                                                             float *rope_cs, uint32_t half_dim) {
  const uint32_t t = blockIdx.x, pos = table->seq[t].position;
  if (rope_freq != nullptr) {
    for (uint32_t i = threadIdx.x; i < half_dim; i += kBlock) {
      float sn, cs;
      sincosf(static_cast<float>(pos) / rope_freq[i], &sn, &cs);
      rope_cs[static_cast<uint64_t>(t) * 2 * half_dim + i] = cs;
      rope_cs[static_cast<uint64_t>(t) * 2 * half_dim + half_dim + i] = sn;
    }
  }
  uint32_t token = pos == 0 ? 0u : table->slots[t][pos - 1].token;
  if (token >= vocab) token = 0;  // sampled ids are < vocab
  const uint16_t *row = emb + static_cast<uint64_t>(token) * hidden;
  for (uint32_t i = threadIdx.x; i < hidden; i += kBlock) x[static_cast<uint64_t>(t) * hidden + i] = dec16<DT>(row[i]);
}

// Batch step: the slot every sequence has just published, side by side, for one copy to the host instead of one
// per sequence (a slot is 10 words; thread = (sequence, word)).
__global__ void gather_slots_kernel(const BatchTable *table, uint32_t count, Slot *out) {
  constexpr uint32_t kWords = sizeof(Slot) / sizeof(uint32_t);
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x, t = i / kWords, w = i % kWords;
  if (t >= count) return;
  const Slot *slot = table->slots[t] + table->seq[t].position;
  reinterpret_cast<uint32_t *>(out + t)[w] = reinterpret_cast<const uint32_t *>(slot)[w];
}

__global__ void set_state_kernel(uint32_t *state, uint32_t cursor, uint32_t prompt_count, uint32_t clear_fault) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    state[0] = cursor;
    state[1] = prompt_count;
    if (clear_fault) state[3] = 0u;
  }
}

// A pass of launches without the embedding launch in front: the step counter moves on, and the attention plan
// takes the new number (the tags of the split partials derive from it and must differ from launch to launch).
__global__ void bump_step_counter_kernel(uint32_t *state, uint32_t *attn_plan) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    state[2] = state[2] + 1u;
    if (attn_plan != nullptr) attn_plan[4] = state[2];
  }
}

__global__ void advance_cursor_kernel(uint32_t *state, uint32_t max_steps) {
  if (threadIdx.x == 0 && blockIdx.x == 0 && state[0] < max_steps) state[0] = state[0] + 1u;
}

struct Carver {
  uint64_t offset = 0;
  uint64_t take(uint64_t bytes, uint64_t align = 256) {
    const uint64_t at = (offset + align - 1) & ~(align - 1);
    offset = at + ((bytes + 255u) & ~uint64_t{255});
    return at;
  }
};
// Weight matrices start on 8 MiB boundaries of device memory (the arena's first such boundary is its origin for
// the weight layout). What the gate/up launch costs depends on its matrix's address modulo 8 MiB - the up rows lie
// a fixed 96 MiB behind the gate rows, and the memory channels are chosen by a hash that reaches up to those bits:
// with the rotated walk 31.0 us at 0 modulo 8 MiB, 31.4 at 2 and 6 MiB, 31.8 at 4 MiB, 32.1 at an odd KiB (the
// plain walk: 33.0 / 31.7 / 31.3 / 31.8 / 31.7). At most 8 MiB a matrix is left unused: under 1.2 GB for 36 layers.
constexpr uint64_t kMatrixAlign = 8u << 20;
// The up rows of a layer start 4 KiB behind the end of its gate rows (large matrices only), so that gate row i
// and up row i - which one wave of the decode step's gate/up launch streams side by side - lie half a row apart
// in the memory channels' interleave instead of exactly on top of each other. With the rotated walk the launch
// then takes 31.1 us at every base address modulo 8 MiB (without the gap: 31.1 to 31.9 depending on it, and up to
// 32.7 with the plain walk). Every kernel that reads the pair takes the gap as a parameter.
constexpr uint32_t kPairGapElems = 2048;

bool layer_supported(const NervaHipHfDecodeChainLayer &l) {
  if (l.w_q_gate || l.w_router || l.w_expert_gate_up || l.w_expert_down || l.w_shared_expert_gate ||
      l.w_shared_expert_up || l.w_shared_expert_down || l.w_shared_expert_router || l.w_linear_conv ||
      l.w_linear_qkv || l.w_linear_z || l.w_linear_b || l.w_linear_a || l.w_linear_dt_bias ||
      l.w_linear_a_log || l.w_linear_norm || l.w_linear_out)
    return false;
  if (l.linear_key_heads || l.linear_value_heads || l.linear_key_head_dim || l.linear_value_head_dim ||
      l.linear_conv_kernel)
    return false;
  if (l.mlp_kind != NERVA_HIP_MLP_DENSE || l.attention_kind != NERVA_HIP_ATTENTION_FULL) return false;
  if (l.moe_intermediate || l.shared_expert_intermediate || l.num_experts || l.experts_per_token)
    return false;
  if (l.deepseek_mode || l.deepseek_flags || l.deepseek_hc_mult || l.deepseek_q_lora_rank ||
      l.deepseek_kv_lora_rank || l.deepseek_o_lora_rank || l.deepseek_compress_ratio ||
      l.deepseek_index_topk)
    return false;
  return true;
}

bool layer_has_weights(const NervaHipHfDecodeChainLayer &l) {
  return l.rms_attn_weight && l.rms_mlp_weight && l.w_q && l.w_k && l.w_v && l.w_o && l.w_gate &&
         l.w_up && l.w_down;
}

void destroy_session(Session *s) {
  if (s == nullptr) return;
  if (s->stream) (void)hipStreamSynchronize(s->stream);
  for (int i = 0; i < 3; ++i) {
    if (s->exec[i]) (void)hipGraphExecDestroy(s->exec[i]);
    if (s->graph[i]) (void)hipGraphDestroy(s->graph[i]);
  }
  if (s->ev0) (void)hipEventDestroy(s->ev0);
  if (s->ev1) (void)hipEventDestroy(s->ev1);
  if (s->arena && !s->arena_in_weights) (void)hipFree(s->arena);
  if (s->weights != nullptr && s->weights->refs.fetch_sub(1) == 1) {
    if (s->weights->origin) (void)hipFree(s->weights->origin);
    delete s->weights;
  }
  if (s->pinned) (void)hipHostFree(s->pinned);
  if (s->stream) (void)hipStreamDestroy(s->stream);
  delete s;
}

// Enqueue one step on the session stream (eagerly or under stream capture). With
// `only` >= 0 just the per-layer launches of that kind are enqueued (profiling).
hipError_t enqueue_step(Session *s, StepMode mode, StepProfiler *prof, int only = -1) {
  hipStream_t st = s->stream;
  const uint32_t A = s->heads * s->head_dim, KV = s->kv_heads * s->head_dim;
  hipError_t err = hipSuccess;
  // armed trace: copy an intermediate vector behind the ones already recorded (256-byte slots)
  const bool tracing = s->trace_buf != nullptr && mode == kDecodeStep && only < 0 && prof == nullptr;
  auto snap = [&](const void *src, uint64_t bytes) {
    if (!tracing || err != hipSuccess) return;
    err = hipMemcpyAsync(s->trace_buf + s->trace_used, src, bytes, hipMemcpyDeviceToDevice, st);
    s->trace_used += (bytes + 255u) & ~uint64_t{255};
  };
  // the next trace slot as a destination a kernel writes itself (the RMSNorm prologue's 16-bit vector)
  auto snap_slot = [&](uint64_t bytes) -> uint16_t * {
    if (!tracing) return nullptr;
    uint16_t *at = reinterpret_cast<uint16_t *>(s->trace_buf + s->trace_used);
    s->trace_used += (bytes + 255u) & ~uint64_t{255};
    return at;
  };
#define NV_STEP(kind, expr)                         \
  do {                                              \
    if (only >= 0 && only != (kind)) break;         \
    if (prof && err == hipSuccess) err = prof->before(kind); \
    if (err == hipSuccess) err = (expr);            \
    if (prof && err == hipSuccess) err = prof->after();      \
    if (err != hipSuccess) return err;              \
  } while (0)

  if (only < 0) {
    const uint32_t blocks = std::min<uint32_t>((s->hidden + kBlock - 1) / kBlock, 64u);
    const float *rope_freq = s->theta > 0.0f ? s->rope_freq : nullptr;
    if (prof) err = prof->before(kLEmbed);
    if (err != hipSuccess) return err;
    if (s->dtype == kBF16)
      hipLaunchKernelGGL(embed_kernel<kBF16>, dim3(blocks), dim3(kBlock), 0, st, s->emb, s->prompt,
                         s->slots, s->state, s->max_ctx, s->hidden, s->vocab, s->x, rope_freq, s->rope_cs,
                         s->head_dim / 2, s->attn_plan, s->table, s->attn_splits, s->attn_single_blocks);
    else
      hipLaunchKernelGGL(embed_kernel<kF16>, dim3(blocks), dim3(kBlock), 0, st, s->emb, s->prompt,
                         s->slots, s->state, s->max_ctx, s->hidden, s->vocab, s->x, rope_freq, s->rope_cs,
                         s->head_dim / 2, s->attn_plan, s->table, s->attn_splits, s->attn_single_blocks);
    err = hipGetLastError();
    if (prof && err == hipSuccess) err = prof->after();
    if (err != hipSuccess) return err;
    snap(s->x, static_cast<uint64_t>(s->hidden) * sizeof(float));
  }
  for (uint32_t l = 0; l < s->layers; ++l) {
    const LayerDev &w = s->layer[l];
    {
      GemvParams p{};
      p.w = w.wqkv;
      p.xf = s->x;
      p.gamma = w.rms_attn;
      p.out_f32 = s->qkv;
      p.rows = A + 2 * KV;
      p.cols = s->hidden;
      p.eps = s->eps;
      p.cursor = s->state;
      p.max_steps = s->max_ctx;
      p.x16_dump = snap_slot(static_cast<uint64_t>(s->hidden) * sizeof(uint16_t));
      NV_STEP(kLQkv, launch_gemv(s->dtype, kProRmsNorm, kEpiF32, p, st));
      snap(s->qkv, static_cast<uint64_t>(A + 2 * KV) * sizeof(float));
    }
    {
      AttnParams p{};
      p.heads = s->heads;
      p.kv_heads = s->kv_heads;
      p.head_dim = s->head_dim;
      attn_bind_workspace(p, s->attn_ws);
      p.qkv = s->qkv;
      p.q_norm = w.q_norm;
      p.k_norm = w.k_norm;
      p.q_bias = w.q_bias;
      p.k_bias = w.k_bias;
      p.v_bias = w.v_bias;
      p.k_cache = s->kc;
      p.v_cache = s->vc;
      p.table = s->table;
      p.rope_freq = s->theta > 0.0f ? s->rope_freq : nullptr;
      p.rope_cs = s->theta > 0.0f ? s->rope_cs : nullptr;
      p.out_f32 = nullptr;
      p.out16 = s->attn16;
      p.layer = l;
      p.block_count = s->block_count;
      p.splits = s->attn_splits;
      p.single_split_blocks = s->attn_single_blocks;
      p.eps = s->eps;
      p.cursor = s->state;
      p.max_steps = s->max_ctx;
      p.append = 1;
      p.trace = s->attn_trace != nullptr ? s->attn_trace + 32 * l : nullptr;
      // (a pass of attention launches alone - profiling - follows full steps at the same position, whose
      // embedding launch left the plan of that position)
      p.plan = s->attn_plan;
      p.part_tagged = s->attn_tagged;
      p.fault = s->state + 3;
      p.merge_spin_limit = static_cast<uint32_t>(std::max(tuning(kTuneAttnMergeSpinLimit), 0));
      p.withhold_split = static_cast<uint32_t>(std::max(tuning(kTuneAttnWithholdSplit), 0));
      NV_STEP(kLAttn, launch_attn_decode(s->dtype, p, st));
      snap(s->attn16, static_cast<uint64_t>(A) * sizeof(uint16_t));
    }
    {
      GemvParams p{};
      p.w = w.wo;
      p.x16 = s->attn16;
      p.bias = w.o_bias;
      p.residual = s->x;
      p.out_f32 = s->r;
      p.rows = s->hidden;
      p.cols = A;
      p.cursor = s->state;
      p.max_steps = s->max_ctx;
      NV_STEP(kLO, launch_gemv(s->dtype, kProX16, kEpiResidual, p, st));
      snap(s->r, static_cast<uint64_t>(s->hidden) * sizeof(float));
    }
    {
      GemvParams p{};
      p.w = w.wgu;
      p.pair_gap = s->pair_gap;
      p.xf = s->r;
      p.gamma = w.rms_mlp;
      p.out16 = s->ff16;
      p.rows = s->intermediate;
      p.cols = s->hidden;
      p.eps = s->eps;
      p.cursor = s->state;
      p.max_steps = s->max_ctx;
      p.x16_dump = snap_slot(static_cast<uint64_t>(s->hidden) * sizeof(uint16_t));
      NV_STEP(kLGateUp, launch_gemv(s->dtype, kProRmsNorm, kEpiSwiglu, p, st));
      snap(s->ff16, static_cast<uint64_t>(s->intermediate) * sizeof(uint16_t));
    }
    {
      GemvParams p{};
      p.w = w.wdown;
      p.x16 = s->ff16;
      p.residual = s->r;
      p.out_f32 = s->x;
      p.rows = s->hidden;
      p.cols = s->intermediate;
      // prompt tokens carry a 16-bit hidden state between layers (prefill_kernels.cu:494-508)
      p.round_out = mode == kDecodeStep ? 0u : 1u;
      p.cursor = s->state;
      p.max_steps = s->max_ctx;
      NV_STEP(kLDown, launch_gemv(s->dtype, kProX16, kEpiResidual, p, st));
      snap(s->x, static_cast<uint64_t>(s->hidden) * sizeof(float));
    }
    }
  if (only >= 0) return hipSuccess;
  if (mode == kPromptStep) {
    if (prof) err = prof->before(kLAdvance);
    if (err != hipSuccess) return err;
    hipLaunchKernelGGL(advance_cursor_kernel, dim3(1), dim3(64), 0, st, s->state, s->max_ctx);
    err = hipGetLastError();
    if (prof && err == hipSuccess) err = prof->after();
    return err;
  }
  GemvParams p{};
  p.w = s->lm_head;
  p.xf = s->x;
  p.gamma = s->final_norm;
  p.out_f32 = s->logits;
  p.rows = s->vocab;
  p.cols = s->hidden;
  p.eps = s->eps;
  p.cursor = s->state;
  p.max_steps = s->max_ctx;
  sample_bind_workspace(p.sample, s->sample_ws);
  p.sample.slots = s->slots;
  p.sample.cursor_rw = s->state;
  p.sample.fault = s->state + 3;
  p.x16_dump = snap_slot(static_cast<uint64_t>(s->hidden) * sizeof(uint16_t));
  uint32_t head_blocks = 0;  // workgroups of the LM-head launch = candidates it leaves
  NV_STEP(kLHead, launch_gemv(s->dtype, kProRmsNorm, kEpiArgmax, p, st, nullptr, &head_blocks));
  snap(s->logits, static_cast<uint64_t>(s->vocab) * sizeof(float));
  if (s->sampler.mode == kSamplerGreedy) {
    // one small workgroup reduces the per-workgroup candidates, writes slot[pos], bumps the cursor
    NV_STEP(kLAdvance, launch_sample_finish(p.sample, head_blocks, s->state, s->max_ctx, st));
  } else {
    // temperature sampling from the logits (two launches), then slot[pos] and the cursor as above
    SamplerParams sp{};
    sp.logits = s->logits;
    sp.vocab = s->vocab;
    sp.config = s->sampler_dev;
    sp.keys = s->sampler_keys;
    sp.out = p.sample;
    sp.cursor = s->state;
    sp.max_steps = s->max_ctx;
    NV_STEP(kLAdvance, launch_sampler(sp, st));
  }
#undef NV_STEP
  return hipSuccess;
}

// Steps are launched kernel by kernel instead of as graph replays when NERVA_HIP_EAGER_STEPS=1 is
// set, or when the process runs under the ROCm profiler: with ROCm 7.2 a process traced by
// rocprofv3 --kernel-trace died inside the HIP runtime at its first hipGraphLaunch (no message of its
// own; the tool reported the abort), so a traced process must never reach that call. The profiler is
// recognised by what it puts into the environment of the process it starts (its tool library in
// LD_PRELOAD / ROCP_TOOL_LIBRARIES, ROCPROF_* settings). Results and per-kernel durations are the
// same; the graph counters then report zero replays.
bool profiler_in_environment() {
  for (char **e = ::environ; e != nullptr && *e != nullptr; ++e) {
    const char *v = *e;
    if (strncmp(v, "ROCPROF", 7) == 0 || strncmp(v, "ROCP_TOOL_LIBRARIES=", 20) == 0 ||
        strncmp(v, "ROCPROFILER_", 12) == 0)
      return true;
    if (strncmp(v, "LD_PRELOAD=", 11) == 0 && (strstr(v, "rocprofiler") != nullptr || strstr(v, "rocprof") != nullptr))
      return true;
  }
  return false;
}
bool eager_steps() {
  static const bool eager = [] {
    const char *v = getenv("NERVA_HIP_EAGER_STEPS");
    return (v != nullptr && v[0] == '1') || profiler_in_environment();
  }();
  return eager;
}

// Kernel launches of one step (which = 0: decode step, 1: prompt step).
uint64_t step_launches(const Session *s, int which) {
  // embed + (lm head + greedy finish | lm head + two sampler launches | cursor advance)
  const uint64_t fixed = which == 1 ? 2 : (s->sampler.mode == kSamplerGreedy ? 3 : 4);
  return fixed + 5ull * s->layers;
}

// Launch one step: graph replay, or the same kernels eagerly (tracing mode).
hipError_t launch_step(Session *s, int which, NervaHipHfDecodeSequenceResult *out);

// Index of the captured decode step for the active sampler.
int decode_graph(const Session *s) { return s->sampler.mode == kSamplerGreedy ? 0 : 2; }

// graph index 0 / 2: decode step (greedy finish / sampler), 1: prompt step
hipError_t ensure_graph(Session *s, int which, NervaHipHfDecodeSequenceResult *out) {
  if (eager_steps()) return hipSuccess;
  if (s->exec[which] != nullptr) {
    if (out) {
      out->graph_nodes = s->graph_nodes[which];
      out->graph_cache_hits += 1;
    }
    return hipSuccess;
  }
  hipGraph_t graph = nullptr;
  hipError_t err = hipStreamBeginCapture(s->stream, hipStreamCaptureModeThreadLocal);
  if (err != hipSuccess) return err;
  hipError_t step_err = enqueue_step(s, which == 1 ? kPromptStep : kDecodeStep, nullptr);
  err = hipStreamEndCapture(s->stream, &graph);
  if (step_err != hipSuccess) err = step_err;
  size_t nodes = 0;
  if (err == hipSuccess) err = hipGraphGetNodes(graph, nullptr, &nodes);
  hipGraphExec_t exec = nullptr;
  if (err == hipSuccess) err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (err != hipSuccess) {
    if (graph) (void)hipGraphDestroy(graph);
    return err;
  }
  s->graph[which] = graph;
  s->exec[which] = exec;
  s->graph_nodes[which] = nodes;
  if (out) {
    out->graph_nodes = nodes;
    out->graph_captures += 1;
  }
  return hipSuccess;
}

hipError_t launch_step(Session *s, int which, NervaHipHfDecodeSequenceResult *out) {
  if (s->trace_buf != nullptr && which != 1) {
    // armed by nerva_hip_session_trace_next_step: this one step runs kernel by kernel with copies
    s->trace_used = 0;
    hipError_t err = enqueue_step(s, kDecodeStep, nullptr);
    s->trace_buf = nullptr;
    if (err == hipSuccess) out->kernel_launches += step_launches(s, which);
    return err;
  }
  if (eager_steps()) {
    hipError_t err = enqueue_step(s, which == 1 ? kPromptStep : kDecodeStep, nullptr);
    if (err == hipSuccess)
      out->kernel_launches += step_launches(s, which);
    return err;
  }
  hipError_t err = hipGraphLaunch(s->exec[which], s->stream);
  if (err == hipSuccess) {
    out->graph_replays += 1;
    out->graph_launches += 1;
    out->kernel_launches += s->graph_nodes[which];
  }
  return err;
}

void fill_header(const Session *s, NervaHipHfDecodeSequenceResult *out, uint32_t steps,
                 uint32_t seed_token) {
  out->device_count = 1;
  out->dtype = s->dtype;
  out->hidden = s->hidden;
  out->heads = s->heads;
  out->kv_heads = s->kv_heads;
  out->head_dim = s->head_dim;
  out->intermediate = s->intermediate;
  out->vocab_size = s->vocab;
  out->layer_count = s->layers;
  out->steps = steps;
  out->seed_token = seed_token;
  out->resident_weight_bytes = s->resident_weight_bytes;
  out->planned_weight_blocks = s->planned_weight_blocks;
  out->planned_gpu_resident_blocks = s->planned_gpu_resident_blocks;
  out->planned_gpu_staged_blocks = s->planned_gpu_staged_blocks;
  out->planned_weight_bytes = s->planned_weight_bytes;
  out->planned_gpu_resident_weight_bytes = s->planned_gpu_resident_weight_bytes;
  out->planned_gpu_staged_weight_bytes = s->planned_gpu_staged_weight_bytes;
  out->descriptor_gpu_resident_h2d_bytes = s->planned_gpu_resident_weight_bytes;
  out->descriptor_gpu_staged_h2d_bytes = s->planned_gpu_staged_weight_bytes;
  out->planned_weight_descriptor_count = s->planned_weight_descriptor_count;
  out->planned_weight_descriptor_hash = s->planned_weight_descriptor_hash;
}

// The sampler of the sequence that is about to start: normalised the way the reference's ABI does
// (sampler.cu:422-433; its callers validate before the call, the ABI itself never refuses a
// configuration) and copied to the device words the sampler kernels read. Not on the per-token path.
hipError_t set_sampler(Session *s, const NervaHipHfDecodeSamplerConfig &config) {
  s->sampler = sampler_device_config(config);
  return hipMemcpy(s->sampler_dev, &s->sampler, sizeof(SamplerDev), hipMemcpyHostToDevice);
}

uint32_t observed_count(uint32_t steps, uint32_t has_eos, uint32_t eos, const Slot *slots) {
  uint32_t count = steps;
  for (uint32_t i = 0; i < steps; ++i) {
    if (slots[i].completion != NERVA_HIP_SLOT_DEVICE_COMPLETE) {
      count = i;
      break;
    }
    if (has_eos != 0 && slots[i].token == eos) {
      count = i + 1;
      break;
    }
  }
  return count;
}

// Every field of a slot as the device publishes it (nerva_cuda_api.h:29-37, sampler.cu:394-407).
bool slots_consistent(const Slot *slots, uint32_t count, uint32_t first_index) {
  for (uint32_t i = 0; i < count; ++i) {
    if (slots[i].request_id != NERVA_HIP_SLOT_REQUEST_ID || slots[i].sequence_id != NERVA_HIP_SLOT_SEQUENCE_ID ||
        slots[i].completion != NERVA_HIP_SLOT_DEVICE_COMPLETE || slots[i].token_index != first_index + i ||
        slots[i].version != static_cast<uint64_t>(first_index + i) + 1u || slots[i].host_copied != 0)
      return false;
  }
  return true;
}
// A slot published by a step in which a device-side bounded wait gave up.
bool slots_faulted(const Slot *slots, uint32_t count) {
  for (uint32_t i = 0; i < count; ++i)
    if (slots[i].completion == NERVA_HIP_SLOT_DEVICE_FAULT) return true;
  return false;
}

hipError_t reset_sequence(Session *s, const uint32_t *prompt_tokens, uint32_t prompt_count,
                          NervaHipHfDecodeSequenceResult *out) {
  // Not on the per-token path: the prompt is copied synchronously (the caller's buffer may be
  // reused as soon as this returns) and the cursor is set by a one-thread kernel in stream order.
  hipError_t err = hipStreamSynchronize(s->stream);
  if (err == hipSuccess)
    err = hipMemcpy(s->prompt, prompt_tokens, static_cast<uint64_t>(prompt_count) * sizeof(uint32_t),
                    hipMemcpyHostToDevice);
  if (err == hipSuccess)
    err = hipMemsetAsync(s->slots, 0, static_cast<uint64_t>(s->max_ctx) * sizeof(Slot), s->stream);
  // the attention's tagged split partials: a tag is unique for 2^23 steps, which no sequence reaches, so with
  // the words cleared here none of an earlier sequence's can ever match
  if (err == hipSuccess && s->attn_tagged != nullptr)
    err = hipMemsetAsync(s->attn_tagged, 0, attn_step_workspace_bytes(s->heads), s->stream);
  if (err == hipSuccess) {
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(64), 0, s->stream, s->state, 0u, prompt_count, 1u);
    err = hipGetLastError();
  }
  out->h2d_bytes = static_cast<uint64_t>(prompt_count) * sizeof(uint32_t);
  return err;
}

// Token blocks (prompt blocks, batch steps) of more than one row keep their 16-bit activations -
// normalised rows, attention output, SwiGLU output: the X operands of the multi-row GEMMs - in
// matrix-operand order, which the GEMM reads with full cache lines and which lets the projections share the
// block through LDS. Batch steps of Qwen3-8B shape, [token][column] rows with every wave fetching its own
// X pieces against operand order: 2 sequences 3.68 vs 3.50 ms, 8: 4.03 vs 3.62, 16: 4.70 vs 3.88 (operand
// order through the kernel without the shared block: 4.28, 4.43, 4.78).
// The "block_layout" override forces one layout (1 = rows, 2 = operand order; comparisons).
uint32_t block_operand_tiles(uint32_t tokens) {
  const int forced = tuning(kTuneBlockLayout);
  const bool operand = forced == 1 || forced == 2 ? forced == 2 : tokens > 1;
  return operand ? gemm_packed_tiles(tokens) : 0u;
}

// Prompt tokens 0 .. count-1 through every layer in blocks of up to prefill_block_tokens tokens, with the
// prompt staging (16-bit hidden state between layers, prefill_kernels.cu:494-508): per block and
// layer one RMSNorm launch, the qkv projection as a multi-row GEMM, the K/V rows of the block into the
// cache, the attention of all its tokens in one launch (token z attends to keys 0 .. first + z), and
// the o / gate-up / down projections as multi-row GEMMs. Leaves the cursor at `count`. The reference
// prefills in chunks too (session_decode_prefill.inc.cu:1879-2243).
hipError_t prefill_blocks(Session *s, uint32_t count, uint32_t prompt_count, NervaHipHfDecodeSequenceResult *out) {
  hipStream_t st = s->stream;
  const uint32_t H = s->hidden, A = s->heads * s->head_dim, KV = s->kv_heads * s->head_dim, I = s->intermediate;
  const float *rope_freq = s->theta > 0.0f ? s->rope_freq : nullptr;
  hipError_t err = hipSuccess;
  // "prefill_attention_rows" override = 1: the block's attention as one workgroup set per token (the batch
  // step's kernel) instead of the prompt kernel that shares K/V tiles between tokens; for comparisons
  const bool rows_attention = tuning(kTunePrefillAttentionRows) == 1;
  const int want_prompt_splits = tuning(kTunePromptSplits);
  const uint32_t prompt_splits = want_prompt_splits >= 1 && want_prompt_splits <= static_cast<int>(kAttnMaxSplits)
                                     ? static_cast<uint32_t>(want_prompt_splits)
                                     : 0u;
  for (uint32_t first = 0; err == hipSuccess && first < count; first += s->prefill_block_tokens) {
    const uint32_t T = std::min<uint32_t>(s->prefill_block_tokens, count - first);
    const uint32_t tiles = block_operand_tiles(T);
    if (s->dtype == kBF16)
      hipLaunchKernelGGL(embed_rows_kernel<kBF16>, dim3(T), dim3(kBlock), 0, st, s->emb, s->prompt, first, H, s->vocab,
                         s->px, rope_freq, s->prope, s->head_dim / 2);
    else
      hipLaunchKernelGGL(embed_rows_kernel<kF16>, dim3(T), dim3(kBlock), 0, st, s->emb, s->prompt, first, H, s->vocab,
                         s->px, rope_freq, s->prope, s->head_dim / 2);
    err = hipGetLastError();
    // Where a projection's slice-adding launch can write the following RMSNorm too, it does (one launch less each)
    const bool o_norms = gemm_rows_fuses_norm(kGemmResidual, H, A, T, tiles, s->pgemm_ws_bytes);
    const bool down_norms = gemm_rows_fuses_norm(kGemmResidual, H, I, T, tiles, s->pgemm_ws_bytes);
    for (uint32_t l = 0; err == hipSuccess && l < s->layers; ++l) {
      const LayerDev &w = s->layer[l];
      if (l == 0 || !down_norms) err = launch_rmsnorm_rows(s->dtype, s->px, w.rms_attn, s->eps, T, H, s->pxn16, st, tiles);
      GemmRowsParams g{};
      g.tokens = T;
      if (err == hipSuccess) {
        g.w = w.wqkv;
        g.x16 = s->pxn16;
        g.x_packed = tiles;
        g.out_f32 = s->pqkv;
        g.rows = A + 2 * KV;
        g.cols = H;
        g.workspace = s->pgemm_ws;
        g.workspace_bytes = s->pgemm_ws_bytes;
        err = launch_gemm_rows(s->dtype, kGemmF32, g, st);
      }
      AttnParams a{};
      a.heads = s->heads;
      a.kv_heads = s->kv_heads;
      a.head_dim = s->head_dim;
      attn_bind_workspace(a, s->pattn_ws);
      a.qkv = s->pqkv;
      a.q_norm = w.q_norm;
      a.k_norm = w.k_norm;
      a.q_bias = w.q_bias;
      a.k_bias = w.k_bias;
      a.v_bias = w.v_bias;
      a.k_cache = s->kc;
      a.v_cache = s->vc;
      a.table = s->table;
      a.rope_freq = rope_freq;
      a.rope_cs = rope_freq != nullptr ? s->prope : nullptr;
      a.out16 = s->pattn16;
      a.layer = l;
      a.block_count = s->block_count;
      a.splits = s->attn_splits;
      a.eps = s->eps;
      a.position = first;
      a.tokens = T;
      a.qkv_token_stride = A + 2 * KV;
      a.out_token_stride = A;
      a.rope_token_stride = s->head_dim;
      a.ws_token_stride = s->pattn_ws_stride;
      a.out_packed_tiles = tiles;
      if (err == hipSuccess) err = launch_kv_publish_rows(s->dtype, a, st);
      if (err == hipSuccess) {
        if (rows_attention) {
          err = launch_attn_decode(s->dtype, a, st);   // every token streams the prefix itself
        } else {
          a.splits = prompt_splits;                    // K/V tiles shared by the tokens of the block (0: the launcher chooses)
          err = launch_attn_prompt(s->dtype, a, st);
        }
      }
      if (err == hipSuccess) {
        g = GemmRowsParams{};
        g.tokens = T;
        g.w = w.wo;
        g.x16 = s->pattn16;
        g.x_packed = tiles;
        g.bias = w.o_bias;
        g.residual = s->px;
        g.out_f32 = s->pr;
        g.rows = H;
        g.cols = A;
        g.workspace = s->pgemm_ws;
        g.workspace_bytes = s->pgemm_ws_bytes;
        if (o_norms) {
          g.norm_gamma = w.rms_mlp;
          g.norm_out16 = s->pxn16;
          g.norm_eps = s->eps;
          g.norm_packed_tiles = tiles;
        }
        err = launch_gemm_rows(s->dtype, kGemmResidual, g, st);
      }
      if (err == hipSuccess && !o_norms) err = launch_rmsnorm_rows(s->dtype, s->pr, w.rms_mlp, s->eps, T, H, s->pxn16, st, tiles);
      if (err == hipSuccess) {
        g = GemmRowsParams{};
        g.tokens = T;
        g.w = w.wgu;
        g.pair_gap = s->pair_gap;
        g.x16 = s->pxn16;
        g.x_packed = tiles;
        g.out16 = s->pff16;
        g.out_packed_tiles = tiles;
        g.rows = I;
        g.cols = H;
        g.workspace = s->pgemm_ws;
        g.workspace_bytes = s->pgemm_ws_bytes;
        err = launch_gemm_rows(s->dtype, kGemmSwiglu, g, st);
      }
      if (err == hipSuccess) {
        g = GemmRowsParams{};
        g.tokens = T;
        g.w = w.wdown;
        g.x16 = s->pff16;
        g.x_packed = tiles;
        g.residual = s->pr;
        g.out_f32 = s->px;
        g.rows = H;
        g.cols = I;
        g.round_out = 1;  // prompt tokens carry a 16-bit hidden state between layers
        g.workspace = s->pgemm_ws;
        g.workspace_bytes = s->pgemm_ws_bytes;
        if (down_norms && l + 1 < s->layers) {   // the next layer's attention norm
          g.norm_gamma = s->layer[l + 1].rms_attn;
          g.norm_out16 = s->pxn16;
          g.norm_eps = s->eps;
          g.norm_packed_tiles = tiles;
        }
        err = launch_gemm_rows(s->dtype, kGemmResidual, g, st);
      }
    }
    if (err == hipSuccess) out->kernel_launches += 1 + (rows_attention ? 9ull : 10ull) * s->layers;
  }
  if (err == hipSuccess) {
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(64), 0, st, s->state, count, prompt_count, 0u);
    err = hipGetLastError();
    out->kernel_launches += 1;
  }
  return err;
}

// ---- weights from the caller's plan -----------------------------------------------------------
// A declared weight plan (weights.cu:157-160) comes with descriptors that tile the weight bytes
// [0, resident_weight_bytes) in the reference's arena order - embeddings, then per layer rms_attn,
// w_q, [q_norm], w_k, [k_norm], w_v, w_o, rms_mlp, w_gate, w_up, w_down, [q/k/v/o bias], then the
// final norm and the LM head (weights.cu:484-591, session_api_lifecycle.inc.cu:124-148) - each with a
// host-memory or a file source. The descriptors are then THE source of the weights; the tensor
// pointers of the request only say which optional tensors exist (weights.cu:18-23) and may be null
// otherwise (weights.cu:237-243). This library keeps [q;k;v] and [gate;up] as row-concatenated
// matrices elsewhere in its own arena, so a descriptor's byte range is cut along the tensor
// boundaries of that order and every piece goes to its tensor's place.
constexpr uint32_t kWeightStrategyGpuResident = 1, kWeightStrategyGpuStaged = 2;  // weight_plan.rs:3-4

struct WeightSegment {
  uint64_t logical, bytes;  // position in the reference's arena order
  char *device;
};

template <typename Request>
bool weight_plan_declared(const Request *rq) {
  return rq->planned_weight_blocks != 0 || rq->planned_weight_bytes != 0;
}

void hash_le(uint64_t &hash, uint64_t value, int bytes) {
  for (int i = 0; i < bytes; ++i) {
    hash ^= (value >> (8 * i)) & 0xffu;
    hash *= 0x00000100000001b3ull;
  }
}

bool descriptor_has_file(const NervaHipHfDecodeSequenceWeightBlock &d) {
  return d.source_file != nullptr && d.source_file_len != 0;
}

// weights.cu:411-467: contiguous from 0, even offsets and sizes, a source each, a known strategy, and
// totals, counts and the FNV-1a hash over (block_id, block_version, offset_bytes, bytes, strategy)
// equal to what the plan declares.
bool validate_weight_descriptors(const NervaHipHfDecodeSequenceSessionCreateRequest *rq, uint64_t resident_weight_bytes) {
  uint64_t cursor = 0, hash = 0xcbf29ce484222325ull, resident_bytes = 0, staged_bytes = 0;
  uint32_t resident_blocks = 0, staged_blocks = 0;
  for (uint32_t i = 0; i < rq->planned_weight_descriptor_count; ++i) {
    const NervaHipHfDecodeSequenceWeightBlock &d = rq->planned_weight_descriptors[i];
    if (d.bytes == 0 || d.reserved != 0 || (d.host_source == nullptr && !descriptor_has_file(d)) ||
        d.offset_bytes != cursor || d.offset_bytes % 2 != 0 || d.bytes % 2 != 0)
      return false;
    if (cursor + d.bytes < cursor) return false;
    cursor += d.bytes;
    hash_le(hash, d.block_id, 8);
    hash_le(hash, d.block_version, 8);
    hash_le(hash, d.offset_bytes, 8);
    hash_le(hash, d.bytes, 8);
    hash_le(hash, d.strategy, 4);
    if (d.strategy == kWeightStrategyGpuResident) {
      resident_blocks += 1;
      resident_bytes += d.bytes;
    } else if (d.strategy == kWeightStrategyGpuStaged) {
      staged_blocks += 1;
      staged_bytes += d.bytes;
    } else {
      return false;
    }
  }
  return cursor == resident_weight_bytes && cursor == rq->planned_weight_bytes &&
         hash == rq->planned_weight_descriptor_hash && resident_blocks == rq->planned_gpu_resident_blocks &&
         staged_blocks == rq->planned_gpu_staged_blocks && resident_bytes == rq->planned_gpu_resident_weight_bytes &&
         staged_bytes == rq->planned_gpu_staged_weight_bytes;
}

// weights.cu:797-908: every descriptor to the device, from memory directly or from its file through a
// pinned staging buffer. `segments` is sorted and gapless in the reference's order.
hipError_t copy_weight_descriptors(const NervaHipHfDecodeSequenceSessionCreateRequest *rq,
                                   const std::vector<WeightSegment> &segments, hipStream_t stream, uint64_t *h2d_bytes,
                                   uint64_t *sync_calls) {
  constexpr uint64_t kStagingBytes = 64ull << 20;
  char *staging = nullptr;
  hipError_t err = hipSuccess;
  size_t at = 0;  // descriptors ascend, so the segment cursor only moves forward
  for (uint32_t i = 0; err == hipSuccess && i < rq->planned_weight_descriptor_count; ++i) {
    const NervaHipHfDecodeSequenceWeightBlock &d = rq->planned_weight_descriptors[i];
    FILE *file = nullptr;
    if (d.host_source == nullptr) {
      if (staging == nullptr) err = counted_host_malloc(reinterpret_cast<void **>(&staging), kStagingBytes);
      if (err != hipSuccess) break;
      const std::string path(d.source_file, d.source_file_len);
      file = fopen(path.c_str(), "rb");
      if (file == nullptr) {
        err = hipErrorInvalidValue;
        break;
      }
    }
    uint64_t done = 0;
    while (err == hipSuccess && done < d.bytes) {
      const uint64_t logical = d.offset_bytes + done;
      while (at < segments.size() && segments[at].logical + segments[at].bytes <= logical) ++at;
      if (at == segments.size()) {
        err = hipErrorInvalidValue;
        break;
      }
      const WeightSegment &seg = segments[at];
      const uint64_t inside = logical - seg.logical;
      uint64_t piece = std::min(d.bytes - done, seg.bytes - inside);
      if (file == nullptr) {
        err = hipMemcpyAsync(seg.device + inside, reinterpret_cast<const char *>(d.host_source) + done, piece,
                             hipMemcpyHostToDevice, stream);
      } else {
        piece = std::min(piece, kStagingBytes);
        if (fseeko(file, static_cast<off_t>(d.file_offset_begin + done), SEEK_SET) != 0 ||
            fread(staging, 1, piece, file) != piece) {
          err = hipErrorInvalidValue;
          break;
        }
        err = hipMemcpyAsync(seg.device + inside, staging, piece, hipMemcpyHostToDevice, stream);
        if (err == hipSuccess) err = hipStreamSynchronize(stream);  // the one staging buffer is reused
        *sync_calls += 1;
      }
      done += piece;
    }
    if (file != nullptr) fclose(file);
    *h2d_bytes += done;
  }
  if (err == hipSuccess) err = hipStreamSynchronize(stream);
  if (staging != nullptr) (void)hipHostFree(staging);
  return err;
}

// Everything of a session that is not weights, from the dimensions already in `s`: stream, events,
// the state arena (KV cache, block table, prompt, token slots, cursor words, activations and
// workspaces), the pinned host mirrors, the step modes. Shared by create and fork.
// with_weights: one allocation holds the weights (s->weights->bytes, not allocated yet) and, behind
// them, this session's state; it lives as long as any session uses the weights.
hipError_t setup_state(Session *s, int32_t *failure_stage, bool with_weights) {
  const uint64_t H = s->hidden, A = static_cast<uint64_t>(s->heads) * s->head_dim,
                 KV = static_cast<uint64_t>(s->kv_heads) * s->head_dim, I = s->intermediate, V = s->vocab,
                 L = s->layers, HD = s->head_dim;
  const uint32_t block_count = (s->max_ctx + kKvBlockTokens - 1) / kKvBlockTokens;
  s->block_count = block_count;
  s->attn_splits = attn_default_splits(s->kv_heads, block_count);
  s->attn_single_blocks = kAttnSingleSplitBlocks;
  if (const int want = tuning(kTuneAttnSplits); want >= 1 && want <= static_cast<int>(kAttnMaxSplits)) {
    // (never more than stay resident together: the merges of the step kernel poll)
    s->attn_splits = std::min({static_cast<uint32_t>(want), block_count, attn_resident_splits(s->kv_heads)});
    s->attn_single_blocks = 0;  // a forced factor holds at every context length
  }

  Carver c;
  const uint64_t kv_half = L * block_count * KV * kKvBlockTokens * 2;
  const uint64_t off_kc = c.take(kv_half);
  const uint64_t off_vc = c.take(kv_half);
  s->kv_bytes = 2 * kv_half;
  const uint64_t off_table = c.take(static_cast<uint64_t>(block_count) * 4);
  const uint64_t off_prompt = c.take(static_cast<uint64_t>(s->max_ctx) * 4);
  const uint64_t off_slots = c.take(static_cast<uint64_t>(s->max_ctx) * sizeof(Slot));
  const uint64_t off_state = c.take(64);
  const uint64_t off_x = c.take(H * 4);
  const uint64_t off_r = c.take(H * 4);
  const uint64_t off_qkv = c.take((A + 2 * KV) * 4);
  const uint64_t off_logits = c.take(V * 4);
  const uint64_t off_attn16 = c.take(A * 2);
  const uint64_t off_ff16 = c.take(I * 2);
  const uint64_t off_rope = c.take(HD * 4);
  const uint64_t off_rope_cs = c.take(HD * 4);
  const uint64_t attn_ws_bytes = attn_workspace_bytes(s->heads, s->head_dim);
  const uint64_t off_attn_ws = c.take(attn_ws_bytes);
  const uint64_t off_attn_plan = c.take(attn_plan_bytes(kAttnMaxSplits));
  const uint64_t off_attn_tagged = c.take(attn_step_workspace_bytes(s->heads));
  const uint64_t off_sample_ws = c.take(sample_workspace_bytes());
  const uint64_t pT = kGemmDeepMaxTokens;
  const uint64_t off_px = c.take(pT * H * 4);
  const uint64_t off_pr = c.take(pT * H * 4);
  const uint64_t off_pqkv = c.take(pT * (A + 2 * KV) * 4);
  const uint64_t off_pxn16 = c.take(pT * H * 2);
  const uint64_t off_pattn16 = c.take(pT * A * 2);
  const uint64_t off_pff16 = c.take(pT * I * 2);
  const uint64_t off_prope = c.take(pT * HD * 4);
  const uint64_t pattn_ws_stride = (attn_ws_bytes + 255u) & ~uint64_t{255};
  const uint64_t off_pattn_ws = c.take(pT * pattn_ws_stride);
  const uint64_t pgemm_ws_bytes = gemm_block_workspace_bytes(static_cast<uint32_t>(std::max<uint64_t>(H, A + 2 * KV)));
  const uint64_t off_pgemm_ws = c.take(pgemm_ws_bytes);
  const uint64_t off_sampler_dev = c.take(sizeof(SamplerDev));
  const uint64_t off_sampler_keys = c.take(sampler_workspace_bytes(s->vocab));
  const uint64_t off_attn_trace = c.take(L * 32 * 8);
  {
    // Prompt blocks and batch steps need the matrix-core attention (head_dim 128, GQA factor
    // 1/2/4/8) and shapes the multi-row kernels take.
    const uint32_t group = s->heads / s->kv_heads;
    s->rows_ready = s->head_dim == 128 && (group == 1 || group == 2 || group == 4 || group == 8) && s->hidden <= 16384 &&
                    gemm_rows_supported(static_cast<uint32_t>(A + 2 * KV), s->hidden, 1) &&
                    gemm_rows_supported(s->hidden, static_cast<uint32_t>(A), 1) &&
                    gemm_rows_supported(s->intermediate, s->hidden, 1) &&
                    gemm_rows_supported(s->hidden, s->intermediate, 1);
  }
  const bool batch_head = s->rows_ready && gemm_rows_supported(s->vocab, s->hidden, 1);
  const uint64_t off_blogits = batch_head ? c.take(static_cast<uint64_t>(NERVA_HIP_BATCH_MAX_BLOCK_TOKENS) * V * 4) : 0;
  const uint64_t off_btable = c.take(sizeof(BatchTable));
  const uint64_t off_bslots = c.take(static_cast<uint64_t>(NERVA_HIP_BATCH_MAX_BLOCK_TOKENS) * sizeof(Slot));
  s->state_bytes = c.offset;
  s->arena_bytes = s->weights->bytes + s->state_bytes;

  *failure_stage = 2;
  hipError_t err = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
  if (err == hipSuccess && with_weights) {
    err = counted_malloc(reinterpret_cast<void **>(&s->weights->origin), kMatrixAlign + s->weights->bytes + s->state_bytes);
    if (err == hipSuccess) {
      const uint64_t lead = (kMatrixAlign - (reinterpret_cast<uintptr_t>(s->weights->origin) & (kMatrixAlign - 1))) & (kMatrixAlign - 1);
      s->weights->base = s->weights->origin + lead;
      s->arena = s->weights->base + s->weights->bytes;
      s->arena_in_weights = true;
    }
  } else if (err == hipSuccess) {
    err = counted_malloc(reinterpret_cast<void **>(&s->arena), s->state_bytes);
  }
  if (err != hipSuccess) return err;
  *failure_stage = 3;
  const uint64_t pinned_seq = (static_cast<uint64_t>(s->max_ctx) * (sizeof(Slot) + 4) + 256 + 255u) & ~uint64_t{255};
  const uint64_t pinned_table = (sizeof(BatchTable) + 255u) & ~uint64_t{255};
  s->pinned_bytes = pinned_seq + pinned_table + static_cast<uint64_t>(NERVA_HIP_BATCH_MAX_BLOCK_TOKENS) * sizeof(Slot);
  err = counted_host_malloc(reinterpret_cast<void **>(&s->pinned), s->pinned_bytes);
  if (err == hipSuccess) err = hipEventCreate(&s->ev0);
  if (err == hipSuccess) err = hipEventCreate(&s->ev1);
  if (err != hipSuccess) return err;
  s->host_slots = reinterpret_cast<Slot *>(s->pinned);
  s->host_prompt = reinterpret_cast<uint32_t *>(s->pinned + static_cast<uint64_t>(s->max_ctx) * sizeof(Slot));
  s->host_state = s->host_prompt + s->max_ctx;
  s->host_btable = reinterpret_cast<BatchTable *>(s->pinned + pinned_seq);
  s->host_bslots = reinterpret_cast<Slot *>(s->pinned + pinned_seq + pinned_table);

  auto dev16 = [&](uint64_t off) { return reinterpret_cast<uint16_t *>(s->arena + off); };
  s->kc = dev16(off_kc);
  s->vc = dev16(off_vc);
  s->table = reinterpret_cast<uint32_t *>(s->arena + off_table);
  s->prompt = reinterpret_cast<uint32_t *>(s->arena + off_prompt);
  s->slots = reinterpret_cast<Slot *>(s->arena + off_slots);
  s->state = reinterpret_cast<uint32_t *>(s->arena + off_state);
  s->x = reinterpret_cast<float *>(s->arena + off_x);
  s->r = reinterpret_cast<float *>(s->arena + off_r);
  s->qkv = reinterpret_cast<float *>(s->arena + off_qkv);
  s->logits = reinterpret_cast<float *>(s->arena + off_logits);
  s->attn16 = dev16(off_attn16);
  s->ff16 = dev16(off_ff16);
  s->rope_freq = reinterpret_cast<float *>(s->arena + off_rope);
  s->rope_cs = reinterpret_cast<float *>(s->arena + off_rope_cs);
  s->attn_ws = s->arena + off_attn_ws;
  s->attn_tagged = reinterpret_cast<uint64_t *>(s->arena + off_attn_tagged);
  {
    // the plan serves the step kernel (head_dim 128, 1, 2, 4 or 8 query heads per kv head, 8 waves)
    const uint32_t group = s->kv_heads != 0 ? s->heads / s->kv_heads : 0;
    if (s->head_dim == 128 && (group == 1 || group == 2 || group == 4 || group == 8))
      s->attn_plan = reinterpret_cast<uint32_t *>(s->arena + off_attn_plan);
  }
  s->sample_ws = s->arena + off_sample_ws;
  s->px = reinterpret_cast<float *>(s->arena + off_px);
  s->pr = reinterpret_cast<float *>(s->arena + off_pr);
  s->pqkv = reinterpret_cast<float *>(s->arena + off_pqkv);
  s->pxn16 = dev16(off_pxn16);
  s->pattn16 = dev16(off_pattn16);
  s->pff16 = dev16(off_pff16);
  s->prope = reinterpret_cast<float *>(s->arena + off_prope);
  s->pattn_ws = s->arena + off_pattn_ws;
  s->pattn_ws_stride = pattn_ws_stride;
  s->pgemm_ws = s->arena + off_pgemm_ws;
  s->pgemm_ws_bytes = pgemm_ws_bytes;
  // Prompt blocks of 512 tokens where all four projections of a layer have the kernel for them (256 weight rows x
  // 256 tokens a workgroup: half the X bytes per product of the 256-token kernel), else of 256 tokens where they
  // have that kernel (twice the tokens per weight byte of the 128-token one): Qwen3-8B widths qualify for both;
  // other widths keep 128-token blocks. The "prefill_block_tokens" override caps the choice at 128 or 256.
  const auto all_four = [&](uint32_t (*slices)(int, uint32_t, uint32_t, uint32_t, uint64_t), uint32_t tokens) {
    return slices(kGemmF32, static_cast<uint32_t>(A + 2 * KV), s->hidden, tokens, pgemm_ws_bytes) != 0 &&
           slices(kGemmResidual, s->hidden, static_cast<uint32_t>(A), tokens, pgemm_ws_bytes) != 0 &&
           slices(kGemmSwiglu, s->intermediate, s->hidden, tokens, pgemm_ws_bytes) != 0 &&
           slices(kGemmResidual, s->hidden, s->intermediate, tokens, pgemm_ws_bytes) != 0;
  };
  const int block_cap = tuning(kTunePrefillBlockTokens);
  const bool wide = block_cap != 128 && block_operand_tiles(kGemmWideMaxTokens) != 0 && all_four(gemm_wide_slices, kGemmWideMaxTokens);
  // (a prompt's last block can have any size: 512-token blocks only where the 256-token kernel takes the rest)
  const bool deep = wide && block_cap != 256 && block_operand_tiles(kGemmDeepMaxTokens) != 0 &&
                    all_four(gemm_deep_slices, kGemmDeepMaxTokens) && all_four(gemm_deep_slices, kGemmWideMaxTokens + 1);
  s->prefill_block_tokens = deep ? kGemmDeepMaxTokens : wide ? kGemmWideMaxTokens : kGemmMaxTokens;
  s->blogits = batch_head ? reinterpret_cast<float *>(s->arena + off_blogits) : nullptr;
  s->btable = reinterpret_cast<BatchTable *>(s->arena + off_btable);
  s->bslots = reinterpret_cast<Slot *>(s->arena + off_bslots);
  // ("prefill_walk" override = 1, read here: one prompt step per token where prompt blocks would be possible)
  s->block_prefill = s->rows_ready && tuning(kTunePrefillWalk) != 1;
  s->sampler_dev = reinterpret_cast<SamplerDev *>(s->arena + off_sampler_dev);
  s->sampler_keys = reinterpret_cast<uint64_t *>(s->arena + off_sampler_keys);
  {
    const char *trace = getenv("NERVA_HIP_ATTN_TRACE");
    if (s->layers > 0 && trace != nullptr && trace[0] == '1')
      s->attn_trace = reinterpret_cast<uint64_t *>(s->arena + off_attn_trace);
  }

  *failure_stage = 5;
  {
    std::vector<uint32_t> table(block_count);
    for (uint32_t i = 0; i < block_count; ++i) table[i] = i;  // identity (kernels.cu:733-739)
    err = hipMemcpy(s->table, table.data(), table.size() * 4, hipMemcpyHostToDevice);
  }
  if (err == hipSuccess && s->theta > 0.0f) {
    // powf(theta, 2i/d) evaluated once on the host in f32 (common/rope.rs:69-70); the
    // kernels divide the f32 position by it.
    std::vector<float> freq(HD / 2);
    for (uint32_t i = 0; i < HD / 2; ++i)
      freq[i] = powf(s->theta, static_cast<float>(2 * i) / static_cast<float>(HD));
    err = hipMemcpy(s->rope_freq, freq.data(), freq.size() * 4, hipMemcpyHostToDevice);
  }
  if (err == hipSuccess) err = hipMemsetAsync(s->arena + off_attn_ws, 0, attn_ws_bytes, s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->arena + off_attn_plan, 0, attn_plan_bytes(kAttnMaxSplits), s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->arena + off_attn_tagged, 0, attn_step_workspace_bytes(s->heads), s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->arena + off_sample_ws, 0, sample_workspace_bytes(), s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->arena + off_pattn_ws, 0, pT * pattn_ws_stride, s->stream);
  if (err == hipSuccess && L > 0) err = hipMemsetAsync(s->arena + off_attn_trace, 0, L * 32 * 8, s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->arena + off_kc, 0, 2 * ((kv_half + 255) & ~uint64_t{255}), s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->slots, 0, static_cast<uint64_t>(s->max_ctx) * sizeof(Slot), s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->state, 0, 64, s->stream);
  if (err == hipSuccess) err = hipMemsetAsync(s->sampler_dev, 0, sizeof(SamplerDev), s->stream);
  if (err == hipSuccess) err = hipStreamSynchronize(s->stream);
  return err;
}

void fill_create_result(const Session *s, NervaHipHfDecodeSequenceSessionCreateResult *out) {
  out->device_count = 1;
  out->dtype = s->dtype;
  out->hidden = s->hidden;
  out->heads = s->heads;
  out->kv_heads = s->kv_heads;
  out->head_dim = s->head_dim;
  out->intermediate = s->intermediate;
  out->vocab_size = s->vocab;
  out->layer_count = s->layers;
  out->max_context_tokens = s->max_ctx;
  out->prefill_chunk_tokens = s->block_prefill ? s->prefill_block_tokens : 1;
  out->head_threads = kBlock;
  out->resident_weight_bytes = s->resident_weight_bytes;
  out->planned_weight_blocks = s->planned_weight_blocks;
  out->planned_gpu_resident_blocks = s->planned_gpu_resident_blocks;
  out->planned_gpu_staged_blocks = s->planned_gpu_staged_blocks;
  out->planned_weight_bytes = s->planned_weight_bytes;
  out->planned_gpu_resident_weight_bytes = s->planned_gpu_resident_weight_bytes;
  out->planned_gpu_staged_weight_bytes = s->planned_gpu_staged_weight_bytes;
  out->descriptor_gpu_resident_h2d_bytes = s->planned_gpu_resident_weight_bytes;
  out->descriptor_gpu_staged_h2d_bytes = s->planned_gpu_staged_weight_bytes;
  out->planned_weight_descriptor_count = s->planned_weight_descriptor_count;
  out->planned_weight_descriptor_hash = s->planned_weight_descriptor_hash;
  out->resident_kv_bytes = s->kv_bytes;
  out->device_arena_bytes = s->arena_bytes;
  out->pinned_host_bytes = s->pinned_bytes;
  out->hot_path_allocations = 0;
  {
    // device-reported memory clock x bus width, like session_api_lifecycle.inc.cu:84-106
    int clock_khz = 0, bus_bits = 0;
    if (hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeMemoryClockRate, 0) == hipSuccess &&
        hipDeviceGetAttribute(&bus_bits, hipDeviceAttributeMemoryBusWidth, 0) == hipSuccess)
      out->device_memory_bandwidth_bps = static_cast<uint64_t>(clock_khz) * 1000ull * 2ull * (static_cast<uint64_t>(bus_bits) / 8ull);
  }
}

int create_impl(const NervaHipHfDecodeSequenceSessionCreateRequest *rq, bool synthetic, uint64_t seed,
                float weight_std, uint32_t with_qk_norm, NervaHipHfDecodeSequenceSessionCreateResult *out,
                Session **session_out) {
  if (!begin_result(out)) return -1;
  if (session_out == nullptr) return -1;
  *session_out = nullptr;
  out->failure_stage = 1;
  if (rq == nullptr || rq->dtype > 1 || rq->hidden == 0 || rq->heads == 0 || rq->kv_heads == 0 ||
      rq->head_dim == 0 || rq->intermediate == 0 || rq->vocab_size == 0 || rq->layer_count == 0 ||
      rq->max_context_tokens == 0 || rq->heads % rq->kv_heads != 0 || !(rq->rms_eps >= 0.0f) ||
      !isfinite(rq->rms_eps) || !isfinite(rq->rope_theta))
    return -1;
  if (rq->rope_theta > 0.0f && rq->head_dim % 2 != 0) return -1;
  // with a declared weight plan the descriptors are the source and the tensor pointers may be null
  const bool declared = !synthetic && weight_plan_declared(rq);
  if (!synthetic) {
    if (rq->layers == nullptr) return -1;
    if (!declared) {
      if (rq->embeddings == nullptr || rq->final_norm_weight == nullptr || rq->lm_head == nullptr) return -1;
      for (uint32_t l = 0; l < rq->layer_count; ++l)
        if (!layer_has_weights(rq->layers[l])) return -1;
    }
  }
  if (rq->planned_weight_descriptor_count != 0 && rq->planned_weight_descriptors == nullptr) return -1;
  // session_api_lifecycle.inc.cu:48-55: a declared plan is complete - one descriptor per block, a hash
  if (declared && (rq->planned_weight_blocks == 0 || rq->planned_weight_bytes == 0 || rq->planned_weight_descriptors == nullptr ||
                   rq->planned_weight_descriptor_count != rq->planned_weight_blocks || rq->planned_weight_descriptor_hash == 0))
    return -1;
  // explicit, never silent: features outside the dense full-attention path are refused
  bool supported = rq->experimental_rt_decode == 0 && rq->head_dim <= 512 &&
                   static_cast<uint64_t>(rq->intermediate) * 2 <= 60 * 1024 &&
                   static_cast<uint64_t>(rq->hidden) * 2 <= 60 * 1024 &&
                   static_cast<uint64_t>(rq->heads) * rq->head_dim * 2 <= 60 * 1024;
  if (!synthetic && rq->layers != nullptr)
    for (uint32_t l = 0; l < rq->layer_count && supported; ++l) supported = layer_supported(rq->layers[l]);
  if (!supported) {
    out->hip_error = NERVA_HIP_ERROR_NOT_SUPPORTED;
    return -1;
  }
  if (!device_ready(&out->hip_error)) return -1;
  out->device_count = 1;
  out->dtype = rq->dtype;
  out->hidden = rq->hidden;
  out->heads = rq->heads;
  out->kv_heads = rq->kv_heads;
  out->head_dim = rq->head_dim;
  out->intermediate = rq->intermediate;
  out->vocab_size = rq->vocab_size;
  out->layer_count = rq->layer_count;
  out->max_context_tokens = rq->max_context_tokens;
  out->prefill_chunk_tokens = 1;
  out->head_threads = kBlock;
  out->experimental_rt_decode_requested = rq->experimental_rt_decode;

  const uint64_t H = rq->hidden, A = static_cast<uint64_t>(rq->heads) * rq->head_dim,
                 KV = static_cast<uint64_t>(rq->kv_heads) * rq->head_dim, I = rq->intermediate,
                 V = rq->vocab_size, L = rq->layer_count, HD = rq->head_dim;

  Session *s = new (std::nothrow) Session();
  if (s == nullptr) return -1;
  s->weights = new (std::nothrow) SharedWeights();
  if (s->weights == nullptr) {
    delete s;
    return -1;
  }
  s->dtype = rq->dtype;
  s->hidden = rq->hidden;
  s->heads = rq->heads;
  s->kv_heads = rq->kv_heads;
  s->head_dim = rq->head_dim;
  s->intermediate = rq->intermediate;
  s->vocab = rq->vocab_size;
  s->layers = rq->layer_count;
  s->max_ctx = rq->max_context_tokens;
  s->eps = rq->rms_eps;
  s->theta = rq->rope_theta;
  s->planned_weight_blocks = rq->planned_weight_blocks;
  s->planned_gpu_resident_blocks = rq->planned_gpu_resident_blocks;
  s->planned_gpu_staged_blocks = rq->planned_gpu_staged_blocks;
  s->planned_weight_bytes = rq->planned_weight_bytes;
  s->planned_gpu_resident_weight_bytes = rq->planned_gpu_resident_weight_bytes;
  s->planned_gpu_staged_weight_bytes = rq->planned_gpu_staged_weight_bytes;
  s->planned_weight_descriptor_count = rq->planned_weight_descriptor_count;
  s->planned_weight_descriptor_hash = rq->planned_weight_descriptor_hash;

  // ---- weight arena layout -------------------------------------------------
  struct LayerOff {
    uint64_t rms_attn, rms_mlp, wqkv, q_norm, k_norm, q_bias, k_bias, v_bias, wo, o_bias, wgu, wdown;
  };
  const uint64_t kNone = ~uint64_t{0};
  Carver c;
  uint64_t weight_elems = 0;
  // (matrices of a few MiB - test models - take 8 KiB boundaries instead)
  auto matrix = [&](uint64_t bytes) { return c.take(bytes, bytes >= kMatrixAlign ? kMatrixAlign : 8192u); };
  s->pair_gap = I * H * 2 >= kMatrixAlign ? kPairGapElems : 0u;
  const uint64_t gap_bytes = s->pair_gap * 2ull;
  const uint64_t off_emb = matrix(V * H * 2);
  weight_elems += V * H;
  std::vector<LayerOff> lo(L);
  for (uint32_t l = 0; l < L; ++l) {
    const NervaHipHfDecodeChainLayer *src = synthetic ? nullptr : &rq->layers[l];
    lo[l].rms_attn = c.take(H * 2);
    lo[l].rms_mlp = c.take(H * 2);
    lo[l].wqkv = matrix((A + 2 * KV) * H * 2);
    const bool qn = synthetic ? with_qk_norm != 0 : src->q_norm_weight != nullptr;
    const bool kn = synthetic ? with_qk_norm != 0 : src->k_norm_weight != nullptr;
    lo[l].q_norm = qn ? c.take(HD * 2) : kNone;
    lo[l].k_norm = kn ? c.take(HD * 2) : kNone;
    lo[l].q_bias = (!synthetic && src->q_bias) ? c.take(A * 2) : kNone;
    lo[l].k_bias = (!synthetic && src->k_bias) ? c.take(KV * 2) : kNone;
    lo[l].v_bias = (!synthetic && src->v_bias) ? c.take(KV * 2) : kNone;
    lo[l].wo = matrix(H * A * 2);
    lo[l].o_bias = (!synthetic && src->o_bias) ? c.take(H * 2) : kNone;
    lo[l].wgu = matrix(2 * I * H * 2 + gap_bytes);
    lo[l].wdown = matrix(H * I * 2);
    weight_elems += 2 * H + (A + 2 * KV) * H + H * A + 3 * I * H;
    if (qn) weight_elems += HD;
    if (kn) weight_elems += HD;
    if (lo[l].q_bias != kNone) weight_elems += A;
    if (lo[l].k_bias != kNone) weight_elems += KV;
    if (lo[l].v_bias != kNone) weight_elems += KV;
    if (lo[l].o_bias != kNone) weight_elems += H;
  }
  const uint64_t off_final = c.take(H * 2);
  const uint64_t off_lm = matrix(V * H * 2);
  weight_elems += H + V * H;
  s->resident_weight_bytes = weight_elems * 2;
  s->weights->bytes = c.offset;

  if (declared && !validate_weight_descriptors(rq, s->resident_weight_bytes)) {
    // session_api_lifecycle.inc.cu:156: a weight plan that disagrees with the arena or with its own
    // descriptors is rejected before anything is allocated
    destroy_session(s);
    return -1;
  }

  out->failure_stage = 2;
  hipError_t err = setup_state(s, &out->failure_stage, true);
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    destroy_session(s);
    return -1;
  }

  char *wbase = s->weights->base;
  auto w16 = [&](uint64_t off) -> const uint16_t * { return off == kNone ? nullptr : reinterpret_cast<const uint16_t *>(wbase + off); };
  s->emb = w16(off_emb);
  s->final_norm = w16(off_final);
  s->lm_head = w16(off_lm);
  s->layer.resize(L);
  for (uint32_t l = 0; l < L; ++l) {
    s->layer[l] = LayerDev{w16(lo[l].rms_attn), w16(lo[l].rms_mlp), w16(lo[l].wqkv),
                           w16(lo[l].q_norm),   w16(lo[l].k_norm),  w16(lo[l].q_bias),
                           w16(lo[l].k_bias),   w16(lo[l].v_bias),  w16(lo[l].wo),
                           w16(lo[l].o_bias),   w16(lo[l].wgu),     w16(lo[l].wdown)};
  }

  // ---- weights -------------------------------------------------------------
  out->failure_stage = 4;
  uint64_t h2d = 0;
  auto upload = [&](uint64_t off, const uint16_t *src, uint64_t elems) {
    if (err != hipSuccess || off == kNone) return;
    err = hipMemcpy(wbase + off, src, elems * 2, hipMemcpyHostToDevice);
    h2d += elems * 2;
  };
  auto fill = [&](uint64_t off, uint64_t tensor_id, uint64_t elems, float mean) {
    if (err != hipSuccess || off == kNone) return;
    err = launch_synth_16(wbase + off, s->dtype, seed, tensor_id, elems, mean, weight_std, s->stream);
  };
  uint64_t setup_syncs = 1;
  if (declared) {
    // the reference's arena order, piece by piece, onto this library's layout
    std::vector<WeightSegment> segments;
    uint64_t logical = 0;
    auto segment = [&](uint64_t off, uint64_t elems) {
      if (off == kNone) return;
      segments.push_back(WeightSegment{logical, elems * 2, wbase + off});
      logical += elems * 2;
    };
    segment(off_emb, V * H);
    for (uint32_t l = 0; l < L; ++l) {
      segment(lo[l].rms_attn, H);
      segment(lo[l].wqkv, A * H);
      segment(lo[l].q_norm, HD);
      segment(lo[l].wqkv + A * H * 2, KV * H);
      segment(lo[l].k_norm, HD);
      segment(lo[l].wqkv + (A + KV) * H * 2, KV * H);
      segment(lo[l].wo, H * A);
      segment(lo[l].rms_mlp, H);
      segment(lo[l].wgu, I * H);
      segment(lo[l].wgu + I * H * 2 + gap_bytes, I * H);
      segment(lo[l].wdown, H * I);
      segment(lo[l].q_bias, A);
      segment(lo[l].k_bias, KV);
      segment(lo[l].v_bias, KV);
      segment(lo[l].o_bias, H);
    }
    segment(off_final, H);
    segment(off_lm, V * H);
    err = logical == s->resident_weight_bytes ? copy_weight_descriptors(rq, segments, s->stream, &h2d, &setup_syncs)
                                              : hipErrorInvalidValue;
  } else if (synthetic) {
    fill(off_emb, 1, V * H, 0.0f);
    fill(off_final, 2, H, 1.0f);
    fill(off_lm, 3, V * H, 0.0f);
    for (uint32_t l = 0; l < L; ++l) {
      const uint64_t base = 16ull * (l + 1);
      fill(lo[l].rms_attn, base + 0, H, 1.0f);
      fill(lo[l].rms_mlp, base + 1, H, 1.0f);
      fill(lo[l].wqkv, base + 2, A * H, 0.0f);
      fill(lo[l].wqkv + A * H * 2, base + 4, KV * H, 0.0f);
      fill(lo[l].q_norm, base + 5, HD, 1.0f);
      fill(lo[l].k_norm, base + 6, HD, 1.0f);
      fill(lo[l].wqkv + (A + KV) * H * 2, base + 7, KV * H, 0.0f);
      fill(lo[l].wo, base + 8, H * A, 0.0f);
      fill(lo[l].wgu, base + 13, I * H, 0.0f);
      fill(lo[l].wgu + I * H * 2 + gap_bytes, base + 14, I * H, 0.0f);
      fill(lo[l].wdown, base + 15, H * I, 0.0f);
    }
    if (err == hipSuccess) err = hipStreamSynchronize(s->stream);
  } else {
    upload(off_emb, rq->embeddings, V * H);
    upload(off_final, rq->final_norm_weight, H);
    upload(off_lm, rq->lm_head, V * H);
    for (uint32_t l = 0; l < L; ++l) {
      const NervaHipHfDecodeChainLayer &src = rq->layers[l];
      upload(lo[l].rms_attn, src.rms_attn_weight, H);
      upload(lo[l].rms_mlp, src.rms_mlp_weight, H);
      // [q; k; v] rows back to back = one (A + 2KV) x H matrix (kernels.cu:741-769)
      upload(lo[l].wqkv, src.w_q, A * H);
      upload(lo[l].wqkv + A * H * 2, src.w_k, KV * H);
      upload(lo[l].wqkv + (A + KV) * H * 2, src.w_v, KV * H);
      upload(lo[l].q_norm, src.q_norm_weight, HD);
      upload(lo[l].k_norm, src.k_norm_weight, HD);
      upload(lo[l].q_bias, src.q_bias, A);
      upload(lo[l].k_bias, src.k_bias, KV);
      upload(lo[l].v_bias, src.v_bias, KV);
      upload(lo[l].wo, src.w_o, H * A);
      upload(lo[l].o_bias, src.o_bias, H);
      // [gate; up] rows back to back (kernels.cu:771-802)
      upload(lo[l].wgu, src.w_gate, I * H);
      upload(lo[l].wgu + I * H * 2 + gap_bytes, src.w_up, I * H);
      upload(lo[l].wdown, src.w_down, H * I);
    }
  }
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    destroy_session(s);
    return -1;
  }
  out->failure_stage = 0;
  fill_create_result(s, out);
  out->h2d_bytes = h2d;
  out->sync_calls = setup_syncs;
  out->status = 0;
  *session_out = s;
  return 0;
}


// One decode step for `T` sequences on the weights and workspaces of `lead`: the token rows of all
// sequences go through every projection as one multi-row GEMM (one stream of the weights for all),
// attention runs per sequence on its own cache and position inside one launch, and every sequence
// samples with its own sampler. Decode staging (f32 hidden state between layers), like enqueue_step.
// Reference: session_api_layer_projection_batch.inc.cu (qkv, o, gate/up, down per layer) and
// session_api_batch_fork_destroy.inc.cu:166-259 (layers, LM head, one sampler launch per session).
hipError_t enqueue_batch_step(Session *lead, Session *const *seqs, uint32_t T,
                              NervaHipHfDecodeSequenceBatchAdvanceResult *out) {
  hipStream_t st = lead->stream;
  const uint32_t H = lead->hidden, A = lead->heads * lead->head_dim, KV = lead->kv_heads * lead->head_dim,
                 I = lead->intermediate;
  const float *rope_freq = lead->theta > 0.0f ? lead->rope_freq : nullptr;
  const uint32_t tiles = block_operand_tiles(T);
  BatchTable *host = lead->host_btable;
  uint32_t min_blocks = ~0u;
  for (uint32_t t = 0; t < T; ++t) {
    const Session *q = seqs[t];
    host->seq[t] = AttnSeq{q->kc, q->vc, q->table, q->block_count, q->cursor};
    host->slots[t] = q->slots;
    // slot[position], cursor -> position + 1, with the sequence's own sampler and random-number counter
    SamplerParams &sp = host->sample[t];
    sp = SamplerParams{};
    sp.logits = lead->blogits + static_cast<uint64_t>(t) * lead->vocab;
    sp.vocab = q->vocab;
    sp.config = q->sampler_dev;
    sp.keys = q->sampler_keys;
    sample_bind_workspace(sp.out, q->sample_ws);
    sp.out.slots = q->slots;
    sp.out.cursor_rw = q->state;
    sp.out.fault = q->state + 3;
    sp.cursor = q->state;
    sp.max_steps = q->max_ctx;
    min_blocks = std::min(min_blocks, q->block_count);
  }
  // kv_heads x T workgroups per split already fill the chip at T = 32; measured on MI355X (Qwen3-8B
  // shapes, contexts 128 .. 8192) further splits only add merge work, so: as many as it takes to reach
  // one workgroup per CU
  uint32_t batch_splits = std::max<uint32_t>(1u, std::min<uint32_t>(attn_default_splits(lead->kv_heads, min_blocks),
                                                                   (256u + lead->kv_heads * T - 1) / (lead->kv_heads * T)));
  if (const int want = tuning(kTuneBatchSplits); want >= 1 && want <= static_cast<int>(kAttnMaxSplits))
    batch_splits = std::min<uint32_t>(static_cast<uint32_t>(want), min_blocks);
  hipError_t err = hipMemcpyAsync(lead->btable, host, sizeof(BatchTable), hipMemcpyHostToDevice, st);
  if (err != hipSuccess) return err;
  if (lead->dtype == kBF16)
    hipLaunchKernelGGL(embed_batch_kernel<kBF16>, dim3(T), dim3(kBlock), 0, st, lead->emb, lead->btable, H, lead->vocab,
                       lead->px, rope_freq, lead->prope, lead->head_dim / 2);
  else
    hipLaunchKernelGGL(embed_batch_kernel<kF16>, dim3(T), dim3(kBlock), 0, st, lead->emb, lead->btable, H, lead->vocab,
                       lead->px, rope_freq, lead->prope, lead->head_dim / 2);
  err = hipGetLastError();
  out->pack_kernel_launches += 1;
  // where the down projection's K slices are added by a launch of their own, that launch writes the RMSNorm that
  // follows as well (the next layer's attention norm, or the final norm): one launch less per layer
  const bool down_norms = gemm_rows_fuses_norm(kGemmResidual, H, I, T, tiles, lead->pgemm_ws_bytes);
  const bool o_norms = gemm_rows_fuses_norm(kGemmResidual, H, A, T, tiles, lead->pgemm_ws_bytes);   // likewise the MLP norm
  // where the q/k/v projection runs in a few K slices the attention adds them as it reads its inputs: no launch of
  // its own for that
  uint32_t qkv_slice_stride = 0;
  const uint32_t qkv_slices = gemm_rows_partial_slices(A + 2 * KV, H, T, tiles, lead->pgemm_ws_bytes, &qkv_slice_stride);
  for (uint32_t l = 0; err == hipSuccess && l < lead->layers; ++l) {
    const LayerDev &w = lead->layer[l];
    if (l == 0 || !down_norms) err = launch_rmsnorm_rows(lead->dtype, lead->px, w.rms_attn, lead->eps, T, H, lead->pxn16, st, tiles);
    GemmRowsParams g{};
    if (err == hipSuccess) {
      g.tokens = T;
      g.w = w.wqkv;
      g.x16 = lead->pxn16;
      g.x_packed = tiles;
      g.out_f32 = lead->pqkv;
      g.rows = A + 2 * KV;
      g.cols = H;
      g.workspace = lead->pgemm_ws;
      g.workspace_bytes = lead->pgemm_ws_bytes;
      g.keep_partials = qkv_slices != 0;
      err = launch_gemm_rows(lead->dtype, kGemmF32, g, st);
    }
    AttnParams a{};
    a.heads = lead->heads;
    a.kv_heads = lead->kv_heads;
    a.head_dim = lead->head_dim;
    attn_bind_workspace(a, lead->pattn_ws);
    a.qkv = qkv_slices != 0 ? reinterpret_cast<const float *>(lead->pgemm_ws) : lead->pqkv;
    a.qkv_slices = qkv_slices;
    a.qkv_slice_stride = qkv_slice_stride;
    a.q_norm = w.q_norm;
    a.k_norm = w.k_norm;
    a.q_bias = w.q_bias;
    a.k_bias = w.k_bias;
    a.v_bias = w.v_bias;
    a.rope_freq = rope_freq;
    a.rope_cs = rope_freq != nullptr ? lead->prope : nullptr;
    a.out16 = lead->pattn16;
    a.layer = l;
    a.splits = batch_splits;
    a.eps = lead->eps;
    a.tokens = T;
    a.qkv_token_stride = A + 2 * KV;
    a.out_token_stride = A;
    a.rope_token_stride = lead->head_dim;
    a.ws_token_stride = lead->pattn_ws_stride;
    a.seqs = lead->btable->seq;
    a.out_packed_tiles = tiles;
    a.append = 1;  // each sequence's K/V row goes into its own cache inside the attention launch
    if (err == hipSuccess) err = launch_attn_decode(lead->dtype, a, st);
    if (err == hipSuccess) {
      g = GemmRowsParams{};
      g.tokens = T;
      g.w = w.wo;
      g.x16 = lead->pattn16;
      g.x_packed = tiles;
      g.bias = w.o_bias;
      g.residual = lead->px;
      g.out_f32 = lead->pr;
      g.rows = H;
      g.cols = A;
      g.workspace = lead->pgemm_ws;
      g.workspace_bytes = lead->pgemm_ws_bytes;
      if (o_norms) {
        g.norm_gamma = w.rms_mlp;
        g.norm_out16 = lead->pxn16;
        g.norm_eps = lead->eps;
        g.norm_packed_tiles = tiles;
      }
      err = launch_gemm_rows(lead->dtype, kGemmResidual, g, st);
    }
    if (err == hipSuccess && !o_norms)
      err = launch_rmsnorm_rows(lead->dtype, lead->pr, w.rms_mlp, lead->eps, T, H, lead->pxn16, st, tiles);
    if (err == hipSuccess) {
      g = GemmRowsParams{};
      g.tokens = T;
      g.w = w.wgu;
      g.pair_gap = lead->pair_gap;
      g.x16 = lead->pxn16;
      g.x_packed = tiles;
      g.out16 = lead->pff16;
      g.out_packed_tiles = tiles;
      g.rows = I;
      g.cols = H;
      g.workspace = lead->pgemm_ws;
      g.workspace_bytes = lead->pgemm_ws_bytes;
      err = launch_gemm_rows(lead->dtype, kGemmSwiglu, g, st);
    }
    if (err == hipSuccess) {
      g = GemmRowsParams{};
      g.tokens = T;
      g.w = w.wdown;
      g.x16 = lead->pff16;
      g.x_packed = tiles;
      g.residual = lead->pr;
      g.out_f32 = lead->px;
      g.rows = H;
      g.cols = I;
      g.workspace = lead->pgemm_ws;
      g.workspace_bytes = lead->pgemm_ws_bytes;
      if (down_norms) {
        g.norm_gamma = l + 1 < lead->layers ? lead->layer[l + 1].rms_attn : lead->final_norm;
        g.norm_out16 = lead->pxn16;
        g.norm_eps = lead->eps;
        g.norm_packed_tiles = tiles;
      }
      err = launch_gemm_rows(lead->dtype, kGemmResidual, g, st);
    }
    out->pack_kernel_launches += (down_norms && l != 0 ? 0 : 1) + (o_norms ? 0 : 1);
    out->projection_kernel_launches += 4;
    out->dependency_kernel_launches += 1;
  }
  if (err == hipSuccess && !down_norms)
    err = launch_rmsnorm_rows(lead->dtype, lead->px, lead->final_norm, lead->eps, T, H, lead->pxn16, st, tiles);
  if (err == hipSuccess) {
    GemmRowsParams g{};
    g.tokens = T;
    g.w = lead->lm_head;
    g.x16 = lead->pxn16;
    g.x_packed = tiles;
    g.out_f32 = lead->blogits;
    g.rows = lead->vocab;
    g.cols = H;
    g.workspace = lead->pgemm_ws;
    g.workspace_bytes = lead->pgemm_ws_bytes;
    err = launch_gemm_rows(lead->dtype, kGemmF32, g, st);
    out->pack_kernel_launches += 1;
    out->projection_kernel_launches += 1;
  }
  if (err == hipSuccess) {
    err = launch_sampler_batch(lead->btable->sample, T, lead->vocab, st);
    out->sampling_kernel_launches += 2;
  }
  return err;
}

}  // namespace

extern "C" {

int nerva_hip_hf_decode_sequence_session_fork_shared_weights(
    const NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest *request,
    NervaHipHfDecodeSequenceSessionCreateResult *out, NervaHipHfDecodeSequenceSession **session_out) {
  if (!begin_result(out)) return -1;
  if (session_out == nullptr) return -1;
  *session_out = nullptr;
  out->failure_stage = 1;
  if (request == nullptr || request->parent == nullptr || request->parent->weights == nullptr) return -1;
  Session *parent = request->parent;
  // session_api_batch_fork_destroy.inc.cu:331-333: a sequence under way is carried over
  const bool clone = parent->started && !parent->finished && parent->prompt_count != 0;
  if (!device_ready(&out->hip_error)) return -1;

  Session *s = new (std::nothrow) Session();
  if (s == nullptr) return -1;
  s->dtype = parent->dtype;
  s->hidden = parent->hidden;
  s->heads = parent->heads;
  s->kv_heads = parent->kv_heads;
  s->head_dim = parent->head_dim;
  s->intermediate = parent->intermediate;
  s->pair_gap = parent->pair_gap;
  s->vocab = parent->vocab;
  s->layers = parent->layers;
  s->max_ctx = parent->max_ctx;
  s->eps = parent->eps;
  s->theta = parent->theta;
  s->planned_weight_blocks = parent->planned_weight_blocks;
  s->planned_gpu_resident_blocks = parent->planned_gpu_resident_blocks;
  s->planned_gpu_staged_blocks = parent->planned_gpu_staged_blocks;
  s->planned_weight_bytes = parent->planned_weight_bytes;
  s->planned_gpu_resident_weight_bytes = parent->planned_gpu_resident_weight_bytes;
  s->planned_gpu_staged_weight_bytes = parent->planned_gpu_staged_weight_bytes;
  s->planned_weight_descriptor_count = parent->planned_weight_descriptor_count;
  s->planned_weight_descriptor_hash = parent->planned_weight_descriptor_hash;
  s->resident_weight_bytes = parent->resident_weight_bytes;
  s->weights = parent->weights;
  s->weights->refs.fetch_add(1);
  s->emb = parent->emb;
  s->final_norm = parent->final_norm;
  s->lm_head = parent->lm_head;
  s->layer = parent->layer;

  hipError_t err = setup_state(s, &out->failure_stage, false);
  uint64_t syncs = 1;
  if (err == hipSuccess && clone) {
    err = hipStreamSynchronize(parent->stream);
    syncs += 1;
    memcpy(s->host_slots, parent->host_slots, static_cast<uint64_t>(s->max_ctx) * sizeof(Slot));
    const uint64_t kv_half = s->kv_bytes / 2;
    auto copy = [&](void *dst, const void *src, uint64_t bytes) {
      if (err == hipSuccess) err = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s->stream);
    };
    copy(s->prompt, parent->prompt, static_cast<uint64_t>(s->max_ctx) * 4);
    copy(s->slots, parent->slots, static_cast<uint64_t>(s->max_ctx) * sizeof(Slot));
    copy(s->state, parent->state, 64);
    copy(s->kc, parent->kc, kv_half);
    copy(s->vc, parent->vc, kv_half);
    copy(s->sampler_dev, parent->sampler_dev, sizeof(SamplerDev));
    s->sampler = parent->sampler;
    s->prompt_count = parent->prompt_count;
    s->has_eos = parent->has_eos;
    s->eos = parent->eos;
    s->seed_token = parent->seed_token;
    s->observed = parent->observed;
    s->cursor = parent->cursor;
    s->started = parent->started;
    s->finished = parent->finished;
    if (err == hipSuccess) err = hipStreamSynchronize(s->stream);
  }
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    destroy_session(s);
    return -1;
  }
  out->failure_stage = 0;
  fill_create_result(s, out);
  out->sync_calls = syncs;
  out->status = 0;
  *session_out = s;
  return 0;
}

int nerva_hip_hf_decode_sequence_batch_advance_one(const NervaHipHfDecodeSequenceBatchAdvanceRequest *request,
                                                   NervaHipHfDecodeSequenceBatchAdvanceResult *out) {
  if (!begin_result(out)) return -1;
  out->reason = NERVA_HIP_BATCH_INVALID_REQUEST;
  if (request == nullptr) return -1;
  out->requested_session_count = request->session_count;
  out->target_block_tokens = request->target_block_tokens == 0 ? 1u : request->target_block_tokens;
  out->min_block_tokens = request->min_block_tokens == 0 ? 1u : request->min_block_tokens;
  if (request->session_count == 0) {
    out->reason = NERVA_HIP_BATCH_NO_SESSIONS;
    out->status = 0;
    return 0;
  }
  if (request->sessions == nullptr || request->output_tokens == nullptr ||
      request->output_token_capacity < request->session_count)
    return -1;
  if (!device_ready(&out->hip_error)) return -1;
  out->device_count = 1;

  // session_api_batch_fork_destroy.inc.cu:33-45: everything computed so far has been handed out
  auto ready = [](const Session *q) {
    return q != nullptr && q->started && !q->finished && q->prompt_count != 0 && q->cursor < q->max_ctx &&
           static_cast<uint64_t>(q->prompt_count) + q->observed == static_cast<uint64_t>(q->cursor) + 1u;
  };
  // :46-61: same weights by descriptor hash, same dimensions
  auto same_model = [](const Session *a, const Session *b) {
    return a->planned_weight_descriptor_hash != 0 && a->planned_weight_descriptor_hash == b->planned_weight_descriptor_hash &&
           a->dtype == b->dtype && a->hidden == b->hidden && a->heads == b->heads && a->kv_heads == b->kv_heads &&
           a->head_dim == b->head_dim && a->intermediate == b->intermediate && a->vocab == b->vocab &&
           a->layers == b->layers && a->resident_weight_bytes == b->resident_weight_bytes;
  };
  uint32_t ready_count = 0;
  bool any_hash = false;
  for (uint32_t i = 0; i < request->session_count; ++i) {
    const Session *q = request->sessions[i];
    if (!ready(q)) continue;
    ready_count += 1;
    any_hash = any_hash || q->planned_weight_descriptor_hash != 0;
  }
  if (ready_count == 0) {
    out->reason = NERVA_HIP_BATCH_NO_READY_SESSIONS;
    out->status = 0;
    return 0;
  }
  if (!any_hash) {
    out->reason = NERVA_HIP_BATCH_SHARED_WEIGHTS_UNPROVEN;
    out->status = 0;
    return 0;
  }
  Session *lead = nullptr;
  uint32_t lead_count = 0;
  for (uint32_t i = 0; i < request->session_count; ++i) {
    Session *candidate = request->sessions[i];
    if (!ready(candidate) || candidate->planned_weight_descriptor_hash == 0) continue;
    uint32_t compatible = 0;
    for (uint32_t j = 0; j < request->session_count; ++j)
      if (ready(request->sessions[j]) && same_model(candidate, request->sessions[j])) compatible += 1;
    if (compatible > lead_count) {
      lead = candidate;
      lead_count = compatible;
    }
  }
  out->eligible_session_count = lead_count;
  if (lead == nullptr || lead_count < out->min_block_tokens) {
    out->reason = NERVA_HIP_BATCH_INSUFFICIENT_COMPATIBLE_READY;
    out->status = 0;
    return 0;
  }
  const uint32_t max_tokens = std::min<uint32_t>(out->target_block_tokens, NERVA_HIP_BATCH_MAX_BLOCK_TOKENS);
  uint32_t picked[NERVA_HIP_BATCH_MAX_BLOCK_TOKENS];
  Session *seqs[NERVA_HIP_BATCH_MAX_BLOCK_TOKENS];
  uint32_t T = 0;
  for (uint32_t i = 0; i < request->session_count && T < max_tokens; ++i) {
    Session *q = request->sessions[i];
    if (!ready(q) || !same_model(lead, q)) continue;
    bool twice = false;  // a session listed twice advances once
    for (uint32_t t = 0; t < T; ++t) twice = twice || seqs[t] == q;
    if (twice) continue;
    picked[T] = i;
    seqs[T] = q;
    T += 1;
  }
  if (T < out->min_block_tokens) {
    out->reason = NERVA_HIP_BATCH_INSUFFICIENT_COMPATIBLE_READY;
    out->status = 0;
    return 0;
  }
  out->reason = NERVA_HIP_BATCH_READY;
  out->exact = 1;
  out->block_tokens = T;
  out->dtype = lead->dtype;
  out->layer_count = lead->layers;

  const uint64_t allocs_before = allocation_count();
  hipError_t err = hipSuccess;
  // work the sequences queued on their own streams comes first
  for (uint32_t t = 0; err == hipSuccess && t < T; ++t) {
    if (seqs[t] == lead) continue;
    err = hipStreamSynchronize(seqs[t]->stream);
    out->sync_calls += 1;
  }
  const bool shared = lead->rows_ready && lead->blogits != nullptr;
  if (err == hipSuccess && shared) {
    err = hipEventRecord(lead->ev0, lead->stream);
    if (err == hipSuccess) err = enqueue_batch_step(lead, seqs, T, out);
    if (err == hipSuccess) err = hipEventRecord(lead->ev1, lead->stream);
    if (err == hipSuccess) {   // the published slots: gathered on the device, one copy, dealt out on the host
      constexpr uint32_t kWords = sizeof(Slot) / sizeof(uint32_t);
      hipLaunchKernelGGL(gather_slots_kernel, dim3((T * kWords + 255u) / 256u), dim3(256), 0, lead->stream, lead->btable, T,
                         lead->bslots);
      err = hipGetLastError();
      out->pack_kernel_launches += 1;
    }
    if (err == hipSuccess)
      err = hipMemcpyAsync(lead->host_bslots, lead->bslots, static_cast<size_t>(T) * sizeof(Slot), hipMemcpyDeviceToHost,
                           lead->stream);
    out->d2h_bytes += static_cast<uint64_t>(T) * sizeof(Slot);
    if (err == hipSuccess) err = hipStreamSynchronize(lead->stream);
    out->sync_calls += 1;
    for (uint32_t t = 0; err == hipSuccess && t < T; ++t) seqs[t]->host_slots[seqs[t]->cursor] = lead->host_bslots[t];
    if (err == hipSuccess) {
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, lead->ev0, lead->ev1) == hipSuccess && ms > 0.0f)
        out->projection_elapsed_ns = std::max<uint64_t>(1, static_cast<uint64_t>(static_cast<double>(ms) * 1e6));
    }
  } else if (err == hipSuccess) {
    // shapes outside the multi-row kernels: every sequence runs its own captured step on its own stream - one
    // after the other (each stream waits for the step before it): a step's attention launch wants every CU for
    // workgroups that poll for each other, and two such launches side by side could hold each other's CUs
    NervaHipHfDecodeSequenceResult scratch{};
    Session *before = nullptr;
    for (uint32_t t = 0; err == hipSuccess && t < T; ++t) {
      Session *q = seqs[t];
      err = ensure_graph(q, decode_graph(q), &scratch);
      if (err == hipSuccess && before != nullptr) err = hipStreamWaitEvent(q->stream, before->ev1, 0);
      if (err == hipSuccess) err = launch_step(q, decode_graph(q), &scratch);
      if (err == hipSuccess) err = hipEventRecord(q->ev1, q->stream);
      before = q;
      if (err == hipSuccess)
        err = hipMemcpyAsync(&q->host_slots[q->cursor], &q->slots[q->cursor], sizeof(Slot), hipMemcpyDeviceToHost,
                             q->stream);
      out->d2h_bytes += sizeof(Slot);
      out->pack_kernel_launches += 1;
      out->projection_kernel_launches += 4ull * q->layers + 1;
      out->dependency_kernel_launches += q->layers;
      out->sampling_kernel_launches += q->sampler.mode == kSamplerGreedy ? 1 : 2;
    }
    for (uint32_t t = 0; err == hipSuccess && t < T; ++t) {
      err = hipStreamSynchronize(seqs[t]->stream);
      out->sync_calls += 1;
    }
  }
  out->hot_path_allocations = allocation_count() - allocs_before;
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    out->exact = 0;
    return -1;
  }
  uint32_t observed[NERVA_HIP_BATCH_MAX_BLOCK_TOKENS];
  for (uint32_t t = 0; t < T; ++t) {
    Session *q = seqs[t];
    const uint32_t at = q->cursor;  // = prompt_count - 1 + observed
    const Slot &slot = q->host_slots[at];
    if (!slots_consistent(&slot, 1, at)) {
      if (slots_faulted(&slot, 1)) out->hip_error = NERVA_HIP_ERROR_STEP_FAULT;
      out->status = -1;
      return -1;
    }
    request->output_tokens[picked[t]] = slot.token;
    observed[t] = slot.token;
    out->last_token = slot.token;
    q->observed += 1;
    q->cursor += 1;
    q->finished = (q->has_eos != 0 && slot.token == q->eos) || at + 1u >= q->max_ctx;
    out->observed_tokens += 1;
  }
  out->observed_token_hash = fnv1a_bytes(observed, static_cast<size_t>(T) * 4);
  out->status = out->observed_tokens == out->block_tokens ? 0 : -1;
  return out->status == 0 ? 0 : -1;
}

int nerva_hip_hf_decode_sequence_session_create(const NervaHipHfDecodeSequenceSessionCreateRequest *request,
                                                NervaHipHfDecodeSequenceSessionCreateResult *out,
                                                NervaHipHfDecodeSequenceSession **session) {
  return create_impl(request, false, 0, 0.0f, 0, out, session);
}

int nerva_hip_bench_session_create_synthetic(const NervaHipHfDecodeSequenceSessionCreateRequest *request,
                                             uint64_t seed, float weight_std, uint32_t with_qk_norm,
                                             NervaHipHfDecodeSequenceSessionCreateResult *out,
                                             NervaHipHfDecodeSequenceSession **session) {
  return create_impl(request, true, seed, weight_std, with_qk_norm, out, session);
}

int nerva_hip_hf_decode_sequence_session_destroy(NervaHipHfDecodeSequenceSession *session,
                                                 NervaHipHfDecodeSequenceSessionCreateResult *out) {
  if (out != nullptr) {
    memset(out, 0, sizeof(*out));
    out->status = -1;
  }
  if (session == nullptr) return -1;
  if (out != nullptr) {
    out->device_count = 1;
    out->dtype = session->dtype;
    out->hidden = session->hidden;
    out->heads = session->heads;
    out->kv_heads = session->kv_heads;
    out->head_dim = session->head_dim;
    out->intermediate = session->intermediate;
    out->vocab_size = session->vocab;
    out->layer_count = session->layers;
    out->max_context_tokens = session->max_ctx;
    out->resident_weight_bytes = session->resident_weight_bytes;
    out->resident_kv_bytes = session->kv_bytes;
    out->device_arena_bytes = session->arena_bytes;
    out->pinned_host_bytes = session->pinned_bytes;
    out->sync_calls = 1;
    out->status = 0;
  }
  destroy_session(session);
  return 0;
}

int nerva_hip_hf_decode_sequence_session_start(const NervaHipHfDecodeSequenceSessionStartRequest *request,
                                               NervaHipHfDecodeSequenceResult *out) {
  if (!begin_result(out)) return -1;
  if (request == nullptr || request->session == nullptr || request->prompt_tokens == nullptr ||
      request->prompt_token_count == 0)
    return -1;
  Session *s = request->session;
  if (request->prompt_token_count > s->max_ctx) return -1;
  for (uint32_t i = 0; i < request->prompt_token_count; ++i)
    if (request->prompt_tokens[i] >= s->vocab) return -1;
  const uint32_t P = request->prompt_token_count;
  fill_header(s, out, 0, request->prompt_tokens[P - 1]);
  s->started = false;
  hipError_t err = set_sampler(s, request->sampler);   // session_api_lifecycle.inc.cu:1026
  if (err == hipSuccess) err = reset_sequence(s, request->prompt_tokens, P, out);
  // prefill: the first P-1 prompt tokens (in blocks on the matrix cores where the shapes allow,
  // else one captured prompt step per token), then one prompt step with the LM head and sampler
  if (err == hipSuccess && P > 1 && !s->block_prefill) err = ensure_graph(s, 1, out);
  if (err == hipSuccess) err = hipEventRecord(s->ev0, s->stream);
  if (s->block_prefill) {
    if (err == hipSuccess && P > 1) err = prefill_blocks(s, P - 1, P, out);
  } else {
    for (uint32_t i = 0; err == hipSuccess && i + 1 < P; ++i) err = launch_step(s, 1, out);
  }
  if (err == hipSuccess) err = enqueue_step(s, kPromptHeadStep, nullptr);
  if (err == hipSuccess) out->kernel_launches += step_launches(s, 0);
  if (err == hipSuccess) err = hipEventRecord(s->ev1, s->stream);
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    return -1;
  }
  s->prompt_count = P;
  s->has_eos = request->has_eos_token;
  s->eos = request->eos_token;
  s->seed_token = request->prompt_tokens[P - 1];
  s->observed = 0;
  s->cursor = P;
  s->started = true;
  s->finished = false;
  out->resident_kv_bytes = s->kv_bytes;
  out->kv_tokens = P;
  out->device_arena_bytes = s->arena_bytes;
  out->pinned_host_bytes = static_cast<uint64_t>(s->max_ctx) * sizeof(Slot);
  out->status = 0;
  return 0;
}

int nerva_hip_hf_decode_sequence_session_advance(const NervaHipHfDecodeSequenceSessionAdvanceRequest *request,
                                                 NervaHipHfDecodeSequenceResult *out) {
  if (!begin_result(out)) return -1;
  if (request == nullptr || request->session == nullptr || request->output_tokens == nullptr ||
      request->steps == 0 || request->output_token_capacity < request->steps)
    return -1;
  Session *s = request->session;
  if (!s->started || s->finished || s->prompt_count == 0) return -1;
  const uint32_t P = s->prompt_count;
  const uint32_t slot_start = P - 1u + s->observed;
  const uint64_t target64 = static_cast<uint64_t>(P) + s->observed + request->steps - 1u;
  if (target64 > s->max_ctx || target64 < s->cursor) return -1;
  const uint32_t target = static_cast<uint32_t>(target64);
  const uint32_t run_count = target - s->cursor;
  const uint32_t seed = s->observed == 0 ? s->seed_token : s->host_slots[slot_start - 1u].token;
  fill_header(s, out, request->steps, seed);

  hipError_t err = hipSuccess;
  if (run_count != 0) err = ensure_graph(s, decode_graph(s), out);
  const uint64_t allocs_before = allocation_count();
  if (err == hipSuccess && run_count != 0) err = hipEventRecord(s->ev0, s->stream);
  for (uint32_t step = 0; err == hipSuccess && step < run_count; ++step) {
    err = launch_step(s, decode_graph(s), out);
    // With a stop token the host looks at each token so that it can stop launching
    // (session_api_lifecycle.inc.cu:1206-1234); without one the loop never syncs.
    if (err == hipSuccess && s->has_eos != 0) {
      const uint32_t pos = s->cursor + step;
      err = hipMemcpyAsync(&s->host_slots[pos], &s->slots[pos], sizeof(Slot), hipMemcpyDeviceToHost, s->stream);
      if (err == hipSuccess) err = hipStreamSynchronize(s->stream);
      out->sync_calls += 1;
      out->d2h_bytes += sizeof(Slot);
      if (err == hipSuccess && s->host_slots[pos].completion == NERVA_HIP_SLOT_DEVICE_COMPLETE &&
          s->host_slots[pos].token == s->eos)
        break;
    }
  }
  if (err == hipSuccess && run_count != 0) err = hipEventRecord(s->ev1, s->stream);
  const uint64_t slots_bytes = static_cast<uint64_t>(request->steps) * sizeof(Slot);
  if (err == hipSuccess) {
    err = hipMemcpyAsync(s->host_slots + slot_start, s->slots + slot_start, slots_bytes,
                         hipMemcpyDeviceToHost, s->stream);
    out->d2h_bytes += slots_bytes;
  }
  if (err == hipSuccess) {
    err = hipStreamSynchronize(s->stream);
    out->sync_calls += 1;
  }
  out->hot_path_allocations = allocation_count() - allocs_before;
  if (err == hipSuccess && run_count != 0) {
    float ms = 0.0f;
    err = hipEventElapsedTime(&ms, s->ev0, s->ev1);
    if (err == hipSuccess && ms > 0.0f) {
      out->device_elapsed_ns = static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
      if (out->device_elapsed_ns == 0) out->device_elapsed_ns = 1;
    }
  }
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    return -1;
  }
  const Slot *observed = s->host_slots + slot_start;
  out->observed_tokens = observed_count(request->steps, s->has_eos, s->eos, observed);
  for (uint32_t i = 0; i < out->observed_tokens; ++i) request->output_tokens[i] = observed[i].token;
  out->last_token = out->observed_tokens == 0 ? 0 : request->output_tokens[out->observed_tokens - 1];
  out->observed_token_hash = fnv1a_bytes(request->output_tokens, static_cast<size_t>(out->observed_tokens) * 4);
  out->resident_kv_bytes = s->kv_bytes;
  out->kv_tokens = slot_start + out->observed_tokens;
  out->device_arena_bytes = s->arena_bytes;
  out->pinned_host_bytes = static_cast<uint64_t>(s->max_ctx) * sizeof(Slot);
  out->host_causality_edges = 0;
  out->status = out->observed_tokens > 0 && slots_consistent(observed, out->observed_tokens, slot_start) ? 0 : -1;
  if (slots_faulted(observed, request->steps)) {
    // a device-side bounded wait gave up in one of these steps: its token and everything after it is void, and
    // the sequence ends here (start() clears the fault)
    out->status = -1;
    out->hip_error = NERVA_HIP_ERROR_STEP_FAULT;
    s->finished = true;
  }
  if (out->status == 0) {
    s->observed += out->observed_tokens;
    s->cursor = out->observed_tokens < request->steps ? s->max_ctx : target;
    s->finished = out->observed_tokens < request->steps || out->kv_tokens >= s->max_ctx;
  }
  return out->status == 0 ? 0 : -1;
}

int nerva_hip_hf_decode_sequence_session_run(const NervaHipHfDecodeSequenceSessionRunRequest *request,
                                             NervaHipHfDecodeSequenceResult *out) {
  if (!begin_result(out)) return -1;
  if (request == nullptr || request->session == nullptr || request->prompt_tokens == nullptr ||
      request->output_tokens == nullptr || request->steps == 0 || request->prompt_token_count == 0 ||
      request->output_token_capacity < request->steps ||
      request->prompt_tokens[request->prompt_token_count - 1u] != request->seed_token ||
      request->prompt_token_count > UINT32_MAX - request->steps + 1u)
    return -1;
  Session *s = request->session;
  const uint32_t P = request->prompt_token_count;
  const uint32_t context_steps = P + request->steps - 1u;
  if (context_steps > s->max_ctx) return -1;
  for (uint32_t i = 0; i < P; ++i)
    if (request->prompt_tokens[i] >= s->vocab) return -1;
  fill_header(s, out, request->steps, request->seed_token);
  s->started = false;
  hipError_t err = set_sampler(s, request->sampler);   // session_api_lifecycle.inc.cu:770
  if (err == hipSuccess) err = reset_sequence(s, request->prompt_tokens, P, out);
  // the decode-step graph walks every position, prompt included (session_api_lifecycle.inc.cu:748-990)
  if (err == hipSuccess) err = ensure_graph(s, decode_graph(s), out);
  const uint64_t allocs_before = allocation_count();
  if (err == hipSuccess) err = hipEventRecord(s->ev0, s->stream);
  for (uint32_t step = 0; err == hipSuccess && step < context_steps; ++step) {
    err = launch_step(s, decode_graph(s), out);
  }
  if (err == hipSuccess) err = hipEventRecord(s->ev1, s->stream);
  const uint64_t slots_bytes = static_cast<uint64_t>(context_steps) * sizeof(Slot);
  if (err == hipSuccess) {
    err = hipMemcpyAsync(s->host_slots, s->slots, slots_bytes, hipMemcpyDeviceToHost, s->stream);
    out->d2h_bytes = slots_bytes;
  }
  if (err == hipSuccess) {
    err = hipStreamSynchronize(s->stream);
    out->sync_calls += 1;
  }
  out->hot_path_allocations = allocation_count() - allocs_before;
  if (err == hipSuccess) {
    float ms = 0.0f;
    err = hipEventElapsedTime(&ms, s->ev0, s->ev1);
    if (err == hipSuccess && ms > 0.0f) out->device_elapsed_ns = std::max<uint64_t>(1, static_cast<uint64_t>(static_cast<double>(ms) * 1e6));
  }
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    return -1;
  }
  const uint32_t output_start = P - 1u;
  const Slot *observed = s->host_slots + output_start;
  out->observed_tokens = observed_count(request->steps, request->has_eos_token, request->eos_token, observed);
  for (uint32_t i = 0; i < out->observed_tokens; ++i) request->output_tokens[i] = observed[i].token;
  out->last_token = out->observed_tokens == 0 ? 0 : request->output_tokens[out->observed_tokens - 1];
  out->observed_token_hash = fnv1a_bytes(request->output_tokens, static_cast<size_t>(out->observed_tokens) * 4);
  out->resident_kv_bytes = s->kv_bytes;
  out->kv_tokens = output_start + out->observed_tokens;
  out->device_arena_bytes = s->arena_bytes;
  out->pinned_host_bytes = static_cast<uint64_t>(s->max_ctx) * sizeof(Slot);
  out->host_causality_edges = 0;
  out->status = out->observed_tokens > 0 && slots_consistent(observed, out->observed_tokens, output_start) ? 0 : -1;
  if (slots_faulted(observed, request->steps)) {
    out->status = -1;
    out->hip_error = NERVA_HIP_ERROR_STEP_FAULT;
  }
  return out->status == 0 ? 0 : -1;
}

int nerva_hip_hf_decode_sequence_u16(const NervaHipHfDecodeSequenceRequest *rq, NervaHipHfDecodeSequenceResult *out) {
  if (!begin_result(out)) return -1;
  if (rq == nullptr || rq->prompt_tokens == nullptr || rq->prompt_token_count == 0 || rq->steps == 0 ||
      rq->output_tokens == nullptr || rq->output_token_capacity < rq->steps ||
      rq->prompt_token_count > UINT32_MAX - rq->steps + 1u)
    return -1;
  NervaHipHfDecodeSequenceSessionCreateRequest cr{};
  cr.dtype = rq->dtype;
  cr.hidden = rq->hidden;
  cr.heads = rq->heads;
  cr.kv_heads = rq->kv_heads;
  cr.head_dim = rq->head_dim;
  cr.intermediate = rq->intermediate;
  cr.vocab_size = rq->vocab_size;
  cr.layer_count = rq->layer_count;
  cr.max_context_tokens = rq->prompt_token_count + rq->steps - 1u;
  cr.rms_eps = rq->rms_eps;
  cr.rope_theta = rq->rope_theta;
  cr.embeddings = rq->embeddings;
  cr.layers = rq->layers;
  cr.final_norm_weight = rq->final_norm_weight;
  cr.lm_head = rq->lm_head;
  cr.planned_weight_blocks = rq->planned_weight_blocks;
  cr.planned_gpu_resident_blocks = rq->planned_gpu_resident_blocks;
  cr.planned_gpu_staged_blocks = rq->planned_gpu_staged_blocks;
  cr.planned_weight_bytes = rq->planned_weight_bytes;
  cr.planned_gpu_resident_weight_bytes = rq->planned_gpu_resident_weight_bytes;
  cr.planned_gpu_staged_weight_bytes = rq->planned_gpu_staged_weight_bytes;
  cr.planned_weight_descriptors = rq->planned_weight_descriptors;
  cr.planned_weight_descriptor_count = rq->planned_weight_descriptor_count;
  cr.planned_weight_descriptor_hash = rq->planned_weight_descriptor_hash;
  NervaHipHfDecodeSequenceSessionCreateResult cres;
  Session *s = nullptr;
  if (create_impl(&cr, false, 0, 0.0f, 0, &cres, &s) != 0) {
    out->hip_error = cres.hip_error;
    out->device_count = cres.device_count;
    return -1;
  }
  NervaHipHfDecodeSequenceSessionRunRequest run{};
  run.session = s;
  run.steps = rq->steps;
  run.seed_token = rq->seed_token;
  run.prompt_tokens = rq->prompt_tokens;
  run.prompt_token_count = rq->prompt_token_count;
  run.has_eos_token = rq->has_eos_token;
  run.eos_token = rq->eos_token;
  run.output_tokens = rq->output_tokens;
  run.output_token_capacity = rq->output_token_capacity;
  run.sampler = rq->sampler;
  const int rc = nerva_hip_hf_decode_sequence_session_run(&run, out);
  if (rc == 0) out->h2d_bytes += cres.h2d_bytes;
  destroy_session(s);
  return rc;
}

int nerva_hip_session_profile_step(NervaHipHfDecodeSequenceSession *s, uint32_t repeats, NervaHipStepProfile *out) {
  if (!begin_result(out)) return -1;
  if (s == nullptr || repeats == 0 || !s->started) return -1;
  hipError_t err = hipStreamSynchronize(s->stream);
  uint32_t pos = 0;
  if (err == hipSuccess) err = hipMemcpy(&pos, s->state, 4, hipMemcpyDeviceToHost);
  if (err == hipSuccess && pos >= s->max_ctx) err = hipErrorInvalidValue;
  Slot saved;
  if (err == hipSuccess) err = hipMemcpy(&saved, s->slots + pos, sizeof(Slot), hipMemcpyDeviceToHost);
  StepProfiler prof;
  prof.stream = s->stream;
  uint64_t sums[kLKinds] = {0};
  uint64_t counts[kLKinds] = {0};
  uint64_t total = 0;
  for (uint32_t rep = 0; err == hipSuccess && rep < repeats + 1; ++rep) {  // first pass is a warm-up
    prof.used = 0;
    prof.kinds.clear();
    err = enqueue_step(s, kDecodeStep, &prof);
    if (err == hipSuccess) err = hipStreamSynchronize(s->stream);
    // undo the step: cursor and the published slot
    if (err == hipSuccess) err = hipMemcpy(s->state, &pos, 4, hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(s->slots + pos, &saved, sizeof(Slot), hipMemcpyHostToDevice);
    if (err != hipSuccess || rep == 0) continue;
    for (size_t i = 0; i < prof.kinds.size(); ++i) {
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, prof.events[2 * i], prof.events[2 * i + 1]) == hipSuccess) {
        sums[prof.kinds[i]] += static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
        counts[prof.kinds[i]] += 1;
      }
    }
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, prof.events[0], prof.events[prof.used - 1]) == hipSuccess)
      total += static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
    out->launches = static_cast<uint32_t>(prof.kinds.size());
  }
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    return -1;
  }
  // back-to-back pass: all `layers` launches of one kind between a single event pair, so the
  // figure is the kernel's own duration without the per-launch event gaps
  uint64_t stream_ns[kLKinds] = {0};
  for (int kind = kLQkv; err == hipSuccess && kind <= kLDown; ++kind) {
    const uint32_t launches = s->layers;
    uint64_t acc = 0;
    for (uint32_t rep = 0; err == hipSuccess && rep < repeats + 1; ++rep) {
      // no embed launch in this pass: advance the step counter here
      hipLaunchKernelGGL(bump_step_counter_kernel, dim3(1), dim3(64), 0, s->stream, s->state, s->attn_plan);
      err = hipGetLastError();
      if (err == hipSuccess) err = hipEventRecord(s->ev0, s->stream);
      if (err == hipSuccess) err = enqueue_step(s, kDecodeStep, nullptr, kind);
      if (err == hipSuccess) err = hipEventRecord(s->ev1, s->stream);
      if (err == hipSuccess) err = hipStreamSynchronize(s->stream);
      float ms = 0.0f;
      if (err == hipSuccess) err = hipEventElapsedTime(&ms, s->ev0, s->ev1);
      if (rep > 0) acc += static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
    }
    stream_ns[kind] = acc / (static_cast<uint64_t>(repeats) * launches);
  }
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    return -1;
  }
  if (s->attn_trace != nullptr) {
    // timestamps (10 ns ticks from the launch's earliest mark) of: qkv workgroup 0 [0..3] and the last
    // one's end [4]; attention (kv head 0, split 0) [8..13]; the merging workgroup of kv head 0 [16..18];
    // first [20..23] and last [24..27] o workgroup
    std::vector<uint64_t> tr(static_cast<size_t>(s->layers) * 32);
    if (hipMemcpy(tr.data(), s->attn_trace, tr.size() * 8, hipMemcpyDeviceToHost) == hipSuccess) {
      for (uint32_t l = 0; l < s->layers && l < 4; ++l) {
        const uint64_t *t = tr.data() + 32 * l;
        uint64_t first = ~uint64_t{0};
        for (int i = 0; i < 28; ++i)
          if (t[i] > 1000000 && t[i] < first) first = t[i];
        fprintf(stderr, "[attention trace] layer %u:", l);
        for (int i = 0; i < 28; ++i) {
          if (i == 8 || i == 16 || i == 20 || i == 24) fprintf(stderr, " |");
          if (t[i] > 1000000) fprintf(stderr, " %lld", static_cast<long long>(t[i] - first));
          else if (t[i] != 0) fprintf(stderr, " #%lld", static_cast<long long>(t[i]));
          else fprintf(stderr, " -");
        }
        fprintf(stderr, "\n");
      }
    }
  }
  err = hipStreamSynchronize(s->stream);
  if (err != hipSuccess) {
    out->hip_error = static_cast<int32_t>(err);
    return -1;
  }
  out->qkv_stream_ns = stream_ns[kLQkv];
  out->attention_stream_ns = stream_ns[kLAttn];
  out->o_stream_ns = stream_ns[kLO];
  out->gate_up_stream_ns = stream_ns[kLGateUp];
  out->down_stream_ns = stream_ns[kLDown];
  auto avg = [&](int k) { return counts[k] ? sums[k] / counts[k] : 0; };
  out->position = pos;
  out->embed_ns = avg(kLEmbed);
  out->qkv_ns = avg(kLQkv);
  out->attention_ns = avg(kLAttn);
  out->o_ns = avg(kLO);
  out->gate_up_ns = avg(kLGateUp);
  out->down_ns = avg(kLDown);
  out->lm_head_ns = avg(kLHead);
  out->total_ns = total / repeats;
  const uint64_t H = s->hidden, A = static_cast<uint64_t>(s->heads) * s->head_dim,
                 KV = static_cast<uint64_t>(s->kv_heads) * s->head_dim, I = s->intermediate, V = s->vocab;
  // algorithmic bytes per launch: weights + input vector + output vector (+ norm weights / residual)
  out->qkv_bytes = (A + 2 * KV) * H * 2 + H * 4 + H * 2 + (A + 2 * KV) * 4;
  out->attention_bytes = 2 * (static_cast<uint64_t>(pos) + 1) * KV * 2 + (A + 2 * KV) * 4 + 2 * KV * 2 + A * 2;
  out->o_bytes = H * A * 2 + A * 2 + H * 4 + H * 4;
  out->gate_up_bytes = 2 * I * H * 2 + H * 4 + H * 2 + I * 2;
  out->down_bytes = H * I * 2 + I * 2 + H * 4 + H * 4;
  out->lm_head_bytes = V * H * 2 + H * 4 + H * 2 + V * 4;
  out->status = 0;
  return 0;
}

int nerva_hip_session_shares_weight_stream(NervaHipHfDecodeSequenceSession *s) {
  if (s == nullptr) return -1;
  return s->rows_ready && s->blogits != nullptr ? 1 : 0;
}

int nerva_hip_steps_are_eager(void) { return eager_steps() ? 1 : 0; }

uint64_t nerva_hip_session_step_trace_bytes(NervaHipHfDecodeSequenceSession *s) {
  if (s == nullptr) return 0;
  auto slot = [](uint64_t bytes) { return (bytes + 255u) & ~uint64_t{255}; };
  const uint64_t A = static_cast<uint64_t>(s->heads) * s->head_dim, KV = static_cast<uint64_t>(s->kv_heads) * s->head_dim;
  const uint64_t per_layer = slot(s->hidden * 2ull) + slot((A + 2 * KV) * 4) + slot(A * 2) + slot(s->hidden * 4ull) +
                             slot(s->hidden * 2ull) + slot(s->intermediate * 2ull) + slot(s->hidden * 4ull);
  return slot(s->hidden * 4ull) + per_layer * s->layers + slot(s->hidden * 2ull) + slot(s->vocab * 4ull);
}

int nerva_hip_session_trace_next_step(NervaHipHfDecodeSequenceSession *s, void *device_buffer, uint64_t bytes) {
  if (s == nullptr) return -1;
  if (device_buffer == nullptr) {  // disarm
    s->trace_buf = nullptr;
    return 0;
  }
  if (bytes < nerva_hip_session_step_trace_bytes(s)) return -1;
  if (s->sampler.mode != kSamplerGreedy) return -1;  // the greedy step only
  s->trace_buf = static_cast<char *>(device_buffer);
  s->trace_used = 0;
  return 0;
}

int nerva_hip_session_read_logits(NervaHipHfDecodeSequenceSession *s, float *host_logits) {
  if (s == nullptr || host_logits == nullptr) return -1;
  if (hipStreamSynchronize(s->stream) != hipSuccess) return -1;
  return hipMemcpy(host_logits, s->logits, static_cast<uint64_t>(s->vocab) * 4, hipMemcpyDeviceToHost) == hipSuccess ? 0 : -1;
}

int nerva_hip_session_read_slots(NervaHipHfDecodeSequenceSession *s, uint32_t first, uint32_t count,
                                 NervaHipSyntheticTokenSlot *host_slots) {
  if (s == nullptr || host_slots == nullptr || static_cast<uint64_t>(first) + count > s->max_ctx) return -1;
  if (count == 0) return 0;
  if (hipStreamSynchronize(s->stream) != hipSuccess) return -1;
  return hipMemcpy(host_slots, s->slots + first, static_cast<uint64_t>(count) * sizeof(Slot), hipMemcpyDeviceToHost) == hipSuccess ? 0 : -1;
}

int nerva_hip_session_read_kv_range(NervaHipHfDecodeSequenceSession *s, uint32_t layer, uint32_t first_token,
                                    uint32_t token_count, uint16_t *host_k, uint16_t *host_v) {
  if (s == nullptr || host_k == nullptr || host_v == nullptr || layer >= s->layers ||
      static_cast<uint64_t>(first_token) + token_count > s->max_ctx)
    return -1;
  if (token_count == 0) return 0;
  if (hipStreamSynchronize(s->stream) != hipSuccess) return -1;
  const uint32_t hd = s->head_dim, kvh = s->kv_heads;
  const uint64_t KV = static_cast<uint64_t>(kvh) * hd;
  const uint32_t b0 = first_token / kKvBlockTokens, b1 = (first_token + token_count - 1) / kKvBlockTokens;
  // one layer's blocks are contiguous (identity table): copy them whole, then reorder on the host
  const uint64_t per_block = KV * kKvBlockTokens;
  std::vector<uint16_t> kimg((b1 - b0 + 1) * per_block), vimg((b1 - b0 + 1) * per_block);
  const uint64_t off = kv_tile_offset(s->block_count, kvh, hd, layer, b0, 0);
  if (hipMemcpy(kimg.data(), s->kc + off, kimg.size() * 2, hipMemcpyDeviceToHost) != hipSuccess) return -1;
  if (hipMemcpy(vimg.data(), s->vc + off, vimg.size() * 2, hipMemcpyDeviceToHost) != hipSuccess) return -1;
  // in-tile element order of one row, computed once per row index
  std::vector<uint32_t> kmap(kKvBlockTokens * hd), vmap(kKvBlockTokens * hd);
  for (uint32_t row = 0; row < kKvBlockTokens; ++row)
    for (uint32_t d = 0; d < hd; ++d) {
      kmap[row * hd + d] = kv_k_elem(hd, row, d);
      vmap[row * hd + d] = kv_v_elem(hd, row, d);
    }
  for (uint32_t t = 0; t < token_count; ++t) {
    const uint32_t tok = first_token + t, blk = tok / kKvBlockTokens - b0, row = tok % kKvBlockTokens;
    for (uint32_t h = 0; h < kvh; ++h) {
      const uint64_t tile = (static_cast<uint64_t>(blk) * kvh + h) * kKvBlockTokens * hd;
      uint16_t *dk = host_k + t * KV + h * hd, *dv = host_v + t * KV + h * hd;
      for (uint32_t d = 0; d < hd; ++d) {
        dk[d] = kimg[tile + kmap[row * hd + d]];
        dv[d] = vimg[tile + vmap[row * hd + d]];
      }
    }
  }
  return 0;
}

int nerva_hip_session_read_kv(NervaHipHfDecodeSequenceSession *s, uint32_t layer, uint32_t token,
                              uint16_t *host_k, uint16_t *host_v) {
  return nerva_hip_session_read_kv_range(s, layer, token, 1, host_k, host_v);
}

}  // extern "C"
