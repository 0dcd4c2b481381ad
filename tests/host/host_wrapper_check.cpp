// Exercises the C++ host wrapper (nerva_amd/host/nerva_hip.hpp) the way the reference's Rust tests
// exercise its safe wrappers (crates/nerva-cuda/src/tests/decode_sequence_session.rs:21-86,
// decode_sequence.rs:123-223). Mode "cpu": everything that must hold without a device
// (validation before the call, Unavailable when there is no GPU). Mode "gpu": the reference's
// greedy-stream known-answer model through create / start / advance / run.
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "nerva_hip.hpp"

using namespace nerva::hip;

static int failures = 0;
#define CHECK(cond)                                                       \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
      ++failures;                                                         \
    }                                                                     \
  } while (0)

struct KatModel {
  // hidden 2, vocab 4, f16: embeddings [1,0; 0,1; -1,0; 0,-1], layer matrices 0, lm_head [0,-1; 1,0; 0,1; -1,0]
  std::vector<uint16_t> emb{0x3c00, 0x0000, 0x0000, 0x3c00, 0xbc00, 0x0000, 0x0000, 0xbc00};
  std::vector<uint16_t> rms{0x3c00, 0x3c00};
  std::vector<uint16_t> zero{0, 0, 0, 0};
  std::vector<uint16_t> head{0x0000, 0xbc00, 0x3c00, 0x0000, 0x0000, 0x3c00, 0xbc00, 0x0000};
  HipHfDecodeSequenceSessionConfig config() const {
    HipHfDecodeSequenceSessionConfig c;
    c.dtype = NERVA_HIP_DTYPE_F16;
    c.hidden = 2;
    c.heads = 1;
    c.kv_heads = 1;
    c.head_dim = 2;
    c.intermediate = 2;
    c.vocab_size = 4;
    c.max_context_tokens = 16;
    c.rms_eps = 1e-5f;
    c.embeddings = emb;
    c.final_norm_weight = rms;
    c.lm_head = head;
    HipHfDecodeChainLayer l;
    l.rms_attn_weight = rms;
    l.rms_mlp_weight = rms;
    l.w_q = l.w_k = l.w_v = l.w_o = l.w_gate = l.w_up = l.w_down = zero;
    c.layers.push_back(l);
    return c;
  }
  // decode_sequence_descriptor_blocks.rs:223-258: one block per tensor in arena order, the first six
  // GPU-resident, the rest GPU-staged
  std::vector<HipHfDecodeSequenceWeightBlock> blocks() const {
    const uint64_t bytes[12] = {16, 4, 8, 8, 8, 8, 4, 8, 8, 8, 4, 16};
    const std::vector<uint16_t> *sources[12] = {&emb, &rms, &zero, &zero, &zero, &zero, &rms, &zero, &zero, &zero, &rms, &head};
    std::vector<HipHfDecodeSequenceWeightBlock> out;
    uint64_t offset = 0;
    for (int i = 0; i < 12; ++i) {
      HipHfDecodeSequenceWeightBlock b{};
      b.host_source = sources[i]->data();
      b.block_id = static_cast<uint64_t>(i) + 1;
      b.offset_bytes = offset;
      b.bytes = bytes[i];
      b.strategy = i < 6 ? HIP_HF_WEIGHT_STRATEGY_GPU_RESIDENT : HIP_HF_WEIGHT_STRATEGY_GPU_STAGED;
      out.push_back(b);
      offset += bytes[i];
    }
    return out;
  }
  static HipHfDecodeSequenceWeightPlan plan(const std::vector<HipHfDecodeSequenceWeightBlock> &blocks) {
    HipHfDecodeSequenceWeightPlan p;
    p.blocks = 12;
    p.gpu_resident_blocks = 6;
    p.gpu_staged_blocks = 6;
    p.weight_bytes = 100;
    p.gpu_resident_weight_bytes = 52;
    p.gpu_staged_weight_bytes = 48;
    p.descriptor_hash = hash_weight_blocks(blocks);
    return p;
  }
};

static void cpu_checks() {
  KatModel m;
  // validation happens before any native call
  HipHfDecodeSequenceSessionConfig bad = m.config();
  bad.kv_heads = 0;
  auto out = bad.create();
  CHECK(out.summary.status == SmokeStatus::Failed && out.summary.error.has_value() && !out.session);
  bad = m.config();
  bad.layers[0].w_q = Span<uint16_t>(m.zero.data(), 3);
  out = bad.create();
  CHECK(out.summary.status == SmokeStatus::Failed && out.summary.error->find("wrong size") != std::string::npos);
  HipHfDecodeSamplerConfig sampler;
  sampler.top_p = 0.0f;
  CHECK(sampler.validate().has_value());
  CHECK(!HipHfDecodeSamplerConfig::greedy().validate().has_value());
  std::vector<uint32_t> none, outside{7};
  CHECK(detail::validate_loop_start(none, 4).has_value());
  CHECK(detail::validate_loop_start(outside, 4).has_value());
  // weight plan: validated before the call (weight_plan.rs:53-100)
  {
    const std::vector<HipHfDecodeSequenceWeightBlock> blocks = m.blocks();
    HipHfDecodeSequenceSessionConfig planned = m.config();
    planned.weight_plan = KatModel::plan(blocks);
    planned.weight_blocks = blocks;
    CHECK(!planned.validate().has_value());
    planned.embeddings = Span<uint16_t>();          // with a declared plan the tensor spans are not looked at
    CHECK(!planned.validate().has_value());
    planned.weight_plan->descriptor_hash ^= 1;
    CHECK(planned.validate().value_or("").find("hash") != std::string::npos);
    planned.weight_plan = KatModel::plan(blocks);
    planned.weight_plan->blocks = 11;
    CHECK(planned.validate().value_or("").find("count") != std::string::npos);
    planned.weight_plan = KatModel::plan(blocks);
    planned.weight_plan->gpu_staged_blocks = 7;
    CHECK(planned.validate().value_or("").find("block counts") != std::string::npos);
    planned.weight_plan = KatModel::plan(blocks);
    planned.weight_plan->descriptor_hash = 0;
    CHECK(planned.validate().value_or("").find("incomplete") != std::string::npos);
    std::vector<HipHfDecodeSequenceWeightBlock> sourceless = blocks;
    sourceless[3].host_source = nullptr;
    planned.weight_plan = KatModel::plan(sourceless);
    planned.weight_blocks = sourceless;
    CHECK(planned.validate().value_or("").find("source") != std::string::npos);
    CHECK(hash_weight_blocks(Span<HipHfDecodeSequenceWeightBlock>()) == 0xcbf29ce484222325ull);
  }
  // a batch step over nothing is answered without a device (decode_sequence_session.rs:61-86)
  HipHfDecodeSequenceBatchAdvanceSummary nothing = HipHfDecodeSequenceSession::batch_advance_one({}, 8, 2);
  CHECK(nothing.status == SmokeStatus::Ok && nothing.reason == "no_sessions" && !nothing.exact);
  CHECK(nothing.requested_session_count == 0 && nothing.block_tokens == 0 && nothing.observed_tokens == 0);
  CHECK(nothing.tokens.empty() && nothing.hot_path_allocations == 0);
  nothing = HipHfDecodeSequenceLoop::batch_advance_one({}, 8, 2);
  CHECK(nothing.status == SmokeStatus::Ok && nothing.reason == "no_sessions" && nothing.tokens.empty());
  // no device: Unavailable, never a crash, never a silent success
  const HipDeviceSmokeSummary smoke = device_smoke();
  if (smoke.status != SmokeStatus::Ok) {
    CHECK(smoke.status == SmokeStatus::Unavailable);
    out = m.config().create();
    CHECK(out.summary.status == SmokeStatus::Unavailable && !out.session);
    CHECK(out.summary.hip_error == NERVA_HIP_ERROR_NO_DEVICE);
  }
}

static void gpu_checks() {
  KatModel m;
  CHECK(device_smoke().status == SmokeStatus::Ok);
  auto created = m.config().create();
  CHECK(created.summary.status == SmokeStatus::Ok && created.session);
  if (!created.session) return;
  CHECK(created.summary.hot_path_allocations == 0 && created.summary.resident_weight_bytes == 100);
  HipHfDecodeSequenceSession &session = *created.session;
  std::vector<uint32_t> prompt{0};
  // one-call run: [1, 2, 3, 0]
  HipHfDecodeSequenceSummary run = session.run(prompt, 4);
  CHECK(run.status == SmokeStatus::Ok && run.tokens == std::vector<uint32_t>({1, 2, 3, 0}));
  CHECK(run.graph_replays == 4 && run.sync_calls == 1 && run.hot_path_allocations == 0 && run.host_causality_edges == 0);
  // with a stop token the stream ends at it
  run = session.run(prompt, 4, 2u);
  CHECK(run.status == SmokeStatus::Ok && run.tokens == std::vector<uint32_t>({1, 2}) && run.kv_tokens == 2);
  // loop: start, then advance in pieces; a finished loop refuses to advance
  auto started = HipHfDecodeSequenceLoop::start(session, prompt, 3u);
  CHECK(started.summary.status == SmokeStatus::Ok && started.loop_state.has_value());
  if (started.loop_state) {
    HipHfDecodeSequenceSummary a = started.loop_state->advance(2);
    CHECK(a.status == SmokeStatus::Ok && a.tokens == std::vector<uint32_t>({1, 2}));
    HipHfDecodeSequenceSummary b = started.loop_state->advance(4);
    CHECK(b.status == SmokeStatus::Ok && b.tokens == std::vector<uint32_t>({3}) && started.loop_state->finished());
    CHECK(started.loop_state->advance(1).status == SmokeStatus::Failed);
  }
  // refusal before the call: prompt outside the vocabulary
  std::vector<uint32_t> outside{9};
  CHECK(HipHfDecodeSequenceLoop::start(session, outside).summary.status == SmokeStatus::Failed);
  // temperature sampling: served, reproducible for a seed, tokens inside the vocabulary
  HipHfDecodeSamplerConfig hot;
  hot.temperature = 0.8f;
  hot.top_k = 40;
  hot.seed = 11;
  std::vector<uint32_t> first;
  for (int round = 0; round < 2; ++round) {
    auto sampled = HipHfDecodeSequenceLoop::start_with_sampler(session, prompt, std::nullopt, hot);
    CHECK(sampled.summary.status == SmokeStatus::Ok && sampled.loop_state.has_value());
    if (!sampled.loop_state) break;
    HipHfDecodeSequenceSummary a = sampled.loop_state->advance(3);
    CHECK(a.status == SmokeStatus::Ok && a.tokens.size() == 3);
    for (uint32_t tok : a.tokens) CHECK(tok < 4);
    if (round == 0) first = a.tokens;
    else CHECK(a.tokens == first);
  }
}

// decode_sequence_session.rs:253-383, 506-628: two sessions of one model take their second token
// together; forks share the parent's weights; a loop that meets its stop token in a batch step is
// finished.
static void gpu_batch_checks() {
  KatModel m;
  // both sessions from the same declared weight plan (decode_sequence_session.rs:305-333): the
  // descriptors are the source of the weights, the tensor spans stay empty
  const std::vector<HipHfDecodeSequenceWeightBlock> blocks = m.blocks();
  HipHfDecodeSequenceSessionConfig config = m.config();
  config.weight_plan = KatModel::plan(blocks);
  config.weight_blocks = blocks;
  config.embeddings = config.final_norm_weight = config.lm_head = Span<uint16_t>();
  config.layers[0] = HipHfDecodeChainLayer{};
  auto created_a = config.create();
  auto created_b = config.create();
  CHECK(created_a.summary.h2d_bytes == 100 && created_a.summary.resident_weight_bytes == 100);
  CHECK(created_a.session && created_b.session);
  if (!created_a.session || !created_b.session) return;
  std::vector<uint32_t> prompt_a{0}, prompt_b{1};
  // what each sequence does alone: [1, 2, 3] after 0 and [2, 3, 0] after 1
  CHECK(created_a.session->run(prompt_a, 3).tokens == std::vector<uint32_t>({1, 2, 3}));
  CHECK(created_b.session->run(prompt_b, 3).tokens == std::vector<uint32_t>({2, 3, 0}));
  auto loop_a = HipHfDecodeSequenceLoop::start(*created_a.session, prompt_a, std::nullopt);
  auto loop_b = HipHfDecodeSequenceLoop::start(*created_b.session, prompt_b, 0u);   // stop token 0
  CHECK(loop_a.loop_state.has_value() && loop_b.loop_state.has_value());
  if (!loop_a.loop_state || !loop_b.loop_state) return;
  std::vector<HipHfDecodeSequenceSession *> sessions{created_a.session.get(), created_b.session.get()};
  // the first token has not been handed out yet: nothing is ready
  HipHfDecodeSequenceBatchAdvanceSummary batch = HipHfDecodeSequenceSession::batch_advance_one(sessions, 2, 2);
  CHECK(batch.status == SmokeStatus::Ok && batch.reason == "no_ready_sessions" && !batch.exact);
  CHECK(loop_a.loop_state->advance(1).tokens == std::vector<uint32_t>({1}));
  CHECK(loop_b.loop_state->advance(1).tokens == std::vector<uint32_t>({2}));
  batch = HipHfDecodeSequenceSession::batch_advance_one(sessions, 2, 2);
  CHECK(batch.status == SmokeStatus::Ok && batch.reason == "ready" && batch.exact);
  CHECK(batch.block_tokens == 2 && batch.layer_count == 1 && batch.observed_tokens == 2);
  CHECK(batch.tokens == std::vector<uint32_t>({2, 3}) && batch.last_token == 3 && batch.hot_path_allocations == 0);
  // through the loops: b meets its stop token and is finished, a goes on
  std::vector<HipHfDecodeSequenceLoop *> loops{&*loop_a.loop_state, &*loop_b.loop_state};
  batch = HipHfDecodeSequenceLoop::batch_advance_one(loops, 2, 2);
  CHECK(batch.status == SmokeStatus::Ok && batch.tokens == std::vector<uint32_t>({3, 0}));
  CHECK(!loop_a.loop_state->finished() && loop_b.loop_state->finished());
  batch = HipHfDecodeSequenceLoop::batch_advance_one(loops, 2, 2);
  CHECK(batch.status == SmokeStatus::Ok && batch.reason == "insufficient_compatible_ready" && batch.eligible_session_count == 1);
  batch = HipHfDecodeSequenceLoop::batch_advance_one(loops, 2, 1);
  CHECK(batch.status == SmokeStatus::Ok && batch.reason == "ready" && batch.tokens == std::vector<uint32_t>({0, UINT32_MAX}));
  // a fork taken in mid-sequence continues like its parent, on the same weights
  auto forked = created_a.session->fork_shared_weights(false);
  CHECK(forked.summary.status == SmokeStatus::Ok && forked.session);
  if (!forked.session) return;
  CHECK(forked.summary.resident_weight_bytes == created_a.summary.resident_weight_bytes);
  std::vector<HipHfDecodeSequenceSession *> pair{created_a.session.get(), forked.session.get()};
  batch = HipHfDecodeSequenceSession::batch_advance_one(pair, 8, 2);
  CHECK(batch.status == SmokeStatus::Ok && batch.reason == "ready" && batch.tokens == std::vector<uint32_t>({1, 1}));
  created_a.session.reset();   // the parent goes first: the child keeps the weights
  CHECK(forked.session->run(prompt_a, 2).tokens == std::vector<uint32_t>({1, 2}));
}

int main(int argc, char **argv) {
  const std::string mode = argc > 1 ? argv[1] : "cpu";
  cpu_checks();
  if (mode == "gpu") {
    gpu_checks();
    gpu_batch_checks();
  }
  std::printf("%s: %d failure(s)\n", mode.c_str(), failures);
  return failures == 0 ? 0 : 1;
}
