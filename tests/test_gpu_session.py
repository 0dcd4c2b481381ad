"""GPU parity tests of the decode session (create / start / advance / run / destroy) through the
C ABI: the reference's end-to-end known-answer streams, and random small models against the CPU
oracle (logits, KV rows, greedy token streams)."""
import ctypes as C

import numpy as np
import pytest

import nerva_amd as N
import oracle as O
from conftest import hx
from nerva_amd import abi
from nerva_amd.session import decode_sequence_oneshot
from oracle.links import assert_stream_follows_oracle, chain_budget, run_traced_stream

pytestmark = pytest.mark.gpu

BF16, F16 = 1, 0
REL_L2 = 1e-3


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def kat_models(kat, qk_norm):
    k = kat["decode_sequence"]
    one = lambda name: np.array([hx(v) for v in k[name]], np.uint16)
    layer = dict(rms_attn=one("rms"), rms_mlp=one("rms"), w_q=one("matrix"), w_k=one("matrix"),
                 w_v=one("matrix"), w_o=one("matrix"), w_gate=one("matrix"), w_up=one("matrix"),
                 w_down=one("matrix"))
    if qk_norm:
        layer.update(q_norm=one("rms"), k_norm=one("rms"))
    args = (F16, k["hidden"], k["heads"], k["kv_heads"], k["head_dim"], k["intermediate"], k["vocab"],
            k["rms_eps"], k["rope_theta"], one("embeddings"), [layer], one("rms"), one("lm_head"))
    return N.ModelWeights(*args), k


@pytest.mark.parametrize("qk_norm", [False, True])
def test_reference_greedy_stream_kat(kat, qk_norm):
    """hidden 2 / vocab 4 model, prompt [0], 4 steps -> [1,2,3,0]; with eos 2 -> [1,2]
    (crates/nerva-cuda/src/tests/decode_sequence.rs:123-223, decode_sequence_qk_norm.rs:11-91)."""
    weights, k = kat_models(kat, qk_norm)
    rc, res, tokens = decode_sequence_oneshot(weights, k["prompt"], k["steps"])
    assert rc == 0 and res.status == 0
    assert tokens.tolist() == k["tokens"]
    assert res.observed_tokens == 4 and res.last_token == 0 and res.kv_tokens == 4
    assert res.observed_token_hash == O.fnv1a(np.array(k["tokens"], np.uint32))
    assert res.graph_replays == 4 and res.graph_launches == 4 and res.sync_calls == 1
    assert res.host_causality_edges == 0 and res.hot_path_allocations == 0
    assert res.resident_weight_bytes == (108 if qk_norm else 100)
    assert res.kernel_launches == res.graph_replays * res.graph_nodes
    rc, res, tokens = decode_sequence_oneshot(weights, k["prompt"], k["steps"], eos=k["eos_token"])
    assert rc == 0 and tokens.tolist() == k["tokens_with_eos"]
    assert res.kv_tokens == k["kv_tokens_with_eos"] and res.graph_replays == 4


def kat_plan(weights):
    """The reference's 12-block plan of the known-answer model: one block per tensor, the first six
    declared GPU-resident and the rest GPU-staged (decode_sequence_descriptor_blocks.rs:223-258)."""
    plan = N.WeightPlan.from_weights(weights, resident_blocks=6)
    assert [b.bytes for b in plan.blocks] == [16, 4, 8, 8, 8, 8, 4, 8, 8, 8, 4, 16]
    return plan


def test_weight_plan_descriptors_are_the_source_of_the_weights(kat):
    """decode_sequence_descriptors.rs:2093-2181 (descriptors override poisoned tensor pointers) and
    :2182-2187 with decode_sequence_descriptor_blocks.rs:41-97 (null tensor pointers): the stream is the
    known-answer stream, the byte counters are the plan's."""
    weights, k = kat_models(kat, False)
    plan = kat_plan(weights)
    fields = plan.fields()
    assert (fields["planned_weight_blocks"], fields["planned_gpu_resident_blocks"], fields["planned_gpu_staged_blocks"],
            fields["planned_weight_bytes"], fields["planned_gpu_resident_weight_bytes"],
            fields["planned_gpu_staged_weight_bytes"]) == (12, 6, 6, 100, 52, 48)
    # poisoned tensor pointers: zero embeddings and head, all-ones matrices
    one, zero = 0x3C00, 0x0000
    bad_layer = {key: np.full(4, one, np.uint16) for key in ("w_q", "w_k", "w_v", "w_o", "w_gate", "w_up", "w_down")}
    bad_layer.update(rms_attn=np.full(2, zero, np.uint16), rms_mlp=np.full(2, zero, np.uint16))
    poisoned = N.ModelWeights(F16, k["hidden"], k["heads"], k["kv_heads"], k["head_dim"], k["intermediate"], k["vocab"],
                              k["rms_eps"], k["rope_theta"], np.zeros(8, np.uint16), [bad_layer],
                              np.zeros(2, np.uint16), np.zeros(8, np.uint16))
    rc, res, tokens = decode_sequence_oneshot(poisoned, k["prompt"], k["steps"], plan=fields)
    assert rc == 0 and tokens.tolist() == k["tokens"]
    assert res.planned_weight_blocks == 12 and res.planned_weight_bytes == res.resident_weight_bytes == 100
    assert res.descriptor_gpu_resident_h2d_bytes == 52 and res.descriptor_gpu_staged_h2d_bytes == 48
    assert res.planned_weight_descriptor_count == 12 and res.planned_weight_descriptor_hash == plan.descriptor_hash
    # without the plan the poisoned pointers are what runs
    rc, res, bad_tokens = decode_sequence_oneshot(poisoned, k["prompt"], k["steps"])
    assert rc == 0 and bad_tokens.tolist() != k["tokens"]
    # null tensor pointers
    s = N.DecodeSession.create(weights, 16, plan=plan, tensor_pointers=False)
    assert s.create_result.h2d_bytes == 100 and s.create_result.planned_weight_descriptor_hash == plan.descriptor_hash
    rc, res, tokens = s.run(k["prompt"], k["steps"])
    assert rc == 0 and tokens.tolist() == k["tokens"]
    s.destroy()


def test_weight_plan_validation(kat):
    """weights.cu:411-467: what makes a declared plan unacceptable."""
    weights, k = kat_models(kat, False)

    def attempt(change=None, **override):
        plan = kat_plan(weights)
        if change is not None:
            change(plan.blocks)
        fields = plan.fields() if change is None else dict(plan.fields(), planned_weight_descriptor_hash=N.hash_weight_blocks(plan.blocks))
        fields.update(override)
        rc, res, _ = decode_sequence_oneshot(weights, k["prompt"], k["steps"], plan=fields)
        return rc, res

    assert attempt()[0] == 0
    rc, res = attempt(planned_weight_bytes=99)
    assert rc == -1 and res.status == -1                                        # totals disagree with the arena
    assert attempt(planned_weight_descriptor_hash=1234)[0] == -1                # hash of the descriptors
    assert attempt(planned_gpu_resident_blocks=5)[0] == -1                      # block counts
    assert attempt(planned_gpu_resident_weight_bytes=50)[0] == -1               # byte counts
    assert attempt(planned_weight_descriptor_count=11)[0] == -1                 # descriptors stop short of the arena
    assert attempt(planned_weight_descriptor_count=0, planned_weight_descriptors=None)[0] == -1   # a plan without descriptors

    def gap(blocks):
        blocks[3].offset_bytes += 2
    def odd(blocks):
        blocks[2].bytes -= 1
        blocks[3].offset_bytes -= 1
        blocks[3].bytes += 1
    def strategy(blocks):
        blocks[4].strategy = 3
    def reserved(blocks):
        blocks[0].reserved = 1
    def sourceless(blocks):
        blocks[5].host_source = None
    for change in (gap, odd, strategy, reserved, sourceless):
        assert attempt(change)[0] == -1, change.__name__


@pytest.mark.parametrize("source", ["memory", "file"])
def test_weight_plan_blocks_cut_across_tensors(source, tmp_path):
    """Descriptors need not follow tensor boundaries: the arena of a random model (q/k norms and biases
    present, so every optional tensor of the order is exercised) is cut into 5000-byte blocks, from memory
    or from a file, and the session must hold exactly the weights a pointer-fed session holds - same
    logits bit for bit, same K/V rows, same stream."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers = BF16, 256, 4, 2, 64, 520, 300, 2
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 31, 1e4, qk_norm=True, bias=True)
    path = str(tmp_path / "arena.bin") if source == "file" else None
    plan = N.WeightPlan.from_weights(weights, block_bytes=5000, resident_blocks=40, path=path)
    assert len(plan.blocks) > 100 and plan.fields()["planned_gpu_staged_blocks"] == len(plan.blocks) - 40
    prompt = np.random.default_rng(2).integers(0, vocab, 11).astype(np.uint32)
    outcome = []
    for kwargs in (dict(), dict(plan=plan)):
        s = N.DecodeSession.create(weights, 32, **kwargs)
        rc, _ = s.start(prompt)
        assert rc == 0
        logits = s.logits()
        rows = [s.kv_row(layer, 10) for layer in range(layers)]
        rc, _, tokens = s.advance(8)
        assert rc == 0
        outcome.append((logits, rows, tokens.tolist(), s.create_result))
        s.destroy()
    (l0, r0, t0, c0), (l1, r1, t1, c1) = outcome
    assert np.array_equal(l0, l1) and t0 == t1
    for (k0, v0), (k1, v1) in zip(r0, r1):
        assert np.array_equal(k0, k1) and np.array_equal(v0, v1)
    assert c1.resident_weight_bytes == c0.resident_weight_bytes == c1.h2d_bytes == c1.planned_weight_bytes
    assert c1.planned_weight_descriptor_count == len(plan.blocks)
    if source == "file":
        # a file that ends early is an error, not a silent short read
        with open(path, "r+b") as f:
            f.truncate(c1.planned_weight_bytes - 100)
        with pytest.raises(RuntimeError):
            N.DecodeSession.create(weights, 32, plan=plan)


@pytest.mark.parametrize("model_type,shards,qk_norm,bias,tied", [("qwen3", 2, True, False, False),
                                                                 ("llama", 1, False, True, False),
                                                                 ("qwen3", 3, True, False, True)])
def test_session_from_checkpoint_files(model_type, shards, qk_norm, bias, tied, tmp_path):
    """The checkpoint planner end to end: a random model written out as config.json + safetensors shards
    (tensors shuffled across the files) gives, through file-backed descriptors alone, the session a
    pointer-fed create gives - same logits bit for bit, same K/V rows, same stream, same byte counts."""
    from checkpoint_files import write_checkpoint
    from nerva_amd import checkpoint as ckpt
    dtype, hidden, heads, kv, hd, inter, vocab, layers = BF16, 256, 4, 2, 64, 520, 300, 2
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 47, 1e4, qk_norm=qk_norm, bias=bias)
    if tied:
        weights = N.ModelWeights(dtype, hidden, heads, kv, hd, inter, vocab, 1e-6, 1e4, weights.embeddings,
                                 weights.layers, weights.final_norm, weights.embeddings)
    write_checkpoint(str(tmp_path), weights, model_type, shards=shards, seed=shards, tied=tied,
                     extra_config=dict(attention_bias=True) if bias else None)
    prompt = np.random.default_rng(3).integers(0, vocab, 11).astype(np.uint32)
    outcome = []
    for from_files in (False, True):
        plan = None
        if from_files:
            s, plan = ckpt.create_session(str(tmp_path), 32)
        else:
            s = N.DecodeSession.create(weights, 32)
        rc, _ = s.start(prompt)
        assert rc == 0
        logits = s.logits()
        rows = [s.kv_row(layer, 10) for layer in range(layers)]
        rc, _, tokens = s.advance(8)
        assert rc == 0
        outcome.append((logits, rows, tokens.tolist(), s.create_result))
        s.destroy()
    (l0, r0, t0, c0), (l1, r1, t1, c1) = outcome
    assert np.array_equal(l0, l1) and t0 == t1
    for (k0, v0), (k1, v1) in zip(r0, r1):
        assert np.array_equal(k0, k1) and np.array_equal(v0, v1)
    assert c1.resident_weight_bytes == c0.resident_weight_bytes == c1.h2d_bytes == c1.planned_weight_bytes
    assert c1.planned_weight_descriptor_count == len(plan.blocks) and c1.planned_weight_descriptor_hash == plan.descriptor_hash
    # a shard that ends early is an error, not a silent short read
    name, shard, begin, nbytes = plan.entries[-1]
    with open(str(tmp_path / shard), "r+b") as f:
        f.truncate(begin + nbytes - 64)
    with pytest.raises((RuntimeError, ckpt.CheckpointError)):
        ckpt.create_session(str(tmp_path), 32)


def test_session_lifecycle_kat(kat):
    """create -> start -> advance in pieces; token accounting of the reference
    (session_api_lifecycle.inc.cu:992-1311): the first advance(n) does n-1 replays."""
    weights, k = kat_models(kat, True)
    s = N.DecodeSession.create(weights, 16)
    assert s.create_result.status == 0 and s.create_result.hot_path_allocations == 0
    assert s.create_result.resident_weight_bytes == 108 and s.create_result.resident_kv_bytes > 0
    rc, res, _ = s.advance(1)
    assert rc == -1                                   # advance before start
    rc, res = s.start([0])
    assert rc == 0 and res.kv_tokens == 1 and res.seed_token == 0
    rc, res, t1 = s.advance(2)
    assert rc == 0 and t1.tolist() == [1, 2] and res.graph_replays == 1 and res.seed_token == 0
    assert res.hot_path_allocations == 0 and res.host_causality_edges == 0 and res.sync_calls == 1
    rc, res, t2 = s.advance(6)
    assert rc == 0 and t2.tolist() == [3, 0, 1, 2, 3, 0] and res.graph_replays == 6
    assert res.seed_token == 2 and res.kv_tokens == 8 and res.graph_cache_hits == 1
    rc, res, _ = s.advance(20)                        # past max_context_tokens
    assert rc == -1
    # restart on the same session with a 3-token prompt and a stop token
    rc, res = s.start([2, 1, 0], eos=3)
    assert rc == 0 and res.kv_tokens == 3
    rc, res, t3 = s.advance(5)
    assert rc == 0 and t3.tolist() == [1, 2, 3] and res.observed_tokens == 3
    rc, res, _ = s.advance(1)                         # finished after the stop token
    assert rc == -1
    # run(): the step graph walks the prompt too
    rc, res, t4 = s.run([0], 4)
    assert rc == 0 and t4.tolist() == [1, 2, 3, 0] and res.graph_replays == 4
    rc, dres = s.destroy()
    assert rc == 0 and dres.status == 0


def test_argument_validation_on_device(kat):
    weights, k = kat_models(kat, False)
    s = N.DecodeSession.create(weights, 8)
    rc, res = s.start([7])                            # token >= vocab
    assert rc == -1 and res.status == -1
    rc, res = s.start([])
    assert rc == -1
    rc, res = s.start(list(range(4)) * 3)             # prompt longer than the context
    assert rc == -1
    sampler = abi.NervaHipHfDecodeSamplerConfig()
    sampler.temperature, sampler.top_p, sampler.top_k = 0.7, 0.9, 40
    rc, res = s.start([0], sampler=sampler)           # temperature sampling is served
    assert rc == 0
    sampler.top_p = 0.0
    rc, res = s.start([0], sampler=sampler)           # out-of-range top_p is normalised to 1 (sampler.cu:422-433)
    assert rc == 0
    rc, res = s.start([0])
    assert rc == 0
    rc, res, _ = s.advance(3, capacity=2)             # capacity < steps
    assert rc == -1
    rc, res, _ = s.run([0, 1], 3, seed_token=0)       # seed token must be the last prompt token
    assert rc == -1
    s.destroy()


def random_model(dtype, hidden, heads, kv_heads, hd, inter, vocab, layers, seed, theta=1e6, qk_norm=True,
                 bias=False, std=0.05):
    rng = np.random.default_rng(seed)
    e = lambda shape, mean=0.0, s=std: O.encode16(dtype, rng.normal(mean, s, shape))
    A, KV = heads * hd, kv_heads * hd
    ls = []
    for _ in range(layers):
        l = dict(rms_attn=e(hidden, 1.0, 0.02), rms_mlp=e(hidden, 1.0, 0.02), w_q=e((A, hidden)),
                 w_k=e((KV, hidden)), w_v=e((KV, hidden)), w_o=e((hidden, A)), w_gate=e((inter, hidden)),
                 w_up=e((inter, hidden)), w_down=e((hidden, inter)))
        if qk_norm:
            l.update(q_norm=e(hd, 1.0, 0.02), k_norm=e(hd, 1.0, 0.02))
        if bias:
            l.update(q_bias=e(A, 0, 0.1), k_bias=e(KV, 0, 0.1), v_bias=e(KV, 0, 0.1), o_bias=e(hidden, 0, 0.1))
        ls.append(l)
    args = (dtype, hidden, heads, kv_heads, hd, inter, vocab, 1e-6, theta, e((vocab, hidden), 0, 1.0), ls,
            e(hidden, 1.0, 0.02), e((vocab, hidden)))
    return N.ModelWeights(*args), O.Model(*args)


# End-to-end numbers. Every operator is held to relative L2 <= 1e-3 on its own (tests/test_gpu_ops.py)
# and inside a running session on the device's own inputs (tests/test_gpu_parity_links.py: measured
# <= 1.1e-5 for every link). Through a whole model the 16-bit staging points amplify f32
# summation-order noise: one bf16 rounding that lands on the other side of a boundary moves that
# element by 2^-8 relative, and every later layer sees it. So the logits of a whole step are held to
# the chain's budget - one operator tolerance per 16-bit staging point, oracle.links.chain_budget -
# and the measured figure (2e-3..8e-3 on these models, the size by which the reference's own two
# stagings differ from each other) is only reported.


E2E_REL_L2 = chain_budget(3)   # no model here is deeper than 3 layers


GEOMETRIES = [
    # dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias
    (BF16, 512, 4, 1, 128, 1024, 1000, 3, 1e6, True, False),   # fast attention path, group 4 (Qwen3-like)
    (BF16, 1024, 8, 8, 128, 1536, 777, 2, 1e4, False, True),   # MHA, biases, no qk-norm
    (F16, 256, 4, 2, 64, 520, 300, 2, 1e4, True, False),       # generic attention path, guarded GEMV
    (BF16, 96, 6, 2, 16, 200, 50, 2, 0, False, False),         # group 3, no RoPE, cols % 8 == 0 only
    (F16, 512, 4, 1, 128, 1024, 1000, 3, 1e6, True, False),    # fast attention path in f16
    (BF16, 2048, 16, 4, 128, 4096, 1000, 3, 1e6, True, False), # 2048-wide, group 4: the lean GEMV kernel on every projection
    (F16, 2048, 16, 16, 128, 2048, 700, 2, 1e4, False, True),  # same in f16, MHA, o bias
]


@pytest.mark.parametrize("geom", GEOMETRIES)
def test_single_layer_short_prompt_is_tight(geom):
    """One layer and a 1- or 2-token prompt leave no room for 16-bit ties to compound: the whole
    step (embed, norms, GEMVs, RoPE, attention, LM head) must agree with the oracle at 1e-3 in
    f16. In bf16 a single value that sits within 1e-6 of a rounding boundary (attention output,
    SwiGLU output and norm outputs are rounded to 16 bit) may land on the other side, which moves
    one activation by 2^-8 relative and the logits of this tiny model by up to ~3e-3: the bound
    is one such flip, 6e-3."""
    dtype, hidden, heads, kv, hd, inter, vocab, _, theta, qk_norm, bias = geom
    tol = REL_L2 if dtype == F16 else 6e-3
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, 1, hidden + 1, theta, qk_norm, bias)
    s = N.DecodeSession.create(weights, 32)
    for prompt in ([3], [vocab - 1, 11]):
        ctx = O.Context(omodel, 32, staging=1)
        for i, t in enumerate(prompt):
            ctx.forward_token(int(t), prompt_token=True, want_logits=(i == len(prompt) - 1))
        rc, res = s.start(prompt)
        assert rc == 0
        assert rel_l2(s.logits(), ctx.logits()) <= tol
        gk, gv = s.kv_row(0, len(prompt) - 1)
        rk, rv = ctx.read_kv16(0, len(prompt) - 1)
        # summation order may move a value across a 16-bit tie: at most one unit, on few elements
        # (values near zero are compared by magnitude: one unit there is far below the f32 noise)
        for got, ref in ((gk, rk), (gv, rv)):
            gf, rf = O.decode16(dtype, got), O.decode16(dtype, ref)
            units = np.abs(got.astype(np.int32) - ref.astype(np.int32))
            assert np.all((units <= 1) | (np.abs(gf - rf) <= 1e-4 * np.max(np.abs(rf))))
            # one flipped element of the normalised input moves every K/V value by ~1e-5, which
            # carries a few percent of them across their own 16-bit boundary
            assert np.mean(got != ref) <= 0.10
        rc, res, tokens = s.advance(1)
        assert rc == 0 and tokens[0] == O.greedy_argmax(ctx.logits(), skip_nonfinite=True)
    s.destroy()


@pytest.mark.parametrize("geom", GEOMETRIES)
def test_session_matches_oracle_logits_kv_and_stream(geom):
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = geom
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, hidden, theta, qk_norm, bias)
    prompt = np.random.default_rng(1).integers(0, vocab, 21).astype(np.uint32)
    steps = 24
    s = N.DecodeSession.create(weights, 64)
    rc, res = s.start(prompt)
    assert rc == 0
    # logits after prefill: compare with an oracle context that stops right after the prompt
    ctx2 = O.Context(omodel, 64, staging=1)
    for i, t in enumerate(prompt):
        ctx2.forward_token(int(t), prompt_token=True, want_logits=(i == len(prompt) - 1))
    ref_logits = ctx2.logits()
    got_logits = s.logits()
    assert rel_l2(got_logits, ref_logits) <= chain_budget(layers)
    for layer in range(layers):
        for token in (0, 7, len(prompt) - 1):
            gk, gv = s.kv_row(layer, token)
            rk, rv = ctx2.read_kv16(layer, token)
            # layer 0 rows depend on one embedding row only: at most a few 16-bit ties differ
            tol = 2e-3 if layer == 0 else chain_budget(layer)
            assert rel_l2(O.decode16(dtype, gk), O.decode16(dtype, rk)) <= tol
            assert rel_l2(O.decode16(dtype, gv), O.decode16(dtype, rv)) <= tol
    # the stream token by token: every step's logits and token against the oracle that follows the
    # device's tokens (in every step mode; the launch-per-piece step is also traced link by link in
    # tests/test_gpu_parity_links.py)
    stepwise, _, e2e = run_traced_stream(s, omodel, prompt, steps, 64, trace_links=False)
    # the same stream from one call: graph replays back to back, no allocation, one synchronisation
    rc, _ = s.start(prompt)
    rc, res, tokens = s.advance(steps)
    assert rc == 0 and res.observed_tokens == steps and res.graph_replays == steps - 1
    assert res.hot_path_allocations == 0 and res.host_causality_edges == 0 and res.sync_calls == 1
    assert tokens.tolist() == stepwise
    assert res.observed_token_hash == O.fnv1a(tokens)
    # determinism: the same prompt again gives the same stream and hash
    rc, _ = s.start(prompt)
    rc, res2, tokens2 = s.advance(steps)
    assert tokens2.tolist() == tokens.tolist() and res2.observed_token_hash == res.observed_token_hash
    assert res2.graph_captures == 0 and res2.graph_cache_hits == 1
    s.destroy()


def test_run_walks_prompt_with_decode_staging():
    """session_run feeds prompt tokens through the decode-step graph (f32 residual stream,
    no per-layer rounding), unlike start(), which uses the prompt staging."""
    weights, omodel = random_model(BF16, 512, 4, 1, 128, 1024, 500, 2, 77)
    prompt = np.array([5, 17, 400, 3, 250], np.uint32)
    ctx = O.Context(omodel, 32, staging=1)
    for i, t in enumerate(prompt):
        ctx.forward_token(int(t), prompt_token=False, want_logits=True)
    ref = ctx.logits()
    s = N.DecodeSession.create(weights, 32)
    rc, res, tokens = s.run(prompt, 1)
    assert rc == 0 and res.graph_replays == len(prompt)
    assert rel_l2(s.logits(), ref) <= E2E_REL_L2
    assert tokens[0] == O.greedy_argmax(ref, skip_nonfinite=True) or \
        np.sort(ref)[-1] - np.sort(ref)[-2] < E2E_REL_L2 * np.max(np.abs(ref))
    s.destroy()


def test_eager_profile_pass_leaves_state_untouched():
    weights, omodel = random_model(BF16, 512, 4, 1, 128, 1024, 500, 2, 5)
    s = N.DecodeSession.create(weights, 48)
    prompt = np.arange(9, dtype=np.uint32)
    s.start(prompt)
    rc, res, a = s.advance(4)
    rc, prof = s.profile_step(2)
    assert rc == 0 and prof.status == 0 and prof.launches == 3 + 5 * 2
    assert prof.gate_up_ns > 0 and prof.lm_head_ns > 0 and prof.position == len(prompt) + 3
    rc, res, b = s.advance(6)
    s.start(prompt)
    rc, res, full = s.advance(10)
    assert np.concatenate([a, b]).tolist() == full.tolist()   # profiling did not disturb the sequence
    s.destroy()


def test_session_split_factor_override_changes_only_the_summation_order():
    """The split-KV factor of a session's decode attention is a launch-shape choice: sessions created
    under the override hook with 1, 3 and 64 splits of a 700-token context give the default session's
    logits up to the order in which the splits' partial sums meet, and the same greedy tokens."""
    weights, omodel = random_model(BF16, 512, 4, 1, 128, 1024, 500, 2, 6)
    prompt = np.random.default_rng(8).integers(0, 500, 700).astype(np.uint32)
    runs = {}
    try:
        for splits in (0, 1, 3, 64):
            N.Device.set_tuning("attn_splits", splits)
            s = N.DecodeSession.create(weights, 768)
            rc, res = s.start(prompt)
            assert rc == 0
            rc, res, toks = s.advance(6)
            assert rc == 0 and res.graph_replays == 5
            runs[splits] = (toks.tolist(), s.logits())
            s.destroy()
    finally:
        N.Device.set_tuning("attn_splits", 0)
    for splits in (1, 3, 64):
        assert runs[splits][0] == runs[0][0], splits
        assert rel_l2(runs[splits][1], runs[0][1]) <= chain_budget(2), splits


def test_synthetic_session_matches_oracle_weights():
    """Device-generated weights (benchmark path) equal the oracle's generator bit for bit, so the
    CPU baseline can rebuild the same model on the host."""
    cfg = dict(dtype=BF16, hidden=512, heads=4, kv_heads=1, head_dim=128, intermediate=1024, vocab=600,
               layers=2, rms_eps=1e-6, rope_theta=1e6)
    seed, std = 0x4E45525641, 0.02
    s = N.DecodeSession.create_synthetic(cfg, 64, seed=seed, weight_std=std, qk_norm=True)
    H, A, KV, I, V, HD = 512, 512, 128, 1024, 600, 128
    g = lambda tid, n, mean=0.0: O.synth_16(BF16, seed, tid, n, mean, std)
    layers = []
    for l in range(2):
        b = 16 * (l + 1)
        layers.append(dict(rms_attn=g(b, H, 1.0), rms_mlp=g(b + 1, H, 1.0), w_q=g(b + 2, A * H).reshape(A, H),
                           w_k=g(b + 4, KV * H).reshape(KV, H), q_norm=g(b + 5, HD, 1.0), k_norm=g(b + 6, HD, 1.0),
                           w_v=g(b + 7, KV * H).reshape(KV, H), w_o=g(b + 8, H * A).reshape(H, A),
                           w_gate=g(b + 13, I * H).reshape(I, H), w_up=g(b + 14, I * H).reshape(I, H),
                           w_down=g(b + 15, H * I).reshape(H, I)))
    omodel = O.Model(BF16, H, 4, 1, HD, I, V, 1e-6, 1e6, g(1, V * H).reshape(V, H), layers, g(2, H, 1.0),
                     g(3, V * H).reshape(V, H))
    prompt = O.synth_tokens(seed, 1000, 12, V)
    rc, res = s.start(prompt)
    assert rc == 0
    rc, res, tokens = s.advance(8)
    assert rc == 0
    assert_stream_follows_oracle(omodel, prompt, tokens, 64)
    s.destroy()


def oracle_sampled_stream(omodel, prompt, steps, sampler, max_ctx):
    """Token stream of the reference's rule: prompt staging for the prompt, then sample, feed, sample ...
    Returns tokens and the sampler's decision margins."""
    ctx = O.Context(omodel, max_ctx, staging=1)
    for i, t in enumerate(prompt):
        ctx.forward_token(int(t), prompt_token=True, want_logits=(i == len(prompt) - 1))
    tokens, margins = [], []
    for i in range(steps):
        position = len(prompt) - 1 + i                # slot index = position of the token that produced the logits
        tok, margin = O.sample(ctx.logits(), sampler.temperature, sampler.top_p, sampler.top_k, sampler.seed, position)
        tokens.append(tok)
        margins.append(margin)
        if i + 1 < steps:
            ctx.forward_token(tok, prompt_token=False, want_logits=True)
    return tokens, margins


@pytest.mark.parametrize("temperature,top_p,top_k", [(0.8, 0.9, 0), (1.0, 1.0, 0), (0.7, 0.95, 20), (1.3, 1.0, 5)])
def test_session_temperature_sampling_follows_the_rule(temperature, top_p, top_k):
    """Every token the session samples is the oracle rule's token for the logits the session itself
    computed at that step, with the position as the random-number counter (near-ties of the two exp/log
    implementations aside). The logits are checked against the oracle elsewhere; checking the rule on
    the device's own logits keeps this test exact on a random model, whose flat distribution turns any
    end-to-end logit noise into different draws."""
    weights, omodel = random_model(BF16, 512, 4, 1, 128, 1024, 1000, 2, 321, 1e6, True, False)
    sampler = abi.NervaHipHfDecodeSamplerConfig()
    sampler.temperature, sampler.top_p, sampler.top_k, sampler.seed = temperature, top_p, top_k, 0xC0FFEE
    prompt = np.array([3, 141, 59, 26, 535], np.uint32)
    steps = 24
    s = N.DecodeSession.create(weights, 64)
    rc, res = s.start(prompt, sampler=sampler)
    assert rc == 0
    got, close = [], 0
    for i in range(steps):
        if i == 0:
            logits = s.logits()                       # start() has sampled the first token from these
        rc, res, tok = s.advance(1)
        assert rc == 0 and res.hot_path_allocations == 0
        if i > 0:
            logits = s.logits()
            assert res.graph_nodes == 4 + 5 * 2       # lm head + two sampler launches
        want, margin = O.sample(logits, temperature, top_p, top_k, sampler.seed, len(prompt) - 1 + i)
        if int(tok[0]) != want:
            assert margin < 1e-5, (i, int(tok[0]), want, margin)
            close += 1
        got.append(int(tok[0]))
    assert close <= 1 and len(set(got)) > 4
    # the whole-vocabulary branch decides with wide margins on this model: there the complete stream
    # also equals the oracle's own chain (its logits, its samples)
    if top_k == 0 and top_p >= 0.999999:
        want, margins = oracle_sampled_stream(omodel, prompt, steps, sampler, 64)
        for i in range(steps):
            if got[i] != want[i]:
                assert margins[i] < 5e-2, (i, got[i], want[i], margins[i])
                break
    # the same seed gives the same stream; another seed gives another one
    rc, _ = s.start(prompt, sampler=sampler)
    rc, res, again = s.advance(steps)
    assert again.tolist() == got
    sampler.seed = 7
    rc, _ = s.start(prompt, sampler=sampler)
    rc, res, other = s.advance(steps)
    assert other.tolist() != got
    # and the session goes back to the greedy graph when asked to
    rc, _ = s.start(prompt)
    rc, res, greedy = s.advance(4)
    assert rc == 0 and res.graph_nodes == 3 + 5 * 2
    s.destroy()


PREFILL_GEOMETRIES = [
    GEOMETRIES[5],                                                # GQA factor 4: two tokens per wave of the prompt attention
    GEOMETRIES[6],                                                # MHA: eight tokens per wave
    (BF16, 2048, 16, 8, 128, 2048, 640, 2, 1e6, True, True),      # GQA factor 2: four tokens per wave
    (F16, 2048, 16, 2, 128, 2048, 640, 2, 1e4, True, False),      # GQA factor 8: one token per wave
]


@pytest.mark.parametrize("geom", PREFILL_GEOMETRIES)
def test_block_prefill_matches_token_walk_and_oracle(geom, monkeypatch):
    """start() sends the prompt through the layers in blocks of up to 64 tokens (multi-row GEMMs, one
    attention launch per block); the "prefill_walk" override keeps one prompt step per token. Same staging,
    so both agree with each other and with the oracle to the end-to-end tolerance, over three blocks."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = geom
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 1234, theta, qk_norm, bias)
    prompt = np.random.default_rng(8).integers(0, vocab, 150).astype(np.uint32)
    ctx = O.Context(omodel, 160, staging=1)
    for i, tok in enumerate(prompt):
        ctx.forward_token(int(tok), prompt_token=True, want_logits=(i == len(prompt) - 1))
    ref_logits = ctx.logits()
    results = {}
    for mode in ("blocks", "walk"):
        if mode == "walk":
            N.Device.set_tuning("prefill_walk", 1)
        else:
            N.Device.set_tuning("prefill_walk", 0)
        s = N.DecodeSession.create(weights, 160)
        rc, res = s.start(prompt)
        assert rc == 0 and res.hot_path_allocations == 0
        logits = s.logits()
        assert rel_l2(logits, ref_logits) <= E2E_REL_L2
        for layer in range(layers):
            for token in (0, 15, 31, 32, 47, 63, 64, 65, 127, 128, 129, 148, 149):     # block and tile edges included
                gk, gv = s.kv_row(layer, token)
                rk, rv = ctx.read_kv16(layer, token)
                tol = 2e-3 if layer == 0 else E2E_REL_L2
                assert rel_l2(O.decode16(dtype, gk), O.decode16(dtype, rk)) <= tol, (mode, layer, token)
                assert rel_l2(O.decode16(dtype, gv), O.decode16(dtype, rv)) <= tol, (mode, layer, token)
        rc, res, tokens = s.advance(6)
        assert rc == 0
        results[mode] = (logits, tokens.tolist(), res.kernel_launches)
        s.destroy()
    assert rel_l2(results["blocks"][0], results["walk"][0]) <= E2E_REL_L2
    assert results["blocks"][1][0] == results["walk"][1][0] or \
        np.sort(ref_logits)[-1] - np.sort(ref_logits)[-2] < E2E_REL_L2 * np.max(np.abs(ref_logits))


# ---- sessions on shared weights: fork, and one decode step for a batch of them -------------------

def started(session, prompt, sampler=None):
    """start + the advance(1) that hands out the token start computed: the state a batch step takes."""
    rc, _ = session.start(prompt, sampler=sampler)
    assert rc == 0
    rc, _, first = session.advance(1)
    assert rc == 0
    return int(first[0])


def oracle_follow(omodel, max_ctx, prompt, produced):
    """Oracle context that walked the prompt (prompt staging) and then the tokens a device produced
    (decode staging): its K/V rows and logits are what a device at the same history must hold."""
    ctx = O.Context(omodel, max_ctx, staging=1)
    for t in prompt:
        ctx.forward_token(int(t), prompt_token=True, want_logits=False)
    margins = []
    for t in produced:
        ctx.forward_token(int(t), prompt_token=False, want_logits=True)
        top = np.sort(ctx.logits())
        margins.append(float(top[-1] - top[-2]))
    return ctx, margins


@pytest.mark.parametrize("geom", [GEOMETRIES[5], GEOMETRIES[6]])
def test_batch_advance_one_matches_solo_sessions_and_oracle(geom):
    """Five sessions on one set of resident weights (a parent and four forks) at five different
    positions advance together, one token per call through one stream of the weights. Every sequence
    must come out as if it had advanced alone: same tokens as a solo session wherever the oracle's
    margin is clear, and the K/V rows it appended equal to the oracle's for the same token history."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = geom
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 4321, theta, qk_norm, bias)
    rng = np.random.default_rng(17)
    prompts = [rng.integers(0, vocab, n).astype(np.uint32) for n in (1, 5, 17, 33, 40)]
    steps, max_ctx = 6, 64
    plan = N.WeightPlan.from_weights(weights)        # a declared weight plan: its descriptor hash names the model
    parent = N.DecodeSession.create(weights, max_ctx, plan=plan, tensor_pointers=False)
    sessions = [parent] + [parent.fork_shared_weights() for _ in range(4)]
    for child in sessions[1:]:
        assert child.create_result.resident_weight_bytes == parent.create_result.resident_weight_bytes
        assert child.create_result.planned_weight_descriptor_hash == plan.descriptor_hash != 0
    streams = [[started(s, p)] for s, p in zip(sessions, prompts)]
    for step in range(steps):
        rc, res, tokens = N.DecodeSession.batch_advance_one(sessions, 32, 2)
        assert rc == 0 and res.status == 0 and res.reason == abi.NERVA_HIP_BATCH_READY and res.exact == 1
        assert res.block_tokens == 5 and res.eligible_session_count == 5 and res.observed_tokens == 5
        assert parent.shares_weight_stream() and res.hot_path_allocations == 0
        assert res.projection_kernel_launches == 4 * layers + 1 and res.dependency_kernel_launches == layers
        assert res.scatter_kernel_launches == 0 and res.sampling_kernel_launches == 2
        assert res.observed_token_hash == O.fnv1a(tokens) and res.last_token == tokens[-1]
        assert res.layer_count == layers and res.dtype == dtype and res.projection_elapsed_ns > 0
        for stream, tok in zip(streams, tokens):
            stream.append(int(tok))
    # solo: a sixth session on the same weights walks each prompt alone
    solo = parent.fork_shared_weights()
    scale = None
    for prompt, stream, sess in zip(prompts, streams, sessions):
        rc, _ = solo.start(prompt)
        assert rc == 0
        rc, _, alone = solo.advance(steps + 1)
        assert rc == 0
        ctx, margins = oracle_follow(omodel, max_ctx, prompt, stream[:-1])
        scale = float(np.max(np.abs(ctx.logits())))
        for i in range(steps + 1):
            if stream[i] != int(alone[i]):
                # the histories part here; before that the oracle's margin must have been thin
                assert i >= 1 and margins[i - 1] <= E2E_REL_L2 * scale, (len(prompt), i, stream, alone.tolist())
                break
        # K/V rows the batch steps appended (positions P .. P + steps - 1) against the oracle on this history
        P = len(prompt)
        for layer in range(layers):
            for token in (P - 1, P, P + steps - 1):
                gk, gv = sess.kv_row(layer, token)
                rk, rv = ctx.read_kv16(layer, token)
                tol = 2e-3 if layer == 0 else E2E_REL_L2
                assert rel_l2(O.decode16(dtype, gk), O.decode16(dtype, rk)) <= tol, (P, layer, token)
                assert rel_l2(O.decode16(dtype, gv), O.decode16(dtype, rv)) <= tol, (P, layer, token)
        ctx.close()
    # sessions go on alone after batch steps, and back
    rc, res, more = sessions[2].advance(2)
    assert rc == 0 and res.observed_tokens == 2
    rc, res, tokens = N.DecodeSession.batch_advance_one(sessions, 32, 2)
    assert rc == 0 and res.block_tokens == 5
    solo.destroy()
    for s in sessions[1:] + sessions[:1]:     # children first or last: the weights outlive the parent either way
        s.destroy()


@pytest.mark.parametrize("count", [7, 32])
def test_batch_step_at_qwen3_8b_widths_matches_solo_sessions(count):
    """The batch step's own launch shapes at the real widths (hidden 4096, 32 q / 8 kv heads x 128, MLP 12288,
    full vocabulary; 2 layers): three-wave workgroups and the rotated K walk of the gate/up pair, the q/k/v partial
    sums added by the attention, o and down in four K slices with the norms from their slice launches, the LM head
    for a block of rows. Every sequence must come out as if it had advanced alone: the same tokens as a solo session
    on the same weights unless the solo logits' lead is thin, and the same K/V rows to the end-to-end tolerance."""
    cfg = dict(N.Qwen3_8B)
    cfg["layers"] = 2
    max_ctx, steps = 96, 3
    parent = N.DecodeSession.create_synthetic(cfg, max_ctx, seed=20240301, weight_std=0.02, qk_norm=True, weight_hash=1)
    sessions = [parent] + [parent.fork_shared_weights() for _ in range(count - 1)]
    rng = np.random.default_rng(count)
    prompts = [rng.integers(0, cfg["vocab"], 1 + (5 * i) % 41).astype(np.uint32) for i in range(count)]
    streams = [[started(s, p)] for s, p in zip(sessions, prompts)]
    for _ in range(steps):
        rc, res, tokens = N.DecodeSession.batch_advance_one(sessions, 32, 2)
        assert rc == 0 and res.status == 0 and res.block_tokens == count and res.hot_path_allocations == 0
        assert parent.shares_weight_stream()
        for stream, tok in zip(streams, tokens):
            stream.append(int(tok))
    solo = parent.fork_shared_weights()
    for i in sorted({0, 1, count // 2, count - 1}):
        prompt, stream, sess = prompts[i], streams[i], sessions[i]
        rc, _ = solo.start(prompt)
        assert rc == 0
        parted = False
        for k in range(steps + 1):
            rc, _, alone = solo.advance(1)
            assert rc == 0
            logits = solo.logits()                      # of the step that produced the token just handed out
            if int(alone[0]) != stream[k]:
                top = np.sort(logits)
                assert k >= 1 and top[-1] - top[-2] <= E2E_REL_L2 * np.max(np.abs(logits)), (i, k, stream, int(alone[0]))
                parted = True
                break
        if not parted:
            P = len(prompt)
            for layer in range(cfg["layers"]):
                for token in (P, P + steps - 1):
                    gk, gv = sess.kv_row(layer, token)
                    rk, rv = solo.kv_row(layer, token)
                    assert rel_l2(O.decode16(BF16, gk), O.decode16(BF16, rk)) <= E2E_REL_L2, (i, layer, token)
                    assert rel_l2(O.decode16(BF16, gv), O.decode16(BF16, rv)) <= E2E_REL_L2, (i, layer, token)
    solo.destroy()
    for s_ in sessions[1:] + sessions[:1]:
        s_.destroy()


def test_fork_carries_a_running_sequence_and_weights_outlive_the_parent():
    """A fork taken in mid-sequence continues exactly like its parent (same cache, slots, cursor and
    sampler), both independently; destroying the parent first leaves the child's weights in place."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[0]
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 99, theta, qk_norm, bias)
    prompt = np.random.default_rng(3).integers(0, vocab, 9).astype(np.uint32)
    cfg = abi.NervaHipHfDecodeSamplerConfig()
    cfg.temperature, cfg.top_p, cfg.top_k, cfg.seed = 0.9, 0.95, 12, 777
    parent = N.DecodeSession.create(weights, 48)
    rc, _ = parent.start(prompt, sampler=cfg)
    assert rc == 0
    rc, _, head = parent.advance(5)
    assert rc == 0
    child = parent.fork_shared_weights()
    rc, _, a = parent.advance(7)
    assert rc == 0
    parent.destroy()
    rc, _, b = child.advance(7)
    assert rc == 0
    assert a.tolist() == b.tolist()           # same seed and positions: the same draws
    # the child's cache holds the parent's rows
    rc, _ = child.start(prompt)
    assert rc == 0
    child.destroy()


def test_batch_advance_one_eligibility_and_reasons():
    """The planning rules of the reference's batch step: what counts as ready, how sessions are
    grouped, what is reported when nothing runs."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[0]
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 5, theta, qk_norm, bias)
    reasons = N.DecodeSession.BATCH_REASONS
    rc, res, _ = N.DecodeSession.batch_advance_one([], 8, 2)
    assert rc == 0 and res.status == 0 and reasons[res.reason] == "no_sessions"
    hashed = N.DecodeSession.create(weights, 24, plan=N.WeightPlan.from_weights(weights))
    twin = hashed.fork_shared_weights()
    other = N.DecodeSession.create(weights, 24, plan=N.WeightPlan.from_weights(weights, block_bytes=4096))   # another plan
    plain = N.DecodeSession.create(weights, 24)
    rc, res, _ = N.DecodeSession.batch_advance_one([hashed, twin], 8, 2)
    assert rc == 0 and reasons[res.reason] == "no_ready_sessions"            # nothing started
    rc, _ = hashed.start([1, 2, 3])
    assert rc == 0
    rc, res, _ = N.DecodeSession.batch_advance_one([hashed, twin], 8, 1)
    assert reasons[res.reason] == "no_ready_sessions"                        # first token not handed out yet
    rc, _, _ = hashed.advance(1)
    first_plain = started(plain, [4, 5])
    rc, res, _ = N.DecodeSession.batch_advance_one([plain], 8, 1)
    assert rc == 0 and reasons[res.reason] == "shared_weights_unproven"      # no descriptor hash
    rc, res, _ = N.DecodeSession.batch_advance_one([hashed, plain], 8, 2)
    assert rc == 0 and reasons[res.reason] == "insufficient_compatible_ready" and res.eligible_session_count == 1
    started(twin, [7])
    started(other, [9, 9])
    # shapes outside the multi-row kernels (hidden 512): every sequence runs its own step, same contract
    rc, res, tokens = N.DecodeSession.batch_advance_one([other, plain, hashed, twin], 8, 2)
    assert rc == 0 and reasons[res.reason] == "ready" and res.block_tokens == 2 and not hashed.shares_weight_stream()
    assert tokens[0] == 0xFFFFFFFF and tokens[1] == 0xFFFFFFFF and tokens[2] < vocab and tokens[3] < vocab
    # the step is the one a solo advance would have made
    ctx = O.Context(omodel, 24, staging=1)
    otokens, margins = ctx.greedy_decode(np.array([1, 2, 3], np.uint32), 2)
    scale = float(np.max(np.abs(ctx.logits())))
    assert tokens[2] == otokens[1] or min(margins[0], margins[1]) <= E2E_REL_L2 * scale
    # target_block_tokens caps the group in request order; a session listed twice advances once
    rc, res, tokens = N.DecodeSession.batch_advance_one([hashed, hashed, twin], 1, 1)
    assert rc == 0 and res.block_tokens == 1 and tokens[0] < vocab and tokens[2] == 0xFFFFFFFF
    # capacity too small / null pointers
    lib = abi.load()
    req = abi.NervaHipHfDecodeSequenceBatchAdvanceRequest()
    req.session_count = 2
    out = abi.NervaHipHfDecodeSequenceBatchAdvanceResult()
    assert lib.nerva_hip_hf_decode_sequence_batch_advance_one(C.byref(req), C.byref(out)) == -1
    assert reasons[out.reason] == "invalid_request"
    assert lib.nerva_hip_hf_decode_sequence_batch_advance_one(None, C.byref(out)) == -1
    # a finished session (context full) drops out
    for _ in range(40):
        rc, res, _ = N.DecodeSession.batch_advance_one([hashed, twin], 8, 1)
        if reasons[res.reason] != "ready":
            break
    assert reasons[res.reason] == "no_ready_sessions"
    for s in (hashed, twin, other, plain):
        s.destroy()


@pytest.mark.parametrize("length", [1, 2, 3, 9, 17, 32, 33, 34, 64, 65, 66, 129, 130, 257, 258, 300, 513, 514, 520, 700])
def test_block_prefill_edge_lengths_match_token_walk(length, monkeypatch):
    """Prompt lengths around the prefill block sizes (the last prompt token always goes through the
    ordinary head step, so length - 1 tokens are prefilled in blocks): logits, first token and K/V
    rows agree with the token walk to the end-to-end tolerance; a context exactly as long as the
    sequence needs is enough."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[5]
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 2718, theta, qk_norm, bias)
    prompt = np.random.default_rng(length).integers(0, vocab, length).astype(np.uint32)
    outcome = {}
    for mode in ("blocks", "walk"):
        if mode == "walk":
            N.Device.set_tuning("prefill_walk", 1)
        else:
            N.Device.set_tuning("prefill_walk", 0)
        s = N.DecodeSession.create(weights, length + 2)          # room for the prompt and three tokens
        rc, res = s.start(prompt)
        assert rc == 0 and res.kv_tokens == length
        logits = s.logits()
        rows = [s.kv_row(layers - 1, t) for t in sorted({0, length // 2, length - 1})]
        rc, res, tokens = s.advance(3)
        assert rc == 0 and res.observed_tokens == 3
        rc, _, _ = s.advance(1)                                   # the context is full now
        assert rc == -1
        outcome[mode] = (logits, rows, tokens.tolist())
        s.destroy()
    (lb, rb, tb), (lw, rw, tw) = outcome["blocks"], outcome["walk"]
    assert rel_l2(lb, lw) <= E2E_REL_L2
    for (kb, vb), (kw, vw) in zip(rb, rw):
        assert rel_l2(O.decode16(dtype, kb), O.decode16(dtype, kw)) <= E2E_REL_L2
        assert rel_l2(O.decode16(dtype, vb), O.decode16(dtype, vw)) <= E2E_REL_L2
    top = np.sort(lw)
    assert tb[0] == tw[0] or top[-1] - top[-2] < E2E_REL_L2 * np.max(np.abs(lw))


def test_prefill_block_size_changes_only_the_block_boundaries():
    """A session whose four projections have the kernels for them prefills 512 tokens at a time (256 where only the
    kernel for those blocks takes its widths); the hook "prefill_block_tokens" = 256 or 128 keeps the smaller
    blocks. Same arithmetic per token either way: logits, K/V rows and the first tokens of a 600-token prompt agree
    to the end-to-end tolerance."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[5]
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 99, theta, qk_norm, bias)
    prompt = np.random.default_rng(600).integers(0, vocab, 600).astype(np.uint32)
    outcome = {}
    try:
        for block in (0, 256, 128):
            N.Device.set_tuning("prefill_block_tokens", block)
            s = N.DecodeSession.create(weights, 608)
            assert s.create_result.prefill_chunk_tokens == (block if block else 512)
            rc, res = s.start(prompt)
            assert rc == 0 and res.kv_tokens == 600 and res.hot_path_allocations == 0
            logits = s.logits()
            rows = [s.kv_row(layers - 1, t) for t in (0, 127, 128, 255, 256, 511, 512, 598)]
            rc, res, tokens = s.advance(4)
            assert rc == 0
            outcome[block] = (logits, rows, tokens.tolist())
            s.destroy()
    finally:
        N.Device.set_tuning("prefill_block_tokens", 0)
    lb, rb, tb = outcome[128]
    for other in (0, 256):
        la, ra, ta = outcome[other]
        assert rel_l2(la, lb) <= E2E_REL_L2
        for (ka, va), (kb, vb) in zip(ra, rb):
            assert rel_l2(O.decode16(dtype, ka), O.decode16(dtype, kb)) <= E2E_REL_L2
            assert rel_l2(O.decode16(dtype, va), O.decode16(dtype, vb)) <= E2E_REL_L2
        top = np.sort(lb)
        assert ta[0] == tb[0] or top[-1] - top[-2] < E2E_REL_L2 * np.max(np.abs(lb))


def test_batch_advance_one_fills_contexts_to_the_last_slot():
    """Sessions of different context sizes in one batch: each goes on until its own context is full,
    finishes there (session_api_batch_fork_destroy.inc.cu:296-299), and the others continue."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[5]
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 161, theta, qk_norm, bias)
    plan = N.WeightPlan.from_weights(weights)
    small = N.DecodeSession.create(weights, 18, plan=plan)       # 17 blocks of context: crosses a 16-token tile
    large = N.DecodeSession.create(weights, 40, plan=plan)
    assert small.shares_weight_stream()
    started(small, [3, 4, 5])
    started(large, list(range(20)))
    produced = {0: 1, 1: 1}
    for step in range(30):
        rc, res, tokens = N.DecodeSession.batch_advance_one([small, large], 32, 1)
        assert rc == 0
        if N.DecodeSession.BATCH_REASONS[res.reason] != "ready":
            break
        for i in (0, 1):
            if tokens[i] != 0xFFFFFFFF:
                assert tokens[i] < vocab
                produced[i] += 1
    assert N.DecodeSession.BATCH_REASONS[res.reason] == "no_ready_sessions"
    # prompt + produced - 1 tokens are in the cache: exactly the context size
    assert 3 + produced[0] - 1 == 18 and 20 + produced[1] - 1 == 40
    rc, _, _ = small.advance(1)
    assert rc == -1
    small.destroy()
    large.destroy()


def expected_slot_bytes(position, token):
    """{request_id 1, sequence_id 1, token_index, token, version = index + 1, completion 1, host_copied 0}
    laid out as the 40-byte C struct (nerva_cuda_api.h:29-37, sampler.cu:394-407)."""
    slot = abi.NervaHipSyntheticTokenSlot()
    C.memset(C.byref(slot), 0, C.sizeof(slot))
    slot.request_id, slot.sequence_id, slot.token_index, slot.token = 1, 1, position, token
    slot.version, slot.completion, slot.host_copied = position + 1, 1, 0
    return np.frombuffer(bytes(slot), np.uint8)


def test_token_slots_hold_the_reference_bytes(kat):
    """Every byte of every published slot, downloaded from device memory: the known-answer stream and a random
    model's greedy and sampled streams; slots before the first sampled position and behind the last stay zero."""
    weights, k = kat_models(kat, True)
    session = N.DecodeSession.create(weights, 8)
    rc, _ = session.start(k["prompt"])
    assert rc == 0
    rc, _, tokens = session.advance(4)
    assert rc == 0 and tokens.tolist() == k["tokens"]
    raw = session.slots(0, 8)
    for i, tok in enumerate(k["tokens"]):          # prompt [0]: the first sampled token sits in slot 0
        assert np.array_equal(raw[i], expected_slot_bytes(i, tok)), i
    assert not raw[4:].any()
    session.destroy()

    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[0]
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 606, theta, qk_norm, bias)
    prompt = np.random.default_rng(606).integers(0, vocab, 37).astype(np.uint32)
    session = N.DecodeSession.create(weights, 64)
    for sampler in (None, (0.8, 0.9, 20, 5)):
        cfg = None
        if sampler is not None:
            cfg = abi.NervaHipHfDecodeSamplerConfig()
            cfg.temperature, cfg.top_p, cfg.top_k, cfg.seed = sampler
        rc, _ = session.start(prompt, sampler=cfg)
        assert rc == 0
        rc, _, tokens = session.advance(9)
        assert rc == 0
        raw = session.slots(0, 64)
        P = len(prompt)
        assert not raw[:P - 1].any() and not raw[P - 1 + 9:].any()
        for i, tok in enumerate(tokens):
            assert np.array_equal(raw[P - 1 + i], expected_slot_bytes(P - 1 + i, int(tok))), (sampler, i)
    session.destroy()


def test_step_whose_attention_merge_gives_up_fails_the_advance():
    """A decode step in which a split of the attention never hands its partial over (test hook; the spin limit of
    the merges set to a few polls, every kernel exits normally): the slot of that token says so, advance returns -1
    with the step-fault error and the sequence is over; a session made without the hook decodes the same prompt."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[0]
    weights, _ = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 31, theta, qk_norm, bias)
    prompt = np.random.default_rng(31).integers(0, vocab, 700).astype(np.uint32)     # 44 blocks: the splits merge
    good = N.DecodeSession.create(weights, 720)
    rc, _ = good.start(prompt)
    assert rc == 0
    rc, res, want = good.advance(6)
    assert rc == 0 and res.hip_error == 0
    N.Device.set_tuning("attn_merge_spin_limit", 4)
    N.Device.set_tuning("attn_withhold_split", 1 + 3)
    try:
        bad = N.DecodeSession.create(weights, 720)
        rc, _ = bad.start(prompt)          # the last prompt token's step already runs the decode attention
        assert rc == 0
        rc, res, tokens = bad.advance(6)
    finally:
        N.Device.set_tuning("attn_merge_spin_limit", 0)
        N.Device.set_tuning("attn_withhold_split", 0)
    assert rc == -1 and res.status == -1 and res.hip_error == abi.NERVA_HIP_ERROR_STEP_FAULT
    assert res.observed_tokens == 0 and len(tokens) == 0
    raw = bad.slots(len(prompt) - 1, 1)
    assert raw[0].view(np.uint32)[8] == abi.NERVA_HIP_SLOT_DEVICE_FAULT          # completion word
    rc, res, _ = bad.advance(1)
    assert rc == -1                                                                # the sequence ended with the fault
    bad.destroy()
    rc, res, again = good.advance(3)                                               # the healthy session is untouched
    assert rc == 0
    fresh = N.DecodeSession.create(weights, 720)
    rc, _ = fresh.start(prompt)
    assert rc == 0
    rc, res, tokens = fresh.advance(9)
    assert rc == 0 and tokens.tolist() == want.tolist() + again.tolist()
    for s in (good, fresh):
        s.destroy()


def test_batch_step_of_sessions_with_their_own_steps_at_long_context():
    """Shapes the multi-row kernels do not take (hidden 512) advance a batch as one captured decode step per
    session, one after the other. At contexts of 1000 and more tokens each step's attention launch spreads over
    64 splits that merge inside the launch: tokens equal those of the same sessions advanced alone, and the rows
    appended equal the oracle's on the same history."""
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = GEOMETRIES[0]
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, 88, theta, qk_norm, bias)
    rng = np.random.default_rng(88)
    prompts = [rng.integers(0, vocab, n).astype(np.uint32) for n in (1030, 1333, 1571)]
    steps, max_ctx = 5, 1600
    plan = N.WeightPlan.from_weights(weights)
    parent = N.DecodeSession.create(weights, max_ctx, plan=plan, tensor_pointers=False)
    sessions = [parent, parent.fork_shared_weights(), parent.fork_shared_weights()]
    streams = [[started(s, p)] for s, p in zip(sessions, prompts)]
    for _ in range(steps):
        rc, res, tokens = N.DecodeSession.batch_advance_one(sessions, 8, 2)
        assert rc == 0 and res.status == 0 and res.block_tokens == 3 and not parent.shares_weight_stream()
        for stream, tok in zip(streams, tokens):
            stream.append(int(tok))
    solo = parent.fork_shared_weights()
    for prompt, stream in zip(prompts, streams):
        rc, _ = solo.start(prompt)
        assert rc == 0
        rc, _, alone = solo.advance(steps + 1)
        assert rc == 0 and alone.tolist() == stream, len(prompt)      # the same kernels on the same inputs
    ctx, _ = oracle_follow(omodel, max_ctx, prompts[0], streams[0][:-1])
    P = len(prompts[0])
    for layer in range(layers):
        for token in (P, P + steps - 1):
            gk, gv = sessions[0].kv_row(layer, token)
            rk, rv = ctx.read_kv16(layer, token)
            tol = 2e-3 if layer == 0 else E2E_REL_L2
            assert rel_l2(O.decode16(dtype, gk), O.decode16(dtype, rk)) <= tol, (layer, token)
            assert rel_l2(O.decode16(dtype, gv), O.decode16(dtype, rv)) <= tol, (layer, token)
    ctx.close()
    solo.destroy()
    for s in sessions[::-1]:
        s.destroy()
