"""In-session parity, link by link and step by step (GPU, through the C ABI).

A session runs a greedy stream; every decode step is traced (nerva_hip_session_trace_next_step: same
kernels and launch shapes as the captured step, each kernel's output vector copied out) and every
kernel is compared with the oracle operator on the device's own input at relative L2 <= 1e-3
(oracle/links.py). On top of that the oracle follows the device's tokens (teacher forcing) and
every step of the stream - not just the steps before a first divergence - must give the oracle's
token, unless the oracle's lead over the device's token is within the measured difference of the two
logit vectors, which itself must stay within the budget of the chain: one operator tolerance per
16-bit staging point between the embedding and the logits (6 per layer + the final norm).
"""
import numpy as np
import pytest

import nerva_amd as N
import oracle as O
from oracle.links import REL_L2, chain_budget, check_step_links, rel_l2, run_traced_stream
from test_gpu_session import GEOMETRIES, random_model

pytestmark = pytest.mark.gpu

BF16 = 1
SEED = 0x4E45525641


@pytest.mark.parametrize("geom", GEOMETRIES)
def test_every_link_of_every_step_matches_the_oracle(geom):
    dtype, hidden, heads, kv, hd, inter, vocab, layers, theta, qk_norm, bias = geom
    weights, omodel = random_model(dtype, hidden, heads, kv, hd, inter, vocab, layers, hidden, theta, qk_norm, bias)
    prompt = np.random.default_rng(1).integers(0, vocab, 21).astype(np.uint32)
    steps = 24
    s = N.DecodeSession.create(weights, 64)
    tokens, worst, e2e = run_traced_stream(s, omodel, prompt, steps, 64)
    # the traced stream is the stream the captured graph produces
    rc, _ = s.start(prompt)
    rc, res, replayed = s.advance(steps)
    assert rc == 0 and res.graph_replays == steps - 1 and replayed.tolist() == tokens
    s.destroy()
    print("links (worst rel L2 over %d steps): %s; end-to-end logits %.2e (budget %.1e)"
          % (steps - 1, ", ".join("%s %.1e" % kv_ for kv_ in sorted(worst.items())), e2e, chain_budget(layers)), flush=True)


def test_links_at_qwen3_8b_widths_two_layers_full_vocabulary():
    """hidden 4096, 32 q / 8 kv heads x 128, MLP 12288, vocabulary 151936 (the real launch shapes of
    every GEMV, the LM head's looping launch with its candidates, 32 heads of attention), 2 layers,
    device-generated weights regenerated bit-identically on the host; 150-token prompt (a full
    128-token prefill block and a partial one), 24 greedy tokens, every step traced."""
    cfg = dict(N.Qwen3_8B)
    cfg["layers"] = 2
    max_ctx = 192
    s = N.DecodeSession.create_synthetic(cfg, max_ctx, seed=SEED, weight_std=0.02)
    model = O.synthetic_model(cfg, SEED, 0.02, threads=16)
    prompt = O.synth_tokens(SEED, 99, 150, cfg["vocab"])
    steps = 24
    tokens, worst, e2e = run_traced_stream(s, model, prompt, steps, max_ctx, threads=16)
    rc, _ = s.start(prompt)
    rc, res, replayed = s.advance(steps)
    assert rc == 0 and res.graph_replays == steps - 1 and replayed.tolist() == tokens
    s.destroy()
    print("Qwen3-8B widths: links (worst rel L2): %s; end-to-end logits %.2e"
          % (", ".join("%s %.1e" % kv_ for kv_ in sorted(worst.items())), e2e), flush=True)


def test_long_context_links_at_qwen3_8b_widths():
    """The same two full-width layers at 4200 tokens of context: the prompt goes through 33 prefill
    blocks of 128 tokens, decode steps run with the 32-split attention and as graph replays. The oracle
    cannot walk a 4200-token prompt at this width in test time, so it starts from the device's cache
    (downloaded) - the decode steps are then checked link by link on the device's own inputs, and
    against the teacher-forced oracle, like everywhere else. The block prefill itself is checked
    against the device's token walk: the last prompt rows of both layers and the logits."""
    cfg = dict(N.Qwen3_8B)
    cfg["layers"] = 2
    P, steps, max_ctx = 4200, 6, 4224
    s = N.DecodeSession.create_synthetic(cfg, max_ctx, seed=SEED, weight_std=0.02)
    model = O.synthetic_model(cfg, SEED, 0.02, threads=16)
    dt = model.dtype
    prompt = O.synth_tokens(SEED, 98, P, cfg["vocab"])
    rc, res = s.start(prompt)
    assert rc == 0
    ctx = O.Context(model, max_ctx, staging=1, threads=16)
    for l in range(2):
        k, v = s.kv_range(l, 0, P)
        ctx.load_kv16(l, k, v)
    ctx.set_len(P)
    rc, res, out = s.advance(1)
    assert rc == 0
    tokens = [int(out[0])]
    prefill_logits = s.logits()
    assert tokens[0] == O.greedy_argmax(prefill_logits, skip_nonfinite=True)
    worst, e2e = {}, 0.0
    for step in range(1, steps):
        position = P + step - 1
        ctx.forward_token(tokens[-1], prompt_token=False, want_logits=True)
        if step in (1, steps - 1):
            rc, res, out, trace = s.traced_advance()
            assert rc == 0 and trace is not None
            rows = [s.kv_range(l, 0, position + 1) for l in range(2)]
            errs = check_step_links(model, trace, position, tokens[-1], int(out[0]), [r[0] for r in rows],
                                    [r[1] for r in rows], threads=16)
            for k_, v_ in errs.items():
                worst[k_] = max(worst.get(k_, 0.0), v_)
            dev_logits = trace["logits"]
        else:
            rc, res, out = s.advance(1)
            assert rc == 0 and res.graph_replays == 1 and res.hot_path_allocations == 0
            dev_logits = s.logits()
        tok = int(out[0])
        ora = ctx.logits()
        e = rel_l2(dev_logits, ora)
        e2e = max(e2e, e)
        assert e <= chain_budget(2), (step, e)
        top = O.greedy_argmax(ora, skip_nonfinite=True)
        if top != tok:
            assert float(ora[top] - ora[tok]) <= 2.0 * float(np.max(np.abs(dev_logits - ora))), step
        tokens.append(tok)
    ctx.close()
    # block prefill against the token walk on the device (different summation order in the projections)
    last_rows = [s.kv_row(l, P - 1) for l in range(2)]
    s.destroy()
    N.Device.set_tuning("prefill_walk", 1)
    try:
        w = N.DecodeSession.create_synthetic(cfg, max_ctx, seed=SEED, weight_std=0.02)
        rc, res = w.start(prompt)
        assert rc == 0
        walk_logits = w.logits()
        for l in range(2):
            for got, ref in zip(last_rows[l], w.kv_row(l, P - 1)):
                assert rel_l2(O.decode16(dt, got), O.decode16(dt, ref)) <= (2e-3 if l == 0 else chain_budget(1)), l
        w.destroy()
    finally:
        N.Device.set_tuning("prefill_walk", 0)
    assert rel_l2(prefill_logits, walk_logits) <= chain_budget(2)
    print("4200-token context: links (worst rel L2): %s; end-to-end logits %.2e; block prefill vs walk logits %.2e"
          % (", ".join("%s %.1e" % kv_ for kv_ in sorted(worst.items())), e2e, rel_l2(prefill_logits, walk_logits)),
          flush=True)


def test_full_depth_step_at_8k_context_first_layers_last_layer_and_head():
    """The named workload at its real size: 36 layers of Qwen3-8B widths (one 17.6 GB arena, device-generated
    weights), a prompt of 8192 tokens prefilled in blocks, then decode steps with the 32-split attention. One
    step is traced and layers 0, 1 and 35 and the head are checked link by link on the device's own inputs -
    weights of those layers regenerated bit for bit on the host, their K/V rows downloaded - and the step after
    it, a graph replay, must start from the token the traced step published."""
    cfg = dict(N.Qwen3_8B)
    P, max_ctx, ids = 8192, 8192 + 16, [0, 1, 35]
    s = N.DecodeSession.create_synthetic(cfg, max_ctx, seed=SEED, weight_std=0.02, qk_norm=True)
    assert s.create_result.layer_count == 36
    prompt = O.synth_tokens(SEED, 97, P, cfg["vocab"])
    rc, res = s.start(prompt)
    assert rc == 0
    rc, res, out = s.advance(2)
    assert rc == 0 and res.graph_replays == 1 and res.hot_path_allocations == 0
    token, position = int(out[1]), P + 1
    model = O.synthetic_model(cfg, SEED, 0.02, layer_ids=ids, embedding_rows=[token], threads=16)
    rc, res, out, trace = s.traced_advance()
    assert rc == 0 and trace is not None and len(trace["layers"]) == 36
    rows = [s.kv_range(l, 0, position + 1) for l in ids]
    errs = check_step_links(model, trace, position, token, int(out[0]), [r[0] for r in rows], [r[1] for r in rows],
                            threads=16, layer_ids=ids)
    rc, res, after = s.advance(1)
    assert rc == 0 and res.graph_replays == 1
    raw = s.slots(position, 2).view(np.uint32)
    assert raw[0][4] == int(out[0]) and raw[1][4] == int(after[0])       # token words of the two slots
    s.destroy()
    print("36 layers, context %d: layers 0, 1, 35 and head (worst rel L2): %s"
          % (position, ", ".join("%s %.1e" % kv_ for kv_ in sorted(errs.items()))), flush=True)


def test_lm_head_full_vocabulary_tie_and_nonfinite_rows():
    """The LM head at its real size (151936 x 4096, the looping launch that leaves one candidate per
    workgroup, then the finishing launch) inside a session whose one layer is small: two identical rows
    far apart must tie and give the lower index, and a row whose logit is not finite must be skipped
    although it comes first (sampler.cu:35-40, 89-119)."""
    dtype, hidden, heads, kv, hd, inter, vocab = BF16, 4096, 4, 1, 128, 1024, 151936
    rng = np.random.default_rng(5)
    e = lambda shape, mean=0.0, sd=0.02: O.encode16(dtype, rng.normal(mean, sd, shape).astype(np.float32))
    layer = dict(rms_attn=e(hidden, 1.0), rms_mlp=e(hidden, 1.0), w_q=e((heads * hd, hidden)), w_k=e((kv * hd, hidden)),
                 w_v=e((kv * hd, hidden)), w_o=e((hidden, heads * hd)), q_norm=e(hd, 1.0), k_norm=e(hd, 1.0),
                 w_gate=e((inter, hidden)), w_up=e((inter, hidden)), w_down=e((hidden, inter)))
    emb = O.synth_16(dtype, SEED, 1, vocab * hidden, 0.0, 1.0).reshape(vocab, hidden)
    lm_head = O.synth_16(dtype, SEED, 3, vocab * hidden, 0.0, 0.02).reshape(vocab, hidden).copy()
    final_norm = e(hidden, 1.0)
    args = lambda head: (dtype, hidden, heads, kv, hd, inter, vocab, 1e-6, 1e6, emb, [layer], final_norm, head)
    prompt = np.array([7, 150000, 31], np.uint32)
    # first pass: the plain head; the decode step at position 3 is traced and its logits are checked
    # against the oracle on the device's own final hidden state
    s = N.DecodeSession.create(N.ModelWeights(*args(lm_head)), 16)
    rc, res = s.start(prompt)
    assert rc == 0
    rc, res, out = s.advance(1)
    token0 = int(out[0])
    rc, res, out, trace = s.traced_advance()
    assert rc == 0 and trace is not None
    h16 = trace["h16"]
    assert np.max(np.abs(h16.astype(np.int32) - O.encode16(dtype, O.rms_norm(dtype, trace["layers"][0]["x"], final_norm,
                                                                           1e-6)).astype(np.int32))) <= 1
    ref = O.gemv(dtype, lm_head, O.decode16(dtype, h16), threads=16)
    assert rel_l2(trace["logits"], ref) <= REL_L2
    assert int(out[0]) == O.greedy_argmax(trace["logits"], skip_nonfinite=True)
    s.destroy()
    # second pass: rows 9 and 140001 both point along that hidden state (a tie far above every other
    # logit), row 3 is all +inf (its logit is inf or NaN: never a candidate). The token of the first pass
    # joins the prompt, so the head sees the same hidden state up to the prompt staging's rounding.
    direction = O.encode16(dtype, np.sign(O.decode16(dtype, h16)).astype(np.float32))
    lm_head[9] = direction
    lm_head[140001] = direction
    lm_head[3] = 0x7F80
    s = N.DecodeSession.create(N.ModelWeights(*args(lm_head)), 16)
    rc, res = s.start(np.append(prompt, np.uint32(token0)))
    assert rc == 0
    logits = s.logits()
    rc, res, out = s.advance(1)
    assert rc == 0
    assert not np.isfinite(logits[3])
    finite = np.isfinite(logits)
    assert logits[9] == logits[140001] == np.max(logits[finite]) and np.sum(logits[finite] == logits[9]) == 2
    assert int(out[0]) == 9
    assert N.argmax(dev(logits), vocab) == 9
    s.destroy()


def dev(a):
    return N.DeviceBuffer.from_numpy(a)
