"""Checker code (test infrastructure, like the rest of this package; the product never imports it).

Link-by-link parity of a running session: every kernel of a traced decode step is checked against
the oracle's statement of the same operator ON THE DEVICE'S OWN INPUT VECTOR (the output the previous
kernel left), so each link is held to the operator tolerance - relative L2 <= 1e-3, indices and
embedding rows bit-exact - no matter how many 16-bit staging points lie before it.

A kernel whose output is rounded to 16 bit is held to the same 1e-3 on the value BEFORE the rounding,
which is where the tolerance is stated (f32 accumulation): the device's 16-bit value must be a rounding
of some value within 1e-3 of the oracle's f32 value, element by element - |dev16 - ref| <= half a
16-bit step at ref + 1e-3 * (|ref| + rms(ref)). Comparing the two ROUNDED vectors in L2 instead would
measure how many elements sit near a rounding boundary (one bf16 step is 4e-3..8e-3 of the element),
not the kernel: one boundary case in the fused RMSNorm's 16-bit output moves every product by ~2e-4,
which carries ~5 % of bf16 outputs over a boundary, 1.2e-3 in L2.

The operators are composed from the oracle's primitives in the order of the CUDA session's step
(session_decode_prefill.inc.cu:74-372; kernels.cu:182-217, 287-432, 577-612, 651-687; sampler.cu:89-119).
"""
import numpy as np

import oracle as O

REL_L2 = 1e-3


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _round16(dtype, v):
    return O.decode16(dtype, O.encode16(dtype, v))


def _bias(dtype, layer, name, n):
    b = layer.get(name)
    return O.decode16(dtype, b).astype(np.float32) if b is not None else np.zeros(n, np.float32)


def _gemv16(dtype, w, x16, threads):
    """W . x for a 16-bit x: sequential f32 on one thread, row-parallel on several (same sums per row)."""
    if threads > 1:
        return O.gemv(dtype, w, O.decode16(dtype, x16), threads=threads)
    return O.gemv_x16(dtype, w, x16)


def check_step_links(model, trace, position, token_in, token_out, k_rows, v_rows, threads=1, layer_ids=None):
    """Checks every link of one traced decode step. `k_rows[l]`, `v_rows[l]`: the device's cache rows
    0..position of layer l in logical order (16-bit), read after the step, so row `position` is the
    one the step appended. `layer_ids`: the session's layers that model.layers[i] (and k_rows[i],
    v_rows[i]) stand for, when the model holds only some of them; every checked layer takes the
    device's own input (the output the trace holds for the layer before it).
    Returns {link name: measured error}; raises AssertionError on a miss."""
    m, dt = model, model.dtype
    H, HD = m.hidden, m.head_dim
    A, KV = m.heads * HD, m.kv_heads * HD
    errs = {}

    def link16(name, got16, ref):
        """16-bit output of a kernel against the oracle's f32 value of it (see the module text)."""
        ref = np.asarray(ref, np.float64)
        got = O.decode16(dt, got16).astype(np.float64)
        mant = 7 if dt == O.BF16 else 10
        mag = np.maximum(np.abs(ref), 2.0 ** -14 if dt != O.BF16 else 2.0 ** -126)
        half_step = 0.5 * 2.0 ** (np.floor(np.log2(mag)) - mant)
        rms = float(np.sqrt(np.mean(ref * ref)))
        excess = (np.abs(got - ref) - half_step) / (np.abs(ref) + rms + 1e-30)
        e = float(max(np.max(excess), 0.0))
        errs[name] = max(errs.get(name, 0.0), e)
        assert e <= REL_L2, "%s at position %d: %.3e of the value beyond the rounding step" % (name, position, e)
        errs[name + "_rounded_l2"] = max(errs.get(name + "_rounded_l2", 0.0), rel_l2(got, _round16(dt, ref.astype(np.float32))))

    def link(name, got, ref, tol=REL_L2):
        e = rel_l2(got, ref)
        errs[name] = max(errs.get(name, 0.0), e)
        assert e <= tol, "%s at position %d: rel L2 %.3e > %.1e" % (name, position, e, tol)

    # embedding: the row of the token the step consumed, bit for bit
    x = trace["x0"]
    assert np.array_equal(x.view(np.uint32), O.decode16(dt, m.embeddings[token_in]).astype(np.float32).view(np.uint32)), \
        "embedding row of token %d" % token_in
    # (a model that holds only the first layers of the session's - the full-size check of the bench -
    # gets those layers checked; the head then takes the x the session's last layer left)
    ids = list(range(len(m.layers))) if layer_ids is None else list(layer_ids)
    for l, w in enumerate(m.layers):
        t = trace["layers"][ids[l]]
        if ids[l] > 0:
            x = trace["layers"][ids[l] - 1]["x"]
        # attention RMSNorm (fused into the qkv launch; its 16-bit output is the projection's input),
        # then the qkv projection (raw: biases are added by the attention kernel)
        link16("attn_norm", t["a16"], O.rms_norm(dt, x, w["rms_attn"], m.rms_eps))
        wqkv = np.concatenate([w["w_q"], w["w_k"], w["w_v"]], axis=0)
        link("qkv", t["qkv"], _gemv16(dt, wqkv, t["a16"], threads))
        # head preparation on the device's qkv: bias, per-head RMSNorm, RoPE, K/V rounded to 16 bit
        q = t["qkv"][:A] + _bias(dt, w, "q_bias", A)
        k = t["qkv"][A:A + KV] + _bias(dt, w, "k_bias", KV)
        v = t["qkv"][A + KV:] + _bias(dt, w, "v_bias", KV)
        if w.get("q_norm") is not None:
            q = O.per_head_rms_norm(dt, w["q_norm"], HD, q, m.rms_eps)
        if w.get("k_norm") is not None:
            k = O.per_head_rms_norm(dt, w["k_norm"], HD, k, m.rms_eps)
        if m.rope_theta:
            q = O.rope(HD, m.heads, position, m.rope_theta, q)
            k = O.rope(HD, m.kv_heads, position, m.rope_theta, k)
        # the appended row: the same inputs, so at most one unit of the 16-bit value apart
        for name, got, ref in (("k_row", k_rows[l][position], O.encode16(dt, k)),
                               ("v_row", v_rows[l][position], O.encode16(dt, v))):
            gf, rf = O.decode16(dt, got), O.decode16(dt, ref)
            units = np.abs(got.astype(np.int32) - ref.astype(np.int32))
            assert np.all((units <= 1) | (np.abs(gf - rf) <= 1e-5 * np.max(np.abs(rf)))), name
            link(name, gf, rf)
        # attention over the device's own cache (rows 0..position as the device holds them)
        n = position + 1
        table0 = np.zeros(1, np.uint32)
        attn = O.attention_paged16(dt, m.heads, m.kv_heads, HD, n, q, k_rows[l][:n], v_rows[l][:n], table0, 0, 1, n)
        link16("attention", t["attn16"], attn)
        # o projection + bias + residual
        r = _gemv16(dt, w["w_o"], t["attn16"], threads) + _bias(dt, w, "o_bias", H) + x
        link("o", t["r"], r)
        # MLP: RMSNorm -> gate/up -> SiLU(gate) * up rounded to 16 bit
        link16("mlp_norm", t["m16"], O.rms_norm(dt, t["r"], w["rms_mlp"], m.rms_eps))
        g, u = _gemv16(dt, w["w_gate"], t["m16"], threads), _gemv16(dt, w["w_up"], t["m16"], threads)
        ff = (g / (np.float32(1) + np.exp(-g, dtype=np.float32))) * u
        link16("gate_up", t["ff16"], ff)
        # down projection + residual (f32 between layers in decode, kernels.cu:661-663)
        link("down", t["x"], t["r"] + _gemv16(dt, w["w_down"], t["ff16"], threads))
        x = t["x"]
    x = trace["layers"][-1]["x"] if trace["layers"] else x
    # final norm, LM head, greedy token
    link16("final_norm", trace["h16"], O.rms_norm(dt, x, m.final_norm, m.rms_eps))
    logits = _gemv16(dt, m.lm_head, trace["h16"], threads)
    link("lm_head", trace["logits"], logits)
    # the device's token is the first maximum of ITS logits, exactly (partials + finish launch)
    assert token_out == O.greedy_argmax(trace["logits"], skip_nonfinite=True), "argmax of the device's logits"
    # and the oracle's token for the same input vector, unless its lead is inside the measured LM-head error
    d = float(np.max(np.abs(trace["logits"] - logits)))
    assert d <= REL_L2 * float(np.max(np.abs(logits))), "LM-head element error %.3e" % d
    top = O.greedy_argmax(logits, skip_nonfinite=True)
    errs["token_margin_used"] = 0.0
    if top != token_out:
        lead = float(logits[top] - logits[token_out])
        assert lead <= 2.0 * d, "token %d vs oracle %d with a lead of %.3e (LM-head error %.3e)" % (token_out, top, lead, d)
        errs["token_margin_used"] = lead
    return errs


def chain_budget(layers):
    """Relative L2 the logits may differ by after `layers` layers when every 16-bit staging point
    (attention-norm output, K row, V row, attention output, MLP-norm output, SwiGLU output per layer,
    final-norm output) contributes at most one operator tolerance."""
    return (6 * layers + 1) * REL_L2


def run_traced_stream(session, model, prompt, steps, max_ctx, threads=1, links_every=1, trace_links=True):
    """start + `steps` tokens, one advance(1) per token; traces and checks every `links_every`-th decode
    step link by link (trace_links=False: never - sessions whose step is not the launch-per-piece one
    cannot be traced) and EVERY step against the oracle that follows the device's tokens: the logits
    within the chain's budget, and the token the oracle's unless the oracle's lead over it is within
    twice the measured logit difference. Returns (tokens, worst link errors, worst logits rel L2)."""
    dt, layers = model.dtype, len(model.layers)
    rc, res = session.start(prompt)
    assert rc == 0, res.hip_error
    ctx = O.Context(model, max_ctx, staging=1, threads=threads)
    for i, t in enumerate(prompt):
        ctx.forward_token(int(t), prompt_token=True, want_logits=(i + 1 == len(prompt)))
    tokens, worst, e2e = [], {}, 0.0

    def teacher_forced(dev_logits, token, step):
        nonlocal e2e
        ora = ctx.logits()
        e = rel_l2(dev_logits, ora)
        e2e = max(e2e, e)
        assert e <= chain_budget(layers), "step %d: logits differ by %.3e (budget %.1e)" % (step, e, chain_budget(layers))
        top = O.greedy_argmax(ora, skip_nonfinite=True)
        if top != token:
            lead, d = float(ora[top] - ora[token]), float(np.max(np.abs(dev_logits - ora)))
            assert lead <= 2.0 * d, "step %d: token %d vs oracle %d, lead %.3e, logit difference %.3e" % (
                step, token, top, lead, d)

    # token 0 comes out of start(): prefill logits against the oracle's prompt walk
    rc, res, out = session.advance(1)
    assert rc == 0 and res.kernel_launches == 0
    tokens.append(int(out[0]))
    assert tokens[0] == O.greedy_argmax(session.logits(), skip_nonfinite=True)
    teacher_forced(session.logits(), tokens[0], 0)
    for step in range(1, steps):
        position = len(prompt) + step - 1
        ctx.forward_token(tokens[-1], prompt_token=False, want_logits=True)
        if trace_links and (step % links_every == 0 or step == 1):
            rc, res, out, trace = session.traced_advance()
            assert rc == 0 and trace is not None and res.graph_replays == 0
            tok = int(out[0])
            rows = [session.kv_range(l, 0, position + 1) for l in range(layers)]
            errs = check_step_links(model, trace, position, tokens[-1], tok, [r[0] for r in rows],
                                    [r[1] for r in rows], threads=threads)
            for k, v in errs.items():
                worst[k] = max(worst.get(k, 0.0), v)
            dev_logits = trace["logits"]
        else:
            rc, res, out = session.advance(1)
            assert rc == 0 and res.graph_replays == 1
            tok, dev_logits = int(out[0]), session.logits()
            assert tok == O.greedy_argmax(dev_logits, skip_nonfinite=True)
        teacher_forced(dev_logits, tok, step)
        tokens.append(tok)
    ctx.close()
    return tokens, worst, e2e


def assert_stream_follows_oracle(model, prompt, device_tokens, max_ctx, threads=1):
    """For streams produced by one multi-step call, where the device's logits of each step are not
    kept: the oracle walks the prompt and then consumes the DEVICE's tokens, and at every step - also
    after a step where the two disagreed - the device's token must be the oracle's choice or trail it by
    no more than twice the chain's budget times the largest logit (the element-wise reading of the
    budget; tests that can see the device's logits use the measured difference instead).
    Returns the number of steps on which the tokens were equal."""
    layers = len(model.layers)
    ctx = O.Context(model, max_ctx, staging=1, threads=threads)
    for i, t in enumerate(prompt):
        ctx.forward_token(int(t), prompt_token=True, want_logits=(i + 1 == len(prompt)))
    equal = 0
    for step, tok in enumerate(device_tokens):
        tok = int(tok)
        if step > 0:
            ctx.forward_token(int(device_tokens[step - 1]), prompt_token=False, want_logits=True)
        ora = ctx.logits()
        top = O.greedy_argmax(ora, skip_nonfinite=True)
        if top == tok:
            equal += 1
        else:
            lead = float(ora[top] - ora[tok])
            assert lead <= 2.0 * chain_budget(layers) * float(np.max(np.abs(ora))), (step, tok, top, lead)
    ctx.close()
    return equal
