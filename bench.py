#!/usr/bin/env python3
"""Benchmark of the batch-1 decode hot path on one MI355X.

Workload (BASELINE.json configs[4], the one the metric is quoted on): Qwen3-8B-architecture
decoder, random-init bf16 weights generated on the device, batch 1, a prompt of 8192 random
token ids prefilled into the paged KV cache, then greedy decode under hipGraph replay.
A "step" is one decoded token (one graph replay = the whole per-token weight + KV stream).

Prints ONE JSON line: whole-step tok/s, plus
  roofline     - the dominant kernel (fused gate_up GEMV): algorithmic bytes / average launch
                 duration measured with hipEvents on the session stream, vs 8 TB/s HBM;
  cpu_baseline - the CPU oracle (scalar port of the reference's CPU path) timed on this
                 host on a bounded sample of the same decode step, extrapolated to tok/s.
"""
import argparse
import concurrent.futures
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes one gate_up launch moves at the Qwen3-8B shape (24576x4096 bf16): FETCH_SIZE + WRITE_SIZE
# per dispatch from two `rocprofv3 --pmc` runs, each scaled by what the counter reads for a plain
# 256 MiB copy kernel (profiles/gate_up_gemv_hbm_traffic_pmc.txt). Not measurable in-process.
# Keyed to the launch the figure was measured for - (hidden, intermediate, kernel variant, workgroups,
# rotated walk, chunks per request batch) as nerva_hip_gemv_launch_shape reports them - so that a
# changed plan reports null instead of a stale number.
GATE_UP_TRAFFIC_BYTES = {(4096, 12288, 3, 2048, True, 2): 201743448}
SEED = 0x4E45525641
WEIGHT_STD = 0.02


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def step_bytes(cfg, ctx_tokens):
    """Algorithmic bytes one decode step must move: every weight once + the KV read + KV write."""
    H, A = cfg["hidden"], cfg["heads"] * cfg["head_dim"]
    KV, I, V, L, HD = cfg["kv_heads"] * cfg["head_dim"], cfg["intermediate"], cfg["vocab"], cfg["layers"], cfg["head_dim"]
    per_layer = ((A + 2 * KV) * H + H * A + 3 * I * H) * 2
    norms = (L * (2 * H + 2 * HD) + H) * 2
    weights = L * per_layer + V * H * 2 + norms + H * 2
    kv_read = L * 2 * KV * 2 * ctx_tokens
    kv_write = L * 2 * KV * 2
    return weights + kv_read + kv_write, weights


def cpu_baseline(session, cfg, position, token, layers_sampled, threads_all):
    """Time the oracle on `layers_sampled` layers + LM head of one decode step at `position`,
    on 1 core and on all cores, with the device's own weights (regenerated bit-identically on
    the host) and the KV cache downloaded from the device prefill. Then, checker only, the device
    runs that token with its step traced and every kernel of the sampled layers and of the head is
    compared with the oracle operator on the device's own input (oracle/links.py)."""
    import oracle as O
    from oracle.links import check_step_links
    dt = cfg["dtype"]
    t0 = time.time()
    model = O.synthetic_model(cfg, SEED, WEIGHT_STD, layers=layers_sampled, embedding_rows=[token], threads=threads_all)
    kv = [session.kv_range(l, 0, position) for l in range(layers_sampled)]
    log("[cpu] host weights + KV ready in %.1f s" % (time.time() - t0))
    result = {}
    for threads in (1, threads_all):
        os.environ["OMP_NUM_THREADS"] = str(threads)
        ctx = O.Context(model, position + 2, staging=1, threads=threads)
        for l, (k, v) in enumerate(kv):
            ctx.load_kv16(l, k, v)
        ctx.set_len(position)
        t0 = time.time()
        hidden = ctx.forward_token(token, prompt_token=False, want_logits=False)
        t_layers = time.time() - t0
        t0 = time.time()
        normed = O.decode16(dt, O.encode16(dt, O.rms_norm(dt, hidden, model.final_norm, cfg["rms_eps"])))
        O.gemv(dt, model.lm_head, normed, threads=threads)
        t_head = time.time() - t0
        per_token = t_layers * cfg["layers"] / layers_sampled + t_head
        result[threads] = dict(tok_s=1.0 / per_token, layers_s=t_layers, head_s=t_head)
        log("[cpu] %d thread(s): %d layers %.2f s, lm_head %.2f s -> %.4f tok/s (extrapolated)"
            % (threads, layers_sampled, t_layers, t_head, 1.0 / per_token))
        ctx.close()
    # Full-size parity, checker only: the traced step at the workload's real sizes and context. Layers
    # 0..layers_sampled-1 (norms, 6144x4096 qkv, attention over the whole context, o, gate/up, down) and
    # the head (final norm, 151936x4096 logits, greedy token) link by link on the device's own inputs.
    rc, _, out, trace = session.traced_advance()
    assert rc == 0 and trace is not None
    k_rows, v_rows = [], []
    for l, (k, v) in enumerate(kv):
        rk, rv = session.kv_row(l, position)
        k_rows.append(np.vstack([k, rk[None]]))
        v_rows.append(np.vstack([v, rv[None]]))
    try:
        links = check_step_links(model, trace, position, token, int(out[0]), k_rows, v_rows, threads=threads_all)
        result["parity_ok"] = True
    except AssertionError as e:
        links = {"failed": str(e)}
        result["parity_ok"] = False
    log("[cpu] device kernels vs oracle operators on the device's own inputs at position %d: %s"
        % (position, ", ".join("%s %.1e" % kv_ for kv_ in sorted(links.items()) if not isinstance(kv_[1], str)) or links))
    result["links"] = links
    return result


def cpu_operator_baselines(threads_all):
    """The four operator configurations on the CPU oracle, each timed in full: the scalar single-core loop the
    reference's CPU path is, and the same work spread over `threads_all` host threads (rows of a GEMV through
    the oracle's OpenMP loop; kv heads of the attention and experts of the MoE as independent calls from a
    thread pool). Inputs have the configurations' shapes and value ranges; nothing here is checked against the
    device (the parity tests do that) - this is the reported CPU baseline beside each GPU row.
    Returns {config key: {"cpu_1core_us", "cpu_Ncore_us", "cpu_cores"}}."""
    import oracle as O
    BF16 = 1
    rng = np.random.default_rng(SEED)
    pool = concurrent.futures.ThreadPoolExecutor(max_workers=threads_all)

    def clock(fn):
        t0 = time.perf_counter()
        fn()
        return (time.perf_counter() - t0) * 1e6

    def w16(tid, rows, cols):
        return O.synth_16(BF16, SEED, tid, rows * cols, 0.0, WEIGHT_STD).reshape(rows, cols)

    out = {}
    # 1: q_proj GEMV 4096 x 4096, bf16 in, f32 accumulate, bf16 out
    w, x = w16(11, 4096, 4096), O.decode16(BF16, O.synth_16(BF16, SEED, 12, 4096, 0.0, 1.0))
    out["configs[0]"] = dict(cpu_1core_us=clock(lambda: O.encode16(BF16, O.gemv(BF16, w, x, threads=1))),
                             cpu_Ncore_us=clock(lambda: O.encode16(BF16, O.gemv(BF16, w, x, threads=threads_all))))
    # 2: MLP block: RMSNorm -> gate/up GEMVs -> SiLU(gate) * up -> down GEMV -> + residual
    H, I = 4096, 12288
    wg, wu, wd = w16(21, I, H), w16(22, I, H), w16(23, H, I)
    gamma = O.synth_16(BF16, SEED, 24, H, 1.0, 0.02)
    h = O.synth_f32(SEED, 25, H, 0.0, 1.0)

    def mlp(threads):
        n16 = O.decode16(BF16, O.encode16(BF16, O.rms_norm(BF16, h, gamma, 1e-6)))
        g, u = O.gemv(BF16, wg, n16, threads=threads), O.gemv(BF16, wu, n16, threads=threads)
        ff = O.decode16(BF16, O.encode16(BF16, (g / (np.float32(1) + np.exp(-g, dtype=np.float32))) * u))
        return h + O.gemv(BF16, wd, ff, threads=threads)
    out["configs[1]"] = dict(cpu_1core_us=clock(lambda: mlp(1)), cpu_Ncore_us=clock(lambda: mlp(threads_all)))
    del wg, wu, wd
    # 3: paged GQA decode attention, 32 q / 8 kv heads x 128, 4096 cached keys + the appended one
    heads, kvh, hd, tokens = 32, 8, 128, 4096
    blocks = tokens // 16 + 1
    table = rng.permutation(blocks).astype(np.uint32)
    kc = O.synth_16(BF16, SEED, 31, blocks * 16 * kvh * hd, 0.0, 1.0).reshape(1, blocks, 16, kvh * hd)
    vc = O.synth_16(BF16, SEED, 32, blocks * 16 * kvh * hd, 0.0, 1.0).reshape(1, blocks, 16, kvh * hd)
    qkv = O.synth_f32(SEED, 33, (heads + 2 * kvh) * hd, 0.0, 1.0)
    qn, kn = O.synth_16(BF16, SEED, 34, hd, 1.0, 0.02), O.synth_16(BF16, SEED, 35, hd, 1.0, 0.02)

    def attention(threads):
        A, KV = heads * hd, kvh * hd
        q = O.rope(hd, heads, tokens, 1e6, O.per_head_rms_norm(BF16, qn, hd, qkv[:A], 1e-6))
        k = O.rope(hd, kvh, tokens, 1e6, O.per_head_rms_norm(BF16, kn, hd, qkv[A:A + KV], 1e-6))
        kc[0, table[tokens // 16], tokens % 16] = O.encode16(BF16, k)
        vc[0, table[tokens // 16], tokens % 16] = O.encode16(BF16, qkv[A + KV:])
        if threads == 1:
            return O.attention_paged16(BF16, heads, kvh, hd, 16, q, kc, vc, table, 0, blocks, tokens + 1)
        G = heads // kvh   # one call per kv head: its query heads over its slice of the cache

        def head_group(j):
            return O.attention_paged16(BF16, G, 1, hd, 16, q[j * G * hd:(j + 1) * G * hd],
                                       np.ascontiguousarray(kc[..., j * hd:(j + 1) * hd]),
                                       np.ascontiguousarray(vc[..., j * hd:(j + 1) * hd]), table, 0, blocks, tokens + 1)
        return np.concatenate(list(pool.map(head_group, range(kvh))))
    out["configs[2]"] = dict(cpu_1core_us=clock(lambda: attention(1)), cpu_Ncore_us=clock(lambda: attention(threads_all)))
    # 4: FP8 MoE, 8 routed + 1 shared expert, hidden 7168, expert MLP 2048, 128 x 128 f32 block scales
    H, I, E, blk = 7168, 2048, 9, 128
    sH, sI = H // blk, I // blk
    fp8 = lambda n: (rng.integers(0, 0x78, n, dtype=np.uint8) | (rng.integers(0, 2, n, dtype=np.uint8) << 7))
    wg8, wu8, wd8 = fp8(E * I * H), fp8(E * I * H), fp8(E * H * I)
    sg, su, sd = (np.full(E * sI * sH, 0.02 / 448, np.float32) for _ in range(3))
    x16 = O.synth_16(BF16, SEED, 41, H, 0.0, 1.0)
    ids, wts = np.arange(8, dtype=np.uint32), np.full(8, 0.125, np.float32)

    def moe(threads):
        if threads == 1:
            return O.moe_fp8_forward(H, I, E, blk, x16, ids, wts, wg8, sg, wu8, su, wd8, sd, shared_index=8)
        one = lambda e: O.moe_fp8_forward(H, I, E, blk, x16, np.array([e], np.uint32),
                                          np.array([0.125 if e < 8 else 1.0], np.float32), wg8, sg, wu8, su, wd8, sd)
        return np.sum(list(pool.map(one, range(E))), axis=0)
    out["configs[3]"] = dict(cpu_1core_us=clock(lambda: moe(1)), cpu_Ncore_us=clock(lambda: moe(threads_all)))
    pool.shutdown()
    for key, row in out.items():
        row["cpu_1core_us"], row["cpu_Ncore_us"], row["cpu_cores"] = round(row["cpu_1core_us"], 1), round(row["cpu_Ncore_us"], 1), threads_all
        log("[cpu] %s on the oracle: %.0f us on 1 core, %.0f us on %d threads" % (key, row["cpu_1core_us"], row["cpu_Ncore_us"], threads_all))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=8192, help="prompt tokens prefilled before decoding")
    ap.add_argument("--layers", type=int, default=36, help="(debug) fewer layers = NOT the named workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-layers", type=int, default=2)
    ap.add_argument("--no-operators", action="store_true", help="skip the operator rows (configs 1-4)")
    ap.add_argument("--batch-sessions", type=int, default=32,
                    help="sessions advanced together in the shared-weights leg (0 = skip it)")
    ap.add_argument("--batch-steps", type=int, default=24)
    ap.add_argument("--prefill-block", type=int, default=0, choices=(0, 128, 256, 512),
                    help="prompt block size (0 = the session's choice: 512 tokens at these widths)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also launch one plain copy kernel of this size (memory-counter calibration runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path is a single-device decode loop and no multi-GPU "
              "figure exists for it (--gpus %d refused)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import nerva_amd as N
    rc, smoke = N.Device.smoke()
    if rc != 0:
        log("no usable GPU (hip_error=%d): the HIP path cannot run, and there is no CPU fallback" % smoke.hip_error)
        sys.exit(1)
    if args.prefill_block in (128, 256):
        N.Device.set_tuning("prefill_block_tokens", args.prefill_block)
    cfg = dict(N.Qwen3_8B)
    cfg["layers"] = args.layers
    max_ctx = args.prompt + args.warmup + args.steps + min(args.steps, 128) + 16   # + the CPU leg's parity token
    t0 = time.time()
    max_ctx += args.batch_steps + 4
    session = N.DecodeSession.create_synthetic(cfg, max_ctx, seed=SEED, weight_std=WEIGHT_STD, qk_norm=True,
                                               weight_hash=SEED)
    log("[bench] %s: session created in %.1f s, arena %.2f GB (weights %.2f GB, KV %.2f GB)" % (
        smoke.gpu_name.decode(), time.time() - t0, session.create_result.device_arena_bytes / 1e9,
        session.create_result.resident_weight_bytes / 1e9, session.create_result.resident_kv_bytes / 1e9))
    prompt = np.random.default_rng(SEED).integers(0, cfg["vocab"], args.prompt).astype(np.uint32)
    t0 = time.time()
    rc, res = session.start(prompt)
    assert rc == 0, "start failed: hip_error=%d" % res.hip_error
    rc, res, first = session.advance(1)      # token 0 was sampled by the prefill; this only syncs
    assert rc == 0
    prefill_s = time.time() - t0
    log("[bench] prefill of %d tokens: %.2f s (%.0f prompt tok/s)" % (args.prompt, prefill_s, args.prompt / prefill_s))
    if args.warmup:
        rc, res, _ = session.advance(args.warmup)
        assert rc == 0
    if args.copy_probe_mib:
        src, dst = (N.DeviceBuffer.zeros(args.copy_probe_mib << 20) for _ in range(2))
        N.Device.copy(dst, src, args.copy_probe_mib << 20)
        N.Device.synchronize()
    allocs = N.Device.allocation_count()
    t0 = time.perf_counter()
    rc, res, tokens = session.advance(args.steps)
    elapsed = time.perf_counter() - t0
    eager = N.Device.steps_are_eager()   # kernel-tracing mode (asked for, or a profiler is attached)
    assert rc == 0 and res.observed_tokens == args.steps and (eager or res.graph_replays == args.steps)
    assert res.hot_path_allocations == 0 and N.Device.allocation_count() == allocs
    tok_s = args.steps / elapsed
    ctx_mid = args.prompt + 1 + args.warmup + args.steps // 2
    bytes_step, bytes_weights = step_bytes(cfg, ctx_mid)
    log("[bench] %d steps in %.3f s -> %.1f tok/s, %.3f ms/step, device %.3f ms/step, graph nodes %d" % (
        args.steps, elapsed, tok_s, 1e3 * elapsed / args.steps, res.device_elapsed_ns / 1e6 / args.steps, res.graph_nodes))

    # Per-kernel durations, timed live with hipEvents on the session stream. "stream" figures
    # bracket all 36 launches of one kind (one per layer, distinct weights) with ONE event pair and
    # divide by the count: the kernel's own duration, which is what a kernel trace reports. The
    # per-launch event pairs of the eager pass add the event/dispatch gap of every launch.
    rc, prof = session.profile_step(3)
    assert rc == 0
    per_kind = {}
    kinds = ("qkv", "attention", "o", "gate_up", "down", "lm_head")
    for k in kinds:
        paired = getattr(prof, k + "_ns")
        ns = getattr(prof, k + "_stream_ns", 0) or paired
        per_kind[k] = (ns, getattr(prof, k + "_bytes"))
        log("[profile] %-9s %8.2f us (event pair per launch %8.2f us)  %7.1f GB/s  (%.1f%% of HBM peak)" % (
            k, ns / 1e3, paired / 1e3, per_kind[k][1] / max(ns, 1), 100 * per_kind[k][1] / max(ns, 1) / HBM_PEAK_GBS))
    dom_ns, dom_bytes = per_kind["gate_up"]
    dom_name = "gemv_fast_kernel<bf16, rmsnorm prologue, swiglu epilogue> (gate_up 24576x4096)"
    traffic = GATE_UP_TRAFFIC_BYTES.get((cfg["hidden"], cfg["intermediate"]) + N.gemv_launch_plan(
        1, 2, cfg["intermediate"], cfg["hidden"]))
    roofline = dict(bound="hbm", kernel=dom_name,
                    achieved=round(dom_bytes / dom_ns, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(dom_bytes / dom_ns / HBM_PEAK_GBS, 4), traffic=traffic,
                    bytes_per_launch=dom_bytes, avg_launch_us=round(dom_ns / 1e3, 2),
                    whole_step_bytes=bytes_step, whole_step_frac=round(bytes_step * tok_s / 1e9 / HBM_PEAK_GBS, 4),
                    per_kernel_frac={k: round(b / max(ns, 1) / HBM_PEAK_GBS, 4) for k, (ns, b) in per_kind.items()})

    # host-observed latency of single tokens: one advance(1) call (graph launch + synchronisation +
    # slot download) per token, which is how a caller that streams tokens out drives the session
    lat = []
    for _ in range(min(args.steps, 128)):
        t1 = time.perf_counter()
        rc, r1, last = session.advance(1)
        lat.append(time.perf_counter() - t1)
        assert rc == 0
        tokens = last
    lat_ms = np.sort(np.array(lat)) * 1e3
    rank = lambda q: float(lat_ms[min(len(lat_ms) - 1, int(np.ceil(q * len(lat_ms))) - 1)])   # nearest rank
    latency = dict(p50=round(rank(0.50), 4), p95=round(rank(0.95), 4), p99=round(rank(0.99), 4), tokens=len(lat_ms))
    log("[bench] single-token advance(1) latency ms: p50 %.3f  p95 %.3f  p99 %.3f" % (latency["p50"], latency["p95"], latency["p99"]))

    # Sequences on shared weights: forks of the session (each a copy of the running sequence, with a
    # cache of its own) advance together, one token each per call, through one stream of the weights.
    # Reported beside the headline figure, never as it: the metric is batch 1.
    batch = None
    if args.batch_sessions > 1:
        t1 = time.time()
        group = [session] + [session.fork_shared_weights() for _ in range(args.batch_sessions - 1)]
        fork_s = time.time() - t1
        for _ in range(3):
            rc, bres, btok = N.DecodeSession.batch_advance_one(group, args.batch_sessions, 2)
            assert rc == 0 and bres.block_tokens == len(group), (rc, bres.reason, bres.block_tokens)
        t1 = time.perf_counter()
        device_ns = 0
        for _ in range(args.batch_steps):
            rc, bres, btok = N.DecodeSession.batch_advance_one(group, args.batch_sessions, 2)
            assert rc == 0 and bres.block_tokens == len(group) and bres.hot_path_allocations == 0
            device_ns += bres.projection_elapsed_ns
        b_elapsed = time.perf_counter() - t1
        position = args.prompt + args.warmup + args.steps + len(lat) + 3 + args.batch_steps
        batch = dict(sessions=len(group), context=position, steps=args.batch_steps,
                     ms_per_step=round(1e3 * b_elapsed / args.batch_steps, 4),
                     device_ms_per_step=round(device_ns / 1e6 / args.batch_steps, 4),
                     tok_s=round(len(group) * args.batch_steps / b_elapsed, 1),
                     shared_weight_stream=int(session.shares_weight_stream()), fork_s=round(fork_s, 2))
        log("[bench] %d sessions on shared weights at context %d: %.3f ms per batch step (device %.3f) -> %.0f tok/s "
            "aggregate (%.1fx the single sequence)" % (len(group), position, batch["ms_per_step"],
                                                       batch["device_ms_per_step"], batch["tok_s"], batch["tok_s"] / tok_s))
        for child in group[1:]:
            child.destroy()
        rc, r1, tokens = session.advance(1)   # the parent goes on alone
        assert rc == 0

    cpu = None
    if not args.no_cpu:
        try:
            threads_all = min(os.cpu_count() or 1, 16)
            position = args.prompt + args.warmup + args.steps + len(lat)   # tokens now in the KV cache
            if batch is not None:
                position += 3 + args.batch_steps + 1
            layers_sampled = min(args.cpu_layers, cfg["layers"])
            r = cpu_baseline(session, cfg, position, int(tokens[-1]), layers_sampled, threads_all)
            cpu = dict(value=round(r[1]["tok_s"], 5), unit="tok/s", cores=1, kind="port",
                       sample="1 decode token at ctx %d: %d of %d layers + lm_head timed on the oracle, extrapolated to %d layers"
                              % (position, layers_sampled, cfg["layers"], cfg["layers"]),
                       all_cores_value=round(r[threads_all]["tok_s"], 5), all_cores=threads_all,
                       parity="traced step at ctx %d: every kernel of layers 0..%d and the head against the oracle operator on "
                              "the device's own input, 1e-3 on the value before any 16-bit rounding" % (position, layers_sampled - 1),
                       parity_links={k: (v if isinstance(v, str) else float("%.3g" % v)) for k, v in r["links"].items()},
                       parity_ok=r["parity_ok"])
        except Exception as e:  # the CPU leg never hides the GPU result
            log("[cpu] baseline failed: %r" % (e,))

    # The same group size at short context (the parent restarted on a 128-token prompt): there the step is the
    # weights' stream, not the sequences' K/V. Last use of the session: its long sequence is gone after this.
    batch_short = None
    if batch is not None and args.prompt > 1024:
        try:
            rc, _ = session.start(prompt[:128])
            assert rc == 0
            rc, _, _ = session.advance(2)
            assert rc == 0
            group = [session] + [session.fork_shared_weights() for _ in range(args.batch_sessions - 1)]
            for _ in range(3):
                rc, bres, btok = N.DecodeSession.batch_advance_one(group, args.batch_sessions, 2)
                assert rc == 0 and bres.block_tokens == len(group), (rc, bres.reason, bres.block_tokens)
            t1 = time.perf_counter()
            device_ns = 0
            for _ in range(args.batch_steps):
                rc, bres, btok = N.DecodeSession.batch_advance_one(group, args.batch_sessions, 2)
                assert rc == 0 and bres.block_tokens == len(group) and bres.hot_path_allocations == 0
                device_ns += bres.projection_elapsed_ns
            b_elapsed = time.perf_counter() - t1
            batch_short = dict(sessions=len(group), context=128 + 2 + 3 + args.batch_steps, steps=args.batch_steps,
                               ms_per_step=round(1e3 * b_elapsed / args.batch_steps, 4),
                               device_ms_per_step=round(device_ns / 1e6 / args.batch_steps, 4),
                               tok_s=round(len(group) * args.batch_steps / b_elapsed, 1))
            log("[bench] %d sessions on shared weights at context %d: %.3f ms per batch step (device %.3f) -> %.0f tok/s aggregate"
                % (len(group), batch_short["context"], batch_short["ms_per_step"], batch_short["device_ms_per_step"], batch_short["tok_s"]))
            for child in group[1:]:
                child.destroy()
        except Exception as e:  # a side figure never hides the headline
            log("[bench] short-context batch leg failed: %r" % (e,))
    session.destroy()

    # The operator configurations (1: q_proj GEMV, 2: MLP block, 3: paged GQA attention at 4096 keys,
    # 4: FP8 MoE experts), each over a rotating working set above 1 GB: the "GEMV HBM GB/s as % of
    # peak" half of the metric. Recorded into one hipGraph per case and timed with hipEvents.
    operators = None
    if not args.no_operators:
        from nerva_amd import opbench
        opbench.OUT = sys.stderr
        operators = {}
        for key, case in (("configs[0] q_proj GEMV 4096x4096 bf16", opbench.case_qproj),
                          ("configs[1] MLP block 4096-12288-4096 (2 launches)", opbench.case_mlp),
                          ("configs[2] paged GQA decode attention 32q/8kv x128, 4097 keys", opbench.case_attention),
                          ("configs[3] FP8 MoE 8 routed + 1 shared, 7168/2048 (2 launches)", opbench.case_moe)):
            try:
                operators[key] = case()
            except Exception as e:  # an operator row never hides the headline figure
                log("[bench] operator case %s failed: %r" % (key, e))
                operators[key] = {"failed": repr(e)}
        if not args.no_cpu:
            try:   # the CPU figure of every operator row, timed in full on this host
                for prefix, row in cpu_operator_baselines(min(os.cpu_count() or 1, 16)).items():
                    for key in operators:
                        if key.startswith(prefix):
                            operators[key].update(row)
            except Exception as e:
                log("[cpu] operator baselines failed: %r" % (e,))

    line = dict(metric="decode tok/s Qwen3-8B bs1", value=round(tok_s, 2), unit="tok/s", n_gpus=1,
                steps=args.steps, warmup=args.warmup, ms_per_step=round(1e3 * elapsed / args.steps, 4),
                higher_is_better=True, scaling="weak", vs_baseline=None, dtype="bf16", data="synthetic",
                config=dict(workload="configs[4]: full Qwen3-8B-architecture decode step, %d layers, hidden 4096, "
                                     "32q/8kv x128, MLP 12288, vocab 151936, random-init bf16 N(0,0.02), batch 1, "
                                     "prompt %d prefilled, %d greedy tokens under hipGraph replay"
                                     % (cfg["layers"], args.prompt, args.steps),
                            prompt_tokens=args.prompt, prefill_s=round(prefill_s, 3), prefill_tok_s=round(args.prompt / prefill_s, 1),
                            prefill_block_tokens=int(session.create_result.prefill_chunk_tokens), context_at_mid=ctx_mid, graph_nodes_per_token=int(res.graph_nodes),
                            hot_path_allocations=int(res.hot_path_allocations), hbm_frac_whole_step=roofline["whole_step_frac"],
                            per_token_latency_ms=latency, shared_weight_sessions=batch,
                            shared_weight_sessions_short_context=batch_short, operators=operators,
                            gpu=smoke.gpu_name.decode()),
                roofline=roofline, cpu_baseline=cpu)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
