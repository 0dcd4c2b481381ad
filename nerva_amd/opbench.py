#!/usr/bin/env python3
"""Operator-level measurements of the decode path on one MI355X:

  1. q_proj GEMV 4096x4096 bf16
  2. MLP block (RMSNorm -> gate/up GEMV -> SwiGLU -> down GEMV -> +residual), hidden 4096, MLP 12288
  3. paged GQA decode attention, 32 q / 8 kv heads x 128, 4096 cached tokens + the new one
  4. FP8 (e4m3, 128x128 block scales) MoE: 8 routed + 1 shared expert, hidden 7168, MLP 2048
  5. the token sampler over 151936 logits (greedy, temperature over the whole vocabulary, top-k / top-p)
  6. multi-row projection (1, 8, 32 token rows through one weight stream) for the step's matrices

Each case is timed twice: "rotating" cycles through enough distinct copies of the weights / cache that
the working set exceeds 1 GB (nothing is served from cache), "resident" repeats one copy. The launches
of a case are recorded into one hipGraph and replayed; time is hipEvents around the replays. Bandwidth
is algorithmic bytes (weights + vectors in and out, intermediates excluded) over time, against the
8 TB/s HBM peak. Run: python -m nerva_amd.opbench
"""
import ctypes as C
import os
import sys
import time

import numpy as np

from . import abi, runtime as R
from .runtime import DeviceBuffer, Device

BF16 = 1
SEED = 0x4E45525641
PEAK = 8000.0


OUT = sys.stdout   # a caller that keeps stdout for its own result (bench.py) points this at stderr


def log(*a):
    print(*a, flush=True, file=OUT)


def synth16(count, tid, mean=0.0, std=0.02):
    buf = DeviceBuffer(count * 2)
    assert abi.load().nerva_hip_synth_fill_16(buf.ptr, BF16, SEED, tid, count, mean, std) == 0
    return buf


def synth32(count, tid, std=1.0):
    buf = DeviceBuffer(count * 4)
    assert abi.load().nerva_hip_synth_fill_f32(buf.ptr, SEED, tid, count, 0.0, std) == 0
    return buf


class Timing(float):
    """Average ns per launch group; `shortest` and `median` are the shortest and the median replay of the
    recorded graph, per group (None where single launches were timed by the host clock)."""
    shortest = None
    median = None


def timed(enqueue, launches, warmup=3, replays=10):
    """enqueue(i) issues the i-th launch group; returns the average ns per group as a Timing."""
    lib = abi.load()
    enqueue(0)                       # untimed: primes lazily built tables
    Device.synchronize()
    if os.environ.get("NERVA_OPBENCH_EAGER") == "1" or Device.steps_are_eager():
        # kernel-tracing mode (asked for, or a profiler is attached): plain launches, the profiler
        # reports the per-kernel durations
        t0 = time.perf_counter()
        for i in range(launches):
            enqueue(i)
        Device.synchronize()
        return Timing((time.perf_counter() - t0) * 1e9 / launches)
    assert lib.nerva_hip_timer_capture_begin() == 0
    for i in range(launches):
        enqueue(i)
    nodes, ns, lo, mid = C.c_uint64(0), C.c_double(0.0), C.c_double(0.0), C.c_double(0.0)
    assert lib.nerva_hip_timer_capture_end_stats(warmup, replays, C.byref(nodes), C.byref(ns), C.byref(lo), C.byref(mid)) == 0
    out = Timing(ns.value / launches)
    out.shortest, out.median = lo.value / launches, mid.value / launches
    return out


def report(name, variant, ns, nbytes):
    """Prints one row and returns it: {"us" (average), "us_min", "us_median" over the replays, "GB/s" and "frac"
    of the 8 TB/s peak (both from the average), "bytes"}."""
    gbs = nbytes / ns
    spread = ""
    row = {"us": round(ns / 1e3, 2), "GB/s": round(gbs, 1), "frac": round(gbs / PEAK, 4), "bytes": int(nbytes)}
    if getattr(ns, "shortest", None) is not None:
        row["us_min"], row["us_median"] = round(ns.shortest / 1e3, 2), round(ns.median / 1e3, 2)
        spread = "  min %.2f  median %.2f" % (row["us_min"], row["us_median"])
    log("%-34s %-9s %9.2f us%s  %8.1f GB/s  %5.1f%% of HBM peak   (ideal %.2f us)" % (
        name, variant, ns / 1e3, spread, gbs, 100 * gbs / PEAK, nbytes / PEAK / 1e3))
    return row


def case_qproj():
    rows = cols = 4096
    copies = 40
    w = synth16(copies * rows * cols, 11)
    x = synth16(cols, 12, std=1.0)
    y = DeviceBuffer(rows * 2)
    nbytes = rows * cols * 2 + cols * 2 + rows * 2
    rows_out = {}
    for variant, n in (("rotating", copies), ("resident", 1)):
        ns = timed(lambda i: R.gemv(BF16, w.at((i % n) * rows * cols * 2), rows, cols, input16=x, out16=y,
                                    epilogue=3, sync=False), 80)
        rows_out[variant] = report("1 q_proj GEMV 4096x4096", variant, ns, nbytes)
    return rows_out


def case_mlp():
    """Rows "rotating" / "resident": the matrices as the configuration states them, [gate; up] one row-major
    [2 x 12288][4096] matrix. Row "rotating, session layout": the up rows 4 KiB behind the end of the gate rows,
    which is how a session lays a layer's pair out (the gate/up launch is then indifferent to where in memory the
    matrix starts: a wave streams gate row i and up row i side by side, and without the gap the two lie exactly
    96 MiB apart)."""
    H, I = 4096, 12288
    copies = 4
    stride = 3 * I * H + (4 << 20)   # elements between copies: the matrices and 8 MiB, so every copy starts alike
    w = synth16(copies * stride, 21)
    gamma = synth16(H, 22, mean=1.0)
    h = synth32(H, 23)
    ff = DeviceBuffer(I * 2)
    out = DeviceBuffer(H * 4)
    nbytes = 3 * I * H * 2 + H * 2 + H * 2 + H * 2     # weights + gamma + h + out counted as 16-bit vectors

    def enqueue(i, n, gap):
        base = (i % n) * stride * 2
        R.gemv(BF16, w.at(base), I, H, input_f32=h, gamma=gamma, eps=1e-6, out16=ff, epilogue=2, pair_gap=gap, sync=False)
        R.gemv(BF16, w.at(base + (2 * I * H + gap) * 2), H, I, input16=ff, residual=h, out_f32=out, epilogue=1, sync=False)
    rows_out = {}
    for variant, n, gap in (("rotating", copies, 0), ("resident", 1, 0), ("rotating, session layout", copies, 2048)):
        ns = timed(lambda i: enqueue(i, n, gap), 24)
        rows_out[variant] = report("2 MLP block 4096 -> 12288 -> 4096", variant, ns, nbytes)
    return rows_out


def case_attention(tokens=4096, label="3 paged GQA attention, 4097 keys"):
    heads, kvh, hd = 32, 8, 128
    layers, blocks = 64, tokens // 16 + 1
    rng = np.random.default_rng(3)
    table = rng.permutation(blocks).astype(np.uint32)
    cache = R.PagedKvCache(layers, blocks, kvh, hd, table)
    lib = abi.load()
    assert lib.nerva_hip_synth_fill_16(cache.k.ptr, BF16, SEED, 31, cache.elems, 0.0, 1.0) == 0
    assert lib.nerva_hip_synth_fill_16(cache.v.ptr, BF16, SEED, 32, cache.elems, 0.0, 1.0) == 0
    qkv = synth32((heads + 2 * kvh) * hd, 33)
    qn, kn = synth16(hd, 34, mean=1.0), synth16(hd, 35, mean=1.0)
    ws = R.attention_workspace(heads, hd)
    out16, out32 = DeviceBuffer(heads * hd * 2), DeviceBuffer(heads * hd * 4)
    kv_read = 2 * (tokens + 1) * kvh * hd * 2
    nbytes = kv_read + (heads + 2 * kvh) * hd * 4 + (blocks * 4) + 2 * kvh * hd * 2 + heads * hd * 4
    rows_out = {}
    for variant, n in (("rotating", layers), ("resident", 1)):
        ns = timed(lambda i: R.paged_attention(BF16, heads, kvh, hd, cache, i % n, tokens, qkv, ws, out16,
                                               out_f32=out32, append=True, rope_theta=1e6, q_norm=qn, k_norm=kn,
                                               sync=False), 128)
        rows_out[variant] = report(label, variant, ns, nbytes)
    return rows_out


def case_attention_8k():
    """The decode step's attention at the bench's context (8192 cached tokens + the new one)."""
    return case_attention(8192, "paged GQA attention, 8193 keys")


def case_copy_probe(mib=256):
    """One plain device copy of known size: the launch a counter run reads its byte scale from."""
    src, dst = (DeviceBuffer.zeros(mib << 20) for _ in range(2))
    Device.copy(dst, src, mib << 20)
    Device.synchronize()
    log("copy probe: %d MiB read, %d MiB written by one plain_copy_kernel launch" % (mib, mib))


def case_moe():
    H, I, E, K, blk = 7168, 2048, 96, 8, 128      # 96 experts resident: 12 disjoint routed sets of 8
    lib = abi.load()
    sH, sI = (H + blk - 1) // blk, (I + blk - 1) // blk
    wg, wu, wd = (DeviceBuffer(E * I * H) for _ in range(3))
    sg, su = DeviceBuffer(E * sI * sH * 4), DeviceBuffer(E * sI * sH * 4)
    sd = DeviceBuffer(E * sH * sI * 4)
    for e in range(E):
        assert lib.nerva_hip_synth_fill_fp8_block(wg.ptr + e * I * H, sg.ptr + e * sI * sH * 4, SEED, 1000 + e, I, H, blk, 0.02) == 0
        assert lib.nerva_hip_synth_fill_fp8_block(wu.ptr + e * I * H, su.ptr + e * sI * sH * 4, SEED, 2000 + e, I, H, blk, 0.02) == 0
        assert lib.nerva_hip_synth_fill_fp8_block(wd.ptr + e * I * H, sd.ptr + e * sH * sI * 4, SEED, 3000 + e, H, I, blk, 0.02) == 0
    x = synth16(H, 41, std=1.0)
    sets = (E - 1) // K                            # expert E-1 is the shared expert
    ids = [DeviceBuffer.from_numpy(np.arange(s * K, (s + 1) * K, dtype=np.uint32)) for s in range(sets)]
    wts = DeviceBuffer.from_numpy(np.full(K, 1.0 / K, np.float32))
    act = DeviceBuffer((K + 1) * I * 4)
    out = DeviceBuffer(H * 4)
    nbytes = 9 * (3 * I * H + 3 * sI * sH * 4) + H * 2 + H * 2
    rows_out = {}
    for variant, n in (("rotating", sets), ("resident", 1)):
        ns = timed(lambda i: R.moe_fp8_experts(H, I, E, K, blk, x, ids[i % n], wts, wg, sg, wu, su, wd, sd, act, out,
                                               shared_index=E - 1, sync=False), 33)
        rows_out[variant] = report("4 FP8 MoE, 8 routed + 1 shared", variant, ns, nbytes)
    # the two launches on their own (rotating): gate/up + SwiGLU (two thirds of the weights), down + combine
    for phase, label, part in ((1, "gate_up", 9 * (2 * I * H + 2 * sI * sH * 4) + H * 2), (2, "down", 9 * (I * H + sI * sH * 4) + H * 4)):
        ns = timed(lambda i: R.moe_fp8_experts(H, I, E, K, blk, x, ids[i % sets], wts, wg, sg, wu, su, wd, sd, act, out,
                                               shared_index=E - 1, sync=False, phases=phase), 33)
        rows_out[label] = report("4 FP8 MoE, %s launch" % label, "rotating", ns, part)
    return rows_out


def case_fp8_gemv():
    """One FP8 block-scaled GEMV at DeepSeek-V3's dense shapes (o projection 7168x16384, dense-layer gate
    18432x7168, and the two low-rank expansions whose K is no multiple of 1024: q_b 24576x1536, kv_b 32768x512):
    e4m3fn weights, 128x128 f32 scales, bf16 activations, f32 output."""
    lib = abi.load()
    blk = 128
    for name, rows, cols, copies in (("o 7168x16384", 7168, 16384, 10), ("gate 18432x7168", 18432, 7168, 9),
                                     ("q_b 24576x1536", 24576, 1536, 30), ("kv_b 32768x512", 32768, 512, 64)):
        sr, sc = (rows + blk - 1) // blk, (cols + blk - 1) // blk
        w = DeviceBuffer(copies * rows * cols)
        s = DeviceBuffer(copies * sr * sc * 4)
        for i in range(copies):
            assert lib.nerva_hip_synth_fill_fp8_block(w.ptr + i * rows * cols, s.ptr + i * sr * sc * 4, SEED, 4000 + i,
                                                      rows, cols, blk, 0.02) == 0
        x = synth16(cols, 43, std=1.0)
        y = DeviceBuffer(rows * 4)
        nbytes = rows * cols + sr * sc * 4 + cols * 2 + rows * 4
        for variant, n in (("rotating", copies), ("resident", 1)):
            ns = timed(lambda i: R.fp8_gemv(w.ptr + (i % n) * rows * cols, s.ptr + (i % n) * sr * sc * 4, rows, cols,
                                            blk, blk, y, input16=x, sync=False), 3 * copies)
            report("7 FP8 GEMV " + name, variant, ns, nbytes)


def case_gemm_rows():
    """Token blocks through the step's weight matrices on the matrix cores: the weights are streamed once
    per block, so 32 tokens should cost about what one token costs."""
    shapes = (("qkv 6144x4096", 6144, 4096, 0), ("o 4096x4096", 4096, 4096, 0),
              ("gate_up 2x12288x4096 +SwiGLU", 12288, 4096, 2), ("down 4096x12288", 4096, 12288, 0),
              ("lm_head 151936x4096", 151936, 4096, 0))
    for name, rows, cols, epi in shapes:
        wrows = rows * (2 if epi == 2 else 1)
        copies = max(2, (1 << 30) // (wrows * cols * 2) + 1)
        w = synth16(copies * wrows * cols, 61)
        ws = DeviceBuffer(R.gemm_rows_workspace_bytes(wrows))   # K slices of the large-block kernel
        for tokens in (1, 8, 32, 64, 128) + ((256, 512) if rows <= 12288 else ()):
            x = synth16(max(tokens, 128) * cols, 62, std=1.0)
            y32 = DeviceBuffer(tokens * rows * 4)
            y16 = DeviceBuffer(max(tokens, 128) * rows * 2)
            nbytes = wrows * cols * 2 + tokens * cols * 2 + tokens * rows * (2 if epi == 2 else 4)
            # "operand order": the activations in the layout token blocks keep inside the session
            # (blocks of more than 128 tokens exist in operand order only)
            for packed in ((False,) if tokens < 32 else (True,) if tokens > 128 else (False, True)):
                ns = timed(lambda i: R.gemm_rows(BF16, w.at((i % copies) * wrows * cols * 2), rows, cols, tokens, x, epilogue=epi,
                                                 out_f32=y32, out16=y16, sync=False, input_operand_order=packed,
                                                 output16_operand_order=packed and epi == 2, workspace=ws), 2 * copies)
                report("6 %s" % name, "T=%d%s" % (tokens, " operand order" if packed else ""), ns, nbytes)


def case_sampler():
    V = 151936
    lib = abi.load()
    logits = synth32(V, 51, std=3.0)
    ws = DeviceBuffer.zeros(lib.nerva_hip_sample_workspace_bytes(V))
    tok = DeviceBuffer.zeros(16)
    nbytes = V * 4
    for name, temperature, top_p, top_k in (("greedy", 0.0, 1.0, 0), ("T=0.7 whole vocabulary", 0.7, 1.0, 0),
                                            ("T=0.7 top_p 0.9 (k=128)", 0.7, 0.9, 0), ("T=0.7 top_k 40", 0.7, 1.0, 40)):
        req = abi.NervaHipSampleRequest()
        req.vocab, req.logits, req.token, req.workspace = V, logits.ptr, tok.ptr, ws.ptr
        req.sampler.temperature, req.sampler.top_p, req.sampler.top_k, req.sampler.seed = temperature, top_p, top_k, 1
        err = C.c_int32(0)

        def enqueue(i):
            req.position = i
            assert lib.nerva_hip_sample(C.byref(req), None, C.byref(err)) == 0
        ns = timed(enqueue, 16)
        report("5 sampler, 151936 logits", name[:9], ns, nbytes)
        log("    (%s: two launches, after the LM head has left the logits in memory)" % name)


def main():
    only = sys.argv[1:]
    rc, smoke = Device.smoke()
    if rc != 0:
        print("no usable GPU (hip_error=%d): these operators have no CPU path" % smoke.hip_error, file=sys.stderr)
        sys.exit(1)
    log("device: %s" % smoke.gpu_name.decode())
    cases = dict(qproj=case_qproj, mlp=case_mlp, attention=case_attention, attention_8k=case_attention_8k, copy_probe=case_copy_probe,
                 moe=case_moe, fp8_gemv=case_fp8_gemv,
                 sampler=case_sampler,
                 gemm_rows=case_gemm_rows)
    for name, case in cases.items():      # `python -m nerva_amd.opbench gemm_rows sampler` runs only those
        if not only or name in only:
            case()


if __name__ == "__main__":
    main()
