"""GPU parity tests of the operator entry points, through the C ABI, against the CPU oracle.

Tolerances (stated by the task): relative L2 <= 1e-3 for BF16/FP8 GEMV and attention with
FP32 accumulation; integer/byte results (codecs, generator, argmax, routing ids) bit-exact.
"""
import numpy as np
import pytest

import nerva_amd as N
import oracle as O
from nerva_amd import abi
from nerva_amd.runtime import attention_workspace

pytestmark = pytest.mark.gpu

BF16, F16 = 1, 0
SEED = 0x4E45525641
REL_L2 = 1e-3


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def dev(a):
    return N.DeviceBuffer.from_numpy(a)


def test_device_smoke():
    rc, res = N.Device.smoke()
    assert rc == 0 and res.status == 0 and res.device_count >= 1
    assert res.value == 0x4E455256
    print("GPU:", res.gpu_name.decode(), "mem", res.total_global_mem >> 30, "GiB", flush=True)


def test_synthetic_generator_matches_oracle_bit_for_bit():
    lib = abi.load()
    n = 100003
    for dtype in (BF16, F16):
        buf = N.DeviceBuffer(n * 2)
        assert lib.nerva_hip_synth_fill_16(buf.ptr, dtype, SEED, 7, n, 1.0, 0.02) == 0
        assert np.array_equal(buf.numpy(np.uint16), O.synth_16(dtype, SEED, 7, n, 1.0, 0.02))
    buf = N.DeviceBuffer(n * 4)
    assert lib.nerva_hip_synth_fill_f32(buf.ptr, SEED, 8, n, 0.0, 1.0) == 0
    assert np.array_equal(buf.numpy(np.float32).view(np.uint32), O.synth_f32(SEED, 8, n, 0.0, 1.0).view(np.uint32))
    rows, cols, block = 130, 260, 128
    w = N.DeviceBuffer(rows * cols)
    s = N.DeviceBuffer(2 * 3 * 4)
    assert lib.nerva_hip_synth_fill_fp8_block(w.ptr, s.ptr, SEED, 9, rows, cols, block, 0.02) == 0
    ow, os_ = O.synth_fp8_block(SEED, 9, rows, cols, block, 0.02)
    assert np.array_equal(s.numpy(np.float32).view(np.uint32), os_.ravel().view(np.uint32))
    assert np.array_equal(w.numpy(np.uint8), ow.ravel())


# ---------------------------------------------------------------------------
# BF16/F16 GEMV family
# ---------------------------------------------------------------------------

def _gemv_case(dtype, rows, cols, seed, std=0.02):
    rng = np.random.default_rng(seed)
    w = O.encode16(dtype, rng.normal(0, std, (rows, cols)))
    x = O.encode16(dtype, rng.normal(0, 1, cols))
    return w, x


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("rows,cols", [(4096, 4096), (6144, 4096), (1030, 12288), (37, 520), (5, 2), (3, 4104), (2, 7),
                                       (515, 14336), (260, 25600), (130, 28672), (1027, 5120), (66, 30720)])
def test_gemv_plain_matches_oracle(dtype, rows, cols):
    """Config 1 (q_proj 4096x4096 bf16, x bf16, bf16 out) plus ragged / unaligned shapes, rows of other models'
    widths (batches of 1024 columns: 5120, 25600; more than 12288 columns: the input copied into LDS by a loop)."""
    w, x = _gemv_case(dtype, rows, cols, rows * 31 + cols)
    ref = O.gemv_x16(dtype, w, x)
    dw, dx = dev(w), dev(x)
    y32 = N.DeviceBuffer(rows * 4)
    N.gemv(dtype, dw, rows, cols, input16=dx, out_f32=y32, epilogue=0)
    got = y32.numpy(np.float32)
    assert rel_l2(got, ref) <= REL_L2
    assert np.max(np.abs(got - ref)) <= 1e-3 * max(1.0, np.max(np.abs(ref)))
    y16 = N.DeviceBuffer(max(16, rows * 2))
    N.gemv(dtype, dw, rows, cols, input16=dx, out16=y16, epilogue=3)
    got16 = O.decode16(dtype, y16.numpy(np.uint16, rows))
    assert rel_l2(got16, O.decode16(dtype, O.encode16(dtype, ref))) <= 4e-3  # one 16-bit rounding of y
    # rounding the device's own f32 result reproduces its 16-bit output exactly
    assert np.array_equal(y16.numpy(np.uint16, rows), O.encode16(dtype, got))


def test_gemv_linearity_and_unit_vectors_full_size():
    """Size-independent properties at the full q_proj size: W.e_j = column j; W.(a+b) = W.a + W.b."""
    rows = cols = 4096
    w = O.synth_16(BF16, SEED, 100, rows * cols, 0.0, 0.02).reshape(rows, cols)
    dw = dev(w)
    y = N.DeviceBuffer(rows * 4)
    e = np.zeros(cols, np.float32)
    e[1234] = 1.0
    N.gemv(BF16, dw, rows, cols, input16=dev(O.encode16(BF16, e)), out_f32=y)
    assert np.array_equal(y.numpy(np.float32), O.decode16(BF16, w[:, 1234]))
    a = O.encode16(BF16, np.random.default_rng(1).integers(-8, 8, cols).astype(np.float32))
    b = O.encode16(BF16, np.random.default_rng(2).integers(-8, 8, cols).astype(np.float32))
    ab = O.encode16(BF16, O.decode16(BF16, a) + O.decode16(BF16, b))  # small integers: exact in bf16
    outs = []
    for v in (a, b, ab):
        N.gemv(BF16, dw, rows, cols, input16=dev(v), out_f32=y)
        outs.append(y.numpy(np.float32).astype(np.float64))
    assert rel_l2(outs[2], outs[0] + outs[1]) < 1e-5


@pytest.mark.parametrize("dtype", [BF16, F16])
def test_gemv_keeps_16_bit_denormals(dtype):
    """The lean GEMV multiplies 16-bit pairs with the packed dot instruction (f32 accumulation): weights that
    are denormal in their 16-bit type must count in full (no flush to zero) - every weight of this matrix is a
    denormal, the activations are large, and the result equals the oracle's exactly."""
    rows = cols = 4096
    w = np.full((rows, cols), 0x0001, np.uint16)                     # the smallest denormal of either type
    w[1::2] = 0x03FF if dtype == F16 else 0x007F                     # the largest
    x = O.encode16(dtype, np.full(cols, 1024.0 if dtype == F16 else 2.0 ** 100, np.float32))
    ref = O.gemv_x16(dtype, w, x)
    assert np.all(ref > 0)
    y = N.DeviceBuffer(rows * 4)
    N.gemv(dtype, dev(w), rows, cols, input16=dev(x), out_f32=y)
    assert np.array_equal(y.numpy(np.float32), ref)


@pytest.mark.parametrize("shape", ["o", "qkv", "down", "ragged rows"])
def test_gemv_start_up_variants_are_the_same_function(shape):
    """The lean GEMV has two start-up orders (requests under branches, or unconditional with exact waits;
    the launcher picks per shape). Forced on and forced off they must give bit-identical results - the
    arithmetic and its order are the same - at the step's shapes, with the residual epilogue and with a
    row count that leaves waves without a row."""
    rows, cols, pro, epi = {"o": (4096, 4096, 0, 1), "qkv": (6144, 4096, 1, 0), "down": (4096, 12288, 0, 1),
                            "ragged rows": (4090, 4096, 0, 1)}[shape]
    rng = np.random.default_rng(rows + cols)
    w = O.synth_16(BF16, SEED, 140, rows * cols, 0.0, 0.02).reshape(rows, cols)
    x16 = O.encode16(BF16, rng.normal(0, 1, cols).astype(np.float32))
    xf = rng.normal(0, 1, cols).astype(np.float32)
    gamma = O.encode16(BF16, rng.normal(1, 0.1, cols).astype(np.float32))
    res = rng.normal(0, 1, rows).astype(np.float32)
    dw, y = dev(w), N.DeviceBuffer(rows * 4)
    outs = {}
    try:
        for mode in (2, 1, 0):
            N.Device.set_tuning("gemv_exact_start", mode)
            N.Device.set_tuning("gemv_x_registers", 2 if mode == 1 else 0)   # (1: exact start without the register copy of x)
            if pro == 0:
                N.gemv(BF16, dw, rows, cols, input16=dev(x16), residual=dev(res), out_f32=y, epilogue=epi)
            else:
                N.gemv(BF16, dw, rows, cols, input_f32=dev(xf), gamma=dev(gamma), eps=1e-6, out_f32=y, epilogue=epi)
            outs[mode] = y.numpy(np.float32).copy()
    finally:
        N.Device.set_tuning("gemv_exact_start", 0)
        N.Device.set_tuning("gemv_x_registers", 0)
    assert np.array_equal(outs[1], outs[2]) and np.array_equal(outs[0], outs[2])
    if pro == 0:
        ref = O.gemv_x16(BF16, w, x16) + res
    else:
        ref = O.gemv_x16(BF16, w, O.encode16(BF16, O.rms_norm(BF16, xf, gamma, 1e-6)))
    assert rel_l2(outs[0], ref) <= REL_L2


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("cols,rows", [(4096, 6144), (520, 64), (6, 3), (5120, 1030), (8192, 515), (12288, 70), (13312, 33)])
def test_gemv_rmsnorm_prologue(dtype, cols, rows):
    """qkv projection: x = round16(rmsnorm(h, gamma)) fused in front of the GEMV."""
    rng = np.random.default_rng(cols)
    h = rng.normal(0, 1, cols).astype(np.float32)
    gamma = O.encode16(dtype, rng.normal(1, 0.02, cols))
    w = O.encode16(dtype, rng.normal(0, 0.02, (rows, cols)))
    n16 = O.encode16(dtype, O.rms_norm(dtype, h, gamma, 1e-6))
    ref = O.gemv_x16(dtype, w, n16)
    y = N.DeviceBuffer(rows * 4)
    N.gemv(dtype, dev(w), rows, cols, input_f32=dev(h), gamma=dev(gamma), eps=1e-6, out_f32=y)
    assert rel_l2(y.numpy(np.float32), ref) <= REL_L2


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("rows,cols,tokens", [(64, 2048, 1), (48, 2048, 5), (32, 4096, 16), (16, 2048, 17),
                                               (1000, 2048, 9), (25, 2048, 32),   # row counts off the 16-row grid
                                               (64, 2048, 33), (48, 4096, 49), (1000, 2048, 64), (64, 2048, 65), (1000, 2048, 128),   # more than two token tiles
                                               (6144, 4096, 32), (4096, 12288, 31), (6144, 4096, 64)])
def test_gemm_rows_matches_oracle_per_token(dtype, rows, cols, tokens):
    """Multi-row projection on the matrix cores: every token row equals the oracle's GEMV of that row
    (plain, and with bias + residual + 16-bit rounding as the prompt staging of the down projection uses)."""
    if dtype == F16 and rows > 1000:
        pytest.skip("full-size shapes once, in bf16")
    rng = np.random.default_rng(rows + cols + tokens)
    if rows * cols > 1 << 22:
        w = O.synth_16(dtype, SEED, 300 + tokens, rows * cols, 0.0, 0.02).reshape(rows, cols)
    else:
        w = O.encode16(dtype, rng.normal(0, 0.02, (rows, cols)))
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, cols)))
    bias = O.encode16(dtype, rng.normal(0, 0.1, rows))
    res = rng.normal(0, 1, (tokens, rows)).astype(np.float32)
    ref = np.stack([O.gemv_x16(dtype, w, x[t]) for t in range(tokens)])
    dw, dx = dev(w), dev(x)
    y = N.DeviceBuffer(tokens * rows * 4)
    N.gemm_rows(dtype, dw, rows, cols, tokens, dx, epilogue=0, out_f32=y)
    got = y.numpy(np.float32).reshape(tokens, rows)
    assert rel_l2(got, ref) <= REL_L2
    assert max(rel_l2(got[t], ref[t]) for t in range(tokens)) <= REL_L2
    N.gemm_rows(dtype, dw, rows, cols, tokens, dx, epilogue=1, bias=dev(bias), residual=dev(res), out_f32=y,
                round_output=True)
    got = y.numpy(np.float32).reshape(tokens, rows)
    want = O.decode16(dtype, O.encode16(dtype, (ref + O.decode16(dtype, bias)[None, :]) + res))
    assert rel_l2(got, want) <= 4e-3                       # one 16-bit rounding of the sum
    assert np.array_equal(O.encode16(dtype, got), O.encode16(dtype, got.astype(np.float32)))  # values are 16-bit numbers


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("inter,hidden,tokens", [(64, 2048, 3), (64, 2048, 57), (64, 2048, 111), (12288, 4096, 32), (12288, 4096, 128)])
def test_gemm_rows_swiglu_matches_oracle(dtype, inter, hidden, tokens):
    """Fused gate/up projection of a token block: out16 = round16(silu(gate) * up), gate rows first."""
    if dtype == F16 and inter > 1000:
        pytest.skip("full-size shape once, in bf16")
    rng = np.random.default_rng(inter + tokens)
    if inter > 1000:
        w = O.synth_16(dtype, SEED, 310, 2 * inter * hidden, 0.0, 0.02).reshape(2 * inter, hidden)
    else:
        w = O.encode16(dtype, rng.normal(0, 0.05, (2 * inter, hidden)))
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, hidden)))
    out = N.DeviceBuffer(tokens * inter * 2)
    N.gemm_rows(dtype, dev(w), inter, hidden, tokens, dev(x), epilogue=2, out16=out)
    got = O.decode16(dtype, out.numpy(np.uint16, tokens * inter)).reshape(tokens, inter)
    for t in range(0, tokens, max(1, tokens // 4)):
        gu = O.gemv_x16(dtype, w, x[t])
        g, u = gu[:inter].astype(np.float64), gu[inter:].astype(np.float64)
        want = O.decode16(dtype, O.encode16(dtype, (g / (1.0 + np.exp(-g)) * u).astype(np.float32)))
        assert rel_l2(got[t], want) <= 4e-3


def test_gemm_rows_rejects_unsupported_shapes():
    w, x, y = N.DeviceBuffer(1 << 16), N.DeviceBuffer(1 << 16), N.DeviceBuffer(1 << 16)
    for rows, cols, tokens in ((8, 2048, 4), (16, 1024, 4), (16, 2048, 129), (16, 2048, 0)):
        with pytest.raises(RuntimeError):
            N.gemm_rows(BF16, w, rows, cols, tokens, x, out_f32=y)
    with pytest.raises(RuntimeError):      # rows off the 16-row grid: no residual added in place
        N.gemm_rows(BF16, w, 24, 2048, 4, x, epilogue=1, residual=y, out_f32=y)
    # more than 128 token rows: operand order only, rows a multiple of 128 (gate/up pairs of 64), 256 rows at most
    for rows, cols, tokens, epi in ((64, 2048, 200, 0), (128, 2048, 257, 0), (32, 2048, 130, 2)):
        with pytest.raises(RuntimeError):
            N.gemm_rows(BF16, w, rows, cols, tokens, x, epilogue=epi, out_f32=y, out16=y, input_operand_order=True)
    with pytest.raises(RuntimeError):      # operand order comes in runs of 32 columns: no such output 48 wide
        N.gemm_rows(BF16, w, 48, 2048, 20, x, epilogue=2, out16=y, input_operand_order=True, output16_operand_order=True)


@pytest.mark.parametrize("full", [False, True])
def test_mlp_block_matches_oracle(full):
    """Config 2: RMSNorm -> fused gate+up GEMV -> SiLU(gate)*up -> down GEMV -> residual add."""
    hidden, inter = (4096, 12288) if full else (512, 1536)
    dtype = BF16
    if full:
        wgu = O.synth_16(dtype, SEED, 200, 2 * inter * hidden, 0.0, 0.02).reshape(2 * inter, hidden)
        wd = O.synth_16(dtype, SEED, 201, hidden * inter, 0.0, 0.02).reshape(hidden, inter)
    else:
        rng = np.random.default_rng(5)
        wgu = O.encode16(dtype, rng.normal(0, 0.02, (2 * inter, hidden)))
        wd = O.encode16(dtype, rng.normal(0, 0.02, (hidden, inter)))
    h = O.decode16(dtype, O.synth_16(dtype, SEED, 202, hidden, 0.0, 1.0))
    gamma = O.synth_16(dtype, SEED, 203, hidden, 1.0, 0.02)
    # oracle, device-session staging
    m16 = O.encode16(dtype, O.rms_norm(dtype, h, gamma, 1e-6))
    gu = O.gemv(dtype, wgu, O.decode16(dtype, m16), threads=8)
    g, u = gu[:inter], gu[inter:]
    ff = (g / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float32) * u
    ff16 = O.encode16(dtype, ff)
    ref = h + O.gemv(dtype, wd, O.decode16(dtype, ff16), threads=8)
    # device
    dff = N.DeviceBuffer(inter * 2)
    dout = N.DeviceBuffer(hidden * 4)
    dh = dev(h)
    N.gemv(dtype, dev(wgu), inter, hidden, input_f32=dh, gamma=dev(gamma), eps=1e-6, out16=dff, epilogue=2)
    N.gemv(dtype, dev(wd), hidden, inter, input16=dff, residual=dh, out_f32=dout, epilogue=1)
    got_ff = O.decode16(dtype, dff.numpy(np.uint16))
    assert rel_l2(got_ff, O.decode16(dtype, ff16)) <= 3e-3  # 16-bit rounding of an f32 result
    assert rel_l2(dout.numpy(np.float32), ref) <= REL_L2
    # prompt-token staging: the sum is rounded to 16 bits
    N.gemv(dtype, dev(wd), hidden, inter, input16=dff, residual=dh, out_f32=dout, epilogue=1, round_output=True)
    got = dout.numpy(np.float32)
    assert np.array_equal(got, O.decode16(dtype, O.encode16(dtype, got)))


def test_gemv_bias_and_invalid_arguments():
    rows, cols = 64, 512
    w, x = _gemv_case(BF16, rows, cols, 3)
    bias = O.encode16(BF16, np.random.default_rng(4).normal(0, 1, rows))
    y = N.DeviceBuffer(rows * 4)
    N.gemv(BF16, dev(w), rows, cols, input16=dev(x), bias=dev(bias), out_f32=y)
    assert rel_l2(y.numpy(np.float32), O.gemv_x16(BF16, w, x) + O.decode16(BF16, bias)) <= REL_L2
    lib = abi.load()
    req = abi.NervaHipGemvRequest()
    import ctypes as C
    err = C.c_int32(0)
    assert lib.nerva_hip_gemv(None, None, C.byref(err)) == -1
    assert lib.nerva_hip_gemv(C.byref(req), None, C.byref(err)) == -1 and err.value != 0  # all-null request
    req.dtype, req.rows, req.cols, req.epilogue = 7, 4, 4, 0
    assert lib.nerva_hip_gemv(C.byref(req), None, C.byref(err)) == -1


# ---------------------------------------------------------------------------
# FP8 block-scaled GEMV
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("cols", [1024, 1040, 3])
def test_fp8_decode_all_256_codes(cols):
    """Every e4m3fn code through the device decode (hardware path at cols=1024 and, with all but one lane of the
    last chunk idle, at cols=1040; bit path at cols=3)."""
    w = np.zeros((256, cols), np.uint8)
    w[:, 0] = np.arange(256)
    x = np.zeros(cols, np.float32)
    x[0] = 1.0
    y = N.DeviceBuffer(256 * 4)
    scales = np.ones((2, -(-cols // 128)), np.float32)
    N.fp8_gemv(dev(w), dev(scales), 256, cols, 128, 128, y, input16=dev(O.encode16(BF16, x)))
    got = y.numpy(np.float32)
    want = O.decode_fp8(np.arange(256, dtype=np.uint8))
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan], want[~nan])


def test_fp8_matvec_kat_host_pointer_abi(kat):
    import ctypes as C
    k = kat["fp8_f32_scale_matvec"]
    w = np.array([int(v, 16) for v in k["weights"]], np.uint8)
    s = np.array(k["scales"], np.float32)
    x16 = O.encode16(BF16, np.array(k["input"], np.float32))
    out = np.zeros(k["rows"], np.float32)
    req = abi.NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest()
    req.rows, req.cols, req.block_rows, req.block_cols, req.input_dtype = k["rows"], k["cols"], k["block_rows"], k["block_cols"], BF16
    req.weights, req.scales, req.input, req.output = w.ctypes.data, s.ctypes.data, x16.ctypes.data, out.ctypes.data
    res = abi.NervaHipDeepSeekQuantDequantResult()
    assert abi.load().nerva_hip_deepseek_quant_fp8_f32_scale_encoded_matvec(C.byref(req), C.byref(res)) == 0
    assert out.tolist() == k["expected"]
    assert (res.rows, res.cols, res.block_rows, res.block_cols) == (3, 4, 2, 2)
    assert res.kernel_launches == 1 and res.sync_calls == 1 and res.hot_path_allocations == 0
    assert res.output_hash == O.fnv1a(out) != 0


def test_fp8_gemm_tokens_ragged_kat(kat):
    import ctypes as C
    k = kat["fp8_gemm_tokens_ragged"]
    rows, cols, tokens = k["rows"], k["cols"], k["tokens"]
    pat = [int(v, 16) for v in k["weight_pattern"]]
    w = np.array([pat[i % len(pat)] for i in range(rows * cols)], np.uint8)
    x16 = O.encode16(BF16, np.array([((i % 17) - 8) / 32 for i in range(tokens * cols)], np.float32))
    s = np.array(k["scales"], np.float32)
    out = np.zeros(tokens * rows, np.float32)
    req = abi.NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest()
    req.rows, req.cols, req.tokens, req.block_rows, req.block_cols, req.input_dtype = rows, cols, tokens, 128, 128, BF16
    req.weights, req.scales, req.input, req.output = w.ctypes.data, s.ctypes.data, x16.ctypes.data, out.ctypes.data
    res = abi.NervaHipDeepSeekQuantDequantResult()
    assert abi.load().nerva_hip_deepseek_quant_fp8_f32_scale_encoded_gemm_tokens(C.byref(req), C.byref(res)) == 0
    ref = O.fp8_gemm_tokens(w, s, x16, rows, cols, tokens, 128, 128)
    assert np.max(np.abs(out.reshape(tokens, rows) - ref)) < k["abs_tol"]


@pytest.mark.parametrize("rows,cols,dtype", [(2048, 7168, BF16), (7168, 2048, BF16), (300, 1024, BF16),
                                             (130, 260, BF16), (384, 16384, BF16), (515, 3072, F16),
                                             (515, 1536, BF16), (131, 5008, F16), (64, 528, BF16), (33, 272, BF16),
                                             (66, 30720, BF16), (1027, 512, F16), (34, 20000, BF16), (1, 1024, BF16), (3, 272, F16)])
def test_fp8_gemv_matches_oracle(rows, cols, dtype):
    """16-bit and f32 activations. One token of 16-bit activations over rows of whole 16-byte pieces takes the
    row-pair kernel (a last chunk of fewer than 1024 columns has idle lanes; an odd row count doubles the last
    row), f32 activations with K of 1024-multiples the chunked kernels, other K the byte-wise one."""
    w, s = O.synth_fp8_block(SEED, rows + cols, rows, cols, 128, 0.02)
    x16 = O.synth_16(dtype, SEED, 11, cols, 0.0, 1.0)
    ref = O.fp8_gemm_tokens(w, s, x16, rows, cols, 1, 128, 128, input_dtype=dtype)[0]
    y = N.DeviceBuffer(rows * 4)
    N.fp8_gemv(dev(w), dev(s), rows, cols, 128, 128, y, input16=dev(x16), input_dtype=dtype)
    assert rel_l2(y.numpy(np.float32), ref) <= REL_L2
    if cols * 4 <= 60 * 1024:
        xf = O.decode16(dtype, x16)
        N.fp8_gemv(dev(w), dev(s), rows, cols, 128, 128, y, input_f32=dev(xf))
        assert rel_l2(y.numpy(np.float32), ref) <= REL_L2


@pytest.mark.parametrize("rows,cols,block_rows,block_cols", [(96, 2064, 64, 48), (50, 528, 7, 16), (33, 4096, 128, 4096),
                                                             (70, 1536, 3, 32), (258, 1024, 128, 64)])
def test_fp8_gemv_block_shapes_other_than_128(rows, cols, block_rows, block_cols):
    """Scale blocks of other shapes than 128 x 128 (rows per block arbitrary, columns per block a multiple of 16 so
    that a lane's 16 weights share a scale): random codes without the NaN encodings, random positive scales."""
    rng = np.random.default_rng(rows * 131 + cols)
    w = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    w[(w & 0x7f) == 0x7f] = 0x38   # 0x7f / 0xff are NaN
    w = (w & 0xbf).astype(np.uint8)  # exponent's top bit cleared: magnitudes up to 1.875, sums stay tame
    sr, sc = -(-rows // block_rows), -(-cols // block_cols)
    s = rng.uniform(0.5, 2.0, (sr, sc)).astype(np.float32)
    x16 = O.synth_16(BF16, SEED, 12, cols, 0.0, 1.0)
    ref = O.fp8_gemm_tokens(w, s, x16, rows, cols, 1, block_rows, block_cols, input_dtype=BF16)[0]
    y = N.DeviceBuffer(rows * 4)
    N.fp8_gemv(dev(w), dev(s), rows, cols, block_rows, block_cols, y, input16=dev(x16), input_dtype=BF16)
    assert rel_l2(y.numpy(np.float32), ref) <= REL_L2


# ---------------------------------------------------------------------------
# Paged GQA decode attention
# ---------------------------------------------------------------------------

def _attention_case(dtype, heads, kv_heads, hd, tokens, theta, qk_norm, seed, layers=2, layer=1, bias=False):
    rng = np.random.default_rng(seed)
    kvh = kv_heads * hd
    n_blocks = tokens // 16 + 2
    table = rng.permutation(n_blocks).astype(np.uint32)
    k_rows = O.encode16(dtype, rng.normal(0, 1, (tokens, kvh)))
    v_rows = O.encode16(dtype, rng.normal(0, 1, (tokens, kvh)))
    qkv = rng.normal(0, 1, heads * hd + 2 * kvh).astype(np.float32)
    qn = O.encode16(dtype, rng.normal(1, 0.02, hd)) if qk_norm else None
    kn = O.encode16(dtype, rng.normal(1, 0.02, hd)) if qk_norm else None
    biases = [O.encode16(dtype, rng.normal(0, 0.1, n)) for n in (heads * hd, kvh, kvh)] if bias else [None] * 3
    return dict(dtype=dtype, heads=heads, kv_heads=kv_heads, hd=hd, tokens=tokens, theta=theta, table=table,
                n_blocks=n_blocks, k_rows=k_rows, v_rows=v_rows, qkv=qkv, qn=qn, kn=kn, biases=biases,
                layers=layers, layer=layer)


def _attention_oracle(c, eps=1e-6):
    """Reference staging: bias -> per-head norm -> RoPE -> K/V rounded -> attention over pos+1 keys."""
    dtype, heads, kv_heads, hd = c["dtype"], c["heads"], c["kv_heads"], c["hd"]
    A, KV = heads * hd, kv_heads * hd
    pos = c["tokens"]
    q, k, v = c["qkv"][:A].copy(), c["qkv"][A:A + KV].copy(), c["qkv"][A + KV:].copy()
    for vec, b in zip((q, k, v), c["biases"]):
        if b is not None:
            vec += O.decode16(dtype, b)
    if c["qn"] is not None:
        q = O.per_head_rms_norm(dtype, c["qn"], hd, q, eps)
        k = O.per_head_rms_norm(dtype, c["kn"], hd, k, eps)
    if c["theta"]:
        q = O.rope(hd, heads, pos, c["theta"], q)
        k = O.rope(hd, kv_heads, pos, c["theta"], k)
    k16, v16 = O.encode16(dtype, k), O.encode16(dtype, v)
    # oracle cache layout [layer][block][16][kv_hidden]
    kc = np.zeros((c["layers"], c["n_blocks"], 16, KV), np.uint16)
    vc = np.zeros_like(kc)
    rows_k = np.vstack([c["k_rows"], k16[None]])
    rows_v = np.vstack([c["v_rows"], v16[None]])
    for t in range(pos + 1):
        kc[c["layer"], c["table"][t // 16], t % 16] = rows_k[t]
        vc[c["layer"], c["table"][t // 16], t % 16] = rows_v[t]
    out = O.attention_paged16(dtype, heads, kv_heads, hd, 16, q, kc, vc, c["table"], c["layer"],
                              c["n_blocks"], pos + 1)
    return out, k16, v16


def _attention_device(c, eps=1e-6):
    cache = N.PagedKvCache(c["layers"], c["n_blocks"], c["kv_heads"], c["hd"], c["table"])
    cache.fill(c["layer"], c["k_rows"], c["v_rows"])
    ws = attention_workspace(c["heads"], c["hd"])
    A = c["heads"] * c["hd"]
    out16 = N.DeviceBuffer(max(16, A * 2))
    out32 = N.DeviceBuffer(A * 4)
    opt = lambda a: dev(a) if a is not None else None
    qb, kb, vb = (opt(b) for b in c["biases"])
    N.paged_attention(c["dtype"], c["heads"], c["kv_heads"], c["hd"], cache, c["layer"], c["tokens"],
                      dev(c["qkv"]), ws, out16, out_f32=out32, append=True, eps=eps,
                      rope_theta=c["theta"] or 0.0, q_norm=opt(c["qn"]), k_norm=opt(c["kn"]),
                      q_bias=qb, k_bias=kb, v_bias=vb)
    k_new, v_new = cache.read_row(c["layer"], c["tokens"])
    return out32.numpy(np.float32), out16.numpy(np.uint16, A), k_new, v_new, cache, ws


@pytest.mark.parametrize("tokens", [0, 1, 15, 16, 17, 100, 1000, 4096])
def test_paged_attention_config3_shapes(tokens):
    """Config 3: 32 q / 8 kv heads x 128, bf16 16-token blocks, permuted table, QK-norm, RoPE 1e6."""
    c = _attention_case(BF16, 32, 8, 128, tokens, 1e6, True, 1000 + tokens)
    ref, k16, v16 = _attention_oracle(c)
    got32, got16, k_new, v_new, _, _ = _attention_device(c)
    # the appended K row passes through powf/sincos: allow 1 unit in the last place of the 16-bit value
    assert np.max(np.abs(k_new.astype(np.int32) - k16.astype(np.int32))) <= 1
    assert np.mean(k_new != k16) < 0.02
    assert np.array_equal(v_new, v16)
    assert rel_l2(got32, ref) <= REL_L2
    assert np.array_equal(got16, O.encode16(BF16, got32))


@pytest.mark.parametrize("heads,kv_heads,hd,dtype,theta,qk_norm,bias", [
    (8, 8, 128, BF16, 1e4, False, False),     # MHA, no norm
    (16, 8, 128, F16, 1e6, True, True),       # group 2, f16, biases
    (64, 8, 128, BF16, 0, True, False),       # group 8, no RoPE
    (4, 2, 64, BF16, 1e4, True, True),        # generic path: head_dim 64
    (6, 2, 32, F16, 1e4, False, False),       # generic path: group 3
    (1, 1, 2, F16, 0, False, False),          # tiny known-answer geometry
])
def test_paged_attention_other_geometries(heads, kv_heads, hd, dtype, theta, qk_norm, bias):
    for tokens in (0, 5, 70):
        c = _attention_case(dtype, heads, kv_heads, hd, tokens, theta, qk_norm, heads * 7 + tokens, bias=bias)
        ref, k16, v16 = _attention_oracle(c)
        got32, got16, k_new, v_new, _, _ = _attention_device(c)
        assert np.max(np.abs(k_new.astype(np.int32) - k16.astype(np.int32))) <= 1
        assert np.array_equal(v_new, v16)
        assert rel_l2(got32, ref) <= REL_L2


@pytest.mark.parametrize("heads,kv_heads", [(64, 8), (32, 4), (16, 16)])
def test_paged_attention_step_kernel_group_sizes_at_long_context(heads, kv_heads):
    """GQA factors 8 and 1 and a 4-kv-head layout (64 splits) through the decode-step kernel at contexts where the
    splits merge (and, with few forced splits, where a wave re-requests tiles), up to the largest split factor that
    stays resident for the kv head count: oracle parity, same bits on a second launch."""
    most = int(N.abi.load().nerva_hip_paged_attention_max_splits(kv_heads))
    for tokens, splits in ((333, 0), (1000, 0), (4096, 0), (4096, 3), (2500, most)):
        c = _attention_case(BF16, heads, kv_heads, 128, tokens, 1e6, True, heads + tokens)
        ref, _, _ = _attention_oracle(c)
        cache = N.PagedKvCache(c["layers"], c["n_blocks"], kv_heads, 128, c["table"])
        cache.fill(c["layer"], c["k_rows"], c["v_rows"])
        ws = attention_workspace(heads, 128)
        out16, out32 = N.DeviceBuffer(heads * 128 * 2), N.DeviceBuffer(heads * 128 * 4)
        outs = []
        for _ in range(2):
            N.paged_attention(BF16, heads, kv_heads, 128, cache, c["layer"], tokens, dev(c["qkv"]), ws, out16,
                              out_f32=out32, append=True, rope_theta=1e6, q_norm=dev(c["qn"]), k_norm=dev(c["kn"]),
                              splits=splits)
            outs.append(out32.numpy(np.float32).copy())
        assert rel_l2(outs[0], ref) <= REL_L2, (tokens, splits)
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), (tokens, splits)


def test_paged_attention_permutation_invariance_and_repeatability():
    """Same logical KV under two block tables gives the same bits; so does calling twice."""
    base = _attention_case(BF16, 32, 8, 128, 777, 1e6, True, 42)
    outs = []
    for seed in (1, 2):
        c = dict(base)
        c["table"] = np.random.default_rng(seed).permutation(base["n_blocks"]).astype(np.uint32)
        got32, _, _, _, _, _ = _attention_device(c)
        outs.append(got32)
        got_again, _, _, _, _, _ = _attention_device(c)
        assert np.array_equal(got32, got_again)
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("tokens", [17, 255, 4096, 8191])
def test_paged_attention_split_merge_is_stable_over_many_launches(tokens):
    """The cross-split merge (every split stores its partial as tagged words; the merge jobs of a kv head are
    spread over its first splits' workgroups, which poll the words and fold them in split order) must not depend
    on arrival order or timing: for split factors 2, 8 and 32 (the most that stay resident together with 8 kv
    heads), 200 launches in a row give the bits of the first launch, and those are within tolerance of the
    oracle. Stops at the first mismatch."""
    c = _attention_case(BF16, 32, 8, 128, tokens, 1e6, True, 5000 + tokens)
    ref, _, _ = _attention_oracle(c)
    cache = N.PagedKvCache(c["layers"], c["n_blocks"], 8, 128, c["table"])
    cache.fill(c["layer"], c["k_rows"], c["v_rows"])
    ws = attention_workspace(32, 128)
    out16, out32 = N.DeviceBuffer(4096 * 2), N.DeviceBuffer(4096 * 4)
    qkv, qn, kn = dev(c["qkv"]), dev(c["qn"]), dev(c["kn"])
    outs = {}
    for splits in (2, 8, 32):
        if splits > c["n_blocks"]:
            continue
        first = None
        for launch in range(200):
            N.paged_attention(BF16, 32, 8, 128, cache, c["layer"], tokens, qkv, ws, out16, out_f32=out32, append=True,
                              rope_theta=1e6, q_norm=qn, k_norm=kn, splits=splits)
            bits = out32.numpy(np.uint32)
            if first is None:
                first = bits
                assert rel_l2(first.view(np.float32), ref) <= REL_L2, (tokens, splits)
            assert np.array_equal(bits, first), "context %d, %d splits: launch %d differs from the first" % (tokens, splits, launch)
        outs[splits] = first.view(np.float32)
    # different split factors are different (each deterministic) summation orders of the same sums
    for splits, out in outs.items():
        assert rel_l2(out, outs[min(outs)]) <= 1e-5, splits


def test_paged_attention_split_override_is_validated():
    c = _attention_case(BF16, 32, 8, 128, 40, 1e6, True, 3)
    cache = N.PagedKvCache(c["layers"], c["n_blocks"], 8, 128, c["table"])
    ws = attention_workspace(32, 128)
    out16 = N.DeviceBuffer(4096 * 2)
    for bad in (65, c["n_blocks"] + 1):
        with pytest.raises(RuntimeError):
            N.paged_attention(BF16, 32, 8, 128, cache, 0, 40, dev(c["qkv"]), ws, out16, splits=bad)


def test_paged_attention_refuses_split_factors_that_cannot_be_resident_together():
    """The merges of a kv head's splits poll inside the launch, so kv_heads x splits workgroups have to fit the
    machine at once (one per compute unit): a larger factor is refused on the host and nothing is launched."""
    c = _attention_case(BF16, 64, 8, 128, 2500, 1e6, True, 77)
    cache = N.PagedKvCache(c["layers"], c["n_blocks"], 8, 128, c["table"])
    ws = attention_workspace(64, 128)
    out16 = N.DeviceBuffer(64 * 128 * 2)
    out16.upload(np.full(64 * 128, 0x7fc1, np.uint16))
    most = N.abi.load().nerva_hip_paged_attention_max_splits(8)
    assert 1 <= most < 64
    with pytest.raises(RuntimeError):
        N.paged_attention(BF16, 64, 8, 128, cache, 0, 2500, dev(c["qkv"]), ws, out16, splits=most + 1)
    assert np.all(out16.numpy(np.uint16, 64 * 128) == 0x7fc1)          # nothing ran
    N.paged_attention(BF16, 64, 8, 128, cache, 0, 2500, dev(c["qkv"]), ws, out16, splits=most)
    assert N.paged_attention_status(ws, 64, 128) == (0, 0)


def test_paged_attention_merge_that_gives_up_is_an_error_and_leaves_the_workspace_usable():
    """A split that never hands its partial over (forced by a test hook; its workgroup exits normally) makes the
    merges that wait for it give up after their spin limit (set to a few polls here): the outputs they feed are
    NaN, the status call returns -1 with the step-fault error, and the next launch on the same workspace - whose
    partials carry another tag - is correct again."""
    c = _attention_case(BF16, 32, 8, 128, 4096, 1e6, True, 4242)
    ref, _, _ = _attention_oracle(c)
    cache = N.PagedKvCache(c["layers"], c["n_blocks"], 8, 128, c["table"])
    cache.fill(c["layer"], c["k_rows"], c["v_rows"])
    ws = attention_workspace(32, 128)
    out16, out32 = N.DeviceBuffer(4096 * 2), N.DeviceBuffer(4096 * 4)
    qkv, qn, kn = dev(c["qkv"]), dev(c["qn"]), dev(c["kn"])
    run = lambda: N.paged_attention(BF16, 32, 8, 128, cache, c["layer"], 4096, qkv, ws, out16, out_f32=out32, append=True,
                                    rope_theta=1e6, q_norm=qn, k_norm=kn)
    run()
    good = out32.numpy(np.float32).copy()
    assert rel_l2(good, ref) <= REL_L2 and N.paged_attention_status(ws, 32, 128) == (0, 0)
    N.Device.set_tuning("attn_merge_spin_limit", 4)
    N.Device.set_tuning("attn_withhold_split", 1 + 7)
    try:
        run()
    finally:
        N.Device.set_tuning("attn_merge_spin_limit", 0)
        N.Device.set_tuning("attn_withhold_split", 0)
    assert np.all(np.isnan(out32.numpy(np.float32)))          # every head's merge needed split 7
    rc, err = N.paged_attention_status(ws, 32, 128)
    assert rc == -1 and err == N.abi.NERVA_HIP_ERROR_STEP_FAULT
    assert N.paged_attention_status(ws, 32, 128) == (0, 0)     # reported once
    for _ in range(2):
        run()
        assert np.array_equal(out32.numpy(np.uint32), good.view(np.uint32))
        assert N.paged_attention_status(ws, 32, 128) == (0, 0)


def test_paged_attention_no_append_reads_cache_only():
    c = _attention_case(BF16, 32, 8, 128, 200, 1e6, True, 9)
    cache = N.PagedKvCache(c["layers"], c["n_blocks"], 8, 128, c["table"])
    cache.fill(c["layer"], c["k_rows"], c["v_rows"])
    ws = attention_workspace(32, 128)
    out16, out32 = N.DeviceBuffer(4096 * 2), N.DeviceBuffer(4096 * 4)
    N.paged_attention(BF16, 32, 8, 128, cache, c["layer"], 199, dev(c["qkv"]), ws, out16, out_f32=out32,
                      append=False, rope_theta=1e6, q_norm=dev(c["qn"]), k_norm=dev(c["kn"]))
    q = O.rope(128, 32, 199, 1e6, O.per_head_rms_norm(BF16, c["qn"], 128, c["qkv"][:4096], 1e-6))
    kc = np.zeros((c["layers"], c["n_blocks"], 16, 1024), np.uint16)
    vc = np.zeros_like(kc)
    for t in range(200):
        kc[c["layer"], c["table"][t // 16], t % 16] = c["k_rows"][t]
        vc[c["layer"], c["table"][t // 16], t % 16] = c["v_rows"][t]
    ref = O.attention_paged16(BF16, 32, 8, 128, 16, q, kc, vc, c["table"], c["layer"], c["n_blocks"], 200)
    assert rel_l2(out32.numpy(np.float32), ref) <= REL_L2


# ---------------------------------------------------------------------------
# argmax, MoE
# ---------------------------------------------------------------------------

def test_argmax_matches_oracle_rules():
    rng = np.random.default_rng(0)
    for n in (1, 4, 1000, 151936):
        l = rng.normal(0, 1, n).astype(np.float32)
        assert N.argmax(dev(l), n) == O.greedy_argmax(l, skip_nonfinite=True)
    l = rng.normal(0, 1, 151936).astype(np.float32)
    l[[777, 150000, 90000]] = l.max() + 1.0   # exact three-way tie -> lowest index
    assert N.argmax(dev(l), l.size) == 777
    l[100] = np.nan
    l[777] = np.inf                             # non-finite candidates are skipped
    assert N.argmax(dev(l), l.size) == 90000 == O.greedy_argmax(l, skip_nonfinite=True)
    ws = N.DeviceBuffer.zeros(abi.load().nerva_hip_argmax_workspace_bytes())
    for _ in range(3):                          # the workspace re-arms itself
        assert N.argmax(dev(l), l.size, ws) == 90000


SAMPLER_CONFIGS = [(0.7, 0.9, 0), (1.0, 1.0, 0), (1.5, 0.5, 40), (0.3, 1.0, 3), (1.0, 0.8, 200), (0.0, 1.0, 0),
                   (2.0, 0.9, 1), (0.9, 1.0, 128), (float("nan"), 2.0, 0)]


def test_sampler_matches_oracle_rule():
    """Same token as the oracle's restatement of the reference rule, at the full vocabulary and at ragged
    small ones, with ties and non-finite logits. The selection is integer work and exact; the device's
    exp/log may differ from the host's in the last bit, so a draw closer than 1e-5 (of the kept mass, or
    of the runner-up's score) to a boundary is set aside - and such draws have to stay rare."""
    rng = np.random.default_rng(5)
    close = checked = 0
    for n in (151936, 1000, 1025, 7, 1):
        l = (rng.standard_normal(n) * 3).astype(np.float32)
        if n > 100:
            l[rng.integers(0, n, 4)] = l.max()               # exact ties at the top
            l[rng.integers(0, n, 2)] = np.nan
            l[rng.integers(0, n, 2)] = np.inf
        buf = dev(l)
        ws = N.DeviceBuffer.zeros(abi.load().nerva_hip_sample_workspace_bytes(n))
        for temperature, top_p, top_k in SAMPLER_CONFIGS:
            for position in (0, 1, 8191, 70000):
                seed = int(rng.integers(0, 2 ** 62))
                want, margin = O.sample(l, 0.0 if temperature != temperature else temperature,
                                        1.0 if top_p > 1.0 else top_p, top_k, seed, position)
                got = N.sample(buf, n, temperature, top_p, top_k, seed, position, ws)
                checked += 1
                if got != want:
                    assert margin < 1e-5, (n, temperature, top_p, top_k, position, got, want, margin)
                    close += 1
    assert close <= checked // 50
    # a masked vocabulary: fewer finite logits than top_k asks for, the rest -inf (and a few +inf / NaN): every
    # finite logit is a candidate and nothing else is
    l = np.full(5000, -np.inf, np.float32)
    keep = rng.choice(5000, 50, replace=False)
    l[keep] = (rng.standard_normal(50) * 2).astype(np.float32)
    l[[7, 4000]] = np.inf
    l[11] = np.nan
    buf = dev(l)
    ws = N.DeviceBuffer.zeros(abi.load().nerva_hip_sample_workspace_bytes(l.size))
    for temperature, top_p, top_k in ((0.8, 0.95, 100), (1.5, 0.5, 0), (0.7, 1.0, 60)):
        for position in range(8):
            want, margin = O.sample(l, temperature, top_p, top_k, 5, position)
            got = N.sample(buf, l.size, temperature, top_p, top_k, 5, position, ws)
            assert np.isfinite(l[got]), (temperature, top_p, top_k, position, got)
            assert got == want or margin < 1e-5, (temperature, top_p, top_k, position, got, want, margin)
    # logits piled into the first chunks: the bound from the chunk maxima prunes nothing, and the
    # selection takes its general route (radix selection over all chunk candidates)
    l = (-1e-3 * np.arange(151936)).astype(np.float32)
    l[5] = l[3]                                               # a tie inside the top
    buf = dev(l)
    ws = N.DeviceBuffer.zeros(abi.load().nerva_hip_sample_workspace_bytes(l.size))
    for temperature, top_p, top_k in ((0.01, 1.0 - 1e-4, 0), (0.5, 0.9, 100), (5.0, 0.99, 7)):
        for position in range(6):
            want, margin = O.sample(l, temperature, top_p, top_k, 77, position)
            got = N.sample(buf, l.size, temperature, top_p, top_k, 77, position, ws)
            assert got == want or margin < 1e-5, (temperature, top_p, top_k, position, got, want, margin)


def test_moe_route_matches_oracle():
    rng = np.random.default_rng(3)
    for e, k, norm in ((256, 8, True), (256, 8, False), (64, 6, True), (5, 5, True)):
        logits = rng.normal(0, 1, e).astype(np.float32)
        ids, wts, _, _ = N.moe_route_softmax(logits, k, norm)
        rid, rw = O.moe_route_softmax(logits, k, norm)
        assert ids.tolist() == rid.tolist()
        assert np.allclose(wts, rw, rtol=2e-6, atol=0)
    ids, _, _, _ = N.moe_route_softmax(np.zeros(6, np.float32), 3, True)
    assert ids.tolist() == [0, 1, 2]


@pytest.mark.parametrize("hidden,inter,experts,top_k", [(1024, 1024, 6, 2), (7168, 2048, 12, 8)])
def test_moe_fp8_experts_match_oracle(hidden, inter, experts, top_k):
    """Config 4 geometry (hidden 7168, intermediate 2048, top-8 + 1 shared) on a 12-expert bank."""
    B = 128
    wg = np.empty((experts, inter, hidden), np.uint8)
    wu = np.empty_like(wg)
    wd = np.empty((experts, hidden, inter), np.uint8)
    sg = np.empty((experts, inter // B, hidden // B), np.float32)
    su = np.empty_like(sg)
    sd = np.empty((experts, hidden // B, inter // B), np.float32)
    for e in range(experts):
        wg[e], sg[e] = O.synth_fp8_block(SEED, 300 + e, inter, hidden, B, 0.02)
        wu[e], su[e] = O.synth_fp8_block(SEED, 400 + e, inter, hidden, B, 0.02)
        wd[e], sd[e] = O.synth_fp8_block(SEED, 500 + e, hidden, inter, B, 0.02)
    x16 = O.synth_16(BF16, SEED, 12, hidden, 0.0, 1.0)
    logits = O.synth_f32(SEED, 13, experts - 1, 0.0, 1.0)      # the last expert is the shared one
    ids, wts, dids, dwts = N.moe_route_softmax(logits, top_k, True)
    rid, rw = O.moe_route_softmax(logits, top_k, True)
    assert ids.tolist() == rid.tolist()
    ref = O.moe_fp8_forward(hidden, inter, experts, B, x16, rid, rw, wg, sg, wu, su, wd, sd,
                            shared_index=experts - 1)
    act = N.DeviceBuffer((top_k + 1) * inter * 4)
    out = N.DeviceBuffer(hidden * 4)
    N.moe_fp8_experts(hidden, inter, experts, top_k, B, dev(x16), dids, dwts, dev(wg), dev(sg), dev(wu),
                      dev(su), dev(wd), dev(sd), act, out, shared_index=experts - 1)
    assert rel_l2(out.numpy(np.float32), ref) <= REL_L2
    # no shared expert
    ref2 = O.moe_fp8_forward(hidden, inter, experts, B, x16, rid, rw, wg, sg, wu, su, wd, sd)
    N.moe_fp8_experts(hidden, inter, experts, top_k, B, dev(x16), dids, dwts, dev(wg), dev(sg), dev(wu),
                      dev(su), dev(wd), dev(sd), act, out, shared_index=-1)
    assert rel_l2(out.numpy(np.float32), ref2) <= REL_L2


def test_moe_fp8_experts_in_a_256_expert_bank():
    """Config 4's address space: 256 routed experts + the shared one (index 256), hidden 7168,
    intermediate 2048. Only the experts the route selects hold data (ids 3, 131, 254, 255 among them:
    expert stride x 255 is a 64-bit product), everything else in the 11 GB bank is never touched. The
    oracle sees the same nine experts as a compact bank with the ids renumbered - the same sums in the
    same order. An id outside the bank must poison the output, not pick another expert."""
    hidden, inter, experts, top_k, B = 7168, 2048, 257, 8, 128
    chosen = np.array([3, 131, 254, 255, 0, 77, 128, 200], np.uint32)
    wts = np.random.default_rng(4).dirichlet(np.ones(top_k)).astype(np.float32)
    bank = list(chosen) + [256]
    wg = np.empty((len(bank), inter, hidden), np.uint8)
    wu = np.empty_like(wg)
    wd = np.empty((len(bank), hidden, inter), np.uint8)
    sg = np.empty((len(bank), inter // B, hidden // B), np.float32)
    su = np.empty_like(sg)
    sd = np.empty((len(bank), hidden // B, inter // B), np.float32)
    for j, e in enumerate(bank):
        wg[j], sg[j] = O.synth_fp8_block(SEED, 3000 + int(e), inter, hidden, B, 0.02)
        wu[j], su[j] = O.synth_fp8_block(SEED, 4000 + int(e), inter, hidden, B, 0.02)
        wd[j], sd[j] = O.synth_fp8_block(SEED, 5000 + int(e), hidden, inter, B, 0.02)
    x16 = O.synth_16(BF16, SEED, 12, hidden, 0.0, 1.0)
    ref = O.moe_fp8_forward(hidden, inter, len(bank), B, x16, np.arange(top_k, dtype=np.uint32), wts, wg, sg, wu, su,
                            wd, sd, shared_index=top_k)
    dwg, dwu, dwd = (N.DeviceBuffer(experts * inter * hidden) for _ in range(3))
    dsg, dsu, dsd = (N.DeviceBuffer(experts * (inter // B) * (hidden // B) * 4) for _ in range(3))
    for j, e in enumerate(bank):
        e = int(e)
        for buf, arr in ((dwg, wg), (dwu, wu), (dwd, wd), (dsg, sg), (dsu, su), (dsd, sd)):
            buf.upload(arr[j], offset=e * arr[j].nbytes)
    act = N.DeviceBuffer((top_k + 1) * inter * 4)
    out = N.DeviceBuffer(hidden * 4)
    N.moe_fp8_experts(hidden, inter, experts, top_k, B, dev(x16), dev(chosen), dev(wts), dwg, dsg, dwu, dsu, dwd, dsd,
                      act, out, shared_index=256)
    assert rel_l2(out.numpy(np.float32), ref) <= REL_L2
    bad = chosen.copy()
    bad[2] = 257
    N.moe_fp8_experts(hidden, inter, experts, top_k, B, dev(x16), dev(bad), dev(wts), dwg, dsg, dwu, dsu, dwd, dsd,
                      act, out, shared_index=256)
    assert np.all(np.isnan(out.numpy(np.float32)))


@pytest.mark.parametrize("dtype", [BF16, F16])
def test_moe_lean_kernels_decode_every_fp8_code(dtype):
    """The production-shape MoE kernels turn pairs of e4m3fn weights into packed 16-bit pairs with the
    hardware conversion (gate/up) or into f32 (down) and read the activations in their own LDS order. Here
    every output meets exactly one weight code: gate row i holds code i % 256 in column i and the
    activation vector is all ones, the up rows pick a 1, so act[i] = silu(value of the code) - every finite
    code in four different lanes and pieces; down row h holds code h % 256 in column h, so out[h] =
    value(code) * act[h]. Exact up to f32 rounding of silu."""
    hidden = inter = 1024
    B = 128
    codes = np.arange(256, dtype=np.uint8)
    codes[[0x7f, 0xff]] = 0                                  # the two NaN codes
    values = O.decode_fp8(codes).astype(np.float64)
    wg = np.zeros((1, inter, hidden), np.uint8)
    wu = np.zeros_like(wg)
    wd = np.zeros((1, hidden, inter), np.uint8)
    idx = np.arange(inter)
    wg[0, idx, idx] = codes[idx % 256]
    wu[0, idx, (idx * 7 + 3) % hidden] = 0x38                # 1.0
    wd[0, idx, idx] = codes[(idx + 64) % 256]
    ones = np.ones((1, inter // B, hidden // B), np.float32)
    x16 = O.encode16(dtype, np.ones(hidden))
    ids, wts = np.zeros(1, np.uint32), np.ones(1, np.float32)
    act = N.DeviceBuffer(inter * 4)
    out = N.DeviceBuffer(hidden * 4)
    N.moe_fp8_experts(hidden, inter, 1, 1, B, dev(x16), dev(ids), dev(wts), dev(wg), dev(ones), dev(wu), dev(ones),
                      dev(wd), dev(ones), act, out, input_dtype=dtype)
    g = values[idx % 256]
    want_act = g / (1.0 + np.exp(-g))
    got_act = act.numpy(np.float32).astype(np.float64)
    assert np.allclose(got_act, want_act, rtol=2e-6, atol=1e-9)
    want_out = values[(idx + 64) % 256] * got_act
    assert np.allclose(out.numpy(np.float32), want_out, rtol=1e-6, atol=1e-12)


def test_moe_forward_f32_kat_host_pointer_abi(kat):
    import ctypes as C
    k = kat["moe_routed_clamp"]
    f = lambda v: np.array(v, np.float32)
    x, wg, wu, wd = f(k["input"]), f(k["w_gate"]), f(k["w_up"]), f(k["w_down"])
    ids, wts = np.array(k["expert_ids"], np.uint32), f(k["expert_weights"])
    out = np.zeros(k["hidden"], np.float32)
    req = abi.NervaHipDeepSeekMoeForwardRequest()
    req.hidden_size, req.intermediate_size, req.num_experts, req.top_k = k["hidden"], k["intermediate"], 2, 2
    req.clamp_swiglu, req.swiglu_limit = 1, k["swiglu_limit"]
    req.input, req.expert_ids, req.expert_weights = x.ctypes.data, ids.ctypes.data, wts.ctypes.data
    req.w_gate, req.w_up, req.w_down, req.output = wg.ctypes.data, wu.ctypes.data, wd.ctypes.data, out.ctypes.data
    res = abi.NervaHipDeepSeekMoeForwardResult()
    assert abi.load().nerva_hip_deepseek_moe_forward(C.byref(req), C.byref(res)) == 0
    ref = O.moe_forward_f32(k["hidden"], k["intermediate"], x, ids, wts, wg, wu, wd, limit=k["swiglu_limit"])
    assert np.max(np.abs(out - ref)) < k["tol"]
    assert res.hot_path_allocations == 0 and res.sync_calls == 1
    ids[0] = 9  # out-of-range expert id is refused before touching the device
    assert abi.load().nerva_hip_deepseek_moe_forward(C.byref(req), C.byref(res)) == -1 and res.moe_error != 0


def test_projection_bench_runs_and_checks_itself():
    import ctypes as C
    req = abi.NervaHipProjectionBenchRequest()
    req.dtype, req.rows, req.cols, req.iterations, req.warmup_iterations, req.block_tokens = BF16, 4096, 4096, 40, 5, 1
    res = abi.NervaHipProjectionBenchResult()
    assert abi.load().nerva_hip_projection_bench(C.byref(req), C.byref(res)) == 0
    assert res.mismatch_count == 0 and res.max_abs_diff < 1e-2
    assert res.hot_path_allocations == 0 and res.graph_captures == 1
    assert res.matrix_bytes == 4096 * 4096 * 2 and res.custom_avg_ns > 0 and res.custom_graph_avg_ns > 0
    print("q_proj GEMV eager %d ns, graph %d ns, %.0f GB/s" % (
        res.custom_avg_ns, res.custom_graph_avg_ns,
        (res.matrix_bytes + res.input_bytes + res.output_bytes) / res.custom_graph_avg_ns), flush=True)


def test_plain_copy_kernel_is_exact_and_rejects_unaligned():
    rng = np.random.default_rng(11)
    for nbytes in (16, 4096 + 16, (3 << 20) + 48):
        src = rng.integers(0, 256, nbytes, dtype=np.uint8)
        a, b = dev(src), N.DeviceBuffer.zeros(nbytes)
        N.Device.copy(b, a, nbytes)
        assert np.array_equal(b.numpy(np.uint8, nbytes), src)
    assert abi.load().nerva_hip_copy_d2d(b.ptr, a.ptr, 24, None) == -1
    assert abi.load().nerva_hip_copy_d2d(b.ptr + 4, a.ptr, 16, None) == -1


def test_operator_timer_records_launches_into_a_graph():
    import ctypes as C
    rng = np.random.default_rng(5)
    rows, cols = 256, 4096
    w = O.encode16(BF16, rng.normal(0, 0.05, (rows, cols)))
    x = O.encode16(BF16, rng.normal(0, 1, cols))
    dw, dx, y = dev(w), dev(x), N.DeviceBuffer.zeros(rows * 4)
    lib = abi.load()
    nodes, ns = C.c_uint64(0), C.c_double(0.0)
    assert lib.nerva_hip_timer_capture_end(1, 1, C.byref(nodes), C.byref(ns)) == -1   # nothing being recorded
    assert lib.nerva_hip_timer_capture_begin() == 0
    assert lib.nerva_hip_timer_capture_begin() == -1                                  # one recording at a time
    for _ in range(5):
        N.gemv(BF16, dw, rows, cols, input16=dx, out_f32=y, sync=False)
    assert lib.nerva_hip_timer_capture_end(2, 4, C.byref(nodes), C.byref(ns)) == 0
    assert nodes.value == 5 and ns.value > 0
    assert rel_l2(y.numpy(np.float32), O.gemv(BF16, w, O.decode16(BF16, x))) <= REL_L2


@pytest.mark.parametrize("tokens,rows,cols", [(5, 48, 2048), (32, 1000, 2048), (33, 64, 4096), (64, 4096, 4096), (65, 64, 2048), (128, 4096, 4096)])
def test_gemm_rows_operand_order_is_the_same_arithmetic(tokens, rows, cols):
    """Inputs and SwiGLU outputs in matrix-operand order (what prompt blocks and batch steps keep between
    their kernels) only change where bytes lie: the results are bit-identical to the row-major call."""
    dtype = BF16
    rng = np.random.default_rng(tokens * rows)
    w = O.encode16(dtype, rng.normal(0, 0.05, (rows, cols)))
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, cols)))
    packed, idx = N.gemm_operand_order(x)
    assert np.array_equal(packed[idx], x) and len(np.unique(idx)) == idx.size      # a permutation into the buffer
    dw = dev(w)
    y0, y1 = N.DeviceBuffer(tokens * rows * 4), N.DeviceBuffer(tokens * rows * 4)
    N.gemm_rows(dtype, dw, rows, cols, tokens, dev(x), out_f32=y0)
    N.gemm_rows(dtype, dw, rows, cols, tokens, dev(packed), out_f32=y1, input_operand_order=True)
    # blocks in operand order may take the kernel that shares X through LDS: the same products summed in another order
    same_kernel = rows % 64 != 0 or cols % 512 != 0
    if same_kernel:
        assert np.array_equal(y0.numpy(np.float32), y1.numpy(np.float32))
    else:
        assert rel_l2(y1.numpy(np.float32), y0.numpy(np.float32)) <= 1e-5
    if rows % 2 == 0 and (rows // 2) % 32 == 0:
        inter = rows // 2                                                          # the same matrix as [gate; up]
        o0 = N.DeviceBuffer(tokens * inter * 2)
        o1 = N.DeviceBuffer.zeros(N.gemm_operand_slots(tokens) * inter * 2)
        N.gemm_rows(dtype, dw, inter, cols, tokens, dev(x), epilogue=2, out16=o0)
        N.gemm_rows(dtype, dw, inter, cols, tokens, dev(packed), epilogue=2, out16=o1, input_operand_order=True,
                    output16_operand_order=True)
        rowmajor = o0.numpy(np.uint16, tokens * inter).reshape(tokens, inter)
        _, oidx = N.gemm_operand_order(np.zeros((tokens, inter), np.uint16))
        if same_kernel:
            assert np.array_equal(o1.numpy(np.uint16)[oidx], rowmajor)
        else:
            assert rel_l2(O.decode16(dtype, o1.numpy(np.uint16)[oidx]), O.decode16(dtype, rowmajor)) <= 4e-3


@pytest.mark.parametrize("sliced", [False, True])
@pytest.mark.parametrize("rows,cols,tokens", [(64, 2048, 65), (192, 2048, 100), (4096, 4096, 128), (6144, 4096, 127),
                                               (4096, 12288, 128), (192, 2048, 17), (64, 2048, 33), (4096, 4096, 32),
                                               (6144, 4096, 48), (4096, 12288, 64),
                                               (128, 2048, 129), (256, 4096, 200), (4096, 4096, 256), (6144, 4096, 255),
                                               (4096, 12288, 256), (192, 2048, 140),
                                               (256, 2048, 257), (512, 4096, 300), (4096, 4096, 512), (6144, 4096, 511),
                                               (4096, 12288, 512), (256, 1024, 400), (192, 2048, 300), (576, 1024, 512)])
def test_gemm_rows_large_blocks_share_x_through_lds(rows, cols, tokens, sliced):
    """More than 16 token rows in operand order: the workgroups split rows (and, given a workspace, K) and read
    X from LDS (2, 4, 8 or - blocks of 129..256 rows, three or four wave pairs sharing their W tiles - 16 token tiles;
    blocks of 257..512 rows, 256 weight rows x 256 tokens a workgroup, W and X straight into LDS - 32). Every token
    row equals the oracle's GEMV of that row; bias + residual + rounding on top."""
    dtype = BF16
    rng = np.random.default_rng(rows + cols + tokens)
    if rows * cols > 1 << 22:
        w = O.synth_16(dtype, SEED, 320 + tokens, rows * cols, 0.0, 0.02).reshape(rows, cols)
    else:
        w = O.encode16(dtype, rng.normal(0, 0.02, (rows, cols)))
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, cols)))
    bias = O.encode16(dtype, rng.normal(0, 0.1, rows))
    res = rng.normal(0, 1, (tokens, rows)).astype(np.float32)
    step = 1 if rows * cols <= 1 << 22 else 9
    picks = list(range(0, tokens, step)) + [tokens - 1]
    ref = {t: O.gemv_x16(dtype, w, x[t]) for t in picks}
    packed, _ = N.gemm_operand_order(x)
    ws = N.DeviceBuffer(N.gemm_rows_workspace_bytes(rows)) if sliced else None
    dw, dx = dev(w), dev(packed)
    y = N.DeviceBuffer.zeros(tokens * rows * 4)
    N.gemm_rows(dtype, dw, rows, cols, tokens, dx, epilogue=0, out_f32=y, input_operand_order=True, workspace=ws)
    got = y.numpy(np.float32).reshape(tokens, rows)
    assert max(rel_l2(got[t], ref[t]) for t in picks) <= REL_L2
    N.gemm_rows(dtype, dw, rows, cols, tokens, dx, epilogue=1, bias=dev(bias), residual=dev(res), out_f32=y,
                round_output=True, input_operand_order=True, workspace=ws)
    got = y.numpy(np.float32).reshape(tokens, rows)
    for t in picks:
        want = O.decode16(dtype, O.encode16(dtype, (ref[t] + O.decode16(dtype, bias)) + res[t]))
        assert rel_l2(got[t], want) <= 4e-3
    assert np.array_equal(O.encode16(dtype, got), O.encode16(dtype, got.astype(np.float32)))


def test_gemm_rows_small_block_launch_shapes_agree():
    """The shared-X kernel's launch-shape choices only reorder sums: a common start of every row group's K walk
    against the rotated one, four-wave against three-wave workgroups for the gate/up pair, fewer or more K slices."""
    dtype, inter, hidden, tokens = BF16, 12288, 4096, 32
    w = O.synth_16(dtype, SEED, 340, 2 * inter * hidden, 0.0, 0.02).reshape(2 * inter, hidden)
    rng = np.random.default_rng(11)
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, hidden)))
    packed, _ = N.gemm_operand_order(x)
    dw, dx = dev(w), dev(packed)
    ws = N.DeviceBuffer(N.gemm_rows_workspace_bytes(2 * inter))
    _, oidx = N.gemm_operand_order(np.zeros((tokens, inter), np.uint16))

    def swiglu():
        out = N.DeviceBuffer.zeros(N.gemm_operand_slots(tokens) * inter * 2)
        N.gemm_rows(dtype, dw, inter, hidden, tokens, dx, epilogue=2, out16=out, input_operand_order=True,
                    output16_operand_order=True, workspace=ws)
        return O.decode16(dtype, out.numpy(np.uint16)[oidx])

    def plain(rows):
        y = N.DeviceBuffer.zeros(tokens * rows * 4)
        N.gemm_rows(dtype, dw, rows, hidden, tokens, dx, epilogue=0, out_f32=y, input_operand_order=True, workspace=ws)
        return y.numpy(np.float32).copy()

    try:
        base_pair, base_plain = swiglu(), plain(6144)
        t = 7
        gu = O.gemv_x16(dtype, w, x[t])
        g, u = gu[:inter].astype(np.float64), gu[inter:].astype(np.float64)
        want = O.decode16(dtype, O.encode16(dtype, (g / (1.0 + np.exp(-g)) * u).astype(np.float32)))
        assert rel_l2(base_pair.reshape(tokens, inter)[t], want) <= 4e-3
        for knob, value in (("gemm_block_rotate", 1), ("gemm_block_rotate", 14), ("gemm_block_waves", 4)):
            N.Device.set_tuning(knob, value)
            assert rel_l2(swiglu(), base_pair) <= 4e-3, (knob, value)       # 16-bit outputs: a rounding step apart at most
            N.Device.set_tuning(knob, 0)
        for knob, value in (("gemm_block_rotate", 1), ("gemm_block_slices", 4), ("gemm_block_slices", 1)):
            N.Device.set_tuning(knob, value)
            assert rel_l2(plain(6144), base_plain) <= 1e-5, (knob, value)
            N.Device.set_tuning(knob, 0)
    finally:
        N.Device.reset_tuning()


@pytest.mark.parametrize("tokens", [200, 257, 512])
def test_gemm_rows_large_blocks_in_f16(tokens):
    """The kernels for blocks of 129..256 and of 257..512 rows with f16 operands (the other cases of this family
    run in bf16): every token row against the oracle's GEMV, plain and as a gate/up pair."""
    dtype, rows, cols = F16, 512, 2048
    rng = np.random.default_rng(tokens)
    w = O.encode16(dtype, rng.normal(0, 0.05, (rows, cols)))
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, cols)))
    packed, _ = N.gemm_operand_order(x)
    ws = N.DeviceBuffer(N.gemm_rows_workspace_bytes(rows))
    dw, dx = dev(w), dev(packed)
    y = N.DeviceBuffer.zeros(tokens * rows * 4)
    N.gemm_rows(dtype, dw, rows, cols, tokens, dx, epilogue=0, out_f32=y, input_operand_order=True, workspace=ws)
    got = y.numpy(np.float32).reshape(tokens, rows)
    picks = sorted({0, 1, 127, 128, tokens // 2, tokens - 2, tokens - 1})
    ref = {t: O.gemv_x16(dtype, w, x[t]) for t in picks}
    assert max(rel_l2(got[t], ref[t]) for t in picks) <= REL_L2
    inter = rows // 2
    out = N.DeviceBuffer.zeros(N.gemm_operand_slots(tokens) * inter * 2)
    N.gemm_rows(dtype, dw, inter, cols, tokens, dx, epilogue=2, out16=out, input_operand_order=True,
                output16_operand_order=True)
    _, oidx = N.gemm_operand_order(np.zeros((tokens, inter), np.uint16))
    act = O.decode16(dtype, out.numpy(np.uint16)[oidx]).reshape(tokens, inter)
    for t in picks:
        g, u = ref[t][:inter].astype(np.float64), ref[t][inter:].astype(np.float64)
        want = O.decode16(dtype, O.encode16(dtype, (g / (1.0 + np.exp(-g)) * u).astype(np.float32)))
        assert rel_l2(act[t], want) <= 4e-3


@pytest.mark.parametrize("sliced", [False, True])
@pytest.mark.parametrize("inter,hidden,tokens", [(64, 2048, 77), (12288, 4096, 128), (64, 2048, 24), (12288, 4096, 32), (128, 2048, 50),
                                                 (64, 2048, 130), (128, 2048, 256), (12288, 4096, 250), (96, 2048, 200),
                                                 (128, 2048, 257), (256, 1024, 512), (12288, 4096, 500), (96, 2048, 300), (288, 1024, 512),
                                                 (192, 2048, 20), (96, 2048, 40), (288, 2048, 64)])
def test_gemm_rows_large_blocks_swiglu(inter, hidden, tokens, sliced):
    """The gate/up pair of a large block: out16 = round16(silu(gate) * up), written in operand order."""
    dtype = BF16
    rng = np.random.default_rng(inter + tokens)
    if inter > 1000:
        w = O.synth_16(dtype, SEED, 330, 2 * inter * hidden, 0.0, 0.02).reshape(2 * inter, hidden)
    else:
        w = O.encode16(dtype, rng.normal(0, 0.05, (2 * inter, hidden)))
    x = O.encode16(dtype, rng.normal(0, 1, (tokens, hidden)))
    packed, _ = N.gemm_operand_order(x)
    ws = N.DeviceBuffer(N.gemm_rows_workspace_bytes(2 * inter)) if sliced else None
    out = N.DeviceBuffer.zeros(N.gemm_operand_slots(tokens) * inter * 2)
    N.gemm_rows(dtype, dev(w), inter, hidden, tokens, dev(packed), epilogue=2, out16=out, input_operand_order=True,
                output16_operand_order=True, workspace=ws)
    _, oidx = N.gemm_operand_order(np.zeros((tokens, inter), np.uint16))
    got = O.decode16(dtype, out.numpy(np.uint16)[oidx]).reshape(tokens, inter)
    for t in sorted({0, tokens // 3, tokens - 1}):
        gu = O.gemv_x16(dtype, w, x[t])
        g, u = gu[:inter].astype(np.float64), gu[inter:].astype(np.float64)
        want = O.decode16(dtype, O.encode16(dtype, (g / (1.0 + np.exp(-g)) * u).astype(np.float32)))
        assert rel_l2(got[t], want) <= 4e-3
