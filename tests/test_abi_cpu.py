"""CPU-only checks of the C ABI boundary: the shared library loads, exports every symbol the
header declares, mirrors the reference struct layouts, and fails closed without a device.
No compute is attempted here."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from nerva_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# sizeof/offsetof of the NervaCuda... originals (x86-64 SysV), see include/nerva_hip_layout_check.hpp
REFERENCE_SIZES = {
    "NervaHipDeviceSmokeResult": 232, "NervaHipSyntheticTokenSlot": 40, "NervaHipHfDecodeChainLayer": 440,
    "NervaHipHfDecodeSequenceWeightBlock": 72, "NervaHipHfDecodeSamplerConfig": 24,
    "NervaHipHfDecodeSequenceRequest": 208, "NervaHipHfDecodeSequenceResult": 528,
    "NervaHipHfDecodeSequenceSessionCreateRequest": 176, "NervaHipHfDecodeSequenceSessionCreateResult": 272,
    "NervaHipHfDecodeSequenceSessionRunRequest": 80, "NervaHipHfDecodeSequenceSessionStartRequest": 56,
    "NervaHipHfDecodeSequenceSessionAdvanceRequest": 32, "NervaHipDeepSeekQuantDequantResult": 96,
    "NervaHipDeepSeekQuantFp8F32ScaleEncodedMatvecRequest": 56,
    "NervaHipDeepSeekQuantFp8F32ScaleEncodedGemmTokensRequest": 56, "NervaHipProjectionBenchRequest": 24,
    "NervaHipProjectionBenchResult": 408, "NervaHipDeepSeekMoeForwardRequest": 80,
    "NervaHipDeepSeekMoeForwardResult": 104,
}


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(abi.LIBRARY):
        from nerva_amd import build
        build.build()
    return abi.load()


def test_library_exports_every_declared_symbol(lib):
    names = abi.declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), name
    for required in ("nerva_hip_device_smoke", "nerva_hip_hf_decode_sequence_u16",
                     "nerva_hip_hf_decode_sequence_session_create", "nerva_hip_hf_decode_sequence_session_start",
                     "nerva_hip_hf_decode_sequence_session_advance", "nerva_hip_hf_decode_sequence_session_run",
                     "nerva_hip_hf_decode_sequence_session_destroy",
                     "nerva_hip_deepseek_quant_fp8_f32_scale_encoded_matvec", "nerva_hip_projection_bench",
                     "nerva_hip_deepseek_moe_forward", "nerva_hip_gemv", "nerva_hip_fp8_gemv",
                     "nerva_hip_paged_gqa_decode", "nerva_hip_argmax", "nerva_hip_moe_fp8_experts"):
        assert required in names


def test_struct_layouts_mirror_reference():
    for name, size in REFERENCE_SIZES.items():
        assert C.sizeof(abi.STRUCTS[name]) == size, name
    assert abi.NervaHipSyntheticTokenSlot.version.offset == 24
    assert abi.NervaHipHfDecodeChainLayer.mlp_kind.offset == 280
    assert abi.NervaHipHfDecodeSequenceResult.observed_token_hash.offset == 64
    assert abi.NervaHipHfDecodeSequenceResult.hot_path_allocations.offset == 400
    assert abi.NervaHipHfDecodeSequenceSessionCreateRequest.detailed_profile.offset == 144
    assert abi.NervaHipHfDecodeSequenceSessionStartRequest.sampler.offset == 32


def test_layout_check_header_compiles(tmp_path):
    src = tmp_path / "layout.cpp"
    src.write_text('#include "nerva_hip_layout_check.hpp"\nint main() { return 0; }\n')
    subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(src)], check=True)
    subprocess.run(["gcc", "-std=c99", "-fsyntax-only", "-x", "c", os.path.join(ROOT, "include", "nerva_hip_api.h")],
                   check=True)


def _has_gpu(lib):
    res = abi.NervaHipDeviceSmokeResult()
    return lib.nerva_hip_device_smoke(C.byref(res)) == 0


def test_null_out_and_null_request_fail_closed(lib):
    """out == NULL -> -1; otherwise the result is zeroed and status = -1
    (session_api_lifecycle.inc.cu:5-55, 1117-1144)."""
    assert lib.nerva_hip_device_smoke(None) == -1
    assert lib.nerva_hip_hf_decode_sequence_session_start(None, None) == -1
    res = abi.NervaHipHfDecodeSequenceResult()
    C.memset(C.byref(res), 0xAB, C.sizeof(res))
    assert lib.nerva_hip_hf_decode_sequence_session_start(None, C.byref(res)) == -1
    assert res.status == -1 and res.hip_error == 0 and res.hidden == 0 and res.hot_path_allocations == 0
    C.memset(C.byref(res), 0xAB, C.sizeof(res))
    assert lib.nerva_hip_hf_decode_sequence_session_advance(None, C.byref(res)) == -1 and res.status == -1
    assert lib.nerva_hip_hf_decode_sequence_session_run(None, C.byref(res)) == -1 and res.status == -1
    assert lib.nerva_hip_hf_decode_sequence_u16(None, C.byref(res)) == -1 and res.status == -1
    cres = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    assert lib.nerva_hip_hf_decode_sequence_session_create(None, C.byref(cres), C.byref(handle)) == -1
    assert cres.status == -1 and not handle
    assert lib.nerva_hip_hf_decode_sequence_session_destroy(None, C.byref(cres)) == -1 and cres.status == -1
    q = abi.NervaHipDeepSeekQuantDequantResult()
    assert lib.nerva_hip_deepseek_quant_fp8_f32_scale_encoded_matvec(None, C.byref(q)) == -1 and q.status == -1
    p = abi.NervaHipProjectionBenchResult()
    assert lib.nerva_hip_projection_bench(None, C.byref(p)) == -1 and p.status == -1
    m = abi.NervaHipDeepSeekMoeForwardResult()
    assert lib.nerva_hip_deepseek_moe_forward(None, C.byref(m)) == -1 and m.status == -1


def test_zero_dim_and_missing_weights_are_rejected_before_the_device(lib):
    req = abi.NervaHipHfDecodeSequenceSessionCreateRequest()
    cres = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    req.dtype, req.hidden, req.heads, req.kv_heads, req.head_dim = 1, 0, 1, 1, 2
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    assert cres.status == -1 and cres.hip_error == 0 and cres.failure_stage == 1
    req.hidden, req.intermediate, req.vocab_size, req.layer_count, req.max_context_tokens = 2, 2, 4, 1, 4
    req.rms_eps = 1e-5
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    assert cres.hip_error == 0                      # null weight pointers: invalid argument, not a device error
    req.heads, req.kv_heads = 3, 2                  # heads not divisible by kv_heads
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    req.dtype = 2
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1


def _tiny_request():
    z = np.zeros(8, np.uint16)
    layer = (abi.NervaHipHfDecodeChainLayer * 1)()
    for f in ("rms_attn_weight", "rms_mlp_weight", "w_q", "w_k", "w_v", "w_o", "w_gate", "w_up", "w_down"):
        setattr(layer[0], f, z.ctypes.data)
    req = abi.NervaHipHfDecodeSequenceSessionCreateRequest()
    req.dtype, req.hidden, req.heads, req.kv_heads, req.head_dim = 0, 2, 1, 1, 2
    req.intermediate, req.vocab_size, req.layer_count, req.max_context_tokens = 2, 4, 1, 4
    req.rms_eps = 1e-5
    req.embeddings = req.final_norm_weight = req.lm_head = z.ctypes.data
    req.layers = layer
    return req, layer, z


def test_unsupported_features_are_refused_explicitly(lib):
    """MoE / linear-attention / DeepSeek / RT fields: status -1 with NOT_SUPPORTED, never silently ignored."""
    cres = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    for field, value in (("mlp_kind", 1), ("attention_kind", 2), ("deepseek_mode", 1), ("num_experts", 8),
                         ("linear_key_heads", 2)):
        req, layer, z = _tiny_request()
        setattr(layer[0], field, value)
        assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
        assert cres.hip_error == abi.NERVA_HIP_ERROR_NOT_SUPPORTED, field
    req, layer, z = _tiny_request()
    layer[0].w_router = z.ctypes.data
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    assert cres.hip_error == abi.NERVA_HIP_ERROR_NOT_SUPPORTED
    req, layer, z = _tiny_request()
    req.experimental_rt_decode = 1
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    assert cres.hip_error == abi.NERVA_HIP_ERROR_NOT_SUPPORTED


def test_no_device_reports_error_100(lib):
    """Without a GPU every call that needs one reports status -1, hip_error 100
    (the reference's stub build: crates/nerva-cuda/src/native_stubs.rs:5-33)."""
    if _has_gpu(lib):
        pytest.skip("a GPU is present")
    smoke = abi.NervaHipDeviceSmokeResult()
    assert lib.nerva_hip_device_smoke(C.byref(smoke)) == -1
    assert smoke.status == -1 and smoke.hip_error == abi.NERVA_HIP_ERROR_NO_DEVICE
    req, layer, z = _tiny_request()
    cres = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    assert cres.status == -1 and cres.hip_error == abi.NERVA_HIP_ERROR_NO_DEVICE and not handle
    breq = abi.NervaHipProjectionBenchRequest()
    breq.dtype, breq.rows, breq.cols, breq.iterations = 1, 64, 64, 1
    bres = abi.NervaHipProjectionBenchResult()
    assert lib.nerva_hip_projection_bench(C.byref(breq), C.byref(bres)) == -1
    assert bres.hip_error == abi.NERVA_HIP_ERROR_NO_DEVICE
    ptr = C.c_void_p()
    assert lib.nerva_hip_malloc(C.byref(ptr), 64) == -1 and not ptr.value


def test_python_package_has_no_cpu_fallback():
    """The shipped package must not import the oracle or carry a CPU compute path."""
    pkg = os.path.join(ROOT, "nerva_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cuh", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f
                assert "libnerva_oracle" not in text and "nvo_" not in text, f


def test_weight_plan_hash_and_totals_of_the_reference_twelve_block_plan():
    """Host logic of the weight plan (weight_plan.rs:24-126): the known-answer model's tensors in arena
    order give the reference's 12 blocks (decode_sequence_descriptor_blocks.rs:223-258), and the
    descriptor hash is FNV-1a-64 over the little-endian bytes of (block_id, block_version,
    offset_bytes, bytes: u64; strategy: u32) - checked against the oracle's byte hash, which the
    reference's own hash vectors pin."""
    import struct

    import nerva_amd as N
    import oracle as O

    z4, r2 = np.zeros(4, np.uint16), np.full(2, 0x3C00, np.uint16)
    layer = dict(rms_attn=r2, rms_mlp=r2, w_q=z4, w_k=z4, w_v=z4, w_o=z4, w_gate=z4, w_up=z4, w_down=z4)
    weights = N.ModelWeights(0, 2, 1, 1, 2, 2, 4, 1e-5, 0.0, np.zeros(8, np.uint16), [layer], r2, np.zeros(8, np.uint16))
    plan = N.WeightPlan.from_weights(weights, resident_blocks=6)
    assert [b.bytes for b in plan.blocks] == [16, 4, 8, 8, 8, 8, 4, 8, 8, 8, 4, 16]
    assert [b.offset_bytes for b in plan.blocks] == [0, 16, 20, 28, 36, 44, 52, 56, 64, 72, 80, 84]
    assert [b.block_id for b in plan.blocks] == list(range(1, 13))
    f = plan.fields()
    assert (f["planned_weight_blocks"], f["planned_gpu_resident_blocks"], f["planned_gpu_staged_blocks"],
            f["planned_weight_bytes"], f["planned_gpu_resident_weight_bytes"], f["planned_gpu_staged_weight_bytes"],
            f["planned_weight_descriptor_count"]) == (12, 6, 6, 100, 52, 48, 12)
    packed = b"".join(struct.pack("<QQQQI", b.block_id, b.block_version, b.offset_bytes, b.bytes, b.strategy)
                      for b in plan.blocks)
    assert plan.descriptor_hash == O.fnv1a(np.frombuffer(packed, np.uint8)) == f["planned_weight_descriptor_hash"]
    assert N.hash_weight_blocks([]) == 0xCBF29CE484222325
    # blocks cut across tensors: even sizes, gapless, the last one shorter
    cut = N.WeightPlan.from_weights(weights, block_bytes=14)
    assert [b.bytes for b in cut.blocks] == [14] * 7 + [2] and cut.fields()["planned_weight_bytes"] == 100
    assert all(b.offset_bytes == 14 * i for i, b in enumerate(cut.blocks))


def test_incomplete_weight_plan_is_refused_before_the_device(lib):
    """session_api_lifecycle.inc.cu:48-55: a declared plan needs one descriptor per block and a hash;
    refused as an invalid request (hip_error 0), with or without a GPU."""
    req, layer, z = _tiny_request()
    cres = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    block = (abi.NervaHipHfDecodeSequenceWeightBlock * 1)()
    block[0].host_source, block[0].bytes, block[0].strategy, block[0].block_id = z.ctypes.data, 100, 1, 1
    cases = [dict(planned_weight_blocks=1),                                                     # no byte total
             dict(planned_weight_bytes=100),                                                    # no block count
             dict(planned_weight_blocks=1, planned_weight_bytes=100, planned_weight_descriptor_hash=7),   # no descriptors
             dict(planned_weight_blocks=2, planned_weight_bytes=100, planned_weight_descriptor_hash=7,
                  planned_weight_descriptors=block, planned_weight_descriptor_count=1),         # count != blocks
             dict(planned_weight_blocks=1, planned_weight_bytes=100, planned_weight_descriptors=block,
                  planned_weight_descriptor_count=1)]                                           # no hash
    for fields in cases:
        req, layer, z = _tiny_request()
        for name, value in fields.items():
            setattr(req, name, value)
        assert lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(cres), C.byref(handle)) == -1, fields
        assert cres.status == -1 and cres.hip_error == 0 and cres.failure_stage == 1


def test_batch_step_over_nothing_and_null_fork_need_no_device(lib):
    """decode_sequence_session.rs:61-86: a batch step over no sessions answers "no_sessions" with
    status 0 on any machine; null requests fail closed."""
    import nerva_amd as N
    rc, res, tokens = N.DecodeSession.batch_advance_one([], 8, 2)
    assert rc == 0 and res.status == 0 and N.DecodeSession.BATCH_REASONS[res.reason] == "no_sessions"
    assert res.exact == 0 and res.requested_session_count == 0 and res.block_tokens == 0 and res.observed_tokens == 0
    assert res.target_block_tokens == 8 and res.min_block_tokens == 2 and res.hot_path_allocations == 0
    out = abi.NervaHipHfDecodeSequenceBatchAdvanceResult()
    assert lib.nerva_hip_hf_decode_sequence_batch_advance_one(None, C.byref(out)) == -1
    assert out.status == -1 and out.reason == abi.NERVA_HIP_BATCH_INVALID_REQUEST
    assert lib.nerva_hip_hf_decode_sequence_batch_advance_one(None, None) == -1
    cres = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    req = abi.NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest()
    assert lib.nerva_hip_hf_decode_sequence_session_fork_shared_weights(C.byref(req), C.byref(cres), C.byref(handle)) == -1
    assert cres.status == -1 and cres.failure_stage == 1 and not handle
    assert lib.nerva_hip_hf_decode_sequence_session_fork_shared_weights(None, C.byref(cres), C.byref(handle)) == -1
    assert lib.nerva_hip_session_shares_weight_stream(None) == -1


def test_operand_order_index_is_the_matrix_core_operand_layout(lib):
    """nerva_hip_gemm_operand_index (host arithmetic): per 32 columns and 16 tokens, 64 pieces of 8
    columns in lane order, lane = (column % 32 / 8) * 16 + token % 16 - the B operand of a 16x16x32
    matrix-core product; 2 token tiles per K-step up to 32 tokens, 4 up to 64, 8 above; a bijection onto the buffer."""
    f = lib.nerva_hip_gemm_operand_index
    for tokens, tiles in ((1, 2), (32, 2), (33, 4), (64, 4), (65, 8), (128, 8)):
        cols = 96
        seen = set()
        for t in range(tiles * 16):
            for k in range(cols):
                i = f(tokens, t, k)
                lane = (k % 32 // 8) * 16 + t % 16
                assert i == ((k // 32) * tiles + t // 16) * 512 + lane * 8 + k % 8
                seen.add(i)
        assert seen == set(range(tiles * 16 * cols))


def test_profiled_processes_never_replay_graphs():
    """A process started by the ROCm profiler carries its tool library and settings in the
    environment; such a process must launch its steps kernel by kernel (a traced hipGraphLaunch
    took the process down on this stack). Decided at the first call, so each case is a process."""
    import subprocess
    import sys
    code = "import nerva_amd.abi as a; print(a.load().nerva_hip_steps_are_eager())"
    cases = [({}, "0"), ({"NERVA_HIP_EAGER_STEPS": "1"}, "1"), ({"ROCP_TOOL_LIBRARIES": ""}, "1"),
             ({"ROCPROF_KERNEL_TRACE": "1"}, "1"), ({"ROCPROF_OUTPUT_PATH": "/tmp/x"}, "1")]
    for extra, want in cases:
        env = {k: v for k, v in os.environ.items() if not k.startswith(("ROCPROF", "ROCP_", "NERVA_HIP_"))}
        env.update(extra)
        out = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, capture_output=True, text=True)
        assert out.returncode == 0 and out.stdout.strip() == want, (extra, out.stdout, out.stderr)


def test_launch_shape_and_tuning_hooks_are_host_arithmetic():
    """The GEMV launch shape is decided on the host (measurements are keyed to it), and launch-shape
    overrides go through a named hook, not through the environment."""
    import nerva_amd as N
    # the decode step's launches at Qwen3-8B widths: every one the lean kernel
    assert N.gemv_launch_shape(1, 2, 12288, 4096) == (3, 2048)     # gate_up: oversubscribed long launch
    assert N.gemv_launch_shape(1, 0, 6144, 4096) == (3, 1024)      # qkv: rotated walk, four workgroups a CU
    assert N.gemv_launch_shape(1, 0, 8192, 8192) == (3, 1024)      # another width: two rows per wave in one round
    assert N.gemv_launch_shape(0, 1, 4096, 4096) == (3, 1024)      # o: every row on the machine at once
    assert N.gemv_launch_shape(1, 4, 151936, 4096) == (3, 512)     # LM head: 16-wave workgroups
    assert N.gemv_launch_shape(0, 0, 100, 520)[0] == 1             # 520 columns: the guarded vector kernel
    # other models' widths on the lean kernel: batches of 1024 columns, rows of up to 30720 columns with a 16-bit input
    for pro, epi, rows, cols in ((0, 1, 4096, 14336), (0, 1, 5120, 25600), (1, 0, 10240, 5120), (0, 1, 8192, 28672),
                                 (1, 2, 25600, 5120), (1, 0, 8192, 8192)):
        assert N.gemv_launch_shape(pro, epi, rows, cols)[0] == 3, (pro, epi, rows, cols)
    assert N.gemv_launch_shape(0, 1, 64, 31744)[0] == 2           # past the limit: the general vector kernel
    assert N.gemv_launch_shape(1, 0, 64, 13312)[0] == 2           # the RMSNorm prologue keeps its 12288-column limit
    with pytest.raises(ValueError):
        N.gemv_launch_shape(0, 0, 0, 64)
    for name in ("attn_splits", "batch_splits", "prompt_splits", "gemm_row_tiles", "gemm_k_waves",
                 "gemm_block_slices", "gemm_block_row_tiles", "gemm_block_min_tokens", "gemv_exact_start",
                 "moe_down_shared_first", "gemv_workgroup_waves", "gemv_x_registers", "prefill_block_tokens",
                 "gemv_rotated_walk", "attn_merge_spin_limit", "attn_withhold_split", "block_layout",
                 "prefill_attention_rows", "prefill_walk", "gemm_block_off", "gemm_block_waves", "gemm_block_rotate"):
        N.Device.set_tuning(name, 2)
        N.Device.set_tuning(name, 0)
    with pytest.raises(ValueError):
        N.Device.set_tuning("NERVA_HIP_ATTN_SPLITS", 2)
    csrc = os.path.join(ROOT, "nerva_amd", "csrc")
    src = "".join(open(os.path.join(csrc, f)).read() for f in os.listdir(csrc) if f.endswith((".hip", ".cuh", ".hpp")))
    for knob in ("_SPLITS", "_ROW_TILES", "_K_WAVES", "_SLICES", "_MIN_TOKENS", "_PREFILL", "_PREFILL_ATTN", "_BLOCK_LAYOUT",
                 "_GEMM_BLOCK", "_SPLIT_ARENAS"):
        assert knob + '")' not in src, knob    # no getenv("NERVA_HIP_..._SPLITS") and the like
    N.Device.set_tuning("prefill_walk", 1)
    N.Device.reset_tuning()                     # a null name switches every override off


def test_build_refuses_register_spills_in_kernels_that_issue_loads_by_hand():
    """The build reads hipcc's resource-usage remarks: a kernel that requests data with inline-assembly loads
    must not use scratch memory (a spilled register may still be receiving its data)."""
    from nerva_amd import build
    remarks = "\n".join([
        "a.hip:1:1: remark: Function Name: _ZN2nv12_GLOBAL__N_120moe_down_lean_kernelILi2EEEvNS_12MoeFp8ParamsE [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:1:1: remark:     VGPRs: 96 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:1:1: remark:     ScratchSize [bytes/lane]: 128 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:2:1: remark: Function Name: _ZN2nv16gemv_fast_kernelILj1ELi1ELi4ELi1ELi4ELb0ELi16ELb0EEEvNS_10GemvParamsE [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:2:1: remark:     ScratchSize [bytes/lane]: 8 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:3:1: remark: Function Name: _ZN2nv12_GLOBAL__N_116attn_step_kernelILj1ELi4EEEvNS_10AttnParamsE [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:3:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]",
    ])
    spilling = build._spilling_kernels(remarks)
    assert [s.split(" ")[0] for s in spilling] == [
        "_ZN2nv12_GLOBAL__N_120moe_down_lean_kernelILi2EEEvNS_12MoeFp8ParamsE",
        "_ZN2nv16gemv_fast_kernelILj1ELi1ELi4ELi1ELi4ELb0ELi16ELb0EEEvNS_10GemvParamsE"]
    guarded = [s for s in spilling if any(name in s for name in build.HAND_ISSUED_LOADS)]
    assert len(guarded) == 1 and "moe_down_lean_kernel" in guarded[0]
    # every kernel with inline-assembly loads in the sources is on the list
    import re
    csrc = os.path.join(os.path.dirname(build.__file__), "csrc")
    for name in os.listdir(csrc):
        if not name.endswith((".hip", ".cuh")):
            continue
        text = open(os.path.join(csrc, name)).read()
        if not re.search(r'asm volatile\(\s*"(global_load_|ds_read_)', text):
            continue
        kernels = re.findall(r"__global__[^;{]*?void (\w+)\(", text)
        assert any(k in build.HAND_ISSUED_LOADS for k in kernels), name
