"""numpy <-> device plumbing over the C ABI (no torch: the library owns its HIP runtime)."""
import ctypes as C

import numpy as np

from . import abi

F16, BF16 = 0, 1


def device_available():
    """True when libnerva_hip.so loads and reports a usable GPU."""
    lib = abi.load()
    res = abi.NervaHipDeviceSmokeResult()
    return lib.nerva_hip_device_smoke(C.byref(res)) == 0


class Device:
    @staticmethod
    def smoke():
        res = abi.NervaHipDeviceSmokeResult()
        rc = abi.load().nerva_hip_device_smoke(C.byref(res))
        return rc, res

    @staticmethod
    def synchronize():
        if abi.load().nerva_hip_stream_synchronize(None) != 0:
            raise RuntimeError("stream synchronize failed")

    @staticmethod
    def allocation_count():
        return int(abi.load().nerva_hip_allocation_count())

    @staticmethod
    def set_tuning(name, value):
        """Overrides one launch-shape choice for the process (0 restores the built-in one): a hook for
        measurements and tests, see nerva_hip_test_set_tuning."""
        if abi.load().nerva_hip_test_set_tuning(name.encode(), int(value)) != 0:
            raise ValueError("unknown tuning name %r" % name)

    @staticmethod
    def reset_tuning():
        """Every override off: the library's built-in launch shapes and modes."""
        abi.load().nerva_hip_test_set_tuning(None, 0)

    @staticmethod
    def steps_are_eager():
        """True when sessions launch a step's kernels one by one instead of replaying the captured
        graph: asked for through NERVA_HIP_EAGER_STEPS=1, or forced because a profiler is attached."""
        return bool(abi.load().nerva_hip_steps_are_eager())

    @staticmethod
    def copy(dst, src, nbytes):
        """Plain device copy kernel of a known size (memory-counter calibration)."""
        if abi.load().nerva_hip_copy_d2d(dst.ptr, src.ptr, nbytes, None) != 0:
            raise RuntimeError("copy_d2d failed")


class DeviceBuffer:
    """A device allocation made through nerva_hip_malloc."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        ptr = C.c_void_p()
        if abi.load().nerva_hip_malloc(C.byref(ptr), self.nbytes) != 0 or not ptr.value:
            raise MemoryError("nerva_hip_malloc(%d) failed" % self.nbytes)
        self.ptr = ptr.value

    @classmethod
    def from_numpy(cls, array):
        array = np.ascontiguousarray(array)
        buf = cls(max(array.nbytes, 16))
        buf.dtype, buf.shape = array.dtype, array.shape
        if array.nbytes:
            buf.upload(array)
        return buf

    @classmethod
    def zeros(cls, nbytes):
        buf = cls(nbytes)
        if abi.load().nerva_hip_memset(buf.ptr, 0, buf.nbytes) != 0:
            raise RuntimeError("memset failed")
        return buf

    def upload(self, array, offset=0):
        array = np.ascontiguousarray(array)
        assert offset + array.nbytes <= self.nbytes
        if abi.load().nerva_hip_memcpy_h2d(self.ptr + offset, array.ctypes.data, array.nbytes) != 0:
            raise RuntimeError("h2d copy failed")

    def numpy(self, dtype, count=None, offset=0):
        dtype = np.dtype(dtype)
        count = (self.nbytes - offset) // dtype.itemsize if count is None else count
        out = np.empty(count, dtype)
        if abi.load().nerva_hip_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes) != 0:
            raise RuntimeError("d2h copy failed")
        return out

    def at(self, byte_offset):
        return self.ptr + byte_offset

    def free(self):
        if getattr(self, "ptr", None):
            abi.load().nerva_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _check(rc, err, what):
    if rc != 0:
        raise RuntimeError("%s failed (hip_error=%d)" % (what, err.value))


def _ptr(buf):
    if buf is None:
        return None
    return buf.ptr if isinstance(buf, DeviceBuffer) else int(buf)


def gemv(dtype, weights, rows, cols, *, input16=None, input_f32=None, gamma=None, eps=0.0, bias=None,
         residual=None, out_f32=None, out16=None, epilogue=0, round_output=False, pair_gap=0, sync=True):
    """Launch nerva_hip_gemv on device buffers. prologue is implied by which input is given.
    pair_gap (epilogue 2): elements between the end of the gate rows and the first up row."""
    req = abi.NervaHipGemvRequest()
    req.dtype, req.rows, req.cols = dtype, rows, cols
    req.prologue = 0 if input16 is not None else 1
    req.epilogue = epilogue
    req.round_output = int(round_output)
    req.rms_eps = eps
    req.pair_gap = pair_gap
    req.weights, req.input16, req.input_f32 = _ptr(weights), _ptr(input16), _ptr(input_f32)
    req.gamma, req.bias, req.residual = _ptr(gamma), _ptr(bias), _ptr(residual)
    req.output_f32, req.output16 = _ptr(out_f32), _ptr(out16)
    err = C.c_int32(0)
    _check(abi.load().nerva_hip_gemv(C.byref(req), None, C.byref(err)), err, "nerva_hip_gemv")
    if sync:
        Device.synchronize()


def gemv_launch_plan(prologue, epilogue, rows, cols):
    """(kernel variant, workgroups, rotated walk, 1 KiB chunks per request batch) of the launch nerva_hip_gemv
    chooses for these sizes (host arithmetic)."""
    kernel, groups = C.c_uint32(0), C.c_uint32(0)
    if abi.load().nerva_hip_gemv_launch_shape(prologue, epilogue, rows, cols, C.byref(kernel), C.byref(groups)) != 0:
        raise ValueError("no launch shape for these sizes")
    return int(kernel.value) & 15, int(groups.value), bool(kernel.value & 16), int(kernel.value) >> 8


def gemv_launch_shape(prologue, epilogue, rows, cols):
    """(kernel variant, workgroups) of that launch."""
    return gemv_launch_plan(prologue, epilogue, rows, cols)[:2]


def fp8_gemv(weights, scales, rows, cols, block_rows, block_cols, out, *, input16=None, input_f32=None,
             input_dtype=BF16, sync=True):
    req = abi.NervaHipFp8GemvRequest()
    req.rows, req.cols, req.block_rows, req.block_cols = rows, cols, block_rows, block_cols
    req.input_dtype = input_dtype
    req.weights, req.scales = _ptr(weights), _ptr(scales)
    req.input16, req.input_f32, req.output = _ptr(input16), _ptr(input_f32), _ptr(out)
    err = C.c_int32(0)
    _check(abi.load().nerva_hip_fp8_gemv(C.byref(req), None, C.byref(err)), err, "nerva_hip_fp8_gemv")
    if sync:
        Device.synchronize()


class PagedKvCache:
    """K/V arrays in the library's layout [layer][block][kv_head][16-token tile] + a block table."""

    def __init__(self, layers, block_count, kv_heads, head_dim, table=None):
        self.layers, self.block_count, self.kv_heads, self.head_dim = layers, block_count, kv_heads, head_dim
        self.elems = layers * block_count * kv_heads * 16 * head_dim
        self.k = DeviceBuffer.zeros(self.elems * 2)
        self.v = DeviceBuffer.zeros(self.elems * 2)
        table = np.arange(block_count, dtype=np.uint32) if table is None else np.asarray(table, np.uint32)
        self.table_host = table
        self.table = DeviceBuffer.from_numpy(table)

    def tile_offset(self, layer, token, kv_head):
        """Element offset of the (block, kv_head) tile that holds `token`."""
        lib = abi.load()
        return int(lib.nerva_hip_kv_cache_offset(self.block_count, self.kv_heads, self.head_dim, layer,
                                                 int(self.table_host[token // 16]), kv_head, 0, 0, 0))

    def _tile_maps(self):
        """In-tile element index of (row, dim) for K and V, as the library lays tiles out."""
        if getattr(self, "_maps", None) is None:
            lib = abi.load()
            hd = self.head_dim
            kmap = np.empty((16, hd), np.int64)
            vmap = np.empty((16, hd), np.int64)
            for row in range(16):
                for d in range(hd):
                    kmap[row, d] = lib.nerva_hip_kv_cache_offset(1, 1, hd, 0, 0, 0, row, d, 0)
                    vmap[row, d] = lib.nerva_hip_kv_cache_offset(1, 1, hd, 0, 0, 0, row, d, 1)
            assert sorted(kmap.ravel()) == list(range(16 * hd)) and sorted(vmap.ravel()) == list(range(16 * hd))
            self._maps = (kmap, vmap)
        return self._maps

    def host_layout(self, layer, k_rows, v_rows):
        """Scatter [tokens, kv_heads*head_dim] 16-bit rows into host images of the cache arrays."""
        kimg = np.zeros(self.elems, np.uint16)
        vimg = np.zeros(self.elems, np.uint16)
        kmap, vmap = self._tile_maps()
        tokens = k_rows.shape[0]
        hd = self.head_dim
        for t in range(tokens):
            for h in range(self.kv_heads):
                o = self.tile_offset(layer, t, h)
                kimg[o + kmap[t % 16]] = k_rows[t, h * hd:(h + 1) * hd]
                vimg[o + vmap[t % 16]] = v_rows[t, h * hd:(h + 1) * hd]
        return kimg, vimg

    def fill(self, layer, k_rows, v_rows):
        kimg, vimg = self.host_layout(layer, k_rows, v_rows)
        self.k.upload(kimg)
        self.v.upload(vimg)

    def read_row(self, layer, token):
        hd = self.head_dim
        kmap, vmap = self._tile_maps()
        k = np.empty(self.kv_heads * hd, np.uint16)
        v = np.empty(self.kv_heads * hd, np.uint16)
        for h in range(self.kv_heads):
            o = self.tile_offset(layer, token, h)
            ktile = self.k.numpy(np.uint16, 16 * hd, o * 2)
            vtile = self.v.numpy(np.uint16, 16 * hd, o * 2)
            k[h * hd:(h + 1) * hd] = ktile[kmap[token % 16]]
            v[h * hd:(h + 1) * hd] = vtile[vmap[token % 16]]
        return k, v


def paged_attention(dtype, heads, kv_heads, head_dim, cache, layer, position, qkv_f32, workspace, out16,
                    *, out_f32=None, append=True, eps=1e-6, rope_theta=0.0, q_norm=None, k_norm=None,
                    q_bias=None, k_bias=None, v_bias=None, sync=True, splits=0):
    req = abi.NervaHipPagedAttentionRequest()
    req.splits = splits
    req.dtype, req.heads, req.kv_heads, req.head_dim = dtype, heads, kv_heads, head_dim
    req.layer, req.block_count, req.position, req.append = layer, cache.block_count, position, int(append)
    req.rms_eps, req.rope_theta = eps, rope_theta
    req.qkv_f32 = _ptr(qkv_f32)
    req.q_norm, req.k_norm = _ptr(q_norm), _ptr(k_norm)
    req.q_bias, req.k_bias, req.v_bias = _ptr(q_bias), _ptr(k_bias), _ptr(v_bias)
    req.k_cache, req.v_cache, req.block_table = cache.k.ptr, cache.v.ptr, cache.table.ptr
    req.workspace, req.output_f32, req.output16 = _ptr(workspace), _ptr(out_f32), _ptr(out16)
    err = C.c_int32(0)
    _check(abi.load().nerva_hip_paged_gqa_decode(C.byref(req), None, C.byref(err)), err,
           "nerva_hip_paged_gqa_decode")
    if sync:
        Device.synchronize()


def attention_workspace(heads, head_dim):
    return DeviceBuffer.zeros(abi.load().nerva_hip_paged_attention_workspace_bytes(heads, head_dim))


def paged_attention_status(workspace, heads, head_dim):
    """(rc, hip_error) of nerva_hip_paged_attention_status: synchronises, then (0, 0), or (-1, NERVA_HIP_ERROR_STEP_FAULT)
    when a launch on this workspace gave up waiting for a split's partial (the report is cleared by the call)."""
    err = C.c_int32(0)
    rc = abi.load().nerva_hip_paged_attention_status(_ptr(workspace), heads, head_dim, None, C.byref(err))
    return rc, int(err.value)


def argmax(logits_buf, count, workspace=None):
    lib = abi.load()
    ws = workspace or DeviceBuffer.zeros(lib.nerva_hip_argmax_workspace_bytes())
    tok = DeviceBuffer.zeros(16)
    req = abi.NervaHipArgmaxRequest()
    req.count, req.logits, req.token, req.workspace = count, _ptr(logits_buf), tok.ptr, ws.ptr
    err = C.c_int32(0)
    _check(lib.nerva_hip_argmax(C.byref(req), None, C.byref(err)), err, "nerva_hip_argmax")
    Device.synchronize()
    return int(tok.numpy(np.uint32, 1)[0])


def argmax_static(logits_buf, count, token_buf):
    """nerva_hip_argmax_static: launches only, no allocation inside the library; the caller owns the
    logits and the token word. Returns (rc, hip_error); synchronises when rc == 0."""
    err = C.c_int32(0)
    rc = abi.load().nerva_hip_argmax_static(_ptr(logits_buf), count, _ptr(token_buf), None, C.byref(err))
    if rc == 0:
        Device.synchronize()
    return rc, err.value


def gemm_operand_slots(tokens):
    """Token slots of a buffer in matrix-operand order for a block of `tokens` rows."""
    return 32 if tokens <= 32 else 64 if tokens <= 64 else 128 if tokens <= 128 else 256 if tokens <= 256 else 512


def gemm_operand_order(x, tokens=None):
    """A [tokens][cols] block of 16-bit rows rearranged into the matrix-operand order the multi-row GEMM
    reads fastest (index of every element from the library); slots past `tokens` stay zero."""
    lib = abi.load()
    x = np.ascontiguousarray(x, np.uint16)
    tokens = x.shape[0] if tokens is None else tokens
    cols = x.shape[1]
    out = np.zeros(gemm_operand_slots(tokens) * cols, np.uint16)
    t, k = np.meshgrid(np.arange(tokens), np.arange(cols), indexing="ij")
    # the index is affine in (token % 16, token // 16) and in the column's three digits: probe it once per digit
    base = lambda tt, kk: int(lib.nerva_hip_gemm_operand_index(tokens, tt, kk))
    idx = (np.array([base(i, 0) for i in range(tokens)])[t]
           + np.array([base(0, j) for j in range(cols)])[k])
    out[idx] = x[:tokens]
    return out, idx


def gemm_rows(dtype, weights, rows, cols, tokens, input16, epilogue=0, bias=None, residual=None, out_f32=None,
              out16=None, round_output=False, sync=True, input_operand_order=False, output16_operand_order=False,
              workspace=None):
    """Y[t] = W . X[t] for up to 128 token rows on the matrix cores (weights streamed once); up to 256 rows
    with the input in operand order where the kernel for wide blocks takes the shape (rows a multiple of 128,
    gate/up pairs of 64, cols of 512); up to 512 where the kernel with 256 (or 192) x 256 workgroup tiles does
    (rows a multiple of 192 or 256, gate/up pairs of 96 or 128, cols of 128).
    `workspace`: optional DeviceBuffer of gemm_rows_workspace_bytes(rows) for the K-sliced large-block kernels."""
    lib = abi.load()
    req = abi.NervaHipGemmRowsRequest()
    if workspace is not None:
        req.workspace, req.workspace_bytes = workspace.ptr, workspace.nbytes
    req.input_operand_order, req.output16_operand_order = int(input_operand_order), int(output16_operand_order)
    req.dtype, req.rows, req.cols, req.tokens, req.epilogue, req.round_output = dtype, rows, cols, tokens, epilogue, int(round_output)
    req.weights, req.input16, req.bias, req.residual = _ptr(weights), _ptr(input16), _ptr(bias), _ptr(residual)
    req.output_f32, req.output16 = _ptr(out_f32), _ptr(out16)
    err = C.c_int32(0)
    _check(lib.nerva_hip_gemm_rows(C.byref(req), None, C.byref(err)), err, "nerva_hip_gemm_rows")
    if sync:
        Device.synchronize()


def gemm_rows_workspace_bytes(rows):
    lib = abi.load()
    lib.nerva_hip_gemm_rows_workspace_bytes.restype = C.c_uint64
    return int(lib.nerva_hip_gemm_rows_workspace_bytes(C.c_uint32(rows)))


def sample(logits_buf, vocab, temperature, top_p, top_k, seed, position, workspace=None):
    """One token from device logits by the session's sampler rule (greedy / Gumbel-max / top-k + top-p)."""
    lib = abi.load()
    ws = workspace or DeviceBuffer.zeros(lib.nerva_hip_sample_workspace_bytes(vocab))
    tok = DeviceBuffer.zeros(16)
    req = abi.NervaHipSampleRequest()
    req.vocab, req.position, req.logits, req.token, req.workspace = vocab, position, _ptr(logits_buf), tok.ptr, ws.ptr
    req.sampler.temperature, req.sampler.top_p, req.sampler.top_k, req.sampler.seed = temperature, top_p, top_k, seed
    err = C.c_int32(0)
    _check(lib.nerva_hip_sample(C.byref(req), None, C.byref(err)), err, "nerva_hip_sample")
    Device.synchronize()
    return int(tok.numpy(np.uint32, 1)[0])


def moe_route_softmax(logits, top_k, normalize=True):
    logits = np.ascontiguousarray(logits, np.float32)
    dl = DeviceBuffer.from_numpy(logits)
    ids = DeviceBuffer.zeros(max(16, top_k * 4))
    wts = DeviceBuffer.zeros(max(16, top_k * 4))
    req = abi.NervaHipMoeRouteRequest()
    req.num_experts, req.top_k, req.normalize = logits.size, top_k, int(normalize)
    req.logits, req.expert_ids, req.expert_weights = dl.ptr, ids.ptr, wts.ptr
    err = C.c_int32(0)
    _check(abi.load().nerva_hip_moe_route_softmax(C.byref(req), None, C.byref(err)), err,
           "nerva_hip_moe_route_softmax")
    Device.synchronize()
    return ids.numpy(np.uint32, top_k), wts.numpy(np.float32, top_k), ids, wts


def moe_fp8_experts(hidden, inter, num_experts, top_k, block, x16, ids, weights, w_gate, s_gate, w_up,
                    s_up, w_down, s_down, act, out, *, shared_index=-1, input_dtype=BF16, sync=True, phases=0):
    req = abi.NervaHipMoeFp8Request()
    req.phases = phases
    req.hidden, req.intermediate, req.num_experts, req.top_k = hidden, inter, num_experts, top_k
    req.block, req.input_dtype, req.shared_index = block, input_dtype, shared_index
    req.input16, req.expert_ids, req.expert_weights = _ptr(x16), _ptr(ids), _ptr(weights)
    req.w_gate, req.w_up, req.w_down = _ptr(w_gate), _ptr(w_up), _ptr(w_down)
    req.s_gate, req.s_up, req.s_down = _ptr(s_gate), _ptr(s_up), _ptr(s_down)
    req.activation, req.output = _ptr(act), _ptr(out)
    err = C.c_int32(0)
    _check(abi.load().nerva_hip_moe_fp8_experts(C.byref(req), None, C.byref(err)), err,
           "nerva_hip_moe_fp8_experts")
    if sync:
        Device.synchronize()
