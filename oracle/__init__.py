"""ctypes binding of the CPU oracle (oracle/libnerva_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py. The shipped package (nerva_amd) never imports
this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libnerva_oracle.so")

F16, BF16 = 0, 1


def build(force=False):
    """Compile the oracle with g++ (oracle/Makefile)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


lib = _load()

u8p, u16p, u32p, u64p, f32p = (C.POINTER(t) for t in (C.c_uint8, C.c_uint16, C.c_uint32, C.c_uint64, C.c_float))


def _p(a, t):
    return a.ctypes.data_as(t) if a is not None else None


class NvoLayer(C.Structure):
    _fields_ = [(n, u16p) for n in (
        "rms_attn", "rms_mlp", "w_q", "w_k", "w_v", "w_o", "q_norm", "k_norm",
        "q_bias", "k_bias", "v_bias", "o_bias", "w_gate", "w_up", "w_down")]


class NvoModel(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "dtype", "hidden", "heads", "kv_heads", "head_dim", "intermediate", "vocab", "layers")] + [
        ("rms_eps", C.c_float), ("rope_theta", C.c_float),
        ("embeddings", u16p), ("layer", C.POINTER(NvoLayer)), ("final_norm", u16p), ("lm_head", u16p)]


def _sig(name, res, *args):
    f = getattr(lib, name)
    f.restype = res
    f.argtypes = list(args)
    return f


_sig("nvo_bf16_to_f32", C.c_float, C.c_uint16)
_sig("nvo_f32_to_bf16", C.c_uint16, C.c_float)
_sig("nvo_f16_to_f32", C.c_float, C.c_uint16)
_sig("nvo_f32_to_f16", C.c_uint16, C.c_float)
_sig("nvo_fp8_e4m3fn_to_f32", C.c_float, C.c_uint8)
_sig("nvo_f32_to_fp8_e4m3fn", C.c_uint8, C.c_float)
_sig("nvo_e8m0_to_f32", C.c_float, C.c_uint8)
_sig("nvo_silu", C.c_float, C.c_float)
_sig("nvo_encode16", None, C.c_uint32, f32p, u16p, C.c_uint64)
_sig("nvo_decode16", None, C.c_uint32, u16p, f32p, C.c_uint64)
_sig("nvo_encode_fp8", None, f32p, u8p, C.c_uint64)
_sig("nvo_decode_fp8", None, u8p, f32p, C.c_uint64)
_sig("nvo_fnv1a", C.c_uint64, u8p, C.c_uint64)
_sig("nvo_gemv_encoded", None, C.c_uint32, u16p, C.c_uint64, C.c_uint64, f32p, f32p)
_sig("nvo_gemv_encoded_mt", None, C.c_uint32, u16p, C.c_uint64, C.c_uint64, f32p, f32p)
_sig("nvo_gemv_encoded_x16", None, C.c_uint32, u16p, C.c_uint64, C.c_uint64, u16p, f32p)
_sig("nvo_fp8_f32_scale_gemm_tokens", None, u8p, f32p, u16p, C.c_uint32, C.c_uint64, C.c_uint64,
     C.c_uint64, C.c_uint64, C.c_uint64, f32p)
_sig("nvo_rms_norm_encoded", None, C.c_uint32, f32p, u16p, C.c_uint64, C.c_float, f32p)
_sig("nvo_per_head_rms_norm", None, C.c_uint32, u16p, C.c_uint64, f32p, C.c_uint64, C.c_float)
_sig("nvo_rope", None, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float, f32p)
_sig("nvo_attention_blockwise", C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, f32p,
     C.POINTER(f32p), C.POINTER(f32p), u64p, C.c_uint64, f32p)
_sig("nvo_attention_paged16", C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32,
     f32p, u16p, u16p, u32p, C.c_uint64, C.c_uint64, C.c_uint64, f32p)
_sig("nvo_greedy_argmax", C.c_int, f32p, C.c_uint64, C.c_int, u32p)
_sig("nvo_sampler_mix64", C.c_uint64, C.c_uint64)
_sig("nvo_sampler_uniform", C.c_float, C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32)
_sig("nvo_sample", C.c_int, f32p, C.c_uint32, C.c_float, C.c_float, C.c_uint32, C.c_uint64, C.c_uint32, u32p, f32p)
_sig("nvo_moe_route_softmax", C.c_int, f32p, C.c_uint32, C.c_uint32, C.c_uint32, u32p, f32p)
_sig("nvo_moe_forward_f32", C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32,
     C.c_float, f32p, u32p, f32p, f32p, f32p, f32p, C.c_uint32, f32p, f32p, f32p, f32p)
_sig("nvo_moe_fp8_forward", C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32,
     C.c_uint32, u16p, u32p, f32p, u8p, f32p, u8p, f32p, u8p, f32p, C.c_int32, C.c_int, f32p)
_sig("nvo_ctx_create", C.c_void_p, C.POINTER(NvoModel), C.c_uint64, C.c_int, C.c_int)
_sig("nvo_ctx_destroy", None, C.c_void_p)
_sig("nvo_ctx_reset", None, C.c_void_p)
_sig("nvo_ctx_len", C.c_uint64, C.c_void_p)
_sig("nvo_ctx_logits", f32p, C.c_void_p)
_sig("nvo_ctx_load_kv16", C.c_int, C.c_void_p, C.c_uint32, u16p, u16p, C.c_uint64)
_sig("nvo_ctx_set_len", None, C.c_void_p, C.c_uint64)
_sig("nvo_ctx_read_kv16", C.c_int, C.c_void_p, C.c_uint32, C.c_uint64, u16p, u16p)
_sig("nvo_ctx_forward_token", C.c_int, C.c_void_p, C.c_uint32, C.c_int, C.c_int, f32p)
_sig("nvo_greedy_decode", C.c_int, C.c_void_p, u32p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32,
     u32p, f32p)
_sig("nvo_block_forward", C.c_int, C.POINTER(NvoModel), u16p, C.c_uint64, C.c_int, u16p)
_sig("nvo_synth_f32", None, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float, C.c_float, f32p)
_sig("nvo_synth_16", None, C.c_uint32, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float,
     C.c_float, u16p)
_sig("nvo_synth_tokens", None, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint32, u32p)
_sig("nvo_synth_fp8_block", None, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64,
     C.c_float, u8p, f32p)


# ---- numpy conveniences ---------------------------------------------------

def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u16(a):
    return np.ascontiguousarray(a, dtype=np.uint16)


def encode16(dtype, values):
    v = _f32(values).ravel()
    out = np.empty(v.size, np.uint16)
    lib.nvo_encode16(dtype, _p(v, f32p), _p(out, u16p), v.size)
    return out.reshape(np.shape(values))


def decode16(dtype, bits):
    b = _u16(bits).ravel()
    out = np.empty(b.size, np.float32)
    lib.nvo_decode16(dtype, _p(b, u16p), _p(out, f32p), b.size)
    return out.reshape(np.shape(bits))


def encode_fp8(values):
    v = _f32(values).ravel()
    out = np.empty(v.size, np.uint8)
    lib.nvo_encode_fp8(_p(v, f32p), _p(out, u8p), v.size)
    return out.reshape(np.shape(values))


def decode_fp8(bits):
    b = np.ascontiguousarray(bits, dtype=np.uint8).ravel()
    out = np.empty(b.size, np.float32)
    lib.nvo_decode_fp8(_p(b, u8p), _p(out, f32p), b.size)
    return out.reshape(np.shape(bits))


def fnv1a(array):
    b = np.ascontiguousarray(array).view(np.uint8).ravel()
    return int(lib.nvo_fnv1a(_p(b, u8p), b.size))


def gemv(dtype, w, x, threads=1):
    """y = W.x with f32 x (reference CPU contract)."""
    w = _u16(w)
    x = _f32(x)
    rows, cols = w.shape
    y = np.empty(rows, np.float32)
    f = lib.nvo_gemv_encoded_mt if threads > 1 else lib.nvo_gemv_encoded
    f(dtype, _p(w, u16p), rows, cols, _p(x, f32p), _p(y, f32p))
    return y


def gemv_x16(dtype, w, x16):
    w = _u16(w)
    x16 = _u16(x16)
    rows, cols = w.shape
    y = np.empty(rows, np.float32)
    lib.nvo_gemv_encoded_x16(dtype, _p(w, u16p), rows, cols, _p(x16, u16p), _p(y, f32p))
    return y


def fp8_gemm_tokens(w, scales, x16, rows, cols, tokens, block_rows, block_cols, input_dtype=BF16):
    w = np.ascontiguousarray(w, np.uint8)
    scales = _f32(scales)
    x16 = _u16(x16)
    out = np.empty(tokens * rows, np.float32)
    lib.nvo_fp8_f32_scale_gemm_tokens(_p(w, u8p), _p(scales, f32p), _p(x16, u16p), input_dtype, rows,
                                      cols, tokens, block_rows, block_cols, _p(out, f32p))
    return out.reshape(tokens, rows)


def rms_norm(dtype, x, gamma16, eps):
    x = _f32(x)
    g = _u16(gamma16)
    out = np.empty_like(x)
    lib.nvo_rms_norm_encoded(dtype, _p(x, f32p), _p(g, u16p), x.size, eps, _p(out, f32p))
    return out


def per_head_rms_norm(dtype, gamma16, head_dim, values, eps):
    v = _f32(values).copy()
    g = _u16(gamma16)
    lib.nvo_per_head_rms_norm(dtype, _p(g, u16p), head_dim, _p(v, f32p), v.size, eps)
    return v


def rope(head_dim, heads, position, theta, values):
    v = _f32(values).copy()
    lib.nvo_rope(head_dim, heads, position, theta, _p(v, f32p))
    return v


def attention_blockwise(heads, kv_heads, head_dim, q, blocks):
    """blocks: list of (keys[t, kv_hidden], values[t, kv_hidden]) f32 arrays."""
    q = _f32(q)
    ks = [_f32(k) for k, _ in blocks]
    vs = [_f32(v) for _, v in blocks]
    n = len(blocks)
    kp = (f32p * n)(*[_p(k, f32p) for k in ks])
    vp = (f32p * n)(*[_p(v, f32p) for v in vs])
    counts = np.array([k.shape[0] if k.size else 0 for k in ks], np.uint64)
    out = np.empty(heads * head_dim, np.float32)
    rc = lib.nvo_attention_blockwise(heads, kv_heads, head_dim, _p(q, f32p), kp, vp,
                                     _p(counts, u64p), n, _p(out, f32p))
    if rc != 0:
        raise ValueError("blockwise attention rejected the input")
    return out


def attention_paged16(dtype, heads, kv_heads, head_dim, block_tokens, q, kcache, vcache, table,
                      layer, n_blocks, kv_tokens):
    q = _f32(q)
    kcache = _u16(kcache)
    vcache = _u16(vcache)
    table = np.ascontiguousarray(table, np.uint32)
    out = np.empty(heads * head_dim, np.float32)
    rc = lib.nvo_attention_paged16(dtype, heads, kv_heads, head_dim, block_tokens, _p(q, f32p),
                                   _p(kcache, u16p), _p(vcache, u16p), _p(table, u32p), layer,
                                   n_blocks, kv_tokens, _p(out, f32p))
    if rc != 0:
        raise ValueError("paged attention rejected the input")
    return out


def greedy_argmax(logits, skip_nonfinite=False):
    l = _f32(logits)
    out = C.c_uint32(0)
    rc = lib.nvo_greedy_argmax(_p(l, f32p), l.size, int(skip_nonfinite), C.byref(out))
    if rc != 0:
        raise ValueError("greedy argmax rejected the logits")
    return out.value


def sampler_mix64(value):
    return int(lib.nvo_sampler_mix64(C.c_uint64(value & 0xFFFFFFFFFFFFFFFF)))


def sampler_uniform(seed, position, token, salt):
    return float(lib.nvo_sampler_uniform(C.c_uint64(seed), position, token, salt))


def sample(logits, temperature, top_p, top_k, seed, position):
    """(token, margin) of the device sampler's rule (greedy / Gumbel-max / top-k + top-p draw)."""
    l = _f32(logits)
    token, margin = C.c_uint32(0), C.c_float(0.0)
    rc = lib.nvo_sample(_p(l, f32p), l.size, temperature, top_p, top_k, C.c_uint64(seed), position,
                        C.byref(token), C.byref(margin))
    if rc != 0:
        raise ValueError("sampler rejected the logits")
    return token.value, margin.value


def moe_route_softmax(logits, top_k, normalize):
    l = _f32(logits)
    ids = np.empty(top_k, np.uint32)
    w = np.empty(top_k, np.float32)
    rc = lib.nvo_moe_route_softmax(_p(l, f32p), l.size, top_k, int(normalize), _p(ids, u32p), _p(w, f32p))
    if rc != 0:
        raise ValueError("route rejected")
    return ids, w


def moe_forward_f32(hidden, inter, x, ids, weights, w_gate, w_up, w_down, limit=None, shared=None):
    x = _f32(x)
    ids = np.ascontiguousarray(ids, np.uint32)
    weights = _f32(weights)
    w_gate, w_up, w_down = _f32(w_gate), _f32(w_up), _f32(w_down)
    num_experts = w_gate.size // (inter * hidden)
    out = np.empty(hidden, np.float32)
    if shared is not None:
        s_inter, sg, su, sd = shared
        sg, su, sd = _f32(sg), _f32(su), _f32(sd)
    else:
        s_inter, sg, su, sd = 0, None, None, None
    rc = lib.nvo_moe_forward_f32(hidden, inter, num_experts, ids.size, int(limit is not None),
                                 float(limit or 0.0), _p(x, f32p), _p(ids, u32p), _p(weights, f32p),
                                 _p(w_gate, f32p), _p(w_up, f32p), _p(w_down, f32p), s_inter,
                                 _p(sg, f32p), _p(su, f32p), _p(sd, f32p), _p(out, f32p))
    if rc != 0:
        raise ValueError("moe rejected")
    return out


def moe_fp8_forward(hidden, inter, num_experts, block, x16, ids, weights, w_gate, s_gate, w_up, s_up,
                    w_down, s_down, shared_index=-1, input_dtype=BF16):
    x16 = _u16(x16)
    ids = np.ascontiguousarray(ids, np.uint32)
    weights = _f32(weights)
    arrs = [np.ascontiguousarray(a, np.uint8) for a in (w_gate, w_up, w_down)]
    scs = [_f32(a) for a in (s_gate, s_up, s_down)]
    out = np.empty(hidden, np.float32)
    rc = lib.nvo_moe_fp8_forward(hidden, inter, num_experts, ids.size, block, input_dtype,
                                 _p(x16, u16p), _p(ids, u32p), _p(weights, f32p),
                                 _p(arrs[0], u8p), _p(scs[0], f32p), _p(arrs[1], u8p), _p(scs[1], f32p),
                                 _p(arrs[2], u8p), _p(scs[2], f32p), shared_index, 1, _p(out, f32p))
    if rc != 0:
        raise ValueError("moe fp8 rejected")
    return out


def synth_f32(seed, tensor_id, n, mean, std, offset=0):
    out = np.empty(n, np.float32)
    lib.nvo_synth_f32(seed, tensor_id, offset, n, mean, std, _p(out, f32p))
    return out


def synth_16(dtype, seed, tensor_id, n, mean, std, offset=0):
    out = np.empty(n, np.uint16)
    lib.nvo_synth_16(dtype, seed, tensor_id, offset, n, mean, std, _p(out, u16p))
    return out


def synth_tokens(seed, tensor_id, n, vocab):
    out = np.empty(n, np.uint32)
    lib.nvo_synth_tokens(seed, tensor_id, n, vocab, _p(out, u32p))
    return out


def synth_fp8_block(seed, tensor_id, rows, cols, block, std):
    w = np.empty((rows, cols), np.uint8)
    s = np.empty((-(-rows // block), -(-cols // block)), np.float32)
    lib.nvo_synth_fp8_block(seed, tensor_id, rows, cols, block, std, _p(w, u8p), _p(s, f32p))
    return w, s


class Model:
    """Host weights of a dense decoder (16-bit arrays) + the NvoModel view of them.

    layers: list of dicts with keys rms_attn, rms_mlp, w_q, w_k, w_v, w_o,
    w_gate, w_up, w_down and optional q_norm, k_norm, q_bias, k_bias, v_bias, o_bias.
    """

    def __init__(self, dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab, rms_eps,
                 rope_theta, embeddings, layers, final_norm, lm_head):
        self.dtype, self.hidden, self.heads, self.kv_heads = dtype, hidden, heads, kv_heads
        self.head_dim, self.intermediate, self.vocab = head_dim, intermediate, vocab
        self.rms_eps, self.rope_theta = rms_eps, rope_theta
        self.embeddings = _u16(embeddings)
        self.final_norm = _u16(final_norm)
        self.lm_head = _u16(lm_head)
        self.layers = [{k: (_u16(v) if v is not None else None) for k, v in l.items()} for l in layers]
        self._c_layers = (NvoLayer * len(layers))()
        for cl, l in zip(self._c_layers, self.layers):
            for name, _ in NvoLayer._fields_:
                setattr(cl, name, _p(l.get(name), u16p))
        self.c = NvoModel(dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab, len(layers),
                          rms_eps, rope_theta or 0.0, _p(self.embeddings, u16p), self._c_layers,
                          _p(self.final_norm, u16p), _p(self.lm_head, u16p))


def synthetic_model(cfg, seed, weight_std, layers=None, embedding_rows=None, threads=8, layer_ids=None):
    """Host copy of the weights nerva_hip_bench_session_create_synthetic generates on the device
    (same counter-based generator, same tensor ids), as a Model. `layers` keeps the first n layers, or
    `layer_ids` exactly those layers of the device's model (in that order);
    `embedding_rows` keeps only those rows of the embedding table (the others stay zero)."""
    import concurrent.futures
    dt, H, HD = cfg["dtype"], cfg["hidden"], cfg["head_dim"]
    A, KV, I, V = cfg["heads"] * HD, cfg["kv_heads"] * HD, cfg["intermediate"], cfg["vocab"]
    layers = cfg["layers"] if layers is None else layers

    def gen(tid, n, mean=0.0):
        chunk = 1 << 24
        out = np.empty(n, np.uint16)

        def work(start):
            m = min(chunk, n - start)
            out[start:start + m] = synth_16(dt, seed, tid, m, mean, weight_std, offset=start)
        if n <= chunk:
            work(0)
        else:
            with concurrent.futures.ThreadPoolExecutor(max_workers=threads) as pool:
                list(pool.map(work, range(0, n, chunk)))
        return out

    ls = []
    for l in (range(layers) if layer_ids is None else layer_ids):
        b = 16 * (l + 1)
        ls.append(dict(rms_attn=gen(b, H, 1.0), rms_mlp=gen(b + 1, H, 1.0), w_q=gen(b + 2, A * H).reshape(A, H),
                       w_k=gen(b + 4, KV * H).reshape(KV, H), q_norm=gen(b + 5, HD, 1.0), k_norm=gen(b + 6, HD, 1.0),
                       w_v=gen(b + 7, KV * H).reshape(KV, H), w_o=gen(b + 8, H * A).reshape(H, A),
                       w_gate=gen(b + 13, I * H).reshape(I, H), w_up=gen(b + 14, I * H).reshape(I, H),
                       w_down=gen(b + 15, H * I).reshape(H, I)))
    if embedding_rows is None:
        emb = gen(1, V * H).reshape(V, H)
    else:
        emb = np.zeros((V, H), np.uint16)
        for t in embedding_rows:
            emb[t] = synth_16(dt, seed, 1, H, 0.0, weight_std, offset=int(t) * H)
    return Model(dt, H, cfg["heads"], cfg["kv_heads"], HD, I, V, cfg["rms_eps"], cfg["rope_theta"], emb, ls,
                 gen(2, H, 1.0), gen(3, V * H).reshape(V, H))


class Context:
    def __init__(self, model, max_ctx, staging=1, threads=1):
        self.model = model
        self.h = lib.nvo_ctx_create(C.byref(model.c), max_ctx, staging, threads)

    def close(self):
        if self.h:
            lib.nvo_ctx_destroy(self.h)
            self.h = None

    __del__ = close

    def forward_token(self, token, prompt_token=False, want_logits=True):
        hidden = np.empty(self.model.hidden, np.float32)
        rc = lib.nvo_ctx_forward_token(self.h, token, int(prompt_token), int(want_logits), _p(hidden, f32p))
        if rc != 0:
            raise ValueError("forward_token failed")
        return hidden

    def logits(self):
        return np.ctypeslib.as_array(lib.nvo_ctx_logits(self.h), shape=(self.model.vocab,)).copy()

    def greedy_decode(self, prompt, steps, eos=None):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        out = np.zeros(steps, np.uint32)
        margins = np.zeros(steps, np.float32)
        n = lib.nvo_greedy_decode(self.h, _p(prompt, u32p), prompt.size, steps, int(eos is not None),
                                  int(eos or 0), _p(out, u32p), _p(margins, f32p))
        if n < 0:
            raise ValueError("greedy decode failed")
        return out[:n], margins[:n]

    def load_kv16(self, layer, k, v):
        k, v = _u16(k), _u16(v)
        tokens = k.shape[0]
        if lib.nvo_ctx_load_kv16(self.h, layer, _p(k, u16p), _p(v, u16p), tokens) != 0:
            raise ValueError("load_kv16 failed")

    def set_len(self, n):
        lib.nvo_ctx_set_len(self.h, n)

    def read_kv16(self, layer, token):
        kvh = self.model.kv_heads * self.model.head_dim
        k = np.empty(kvh, np.uint16)
        v = np.empty(kvh, np.uint16)
        if lib.nvo_ctx_read_kv16(self.h, layer, token, _p(k, u16p), _p(v, u16p)) != 0:
            raise ValueError("read_kv16 failed")
        return k, v


def block_forward(model, input16, position=0, staging=0):
    x = _u16(input16)
    out = np.empty_like(x)
    rc = lib.nvo_block_forward(C.byref(model.c), _p(x, u16p), position, staging, _p(out, u16p))
    if rc != 0:
        raise ValueError("block forward failed")
    return out
