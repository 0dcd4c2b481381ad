"""Decode-session wrapper over the C ABI (create / start / advance / run / destroy).

Mirrors the request/summary objects of the reference's host crate
(crates/nerva-cuda/src/decode/hf_sequence/session/request.rs,
crates/nerva-cuda/src/decode/hf_sequence/request.rs): the caller owns host
weights, the library owns the opaque session.
"""
import ctypes as C

import numpy as np

from . import abi

Qwen3_8B = dict(dtype=1, hidden=4096, heads=32, kv_heads=8, head_dim=128, intermediate=12288,
                vocab=151936, layers=36, rms_eps=1e-6, rope_theta=1e6)

_LAYER_FIELDS = {
    "rms_attn": "rms_attn_weight", "rms_mlp": "rms_mlp_weight", "w_q": "w_q", "w_k": "w_k",
    "w_v": "w_v", "w_o": "w_o", "q_norm": "q_norm_weight", "k_norm": "k_norm_weight",
    "q_bias": "q_bias", "k_bias": "k_bias", "v_bias": "v_bias", "o_bias": "o_bias",
    "w_gate": "w_gate", "w_up": "w_up", "w_down": "w_down",
}


def _u16(a):
    return None if a is None else np.ascontiguousarray(a, np.uint16)


class ModelWeights:
    """Host weights (16-bit numpy arrays, row-major [out, in]) of a dense decoder."""

    def __init__(self, dtype, hidden, heads, kv_heads, head_dim, intermediate, vocab, rms_eps,
                 rope_theta, embeddings, layers, final_norm, lm_head):
        self.dtype, self.hidden, self.heads, self.kv_heads = dtype, hidden, heads, kv_heads
        self.head_dim, self.intermediate, self.vocab = head_dim, intermediate, vocab
        self.rms_eps, self.rope_theta = rms_eps, rope_theta
        self.embeddings, self.final_norm, self.lm_head = _u16(embeddings), _u16(final_norm), _u16(lm_head)
        self.layers = [{k: _u16(v) for k, v in layer.items()} for layer in layers]
        self.c_layers = (abi.NervaHipHfDecodeChainLayer * len(self.layers))()
        for cl, layer in zip(self.c_layers, self.layers):
            for key, field in _LAYER_FIELDS.items():
                arr = layer.get(key)
                setattr(cl, field, arr.ctypes.data if arr is not None else None)

    def fill_dims(self, req):
        req.dtype, req.hidden, req.heads, req.kv_heads = self.dtype, self.hidden, self.heads, self.kv_heads
        req.head_dim, req.intermediate, req.vocab_size = self.head_dim, self.intermediate, self.vocab
        req.layer_count = len(self.layers)
        req.rms_eps, req.rope_theta = self.rms_eps, self.rope_theta or 0.0
        req.embeddings = self.embeddings.ctypes.data
        req.layers = self.c_layers
        req.final_norm_weight = self.final_norm.ctypes.data
        req.lm_head = self.lm_head.ctypes.data


WEIGHT_STRATEGY_GPU_RESIDENT, WEIGHT_STRATEGY_GPU_STAGED = 1, 2    # weight_plan.rs:3-4

_ARENA_ORDER = ("rms_attn", "w_q", "q_norm", "w_k", "k_norm", "w_v", "w_o", "rms_mlp", "w_gate", "w_up", "w_down",
                "q_bias", "k_bias", "v_bias", "o_bias")


def arena_order(weights):
    """The model's tensors in the order the reference lays its weight arena out, which is the byte
    space weight descriptors address (weights.cu:484-591, session_api_lifecycle.inc.cu:124-148)."""
    out = [weights.embeddings]
    for layer in weights.layers:
        out += [layer[k] for k in _ARENA_ORDER if layer.get(k) is not None]
    return out + [weights.final_norm, weights.lm_head]


def hash_weight_blocks(blocks):
    """FNV-1a-64 over (block_id, block_version, offset_bytes, bytes) as u64 and strategy as u32,
    little endian, block after block (weight_plan.rs:102-126, weights.cu:90-111)."""
    h = 0xcbf29ce484222325
    for b in blocks:
        for value, width in ((b.block_id, 8), (b.block_version, 8), (b.offset_bytes, 8), (b.bytes, 8), (b.strategy, 4)):
            for i in range(width):
                h = ((h ^ ((value >> (8 * i)) & 0xFF)) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


class WeightPlan:
    """A declared weight plan: descriptors that tile the model's weight bytes in arena order, each
    with a host-memory or a file source, and the totals the session checks them against
    (weight_plan.rs:24-100)."""

    def __init__(self, blocks, keepalive):
        self.blocks = (abi.NervaHipHfDecodeSequenceWeightBlock * len(blocks))(*blocks)
        self._keepalive = keepalive
        self.descriptor_hash = hash_weight_blocks(blocks)

    @classmethod
    def from_weights(cls, weights, block_bytes=None, resident_blocks=None, path=None):
        """block_bytes None: one block per tensor, sourced from the tensor's own memory. Otherwise the
        arena is cut into blocks of block_bytes (even; the last one shorter) over one contiguous copy
        of it - in memory, or in the file `path`, which is written here. The first `resident_blocks`
        blocks are declared GPU-resident, the rest GPU-staged (both end up in device memory)."""
        tensors = arena_order(weights)
        keep, blocks, offset = [tensors], [], 0
        if block_bytes is None:
            pieces = [(t.ctypes.data, t.nbytes) for t in tensors]
        else:
            storage = np.concatenate([t.reshape(-1) for t in tensors])
            keep.append(storage)
            total = storage.nbytes
            pieces = [(storage.ctypes.data + o, min(block_bytes, total - o)) for o in range(0, total, block_bytes)]
            if path is not None:
                storage.tofile(path)
                keep.append(C.create_string_buffer(path.encode()))
        for index, (address, nbytes) in enumerate(pieces):
            b = abi.NervaHipHfDecodeSequenceWeightBlock()
            if path is not None and block_bytes is not None:
                b.source_file = C.cast(keep[-1], C.c_void_p).value
                b.source_file_len = len(path.encode())
                b.file_offset_begin = offset
            else:
                b.host_source = address
            b.block_id, b.block_version, b.offset_bytes, b.bytes = index + 1, 0, offset, nbytes
            resident = resident_blocks is None or index < resident_blocks
            b.strategy = WEIGHT_STRATEGY_GPU_RESIDENT if resident else WEIGHT_STRATEGY_GPU_STAGED
            blocks.append(b)
            offset += nbytes
        return cls(blocks, keep)

    def fields(self):
        resident = [b for b in self.blocks if b.strategy == WEIGHT_STRATEGY_GPU_RESIDENT]
        staged = [b for b in self.blocks if b.strategy == WEIGHT_STRATEGY_GPU_STAGED]
        return dict(planned_weight_blocks=len(self.blocks), planned_gpu_resident_blocks=len(resident),
                    planned_gpu_staged_blocks=len(staged), planned_weight_bytes=sum(b.bytes for b in self.blocks),
                    planned_gpu_resident_weight_bytes=sum(b.bytes for b in resident),
                    planned_gpu_staged_weight_bytes=sum(b.bytes for b in staged),
                    planned_weight_descriptors=self.blocks,
                    planned_weight_descriptor_count=len(self.blocks),
                    planned_weight_descriptor_hash=self.descriptor_hash)


def descriptor_layout_layers(weights, req):
    """What a request with a declared weight plan carries instead of tensor pointers
    (hf_chain/layer.rs:352-399, helpers.rs:13-19): the layer array with only the pointers of the
    optional tensors left, as markers that they exist; every other tensor pointer null."""
    req.embeddings = req.final_norm_weight = req.lm_head = None
    layers = (abi.NervaHipHfDecodeChainLayer * req.layer_count)()
    for dst, src in zip(layers, weights.c_layers):
        for field in ("q_norm_weight", "k_norm_weight", "q_bias", "k_bias", "v_bias", "o_bias"):
            setattr(dst, field, getattr(src, field))
    req.layers = layers
    return layers


def greedy_sampler():
    cfg = abi.NervaHipHfDecodeSamplerConfig()
    cfg.temperature, cfg.top_p, cfg.top_k, cfg.seed = 0.0, 1.0, 0, 0
    return cfg


class DecodeSession:
    def __init__(self, handle, create_result, vocab, kv_hidden):
        self.handle, self.create_result, self.vocab, self.kv_hidden = handle, create_result, vocab, kv_hidden
        self.lib = abi.load()

    @classmethod
    def create(cls, weights, max_context, plan=None, tensor_pointers=True, **extra):
        """plan: a WeightPlan whose descriptors then are the source of the weights; with
        tensor_pointers=False the request carries no tensor pointers at all."""
        lib = abi.load()
        req = abi.NervaHipHfDecodeSequenceSessionCreateRequest()
        weights.fill_dims(req)
        req.max_context_tokens = max_context
        keep = None if tensor_pointers else descriptor_layout_layers(weights, req)
        for k, v in (plan.fields() if plan is not None else {}).items():
            setattr(req, k, v)
        for k, v in extra.items():
            setattr(req, k, v)
        res = abi.NervaHipHfDecodeSequenceSessionCreateResult()
        handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
        rc = lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(res), C.byref(handle))
        if rc != 0:
            raise RuntimeError("session_create failed: status=%d hip_error=%d stage=%d"
                               % (res.status, res.hip_error, res.failure_stage))
        return cls(handle, res, weights.vocab, weights.kv_heads * weights.head_dim)

    @classmethod
    def create_synthetic(cls, cfg, max_context, seed=0x4E45525641, weight_std=0.02, qk_norm=True,
                         weight_hash=0):
        """Session over device-generated weights. `weight_hash` stands in for the weight-plan
        descriptor hash by which batch steps recognise sessions of the same model."""
        lib = abi.load()
        req = abi.NervaHipHfDecodeSequenceSessionCreateRequest()
        req.dtype, req.hidden, req.heads, req.kv_heads = cfg["dtype"], cfg["hidden"], cfg["heads"], cfg["kv_heads"]
        req.head_dim, req.intermediate, req.vocab_size = cfg["head_dim"], cfg["intermediate"], cfg["vocab"]
        req.layer_count, req.max_context_tokens = cfg["layers"], max_context
        req.rms_eps, req.rope_theta = cfg["rms_eps"], cfg["rope_theta"] or 0.0
        req.planned_weight_descriptor_hash = weight_hash
        res = abi.NervaHipHfDecodeSequenceSessionCreateResult()
        handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
        rc = lib.nerva_hip_bench_session_create_synthetic(C.byref(req), seed, weight_std, int(qk_norm),
                                                          C.byref(res), C.byref(handle))
        if rc != 0:
            raise RuntimeError("synthetic session_create failed: status=%d hip_error=%d stage=%d"
                               % (res.status, res.hip_error, res.failure_stage))
        return cls(handle, res, cfg["vocab"], cfg["kv_heads"] * cfg["head_dim"])

    def fork_shared_weights(self, detailed_profile=False):
        """A second session on this one's resident weights (request.rs:380-407); carries a sequence
        that is under way over to the child."""
        req = abi.NervaHipHfDecodeSequenceSessionForkSharedWeightsRequest()
        req.parent, req.detailed_profile = self.handle, int(detailed_profile)
        res = abi.NervaHipHfDecodeSequenceSessionCreateResult()
        handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
        rc = self.lib.nerva_hip_hf_decode_sequence_session_fork_shared_weights(C.byref(req), C.byref(res),
                                                                               C.byref(handle))
        if rc != 0:
            raise RuntimeError("session fork failed: status=%d hip_error=%d stage=%d"
                               % (res.status, res.hip_error, res.failure_stage))
        return DecodeSession(handle, res, self.vocab, self.kv_hidden)

    BATCH_REASONS = ("ready", "invalid_request", "no_sessions", "no_ready_sessions", "shared_weights_unproven",
                     "insufficient_compatible_ready")

    @staticmethod
    def batch_advance_one(sessions, target_block_tokens, min_block_tokens):
        """One more token for every ready session of the same model (request.rs:575-597). Returns
        (rc, result, tokens) with tokens[i] = 0xFFFFFFFF for sessions that did not advance."""
        lib = abi.load()
        handles = (C.POINTER(abi.NervaHipHfDecodeSequenceSession) * max(len(sessions), 1))()
        for i, sess in enumerate(sessions):
            handles[i] = sess.handle
        tokens = np.full(max(len(sessions), 1), 0xFFFFFFFF, np.uint32)
        req = abi.NervaHipHfDecodeSequenceBatchAdvanceRequest()
        req.sessions = handles
        req.session_count = len(sessions)
        req.target_block_tokens, req.min_block_tokens = target_block_tokens, min_block_tokens
        req.output_tokens, req.output_token_capacity = tokens.ctypes.data, len(sessions)
        res = abi.NervaHipHfDecodeSequenceBatchAdvanceResult()
        rc = lib.nerva_hip_hf_decode_sequence_batch_advance_one(C.byref(req), C.byref(res))
        return rc, res, tokens[:len(sessions)]

    def shares_weight_stream(self):
        """Whether a batch step led by this session streams the weights once for all its sequences."""
        return self.lib.nerva_hip_session_shares_weight_stream(self.handle) == 1

    def start(self, prompt, eos=None, sampler=None):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        req = abi.NervaHipHfDecodeSequenceSessionStartRequest()
        req.session = self.handle
        req.prompt_tokens, req.prompt_token_count = prompt.ctypes.data, prompt.size
        req.has_eos_token, req.eos_token = int(eos is not None), int(eos or 0)
        req.sampler = sampler or greedy_sampler()
        res = abi.NervaHipHfDecodeSequenceResult()
        rc = self.lib.nerva_hip_hf_decode_sequence_session_start(C.byref(req), C.byref(res))
        return rc, res

    def advance(self, steps, capacity=None):
        out = np.zeros(capacity if capacity is not None else steps, np.uint32)
        req = abi.NervaHipHfDecodeSequenceSessionAdvanceRequest()
        req.session, req.steps = self.handle, steps
        req.output_tokens, req.output_token_capacity = out.ctypes.data, out.size
        res = abi.NervaHipHfDecodeSequenceResult()
        rc = self.lib.nerva_hip_hf_decode_sequence_session_advance(C.byref(req), C.byref(res))
        return rc, res, out[:res.observed_tokens]

    def run(self, prompt, steps, eos=None, sampler=None, seed_token=None):
        prompt = np.ascontiguousarray(prompt, np.uint32)
        out = np.zeros(steps, np.uint32)
        req = abi.NervaHipHfDecodeSequenceSessionRunRequest()
        req.session, req.steps = self.handle, steps
        req.seed_token = int(prompt[-1]) if seed_token is None else seed_token
        req.prompt_tokens, req.prompt_token_count = prompt.ctypes.data, prompt.size
        req.has_eos_token, req.eos_token = int(eos is not None), int(eos or 0)
        req.output_tokens, req.output_token_capacity = out.ctypes.data, out.size
        req.sampler = sampler or greedy_sampler()
        res = abi.NervaHipHfDecodeSequenceResult()
        rc = self.lib.nerva_hip_hf_decode_sequence_session_run(C.byref(req), C.byref(res))
        return rc, res, out[:res.observed_tokens]

    def profile_step(self, repeats=3):
        res = abi.NervaHipStepProfile()
        rc = self.lib.nerva_hip_session_profile_step(self.handle, repeats, C.byref(res))
        return rc, res

    def traced_advance(self):
        """advance(1) with the step's intermediates read back (nerva_hip_session_trace_next_step).

        Returns (rc, result, tokens, trace); trace = {"x0": f32[hidden], "layers": [{"a16", "qkv", "attn16",
        "r", "m16", "ff16", "x"}...], "h16", "logits": f32[vocab]} - the output vector of every kernel of
        that step, and the 16-bit outputs of the RMSNorm prologues (a16, m16, h16),
        or None when the call launched no step (the first advance hands out the token start() made)."""
        from .runtime import DeviceBuffer
        cr = self.create_result
        nbytes = int(self.lib.nerva_hip_session_step_trace_bytes(self.handle))
        buf = DeviceBuffer.zeros(nbytes)
        if self.lib.nerva_hip_session_trace_next_step(self.handle, buf.ptr, nbytes) != 0:
            raise RuntimeError("trace_next_step refused")
        rc, res, tokens = self.advance(1)
        if rc != 0 or res.kernel_launches == 0:
            self.lib.nerva_hip_session_trace_next_step(self.handle, None, 0)  # disarm
            return rc, res, tokens, None
        raw = buf.numpy(np.uint8)
        at = [0]

        def take(count, dtype):
            n = count * np.dtype(dtype).itemsize
            a = raw[at[0]:at[0] + n].view(dtype).copy()
            at[0] += (n + 255) & ~255
            return a

        A, KV = cr.heads * cr.head_dim, cr.kv_heads * cr.head_dim
        trace = {"x0": take(cr.hidden, np.float32), "layers": []}
        for _ in range(cr.layer_count):
            trace["layers"].append({"a16": take(cr.hidden, np.uint16), "qkv": take(A + 2 * KV, np.float32),
                                    "attn16": take(A, np.uint16), "r": take(cr.hidden, np.float32),
                                    "m16": take(cr.hidden, np.uint16), "ff16": take(cr.intermediate, np.uint16),
                                    "x": take(cr.hidden, np.float32)})
        trace["h16"] = take(cr.hidden, np.uint16)
        trace["logits"] = take(cr.vocab_size, np.float32)
        assert at[0] == nbytes
        return rc, res, tokens, trace

    def logits(self):
        out = np.empty(self.vocab, np.float32)
        if self.lib.nerva_hip_session_read_logits(self.handle, out.ctypes.data) != 0:
            raise RuntimeError("read_logits failed")
        return out

    def slots(self, first, count):
        """The raw 40-byte token slots [first, first + count) as the device wrote them: a (count, 40) uint8 array."""
        out = np.zeros((count, C.sizeof(abi.NervaHipSyntheticTokenSlot)), np.uint8)
        ptr = C.cast(out.ctypes.data, C.POINTER(abi.NervaHipSyntheticTokenSlot))
        if self.lib.nerva_hip_session_read_slots(self.handle, first, count, ptr) != 0:
            raise RuntimeError("read_slots failed")
        return out

    def kv_row(self, layer, token):
        k = np.empty(self.kv_hidden, np.uint16)
        v = np.empty(self.kv_hidden, np.uint16)
        if self.lib.nerva_hip_session_read_kv(self.handle, layer, token, k.ctypes.data, v.ctypes.data) != 0:
            raise RuntimeError("read_kv failed")
        return k, v

    def kv_range(self, layer, first, count):
        k = np.empty((count, self.kv_hidden), np.uint16)
        v = np.empty((count, self.kv_hidden), np.uint16)
        if self.lib.nerva_hip_session_read_kv_range(self.handle, layer, first, count, k.ctypes.data,
                                                    v.ctypes.data) != 0:
            raise RuntimeError("read_kv_range failed")
        return k, v

    def destroy(self):
        if self.handle:
            res = abi.NervaHipHfDecodeSequenceSessionCreateResult()
            rc = self.lib.nerva_hip_hf_decode_sequence_session_destroy(self.handle, C.byref(res))
            self.handle = None
            return rc, res
        return -1, None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def decode_sequence_oneshot(weights, prompt, steps, eos=None, plan=None):
    """nerva_hip_hf_decode_sequence_u16: create + run + destroy in one call."""
    lib = abi.load()
    prompt = np.ascontiguousarray(prompt, np.uint32)
    out = np.zeros(steps, np.uint32)
    req = abi.NervaHipHfDecodeSequenceRequest()
    weights.fill_dims(req)
    req.steps, req.seed_token = steps, int(prompt[-1])
    req.prompt_tokens, req.prompt_token_count = prompt.ctypes.data, prompt.size
    req.has_eos_token, req.eos_token = int(eos is not None), int(eos or 0)
    req.output_tokens, req.output_token_capacity = out.ctypes.data, out.size
    req.sampler = greedy_sampler()
    for k, v in (plan or {}).items():
        setattr(req, k, v)
    res = abi.NervaHipHfDecodeSequenceResult()
    rc = lib.nerva_hip_hf_decode_sequence_u16(C.byref(req), C.byref(res))
    return rc, res, out[:res.observed_tokens]
