"""From a Hugging Face checkpoint directory to the weight plan a decode session is created from.

The reference's runtime does this in three steps: `config.json` -> model metadata
(crates/nerva-model/src/hf/parser.rs:30-110), metadata -> the tensor manifest in arena order
(crates/nerva-model/src/weights/layout/plan.rs:52-160, layout/plan/layer_blocks.rs:9-49,
manifest/names.rs:31-90), manifest x safetensors headers -> one file-backed descriptor per tensor
(crates/nerva-model/src/weights/safetensors/{header,tensor,validation,shard}.rs,
crates/nerva-runtime/src/engine/hf_cuda_decode/file_backed/descriptors.rs:442-521). This module is the
same pipeline for the dense decoder families the session runs (Llama, Mistral, Qwen2, Qwen3): nothing of
the checkpoint is read into host memory here except the headers; the session copies every tensor from
its file range straight into the device arena.
"""
import ctypes as C
import json
import os
import struct

from . import abi
from .session import (WEIGHT_STRATEGY_GPU_RESIDENT, WEIGHT_STRATEGY_GPU_STAGED, DecodeSession, WeightPlan)

_DTYPES = {"float16": (0, "F16"), "bfloat16": (1, "BF16")}          # request dtype code, safetensors name
_DENSE = {"llama": False, "mistral": False, "qwen2": False, "qwen3": True}  # model_type -> per-head q/k norm
_MAX_HEADER = 100 * 1000 * 1000                                       # the format's own bound on header bytes


class CheckpointError(ValueError):
    pass


def parse_config(config):
    """Model dimensions and optional-tensor flags of a dense decoder from its `config.json`
    (hf/parser.rs:30-110; bias rule :464-479, q/k-norm rule :481-499)."""
    text = config.get("text_config", config)
    kind = (text.get("model_type") or config.get("model_type") or "").lower()
    if kind not in _DENSE:
        raise CheckpointError("model_type %r is not a dense decoder this session runs" % kind)

    def need(key):
        value = text.get(key, config.get(key))
        if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
            raise CheckpointError("config.json: %s missing or not a positive integer" % key)
        return value

    dtype = text.get("torch_dtype", config.get("torch_dtype", text.get("dtype", config.get("dtype"))))
    if dtype not in _DTYPES:
        raise CheckpointError("torch_dtype %r: the session takes float16 or bfloat16 weights" % (dtype,))
    hidden, heads = need("hidden_size"), need("num_attention_heads")
    kv_heads = text.get("num_key_value_heads", heads)
    head_dim = text.get("head_dim") or hidden // heads
    attention_bias = text.get("attention_bias")
    qkv_bias = text.get("qkv_bias")
    qk_norm = text.get("qk_norm", text.get("use_qk_norm", _DENSE[kind]))
    return dict(model_type=kind, dtype=_DTYPES[dtype][0], st_dtype=_DTYPES[dtype][1], hidden=hidden, heads=heads,
                kv_heads=kv_heads, head_dim=head_dim, intermediate=need("intermediate_size"),
                vocab=need("vocab_size"), layers=need("num_hidden_layers"),
                rms_eps=float(text.get("rms_norm_eps", 1e-6)), rope_theta=float(text.get("rope_theta", 10000.0)),
                qk_norm=bool(qk_norm), qkv_bias=bool(attention_bias) or bool(qkv_bias),
                o_bias=bool(attention_bias), tied=bool(text.get("tie_word_embeddings", config.get("tie_word_embeddings", False))))


def tensor_manifest(cfg):
    """(name, shape) of every tensor in the order of the weight arena: embeddings, per layer
    norm / q / q_norm / k / k_norm / v / o / mlp norm / gate / up / down / biases, final norm, LM head
    (layout/plan/layer_blocks.rs:9-49, weights.cu:484-591). A tied LM head is the embedding tensor again."""
    H, A, KV, I = cfg["hidden"], cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"], cfg["intermediate"]
    out = [("model.embed_tokens.weight", [cfg["vocab"], H])]
    for l in range(cfg["layers"]):
        p = "model.layers.%d." % l
        out.append((p + "input_layernorm.weight", [H]))
        out.append((p + "self_attn.q_proj.weight", [A, H]))
        if cfg["qk_norm"]:
            out.append((p + "self_attn.q_norm.weight", [cfg["head_dim"]]))
        out.append((p + "self_attn.k_proj.weight", [KV, H]))
        if cfg["qk_norm"]:
            out.append((p + "self_attn.k_norm.weight", [cfg["head_dim"]]))
        out.append((p + "self_attn.v_proj.weight", [KV, H]))
        out.append((p + "self_attn.o_proj.weight", [H, A]))
        out.append((p + "post_attention_layernorm.weight", [H]))
        out.append((p + "mlp.gate_proj.weight", [I, H]))
        out.append((p + "mlp.up_proj.weight", [I, H]))
        out.append((p + "mlp.down_proj.weight", [H, I]))
        if cfg["qkv_bias"]:
            out += [(p + "self_attn.q_proj.bias", [A]), (p + "self_attn.k_proj.bias", [KV]),
                    (p + "self_attn.v_proj.bias", [KV])]
        if cfg["o_bias"]:
            out.append((p + "self_attn.o_proj.bias", [H]))
    out.append(("model.norm.weight", [H]))
    out.append(("model.embed_tokens.weight" if cfg["tied"] else "lm_head.weight", [cfg["vocab"], H]))
    return out


def read_safetensors_header(path):
    """(header dict, file offset of the data section). The rules of header.rs:7-32: an 8-byte little-endian
    length, that many bytes of UTF-8 JSON, all inside the file."""
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) < 8:
            raise CheckpointError("%s: too small to contain a header length" % path)
        (n,) = struct.unpack("<Q", head)
        if n > _MAX_HEADER or 8 + n > size:
            raise CheckpointError("%s: header length %d exceeds the file" % (path, n))
        raw = f.read(n)
    try:
        header = json.loads(raw.decode("utf-8"))
    except (UnicodeDecodeError, ValueError) as err:
        raise CheckpointError("%s: header is not valid UTF-8 JSON (%s)" % (path, err))
    if not isinstance(header, dict):
        raise CheckpointError("%s: header is not a JSON object" % path)
    return header, 8 + n


def _shards(directory):
    """tensor name -> shard file, from `model.safetensors.index.json` (weight_map.rs:8-46) or the single
    `model.safetensors`."""
    index = os.path.join(directory, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as f:
            weight_map = json.load(f).get("weight_map")
        if not isinstance(weight_map, dict) or not weight_map:
            raise CheckpointError("%s: no weight_map" % index)
        return weight_map
    single = os.path.join(directory, "model.safetensors")
    if not os.path.exists(single):
        raise CheckpointError("%s: neither model.safetensors.index.json nor model.safetensors" % directory)
    return None


class CheckpointPlan(WeightPlan):
    """A WeightPlan whose descriptors point into the checkpoint's files, plus the model dimensions."""

    def __init__(self, cfg, entries, blocks, keepalive):
        super().__init__(blocks, keepalive)
        self.cfg, self.entries = cfg, entries   # entries: (name, file, file_offset_begin, bytes) in arena order


def plan_checkpoint(directory, resident_bytes=None):
    """Validates every manifest tensor against its shard's header (dtype, shape, offset span:
    tensor.rs:12-66, validation.rs:43-84) and declares one descriptor per tensor, sourced from the file range
    (descriptors.rs:442-521: block ids count from 1 in manifest order, offsets run through the arena,
    an odd byte count would be padded to the next even one - 16-bit tensors never have one). The first
    `resident_bytes` of the arena are declared GPU-resident and the rest GPU-staged (None: all resident);
    both end up in device memory here."""
    with open(os.path.join(directory, "config.json")) as f:
        cfg = parse_config(json.load(f))
    weight_map = _shards(directory)
    headers, paths, entries, blocks, offset = {}, {}, [], [], 0
    for index, (name, shape) in enumerate(tensor_manifest(cfg)):
        shard = "model.safetensors" if weight_map is None else weight_map.get(name)
        if shard is None:
            raise CheckpointError("weight_map is missing tensor %s" % name)
        if shard not in headers:
            headers[shard] = read_safetensors_header(os.path.join(directory, shard))
            paths[shard] = C.create_string_buffer(os.path.join(directory, shard).encode())
        header, data_start = headers[shard]
        meta = header.get(name)
        if not isinstance(meta, dict):
            raise CheckpointError("safetensors header of %s is missing tensor %s" % (shard, name))
        if meta.get("dtype") != cfg["st_dtype"]:
            raise CheckpointError("tensor %s dtype %r does not match expected %s" % (name, meta.get("dtype"), cfg["st_dtype"]))
        if meta.get("shape") != shape:
            raise CheckpointError("tensor %s shape %r does not match expected %r" % (name, meta.get("shape"), shape))
        nbytes = 2
        for d in shape:
            nbytes *= d
        offsets = meta.get("data_offsets")
        if (not isinstance(offsets, list) or len(offsets) != 2 or not all(isinstance(o, int) for o in offsets)
                or offsets[1] < offsets[0]):
            raise CheckpointError("tensor %s has invalid offsets" % name)
        if offsets[1] - offsets[0] != nbytes:
            raise CheckpointError("tensor %s offset span %d does not match expected bytes %d"
                                  % (name, offsets[1] - offsets[0], nbytes))
        if data_start + offsets[1] > os.path.getsize(os.path.join(directory, shard)):
            raise CheckpointError("tensor %s ends beyond its file %s" % (name, shard))
        b = abi.NervaHipHfDecodeSequenceWeightBlock()
        b.source_file = C.cast(paths[shard], C.c_void_p).value
        b.source_file_len = len(paths[shard].value)
        b.file_offset_begin = data_start + offsets[0]
        b.block_id, b.block_version, b.offset_bytes, b.bytes = index + 1, 0, offset, nbytes
        resident = resident_bytes is None or offset + nbytes <= resident_bytes
        b.strategy = WEIGHT_STRATEGY_GPU_RESIDENT if resident else WEIGHT_STRATEGY_GPU_STAGED
        blocks.append(b)
        entries.append((name, shard, data_start + offsets[0], nbytes))
        offset += nbytes
    return CheckpointPlan(cfg, entries, blocks, [paths])


_MARKER = (C.c_uint16 * 1)(0)


def marker_layers(cfg):
    """The layer array of a descriptor-fed request: every tensor pointer null except the optional tensors',
    which point at a one-element marker saying "this model has it"
    (descriptors.rs:69-170, hf_chain/layer.rs:352-399)."""
    layers = (abi.NervaHipHfDecodeChainLayer * cfg["layers"])()
    mark = C.cast(_MARKER, C.c_void_p).value
    for layer in layers:
        if cfg["qk_norm"]:
            layer.q_norm_weight = layer.k_norm_weight = mark
        if cfg["qkv_bias"]:
            layer.q_bias = layer.k_bias = layer.v_bias = mark
        if cfg["o_bias"]:
            layer.o_bias = mark
    return layers


def create_session(directory, max_context, resident_bytes=None, **extra):
    """A decode session whose weights come from the checkpoint's files through a declared weight plan.
    Returns (session, plan); the plan must outlive the create call only."""
    plan = plan_checkpoint(directory, resident_bytes)
    cfg = plan.cfg
    lib = abi.load()
    req = abi.NervaHipHfDecodeSequenceSessionCreateRequest()
    req.dtype, req.hidden, req.heads, req.kv_heads = cfg["dtype"], cfg["hidden"], cfg["heads"], cfg["kv_heads"]
    req.head_dim, req.intermediate, req.vocab_size = cfg["head_dim"], cfg["intermediate"], cfg["vocab"]
    req.layer_count, req.max_context_tokens = cfg["layers"], max_context
    req.rms_eps, req.rope_theta = cfg["rms_eps"], cfg["rope_theta"]
    layers = marker_layers(cfg)
    req.layers = layers
    for k, v in plan.fields().items():
        setattr(req, k, v)
    for k, v in extra.items():
        setattr(req, k, v)
    res = abi.NervaHipHfDecodeSequenceSessionCreateResult()
    handle = C.POINTER(abi.NervaHipHfDecodeSequenceSession)()
    rc = lib.nerva_hip_hf_decode_sequence_session_create(C.byref(req), C.byref(res), C.byref(handle))
    if rc != 0:
        raise RuntimeError("session_create from %s failed: status=%d hip_error=%d stage=%d"
                           % (directory, res.status, res.hip_error, res.failure_stage))
    return DecodeSession(handle, res, cfg["vocab"], cfg["kv_heads"] * cfg["head_dim"]), plan
