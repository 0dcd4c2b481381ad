"""Writes a ModelWeights object out as a Hugging Face checkpoint directory (config.json, safetensors
shards, index) for the checkpoint-planner tests. The safetensors container is written by hand - an
8-byte little-endian header length, a JSON header, the tensor bytes - so that the tests control tensor
order and shard cuts; test_checkpoint_cpu.py reads the result back with the safetensors library."""
import json
import os
import struct

import numpy as np

_HF_NAMES = {"rms_attn": "input_layernorm.weight", "w_q": "self_attn.q_proj.weight",
             "q_norm": "self_attn.q_norm.weight", "w_k": "self_attn.k_proj.weight",
             "k_norm": "self_attn.k_norm.weight", "w_v": "self_attn.v_proj.weight",
             "w_o": "self_attn.o_proj.weight", "rms_mlp": "post_attention_layernorm.weight",
             "w_gate": "mlp.gate_proj.weight", "w_up": "mlp.up_proj.weight", "w_down": "mlp.down_proj.weight",
             "q_bias": "self_attn.q_proj.bias", "k_bias": "self_attn.k_proj.bias",
             "v_bias": "self_attn.v_proj.bias", "o_bias": "self_attn.o_proj.bias"}


def named_tensors(weights, tied=False):
    out = {"model.embed_tokens.weight": weights.embeddings, "model.norm.weight": weights.final_norm}
    if not tied:
        out["lm_head.weight"] = weights.lm_head
    for l, layer in enumerate(weights.layers):
        for key, arr in layer.items():
            if arr is not None:
                out["model.layers.%d.%s" % (l, _HF_NAMES[key])] = arr
    return out


def write_safetensors(path, tensors, st_dtype, metadata=None):
    header, blob, offset = {}, [], 0
    if metadata:
        header["__metadata__"] = metadata
    for name, arr in tensors:
        raw = np.ascontiguousarray(arr, np.uint16).tobytes()
        header[name] = {"dtype": st_dtype, "shape": list(arr.shape), "data_offsets": [offset, offset + len(raw)]}
        blob.append(raw)
        offset += len(raw)
    text = json.dumps(header, separators=(",", ":")).encode()
    text += b" " * (-len(text) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)))
        f.write(text)
        for raw in blob:
            f.write(raw)


def write_checkpoint(directory, weights, model_type, shards=2, seed=0, tied=False, extra_config=None):
    """Tensors go to `shards` files in a shuffled order (file order must not matter to the planner);
    one file is called model.safetensors and gets no index."""
    os.makedirs(directory, exist_ok=True)
    st_dtype, torch_dtype = ("BF16", "bfloat16") if weights.dtype == 1 else ("F16", "float16")
    config = dict(model_type=model_type, architectures=[model_type], torch_dtype=torch_dtype,
                  hidden_size=weights.hidden, num_attention_heads=weights.heads,
                  num_key_value_heads=weights.kv_heads, head_dim=weights.head_dim,
                  intermediate_size=weights.intermediate, vocab_size=weights.vocab,
                  num_hidden_layers=len(weights.layers), rms_norm_eps=weights.rms_eps,
                  rope_theta=weights.rope_theta, tie_word_embeddings=tied)
    config.update(extra_config or {})
    with open(os.path.join(directory, "config.json"), "w") as f:
        json.dump(config, f)
    items = list(named_tensors(weights, tied).items())
    np.random.default_rng(seed).shuffle(items)
    if shards == 1:
        write_safetensors(os.path.join(directory, "model.safetensors"), items, st_dtype, {"format": "pt"})
        return
    weight_map, total = {}, 0
    for i in range(shards):
        name = "model-%05d-of-%05d.safetensors" % (i + 1, shards)
        part = items[i::shards]
        write_safetensors(os.path.join(directory, name), part, st_dtype, {"format": "pt"})
        for tensor, arr in part:
            weight_map[tensor] = name
            total += arr.nbytes
    with open(os.path.join(directory, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, f)
