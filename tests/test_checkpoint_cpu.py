"""Host logic of the checkpoint planner (config.json -> manifest in arena order -> file-backed weight
descriptors); no device needed. The session side of the same plan is tested on the GPU in
test_gpu_session.py."""
import json
import os

import numpy as np
import pytest

import nerva_amd as N
import oracle as O
from checkpoint_files import named_tensors, write_checkpoint
from nerva_amd import checkpoint as ckpt
from nerva_amd.session import arena_order


def small_weights(dtype=1, qk_norm=True, bias=False, layers=2, seed=5):
    rng = np.random.default_rng(seed)
    hidden, heads, kv, hd, inter, vocab = 64, 4, 2, 32, 96, 50
    e = lambda shape: O.encode16(dtype, rng.normal(0, 0.05, shape))
    A, KV = heads * hd, kv * hd
    ls = []
    for _ in range(layers):
        l = dict(rms_attn=e(hidden), rms_mlp=e(hidden), w_q=e((A, hidden)), w_k=e((KV, hidden)),
                 w_v=e((KV, hidden)), w_o=e((hidden, A)), w_gate=e((inter, hidden)), w_up=e((inter, hidden)),
                 w_down=e((hidden, inter)))
        if qk_norm:
            l.update(q_norm=e(hd), k_norm=e(hd))
        if bias:
            l.update(q_bias=e(A), k_bias=e(KV), v_bias=e(KV), o_bias=e(hidden))
        ls.append(l)
    return N.ModelWeights(dtype, hidden, heads, kv, hd, inter, vocab, 1e-6, 1e4, e((vocab, hidden)), ls,
                          e(hidden), e((vocab, hidden)))


def test_config_rules_follow_the_reference_parser():
    base = dict(model_type="qwen3", torch_dtype="bfloat16", hidden_size=4096, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
                num_hidden_layers=36, rms_norm_eps=1e-6, rope_theta=1e6)
    cfg = ckpt.parse_config(base)
    assert {k: cfg[k] for k in N.Qwen3_8B} == N.Qwen3_8B          # the named workload's dimensions
    assert cfg["qk_norm"] and not cfg["qkv_bias"] and not cfg["o_bias"] and not cfg["tied"]
    # q/k norm defaults by family and can be stated; attention_bias means all four biases, qkv_bias three
    assert not ckpt.parse_config(dict(base, model_type="llama"))["qk_norm"]
    assert ckpt.parse_config(dict(base, model_type="llama", use_qk_norm=True))["qk_norm"]
    assert not ckpt.parse_config(dict(base, qk_norm=False))["qk_norm"]
    both = ckpt.parse_config(dict(base, attention_bias=True))
    assert both["qkv_bias"] and both["o_bias"]
    three = ckpt.parse_config(dict(base, model_type="qwen2", qkv_bias=True))
    assert three["qkv_bias"] and not three["o_bias"]
    # head_dim falls back to hidden / heads; kv heads to heads
    short = {k: v for k, v in base.items() if k not in ("head_dim", "num_key_value_heads")}
    assert ckpt.parse_config(short)["head_dim"] == 128 and ckpt.parse_config(short)["kv_heads"] == 32
    for bad in (dict(base, model_type="gemma"), dict(base, torch_dtype="float32"), dict(base, hidden_size=0),
                {k: v for k, v in base.items() if k != "vocab_size"}):
        with pytest.raises(ckpt.CheckpointError):
            ckpt.parse_config(bad)


def test_manifest_of_the_named_model_adds_up():
    """Qwen3-8B: 399 tensors (1 + 36 x 11 + 2) and the weight bytes of a decode step's stream plus the
    embedding table."""
    cfg = dict(N.Qwen3_8B, qk_norm=True, qkv_bias=False, o_bias=False, tied=False)
    manifest = ckpt.tensor_manifest(cfg)
    assert len(manifest) == 1 + 36 * 11 + 2
    assert manifest[0][0] == "model.embed_tokens.weight" and manifest[-1][0] == "lm_head.weight"
    assert [n.split(".", 3)[3] for n, _ in manifest[1:12]] == [
        "input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.q_norm.weight", "self_attn.k_proj.weight",
        "self_attn.k_norm.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
        "post_attention_layernorm.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight"]
    total = sum(2 * int(np.prod(shape)) for _, shape in manifest)
    per_layer = 2 * (2 * 4096 + 2 * 128 + 4096 * 4096 * 2 + 2 * 1024 * 4096 + 3 * 12288 * 4096)
    assert total == 2 * 2 * 151936 * 4096 + 2 * 4096 + 36 * per_layer


@pytest.mark.parametrize("shards,qk_norm,bias,model_type", [(1, True, False, "qwen3"), (3, False, True, "llama"),
                                                              (2, True, True, "qwen3")])
def test_plan_points_at_every_tensor_in_arena_order(tmp_path, shards, qk_norm, bias, model_type):
    weights = small_weights(qk_norm=qk_norm, bias=bias)
    extra = dict(attention_bias=True) if bias else {}
    write_checkpoint(str(tmp_path), weights, model_type, shards=shards, seed=shards, extra_config=extra)
    plan = ckpt.plan_checkpoint(str(tmp_path))
    tensors = arena_order(weights)
    assert len(plan.blocks) == len(tensors) == len(plan.entries)
    offset = 0
    for block, tensor, (name, shard, begin, nbytes) in zip(plan.blocks, tensors, plan.entries):
        # the bytes the descriptor names are the tensor's bytes, and the arena offsets run on
        assert (block.offset_bytes, block.bytes, block.file_offset_begin) == (offset, tensor.nbytes, begin)
        assert block.host_source is None and block.source_file_len == len(os.path.join(str(tmp_path), shard))
        with open(os.path.join(str(tmp_path), shard), "rb") as f:
            f.seek(begin)
            assert f.read(nbytes) == tensor.tobytes(), name
        offset += tensor.nbytes
    # same identity as a plan declared over the tensors in memory: ids, offsets, sizes, strategies
    assert plan.descriptor_hash == N.WeightPlan.from_weights(weights).descriptor_hash
    fields = plan.fields()
    assert fields["planned_weight_bytes"] == offset == fields["planned_gpu_resident_weight_bytes"]
    # a residency budget declares the tail of the arena staged
    part = ckpt.plan_checkpoint(str(tmp_path), resident_bytes=tensors[0].nbytes + tensors[1].nbytes)
    assert part.fields()["planned_gpu_resident_blocks"] == 2
    assert part.fields()["planned_gpu_staged_weight_bytes"] == offset - tensors[0].nbytes - tensors[1].nbytes


def test_written_shards_are_what_the_safetensors_library_reads(tmp_path):
    """The hand-written container is the real format: the safetensors library returns the same bits."""
    torch = pytest.importorskip("torch")
    from safetensors import safe_open
    weights = small_weights()
    write_checkpoint(str(tmp_path), weights, "qwen3", shards=1)
    with safe_open(os.path.join(str(tmp_path), "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
        expect = named_tensors(weights)
        assert names == set(expect)
        for name in ("model.embed_tokens.weight", "model.layers.1.mlp.down_proj.weight", "model.layers.0.self_attn.q_norm.weight"):
            got = f.get_tensor(name).view(torch.uint16).numpy()
            assert np.array_equal(got, expect[name])


def test_tied_head_reuses_the_embedding_file_range(tmp_path):
    weights = small_weights()
    weights.lm_head = weights.embeddings
    write_checkpoint(str(tmp_path), weights, "qwen3", shards=1, tied=True)
    plan = ckpt.plan_checkpoint(str(tmp_path))
    assert plan.entries[-1][0] == "model.embed_tokens.weight" and plan.entries[-1][2] == plan.entries[0][2]
    assert plan.blocks[len(plan.blocks) - 1].offset_bytes + weights.embeddings.nbytes == plan.fields()["planned_weight_bytes"]


def test_header_and_manifest_mismatches_are_refused(tmp_path):
    weights = small_weights()
    root = str(tmp_path / "ok")
    write_checkpoint(root, weights, "qwen3", shards=2)
    ckpt.plan_checkpoint(root)

    def broken(name, change):
        path = str(tmp_path / name)
        write_checkpoint(path, weights, "qwen3", shards=1)
        file = os.path.join(path, "model.safetensors")
        header, start = ckpt.read_safetensors_header(file)
        with open(file, "rb") as f:
            f.seek(start)
            data = f.read()
        change(header)
        text = json.dumps(header).encode()
        with open(file, "wb") as f:
            f.write(len(text).to_bytes(8, "little") + text + data)
        return path

    def missing(h): del h["model.layers.1.mlp.up_proj.weight"]
    def dtype(h): h["model.norm.weight"]["dtype"] = "F16"
    def shape(h): h["model.layers.0.self_attn.k_proj.weight"]["shape"] = [32, 128]
    def span(h): h["lm_head.weight"]["data_offsets"][1] -= 2
    def backwards(h): h["lm_head.weight"]["data_offsets"] = h["lm_head.weight"]["data_offsets"][::-1]
    def beyond(h):
        size = h["lm_head.weight"]["data_offsets"][1] - h["lm_head.weight"]["data_offsets"][0]
        h["lm_head.weight"]["data_offsets"] = [10 ** 9, 10 ** 9 + size]
    for change in (missing, dtype, shape, span, backwards, beyond):
        with pytest.raises(ckpt.CheckpointError):
            ckpt.plan_checkpoint(broken(change.__name__, change))
    # header length beyond the file, index without the tensor, no checkpoint at all
    cut = str(tmp_path / "cut")
    write_checkpoint(cut, weights, "qwen3", shards=1)
    with open(os.path.join(cut, "model.safetensors"), "r+b") as f:
        f.write((10 ** 8 + 1).to_bytes(8, "little"))
    with pytest.raises(ckpt.CheckpointError):
        ckpt.plan_checkpoint(cut)
    index = os.path.join(root, "model.safetensors.index.json")
    with open(index) as f:
        doc = json.load(f)
    del doc["weight_map"]["model.norm.weight"]
    with open(index, "w") as f:
        json.dump(doc, f)
    with pytest.raises(ckpt.CheckpointError):
        ckpt.plan_checkpoint(root)
    empty = str(tmp_path / "empty")
    os.makedirs(empty)
    with open(os.path.join(empty, "config.json"), "w") as f:
        json.dump(dict(model_type="qwen3", torch_dtype="bfloat16", hidden_size=64, num_attention_heads=4,
                       intermediate_size=96, vocab_size=50, num_hidden_layers=1), f)
    with pytest.raises(ckpt.CheckpointError):
        ckpt.plan_checkpoint(empty)
