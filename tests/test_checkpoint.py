"""Checkpoint loader (host logic): a synthetic model written in the reference's layout and names
(SeedlessEngine.swift:33-144; shards + index as WeightStore reads them, QwispModel.swift:25-44) comes back as the
same model; dtype conventions follow SeedlessFusedVerify.swift:2808-2819."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import orc
from qwisp_amd import checkpoint
from qwisp_amd.synth import ModelConfig


def arr(x):
    return x.numpy() if hasattr(x, "numpy") else x


def bits(x):
    a = np.ascontiguousarray(arr(x))
    return a.view(np.uint8).reshape(-1)


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = ModelConfig(n_layers=4, n_experts=16, vocab=2048, gate_bits=8, norm_f32=True)
    t = orc.generate_host(cfg)
    d = str(tmp_path_factory.mktemp("ckpt"))
    out = dict(t)
    # what a converted checkpoint may hold: scales / biases and small vectors in other float types
    out["layers.0.linear_attn.in_proj_qkv.scales"] = torch.from_numpy(t["layers.0.linear_attn.in_proj_qkv.scales"]).float()
    out["layers.1.mlp.switch_mlp.up_proj.biases"] = torch.from_numpy(t["layers.1.mlp.switch_mlp.up_proj.biases"]).float()
    out["layers.0.input_layernorm.weight"] = torch.from_numpy(t["layers.0.input_layernorm.weight"]).float()
    out["layers.0.linear_attn.A_log"] = torch.from_numpy(t["layers.0.linear_attn.A_log"]).double()
    out["vision_tower.blocks.0.attn.qkv.weight"] = torch.zeros(4, 4)
    checkpoint.save_checkpoint(d, out, shard_bytes=8 << 20)
    return cfg, t, d


def test_layout_on_disk(model):
    cfg, t, d = model
    idx = json.load(open(os.path.join(d, "model.safetensors.index.json")))["weight_map"]
    assert len(set(idx.values())) > 1                                         # several shards
    assert "language_model.model.layers.0.mlp.switch_mlp.gate_proj.weight" in idx
    assert "language_model.lm_head.weight" in idx and "language_model.model.embed_tokens.scales" in idx
    assert "language_model.model.layers.3.self_attn.q_norm.weight" in idx
    from safetensors import safe_open
    with safe_open(os.path.join(d, idx["language_model.model.layers.0.mlp.switch_mlp.down_proj.weight"]), framework="pt") as f:
        assert tuple(f.get_tensor("language_model.model.layers.0.mlp.switch_mlp.down_proj.weight").shape) == (16, 2048, 64)
    with safe_open(os.path.join(d, idx["language_model.model.layers.0.linear_attn.conv1d.weight"]), framework="pt") as f:
        assert tuple(f.get_tensor("language_model.model.layers.0.linear_attn.conv1d.weight").shape) == (8192, 4, 1)


def test_round_trip_gives_the_same_model(model):
    cfg, t, d = model
    cfg2, t2 = checkpoint.load_checkpoint(d)
    assert (cfg2.n_layers, cfg2.n_experts, cfg2.vocab, cfg2.gate_bits, cfg2.norm_f32) == (4, 16, 2048, 8, True)
    assert [cfg2.is_linear(i) for i in range(4)] == [True, True, True, False]
    assert not any("vision" in k for k in t2) and set(t2) == set(t)
    for k in t:
        a, b = arr(t2[k]), t[k]
        assert a.shape == b.shape, k
        assert a.dtype.itemsize == b.dtype.itemsize and np.array_equal(bits(a), bits(b)), k
    assert t2["layers.0.linear_attn.in_proj_qkv.scales"].dtype == torch.float16
    assert t2["layers.0.linear_attn.norm.weight"].dtype == torch.float32
    assert t2["layers.0.linear_attn.A_log"].dtype == torch.float32
    assert t2["layers.0.mlp.gate.weight"].dtype == torch.int32 and tuple(t2["layers.0.mlp.gate.weight"].shape) == (16, 512)
    # and it runs: the loaded model and the original give the same tokens on the CPU oracle
    a = orc.Oracle(cfg, t, max_m=4, max_seq_len=32)
    b = orc.Oracle(cfg2, t2, max_m=4, max_seq_len=32)
    prompt = [3, 1500, 77, 9]
    assert a.greedy_generate(prompt, 6).tolist() == b.greedy_generate(prompt, 6).tolist()


def test_bf16_is_rounded_to_half_and_bad_shapes_are_refused(tmp_path):
    cfg = ModelConfig(n_layers=1, n_experts=8, vocab=0, layer_types=("gdn",))
    t = orc.generate_host(cfg)
    out = dict(t)
    s = torch.from_numpy(t["layers.0.linear_attn.out_proj.scales"]).to(torch.bfloat16)
    out["layers.0.linear_attn.out_proj.scales"] = s
    checkpoint.save_checkpoint(str(tmp_path / "a"), out)
    cfg2, t2 = checkpoint.load_checkpoint(str(tmp_path / "a"))
    assert cfg2.gate_bits == 16 and cfg2.n_layers == 1 and cfg2.is_linear(0) and cfg2.vocab == 0
    assert torch.equal(t2["layers.0.linear_attn.out_proj.scales"], s.to(torch.float16))
    assert tuple(t2["layers.0.mlp.shared_expert_gate.weight"].shape) == (2048,)
    bad = dict(t)
    bad["layers.0.linear_attn.in_proj_z.weight"] = t["layers.0.linear_attn.in_proj_z.weight"][:, :128]
    checkpoint.save_checkpoint(str(tmp_path / "b"), bad)
    with pytest.raises(ValueError, match="in_proj_z"):
        checkpoint.load_checkpoint(str(tmp_path / "b"))
    with pytest.raises(FileNotFoundError):
        checkpoint.load_checkpoint(str(tmp_path / "nothing"))
