"""Seeded synthetic checkpoints in the reference's tensor naming (SeedlessEngine.swift:33-144).

`tensor_specs(cfg)` is the single list of (name, kind, shape, seed, mean, sigma) that defines a
synthetic model; `generate_device` materialises it in HBM with the library's generator kernels
(torch is used only to own the device memory).  Every element is a pure function of
(seed, flat index), so a host implementation of the same rule reproduces the bytes.
"""
import ctypes as C
from dataclasses import dataclass

from . import abi


@dataclass
class ModelConfig:
    n_layers: int = 40
    n_experts: int = 256
    vocab: int = 248320
    full_attn_interval: int = 4       # layer i is full attention iff (i+1) % interval == 0
    seed_base: int = 2000
    layer_types: tuple = None         # optional explicit override, e.g. ("gdn",) or ("attn",)
    gate_bits: int = 16               # 16: fp16 router / shared gate (benchmark configuration); 8: MLX affine 8-bit
    norm_f32: bool = False            # linear_attn.norm.weight in fp32 (the reference's "promote" variant of the gated norm)

    def is_linear(self, i):
        if self.layer_types is not None:
            return self.layer_types[i] == "gdn"
        return (i + 1) % self.full_attn_interval != 0


FULL_35B_A3B = ModelConfig()


def _q4(name, n, k, seed):
    return (name, "q4", (n, k), seed, 0.0, 0.02)


def tensor_specs(cfg):
    """[(name, kind, shape, seed, mean, sigma)]; kind in {"q4", "f16", "f32"}."""
    H, I, E = abi.H, abi.MOE_I, cfg.n_experts
    out = []
    if cfg.vocab > 0:
        out += [_q4("embed_tokens", cfg.vocab, H, 100), _q4("lm_head", cfg.vocab, H, 101),
                ("norm.weight", "f16", (H,), 102, 1.0, 0.1)]
    for i in range(cfg.n_layers):
        s = cfg.seed_base + 100 * i
        p = f"layers.{i}."
        out += [(p + "input_layernorm.weight", "f16", (H,), s + 0, 1.0, 0.1),
                (p + "post_attention_layernorm.weight", "f16", (H,), s + 1, 1.0, 0.1)]
        if cfg.is_linear(i):
            la = p + "linear_attn."
            out += [_q4(la + "in_proj_qkv", abi.CONV_DIM, H, s + 10),
                    _q4(la + "in_proj_z", abi.GDN_HV * abi.GDN_D, H, s + 11),
                    _q4(la + "in_proj_b", abi.GDN_HV, H, s + 12),
                    _q4(la + "in_proj_a", abi.GDN_HV, H, s + 13),
                    _q4(la + "out_proj", H, abi.GDN_HV * abi.GDN_D, s + 14),
                    (la + "conv1d.weight", "f32", (abi.CONV_DIM, abi.CONV_K), s + 15, 0.0, 0.5),
                    (la + "norm.weight", "f32" if cfg.norm_f32 else "f16", (abi.GDN_D,), s + 16, 1.0, 0.1),
                    (la + "A_log", "f32", (abi.GDN_HV,), s + 17, 0.0, 1.0),
                    (la + "dt_bias", "f32", (abi.GDN_HV,), s + 18, 0.0, 1.0)]
        else:
            sa = p + "self_attn."
            out += [_q4(sa + "q_proj", abi.ATT_HEADS * 2 * abi.ATT_D, H, s + 20),
                    _q4(sa + "k_proj", abi.ATT_KV * abi.ATT_D, H, s + 21),
                    _q4(sa + "v_proj", abi.ATT_KV * abi.ATT_D, H, s + 22),
                    _q4(sa + "o_proj", H, abi.ATT_HEADS * abi.ATT_D, s + 23),
                    (sa + "q_norm.weight", "f16", (abi.ATT_D,), s + 24, 1.0, 0.1),
                    (sa + "k_norm.weight", "f16", (abi.ATT_D,), s + 25, 1.0, 0.1)]
        mp = p + "mlp."
        out += [(mp + "gate.weight", "f16", (E, H), s + 30, 0.0, 0.02),
                (mp + "shared_expert_gate.weight", "f16", (H,), s + 31, 0.0, 0.02),
                _q4(mp + "switch_mlp.gate_proj", E * I, H, s + 32),
                _q4(mp + "switch_mlp.up_proj", E * I, H, s + 33),
                _q4(mp + "switch_mlp.down_proj", E * H, I, s + 34),
                _q4(mp + "shared_expert.gate_proj", I, H, s + 35),
                _q4(mp + "shared_expert.up_proj", I, H, s + 36),
                _q4(mp + "shared_expert.down_proj", H, I, s + 37)]
    return out


def weight_bytes(cfg):
    """Bytes of checkpoint tensors (packed weights + scales + biases + small tensors)."""
    total = 0
    for _, kind, shape, *_ in tensor_specs(cfg):
        n = 1
        for d in shape:
            n *= d
        total += {"q4": n // 2 + n // 16, "f16": 2 * n, "f32": 4 * n}[kind]
    return total


def quantize_q8(w):
    """MLX affine quantisation, 8 bits, group 64, of an fp16/fp32 matrix [n, k] (numpy).  Returns packed words
    uint32 [n, k/4] (value j of a word in bits 8j..8j+7), scales and biases fp16 [n, k/64].  Same rule as the
    4-bit generator: the group's edge with the larger magnitude is represented exactly."""
    import numpy as np
    w = np.asarray(w, np.float32)
    n, k = w.shape
    g = w.reshape(n, k // 64, 64)
    lo, hi = g.min(axis=2), g.max(axis=2)
    mask = np.abs(lo) > np.abs(hi)
    scale = np.maximum((hi - lo) / np.float32(255.0), np.float32(1e-7))
    scale = np.where(mask, scale, -scale)
    edge = np.where(mask, lo, hi)
    q0 = np.rint(edge / scale)
    nz = q0 != 0
    scale = np.where(nz, edge / np.where(nz, q0, 1), scale).astype(np.float32)
    bias = np.where(nz, edge, np.float32(0.0)).astype(np.float32)
    s16, b16 = scale.astype(np.float16), bias.astype(np.float16)
    q = np.clip(np.rint((g - bias[..., None]) / scale[..., None]), 0, 255).astype(np.uint32).reshape(n, k // 4, 4)
    words = q[..., 0] | (q[..., 1] << 8) | (q[..., 2] << 16) | (q[..., 3] << 24)
    return words.astype(np.uint32), s16, b16


def generate_device(cfg, lib, device="cuda:0"):
    """Materialise the model in HBM.  Returns dict name -> torch tensor (q4 tensors appear as
    name.weight / name.scales / name.biases)."""
    import torch
    dev = torch.device(device)
    stream = torch.cuda.current_stream(dev).cuda_stream
    t = {}
    for name, kind, shape, seed, mean, sigma in tensor_specs(cfg):
        if kind == "q4":
            n, k = shape
            w = torch.empty((n, k // 8), dtype=torch.int32, device=dev)
            s = torch.empty((n, k // 64), dtype=torch.float16, device=dev)
            b = torch.empty((n, k // 64), dtype=torch.float16, device=dev)
            lib.check(lib.dll.sl_synth_q4(w.data_ptr(), s.data_ptr(), b.data_ptr(), n, k, seed,
                                          C.c_float(sigma), stream), "sl_synth_q4")
            t[name + ".weight"], t[name + ".scales"], t[name + ".biases"] = w, s, b
        elif kind == "f16":
            x = torch.empty(shape, dtype=torch.float16, device=dev)
            lib.check(lib.dll.sl_synth_f16(x.data_ptr(), x.numel(), seed, C.c_float(mean),
                                           C.c_float(sigma), stream), "sl_synth_f16")
            t[name] = x
        else:
            x = torch.empty(shape, dtype=torch.float32, device=dev)
            lib.check(lib.dll.sl_synth_f32(x.data_ptr(), x.numel(), seed, C.c_float(mean),
                                           C.c_float(sigma), stream), "sl_synth_f32")
            t[name] = x
    torch.cuda.synchronize(dev)
    if cfg.gate_bits == 8:
        # the two gates of every layer re-expressed in 8 bits (quantised on the host: 0.5 M values per layer)
        for i in range(cfg.n_layers):
            for nm in (f"layers.{i}.mlp.gate", f"layers.{i}.mlp.shared_expert_gate"):
                w, s, b = quantize_q8(t[nm + ".weight"].float().cpu().numpy().reshape(-1, abi.H))
                t[nm + ".weight"] = torch.from_numpy(w.view("int32")).to(dev)
                t[nm + ".scales"] = torch.from_numpy(s).to(dev)
                t[nm + ".biases"] = torch.from_numpy(b).to(dev)
        torch.cuda.synchronize(dev)
    return t
