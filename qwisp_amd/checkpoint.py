"""Checkpoints in the layout the reference loads (MLX-format safetensors shards + model.safetensors.index.json;
WeightStore, QwispModel.swift:25-44, and the tensor names of SeedlessEngine.swift:33-144).

`load_checkpoint(dir)` returns (ModelConfig, {name: tensor}) ready for `SeedlessFusedForward(cfg, tensors)`:

* names lose their `language_model.model.` / `language_model.` prefix; vision-tower tensors are skipped
  (QwispModel.swift:21-23);
* packed weights stay uint32; scales and biases become fp16 and `conv1d.weight`, `A_log`, `dt_bias` fp32, as the
  reference casts them when it builds its buffers (SeedlessFusedVerify.swift:2808-2819);
* `linear_attn.norm.weight` stays fp32 when stored so (the gated norm then runs its fp32-weight variant,
  SeedlessFusedVerify.swift:2815), every other norm weight becomes fp16;
* the router (`mlp.gate`) and `mlp.shared_expert_gate` may be 8-bit (released checkpoint) or plain fp16 rows;
  every other matrix must be 4-bit, group 64.

Norm weights are used as stored (direct multipliers, the MLX convention).  Nothing is executed from the files:
safetensors only.  `save_checkpoint` writes a model description back in the same layout.
"""
import json
import os

import numpy as np

from . import abi
from .synth import ModelConfig

PREFIX_MODEL = "language_model.model."
PREFIX_HEAD = "language_model."


def _internal_name(name):
    if name.startswith("vision_tower") or "visual" in name:
        return None
    if name.startswith(PREFIX_MODEL):
        return name[len(PREFIX_MODEL):]
    if name.startswith(PREFIX_HEAD):
        return name[len(PREFIX_HEAD):]
    return name


def _want_dtype(name, stored):
    import torch
    if name.endswith(".scales") or name.endswith(".biases"):
        return torch.float16
    if name.endswith("conv1d.weight") or name.endswith("A_log") or name.endswith("dt_bias"):
        return torch.float32
    if name.endswith("linear_attn.norm.weight"):
        return torch.float32 if stored == torch.float32 else torch.float16
    if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
        return torch.float16
    if name.endswith(".weight") and stored in (torch.uint32, torch.int32):
        return torch.int32                      # packed words; torch has no arithmetic on uint32, bits are what matters
    if name.endswith(".weight"):
        return torch.float16                    # unquantised rows (fp16 router / shared gate)
    return stored


def load_checkpoint(model_dir, device=None):
    """Reads every shard named by model.safetensors.index.json (or every *.safetensors file when there is no
    index) tensor by tensor.  `device` (e.g. "cuda:0") places the tensors there; default is host memory."""
    import torch
    from safetensors import safe_open
    idx = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(idx):
        with open(idx) as f:
            shards = sorted(set(json.load(f)["weight_map"].values()))
    else:
        shards = sorted(n for n in os.listdir(model_dir) if n.endswith(".safetensors"))
    if not shards:
        raise FileNotFoundError(f"no safetensors shards in {model_dir}")
    t = {}
    for shard in shards:
        with safe_open(os.path.join(model_dir, shard), framework="pt") as f:
            for key in f.keys():
                name = _internal_name(key)
                if name is None:
                    continue
                x = f.get_tensor(key)
                want = _want_dtype(name, x.dtype)
                if x.dtype == torch.uint32:
                    x = x.view(torch.int32)
                elif x.dtype != want:
                    x = x.to(want)
                if name.endswith("conv1d.weight"):
                    x = x.reshape(x.shape[0], -1)
                if name.endswith("shared_expert_gate.weight") and x.dtype == torch.float16:
                    x = x.reshape(-1)
                t[name] = x.contiguous().to(device) if device else x.contiguous()
    cfg = _infer_config(model_dir, t)
    _validate(cfg, t)
    return cfg, t


def _infer_config(model_dir, t):
    n_layers = 1 + max(int(k.split(".")[1]) for k in t if k.startswith("layers."))
    interval = 4
    cj = os.path.join(model_dir, "config.json")
    if os.path.exists(cj):
        with open(cj) as f:
            c = json.load(f)
        c = c.get("text_config", c)
        interval = int(c.get("full_attention_interval", interval))
    types = tuple("gdn" if f"layers.{i}.linear_attn.in_proj_qkv.weight" in t else "attn" for i in range(n_layers))
    regular = all((types[i] == "attn") == ((i + 1) % interval == 0) for i in range(n_layers))
    gate = t["layers.0.mlp.gate.weight"]
    vocab = int(t["lm_head.weight"].shape[0]) if "lm_head.weight" in t else 0
    gdn0 = next((i for i in range(n_layers) if types[i] == "gdn"), None)
    norm_f32 = gdn0 is not None and "float32" in str(t[f"layers.{gdn0}.linear_attn.norm.weight"].dtype)
    return ModelConfig(n_layers=n_layers, n_experts=int(gate.shape[0]), vocab=vocab, full_attn_interval=interval,
                       layer_types=None if regular else types,
                       gate_bits=8 if "layers.0.mlp.gate.scales" in t else 16, norm_f32=norm_f32)


def _validate(cfg, t):
    """Shapes against the fixed geometry of the engine; a clear error beats a device fault."""
    H, I, E = abi.H, abi.MOE_I, cfg.n_experts

    def q4(name, n, k):
        w, s, b = t[name + ".weight"], t[name + ".scales"], t[name + ".biases"]
        if tuple(w.shape) != (n, k // 8) or tuple(s.shape) != (n, k // 64) or tuple(b.shape) != (n, k // 64):
            raise ValueError(f"{name}: expected 4-bit group-64 [{n}, {k}], found weight {tuple(w.shape)} scales {tuple(s.shape)}")

    def reshape3(name, n, k):      # expert stacks may be stored [E, rows, words]
        for suf, cols in ((".weight", k // 8), (".scales", k // 64), (".biases", k // 64)):
            if t[name + suf].dim() == 3:
                t[name + suf] = t[name + suf].reshape(n, cols)

    if cfg.vocab:
        q4("embed_tokens", cfg.vocab, H)
        q4("lm_head", cfg.vocab, H)
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        if cfg.is_linear(i):
            la = p + "linear_attn."
            q4(la + "in_proj_qkv", abi.CONV_DIM, H); q4(la + "in_proj_z", abi.GDN_HV * abi.GDN_D, H)
            q4(la + "in_proj_b", abi.GDN_HV, H); q4(la + "in_proj_a", abi.GDN_HV, H)
            q4(la + "out_proj", H, abi.GDN_HV * abi.GDN_D)
            if tuple(t[la + "conv1d.weight"].shape) != (abi.CONV_DIM, abi.CONV_K):
                raise ValueError(f"{la}conv1d.weight: {tuple(t[la + 'conv1d.weight'].shape)}")
        else:
            sa = p + "self_attn."
            q4(sa + "q_proj", abi.ATT_HEADS * 2 * abi.ATT_D, H); q4(sa + "k_proj", abi.ATT_KV * abi.ATT_D, H)
            q4(sa + "v_proj", abi.ATT_KV * abi.ATT_D, H); q4(sa + "o_proj", H, abi.ATT_HEADS * abi.ATT_D)
        mp = p + "mlp."
        for nm, n, k in (("switch_mlp.gate_proj", E * I, H), ("switch_mlp.up_proj", E * I, H), ("switch_mlp.down_proj", E * H, I)):
            reshape3(mp + nm, n, k)
            q4(mp + nm, n, k)
        q4(mp + "shared_expert.gate_proj", I, H); q4(mp + "shared_expert.up_proj", I, H); q4(mp + "shared_expert.down_proj", H, I)
        if cfg.gate_bits == 8:
            for nm, n in (("gate", E), ("shared_expert_gate", 1)):
                w = t[mp + nm + ".weight"]
                if tuple(w.shape) != (n, H // 4) or tuple(t[mp + nm + ".scales"].shape) != (n, H // 64):
                    raise ValueError(f"{mp}{nm}: expected 8-bit group-64 [{n}, {H}], found weight {tuple(w.shape)}")
        elif tuple(t[mp + "gate.weight"].shape) != (E, H):
            raise ValueError(f"{mp}gate.weight: {tuple(t[mp + 'gate.weight'].shape)}")


def save_checkpoint(model_dir, tensors, shard_bytes=1 << 30, full_attention_interval=4):
    """Writes {internal name: numpy array or torch tensor} as safetensors shards with the reference's names and
    an index file; expert stacks go out as [E, rows, words] like the released checkpoint."""
    import torch
    from safetensors.torch import save_file
    os.makedirs(model_dir, exist_ok=True)
    shards, cur, cur_bytes, weight_map = [], {}, 0, {}
    for name in sorted(tensors):
        x = tensors[name]
        if isinstance(x, np.ndarray):
            x = torch.from_numpy(x.view(np.int32) if x.dtype == np.uint32 else x)
        x = x.detach().cpu().contiguous()
        if ".switch_mlp." in name:
            E = int(tensors[name.split("switch_mlp.")[0] + "gate.weight"].shape[0])
            x = x.reshape(E, x.shape[0] // E, x.shape[1])
        if name.endswith("conv1d.weight"):
            x = x.reshape(x.shape[0], x.shape[1], 1)
        if name.endswith("shared_expert_gate.weight") and x.dim() == 1:
            x = x.reshape(1, -1)
        key = name if name.startswith("vision_tower") else (PREFIX_HEAD if name.startswith("lm_head.") else PREFIX_MODEL) + name
        nbytes = x.numel() * x.element_size()
        if cur and cur_bytes + nbytes > shard_bytes:
            shards.append(cur); cur, cur_bytes = {}, 0
        cur[key] = x
        cur_bytes += nbytes
    if cur:
        shards.append(cur)
    for i, sh in enumerate(shards):
        fn = f"model-{i + 1:05d}-of-{len(shards):05d}.safetensors"
        save_file(sh, os.path.join(model_dir, fn))
        for key in sh:
            weight_map[key] = fn
    with open(os.path.join(model_dir, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump({"text_config": {"full_attention_interval": full_attention_interval}}, f)
