"""CPU-only checks of the boundary: the shared library loads and exports every function that
include/seedless_hip.h declares, the ctypes mirror matches the C struct layout, and the host-side
model description / byte accounting is consistent.  No compute call is made (there is no GPU here)."""
import ctypes as C
import os
import re
import subprocess
import sys
import textwrap

import numpy as np
import pytest

from qwisp_amd import abi, lib, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "seedless_hip.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(sl_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 30 and "sl_step_argmax" in names and "sl_chained_step_argmax" in names
    L = lib.get()
    for n in names:
        assert hasattr(L.dll, n), f"{n} is declared in include/seedless_hip.h but not exported"
    # and the Python binding covers exactly the declared functions
    assert sorted(lib.SIGNATURES) == names


def test_ctypes_structs_match_the_c_layout(tmp_path):
    """Compile a tiny C program against the header and compare sizeof/offsetof with ctypes."""
    prog = tmp_path / "layout.c"
    prog.write_text(textwrap.dedent("""
        #include <stdio.h>
        #include <stddef.h>
        #include "seedless_hip.h"
        int main(void) {
          printf("%zu %zu %zu %zu %zu %zu %zu\\n", sizeof(sl_q4), sizeof(sl_gdn_w), sizeof(sl_attn_w), sizeof(sl_moe_w),
                 sizeof(sl_layer_desc), sizeof(sl_model_desc), sizeof(sl_snap));
          printf("%zu %zu %zu %zu\\n", sizeof(sl_spec_options), sizeof(sl_spec_stats), sizeof(sl_spec_backend), sizeof(sl_batch_slots));
          printf("%zu %zu %zu %zu\\n", offsetof(sl_layer_desc, gdn), offsetof(sl_layer_desc, attn), offsetof(sl_layer_desc, moe),
                 offsetof(sl_model_desc, embed));
          return 0;
        }"""))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(prog)])
    out = subprocess.check_output([str(exe)]).decode().split()
    sizes = [C.sizeof(t) for t in (abi.Q4, abi.GdnW, abi.AttnW, abi.MoeW, abi.LayerDesc, abi.ModelDesc, abi.Snap,
                                   abi.SpecOptions, abi.SpecStats, abi.SpecBackend, abi.BatchSlots)]
    offs = [abi.LayerDesc.gdn.offset, abi.LayerDesc.attn.offset, abi.LayerDesc.moe.offset, abi.ModelDesc.embed.offset]
    assert [int(x) for x in out] == sizes + offs


def test_layer_pattern_and_tensor_names():
    cfg = synth.FULL_35B_A3B
    kinds = ["gdn" if cfg.is_linear(i) else "attn" for i in range(cfg.n_layers)]
    assert kinds.count("gdn") == 30 and kinds.count("attn") == 10
    assert all(k == "attn" for k in kinds[3::4])          # (i+1) % 4 == 0  (SeedlessEngine.swift:29)
    names = {n for n, *_ in synth.tensor_specs(cfg)}
    for want in ("embed_tokens", "lm_head", "norm.weight", "layers.0.linear_attn.in_proj_qkv",
                 "layers.3.self_attn.q_proj", "layers.39.mlp.switch_mlp.down_proj", "layers.0.mlp.shared_expert_gate.weight"):
        assert want in names
    seeds = [s for _, _, _, s, _, _ in synth.tensor_specs(cfg)]
    assert len(seeds) == len(set(seeds)), "every tensor has its own seed"


def test_byte_accounting_matches_the_model():
    """bench.py's algorithmic bytes per token against the tensor list (4-bit g64 = 0.5625 B/weight)."""
    sys.path.insert(0, ROOT)
    import bench
    cfg = synth.FULL_35B_A3B
    total, head = bench.step_bytes(cfg, 640)
    assert head == 248320 * 2048 * 9 // 16 == 286064640
    assert 1.82e9 < total < 1.85e9
    # resident checkpoint: about 19.5 GB
    assert 19.0e9 < synth.weight_bytes(cfg) < 20.0e9
    # a step reads 8 of 256 experts, the checkpoint holds all of them
    moe_all = 40 * 256 * 3 * 512 * 2048 * 9 // 16
    assert synth.weight_bytes(cfg) - moe_all < total


def test_desc_builder_fills_every_pointer():
    cfg = synth.ModelConfig(n_layers=4, n_experts=8, vocab=64)
    t = {}
    for name, kind, shape, *_ in synth.tensor_specs(cfg):
        if kind == "q4":
            n, k = shape
            t[name + ".weight"] = np.zeros((n, k // 8), np.uint32)
            t[name + ".scales"] = np.zeros((n, k // 64), np.float16)
            t[name + ".biases"] = np.zeros((n, k // 64), np.float16)
        else:
            t[name] = np.zeros(shape, np.float16 if kind == "f16" else np.float32)
    d, keep = abi.build_desc(cfg, t, abi.SL_LOC_HOST)
    assert d.n_layers == 4 and d.vocab == 64 and d.embed.n == 64 and d.embed.k == 2048
    for i in range(4):
        L = d.layers[i]
        assert L.input_ln and L.post_ln and L.moe.router_w and L.moe.sw_down.w
        assert L.moe.sw_gate.n == 8 * 512 and L.moe.sw_down.n == 8 * 2048 and L.moe.sw_down.k == 512
        if L.is_linear:
            assert L.gdn.in_proj_qkv.n == 8192 and L.gdn.out_proj.k == 4096 and L.gdn.conv1d_w
        else:
            assert L.attn.q_proj.n == 8192 and L.attn.k_proj.n == 512 and L.attn.q_norm


def test_engine_needs_the_gpu():
    """Without a device the engine refuses to come up (no CPU fallback)."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    cfg = synth.ModelConfig(n_layers=1, n_experts=8, vocab=0, layer_types=("gdn",))
    t = {}
    for name, kind, shape, *_ in synth.tensor_specs(cfg):
        if kind == "q4":
            n, k = shape
            t[name + ".weight"] = np.zeros((n, k // 8), np.uint32)
            t[name + ".scales"] = np.zeros((n, k // 64), np.float16)
            t[name + ".biases"] = np.zeros((n, k // 64), np.float16)
        else:
            t[name] = np.zeros(shape, np.float16 if kind == "f16" else np.float32)
    from qwisp_amd.engine import SeedlessFusedForward
    with pytest.raises(lib.SeedlessError):
        SeedlessFusedForward(cfg, t, max_m=1, max_seq_len=8)


def test_step_kernel_tags_never_meet_across_the_counter_restart():
    """The single-launch step tags what it exchanges with a counter of stage instances.  The 32-bit tags keep 31 bits
    of it, so the host restarts the counter before it gets near 2^31.  Checked here without a device: for any counter
    value from which a launch is NOT preceded by a restart, every tag of that launch is below the wrap (top bit set,
    strictly increasing with the instance, no carry into the top bit), and from the restart limit on a restart is
    always announced; 16-bit tags of the instances of one step (the farthest a slot's writer can be from its reader)
    are pairwise distinct."""
    L = lib.get()
    t16, t32 = C.c_uint32(), C.c_uint32()

    def tags(base, layer, stage, steps=1, n_layers=40):
        r = L.dll.sl_debug_flow_tags(base, layer, stage, steps, n_layers, C.byref(t16), C.byref(t32))
        return r, t16.value, t32.value

    n_layers, per_step = 40, 8 * 41
    rng = np.random.default_rng(5)
    limit = 0x7FF00000
    bases = [0, 1, per_step, 0x7FFF, 0x8000, 0x12345678] + [int(b) for b in rng.integers(0, limit, 200)]
    # the last counter values from which launches of 1 and of 256 steps still run without a restart
    for steps in (1, 8, 256):
        last = limit - (steps + 1) * per_step
        bases += [last - 1, last]
        assert tags(last, 0, 0, steps)[0] == 0 and tags(last + 1, 0, 0, steps)[0] == 1
        assert tags(0xFFFFFFFF, 0, 0, steps)[0] == 1 and tags(0x80000000, 0, 0, steps)[0] == 1
    for base in bases:
        for steps in (1, 256):
            restart, _, _ = tags(base, 0, 0, steps)
            if restart:
                continue
            # first and last stage instance the launch touches (the token hand-over of the step after the last uses
            # stage 7 of layer 0 at the next step's base)
            first = tags(base, 0, 0, steps)[2]
            end_base = base + steps * per_step
            last = tags(end_base, 0, 7, steps)[2]
            assert first == (0x80000000 | base) and last == (0x80000000 | (end_base + 7))
            assert end_base + per_step < 2 ** 31, "no carry into the tag's top bit"
            assert last > first
    # 16-bit tags: the instances of two consecutive steps never share a tag, and the top bit is always set
    for base in (0, 0x7FF0, 0x7FFF, 0x8000, limit - 3 * per_step):
        seen = {}
        for step in range(2):
            for layer in range(n_layers + 1):
                for stage in range(8):
                    t = tags(base + step * per_step, layer, stage)[1]
                    assert t & 0x8000 and t < 0x10000
                    assert t not in seen, (base, step, layer, stage, seen[t])
                    seen[t] = (step, layer, stage)
