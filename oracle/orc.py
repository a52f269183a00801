"""TEST INFRASTRUCTURE — ctypes binding of the CPU oracle (libseedless_oracle.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from qwisp_amd import abi
from qwisp_amd.synth import tensor_specs

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libseedless_oracle.so")


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "-s"])


def _load():
    if not os.path.exists(_SO):
        build()
    dll = C.CDLL(_SO)
    f32, i32, i64, u64, vp = C.c_float, C.c_int32, C.c_int64, C.c_uint64, C.c_void_p
    sig = {
        "orc_create": (vp, [C.POINTER(abi.ModelDesc), i32, i32]),
        "orc_destroy": (None, [vp]),
        "orc_position": (i32, [vp]),
        "orc_forward_rows": (i32, [vp, vp, i32, i32, vp]),
        "orc_step_argmax": (i32, [vp, vp, i32, vp]),
        "orc_forward_tokens": (i32, [vp, vp, i32, vp]),
        "orc_head_argmax": (i32, [vp, vp, i32, vp]),
        "orc_chained_step_argmax": (i32, [vp, i32, i32, vp]),
        "orc_greedy_generate": (i32, [vp, vp, i32, i32, vp]),
        "orc_logits_row": (i32, [vp, i32, vp]),
        "orc_hidden_rows": (i32, [vp, i32, vp]),
        "orc_read_route": (i32, [vp, i32, i32, vp, vp]),
        "orc_read_layer_cache": (i32, [vp, i32, vp, vp]),
        "orc_load_layer_cache": (i32, [vp, i32, vp, vp, i32]),
        "orc_rollback_one_step": (i32, [vp, i32]),
        "orc_moe_block_rows": (i32, [vp, i32, vp, i32, vp]),
        "orc_gdn_layer_rows": (i32, [vp, i32, vp, i32, vp]),
        "orc_attn_layer_rows": (i32, [vp, i32, vp, i32, vp]),
        "orc_exp": (f32, [f32]), "orc_log": (f32, [f32]), "orc_sigmoid32": (f32, [f32]),
        "orc_sigmoid16": (f32, [f32]), "orc_softplus": (f32, [f32]), "orc_ppnd7": (f32, [f32]),
        "orc_f16r": (f32, [f32]), "orc_f2h": (C.c_uint16, [f32]), "orc_f2h_soft": (C.c_uint16, [f32]),
        "orc_h2f": (f32, [C.c_uint16]), "orc_h2f_soft": (f32, [C.c_uint16]),
        "orc_hash64": (u64, [u64, u64]), "orc_normal01": (f32, [u64, u64]),
        "orc_exp_vec": (None, [vp, vp, i64]), "orc_log_vec": (None, [vp, vp, i64]),
        "orc_ppnd7_vec": (None, [vp, vp, i64]),
        "orc_map_vec": (None, [i32, vp, vp, i64]),
        "orc_qmv": (None, [vp, vp, vp, vp, i32, i32, vp]),
        "orc_qmv_f32": (None, [vp, vp, vp, vp, i32, i32, vp]),
        "orc_dense_f16": (None, [vp, vp, i32, i32, vp]),
        "orc_q8_f32": (None, [vp, vp, vp, vp, i32, i32, vp]),
        "orc_rmsnorm": (None, [vp, vp, i32, vp]),
        "orc_route": (None, [vp, i32, vp, vp]),
        "orc_swiglu": (None, [vp, vp, i32, vp]),
        "orc_sdpa": (None, [vp, vp, vp, i32, vp]),
        "orc_rope_entry": (None, [i32, i32, C.POINTER(f32), C.POINTER(f32)]),
        "orc_norm_rope": (None, [vp, vp, i32, vp]),
        "orc_delta_step": (None, [vp, vp, vp, vp, vp, vp, i32, i32, vp]),
        "orc_gdn_beta": (f32, [f32]), "orc_gdn_decay": (f32, [f32, f32, f32]),
        "orc_conv_silu": (f32, [vp, vp]),
        "orc_synth_q4": (None, [vp, vp, vp, i64, i32, u64, f32]),
        "orc_synth_f16": (None, [vp, i64, u64, f32, f32]),
        "orc_synth_f32": (None, [vp, i64, u64, f32, f32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(dll, name)
        fn.restype, fn.argtypes = res, args
    return dll


dll = _load()


def p(a):
    return a.ctypes.data if a is not None else None


# ---- synthetic tensors on the host ---------------------------------------------------------------
def synth_q4(n, k, seed, sigma=0.02):
    w = np.empty((n, k // 8), np.uint32)
    s = np.empty((n, k // 64), np.float16)
    b = np.empty((n, k // 64), np.float16)
    dll.orc_synth_q4(p(w), p(s), p(b), n, k, seed, sigma)
    return w, s, b


def synth_f16(shape, seed, mean, sigma):
    x = np.empty(shape, np.float16)
    dll.orc_synth_f16(p(x), x.size, seed, mean, sigma)
    return x


def synth_f32(shape, seed, mean, sigma):
    x = np.empty(shape, np.float32)
    dll.orc_synth_f32(p(x), x.size, seed, mean, sigma)
    return x


def generate_host(cfg):
    """dict name -> numpy array for the synthetic model `cfg` (same names as generate_device)."""
    t = {}
    for name, kind, shape, seed, mean, sigma in tensor_specs(cfg):
        if kind == "q4":
            t[name + ".weight"], t[name + ".scales"], t[name + ".biases"] = synth_q4(shape[0], shape[1], seed, sigma)
        elif kind == "f16":
            t[name] = synth_f16(shape, seed, mean, sigma)
        else:
            t[name] = synth_f32(shape, seed, mean, sigma)
    if getattr(cfg, "gate_bits", 16) == 8:      # the two gates re-expressed in 8 bits, as generate_device does
        from qwisp_amd.synth import quantize_q8
        for i in range(cfg.n_layers):
            for nm in (f"layers.{i}.mlp.gate", f"layers.{i}.mlp.shared_expert_gate"):
                t[nm + ".weight"], t[nm + ".scales"], t[nm + ".biases"] = quantize_q8(t[nm + ".weight"].reshape(-1, 2048))
    return t


def dequant(w, s, b):
    """float64 dequantised matrix [n, k] from MLX-affine 4-bit tensors."""
    n, wpr = w.shape
    nib = (w[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))[None, None, :]) & 15
    q = nib.reshape(n, wpr * 8).astype(np.float64)
    return q * np.repeat(s.astype(np.float64), 64, axis=1) + np.repeat(b.astype(np.float64), 64, axis=1)


class Oracle:
    """CPU engine with the surface of qwisp_amd.engine.SeedlessFusedForward."""

    def __init__(self, cfg, tensors, max_m=8, max_seq_len=1024):
        self.cfg = cfg
        self.max_m, self.max_seq_len = max_m, max_seq_len
        self.tensors = {k: np.ascontiguousarray(v) for k, v in tensors.items()}
        self.desc, self._keep = abi.build_desc(cfg, self.tensors, abi.SL_LOC_HOST)
        self.h = dll.orc_create(C.byref(self.desc), max_m, max_seq_len)
        if not self.h:
            raise RuntimeError("orc_create failed")

    def close(self):
        if self.h:
            dll.orc_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    @staticmethod
    def _chk(r, what):
        if r != 0:
            raise RuntimeError(f"{what} -> {r}")

    @property
    def position(self):
        return dll.orc_position(self.h)

    def step_argmax(self, tokens):
        tok = np.asarray(tokens, np.int32)
        out = np.empty(len(tok), np.int32)
        self._chk(dll.orc_step_argmax(self.h, p(tok), len(tok), p(out)), "orc_step_argmax")
        return out

    def chained_step_argmax(self, first, k):
        out = np.empty(k, np.int32)
        self._chk(dll.orc_chained_step_argmax(self.h, int(first), k, p(out)), "orc_chained_step_argmax")
        return out

    def forward_rows(self, x, final_norm=False):
        x = np.ascontiguousarray(x, np.float16)
        out = np.empty_like(x)
        self._chk(dll.orc_forward_rows(self.h, p(x), x.shape[0], int(final_norm), p(out)), "orc_forward_rows")
        return out

    def forward_tokens(self, tokens):
        tok = np.asarray(tokens, np.int32)
        out = np.empty((len(tok), abi.H), np.float16)
        self._chk(dll.orc_forward_tokens(self.h, p(tok), len(tok), p(out)), "orc_forward_tokens")
        return out

    def head_argmax(self, normed):
        x = np.ascontiguousarray(normed, np.float16).reshape(-1, abi.H)
        out = np.empty(x.shape[0], np.int32)
        self._chk(dll.orc_head_argmax(self.h, p(x), x.shape[0], p(out)), "orc_head_argmax")
        return out

    def greedy_generate(self, prompt, n_new):
        pr = np.asarray(prompt, np.int32)
        out = np.empty(n_new, np.int32)
        self._chk(dll.orc_greedy_generate(self.h, p(pr), len(pr), n_new, p(out)), "orc_greedy_generate")
        return out

    def logits_row(self, m):
        out = np.empty(self.cfg.vocab, np.float16)
        self._chk(dll.orc_logits_row(self.h, m, p(out)), "orc_logits_row")
        return out

    def hidden_rows(self, m):
        out = np.empty((m, abi.H), np.float16)
        self._chk(dll.orc_hidden_rows(self.h, m, p(out)), "orc_hidden_rows")
        return out

    def read_route(self, layer, m):
        inds = np.empty((m, abi.TOPK), np.int32)
        sc = np.empty((m, abi.TOPK), np.float16)
        self._chk(dll.orc_read_route(self.h, layer, m, p(inds), p(sc)), "orc_read_route")
        return inds, sc

    def read_layer_cache(self, layer):
        if self.cfg.is_linear(layer):
            a = np.empty((abi.CONV_K - 1, abi.CONV_DIM), np.float16)
            b = np.empty((abi.GDN_HV, abi.GDN_D, abi.GDN_D), np.float32)
        else:
            n = self.position
            a = np.empty((abi.ATT_KV, n, abi.ATT_D), np.float16)
            b = np.empty((abi.ATT_KV, n, abi.ATT_D), np.float16)
        self._chk(dll.orc_read_layer_cache(self.h, layer, p(a), p(b)), "orc_read_layer_cache")
        return a, b

    def load_layer_cache(self, layer, a, b):
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b)
        n = 0 if self.cfg.is_linear(layer) else a.shape[1]
        self._chk(dll.orc_load_layer_cache(self.h, layer, p(a), p(b), n), "orc_load_layer_cache")

    def rollback_one_step(self, pos_before):
        self._chk(dll.orc_rollback_one_step(self.h, pos_before), "orc_rollback_one_step")

    def _block(self, fn, layer, x):
        x = np.ascontiguousarray(x, np.float16)
        out = np.empty_like(x)
        self._chk(fn(self.h, layer, p(x), x.shape[0], p(out)), fn.__name__)
        return out

    def moe_block_rows(self, layer, x):
        return self._block(dll.orc_moe_block_rows, layer, x)

    def gdn_layer_rows(self, layer, x):
        return self._block(dll.orc_gdn_layer_rows, layer, x)

    def attn_layer_rows(self, layer, x):
        return self._block(dll.orc_attn_layer_rows, layer, x)
