"""Float64 numpy statement of the reference's MLX op graph for the decode path, written from the
graph model rather than from the raw kernels, with no intermediate fp16 rounding:
  DecoderLayer.swift:26-36, MoEBlock.swift:69-97, GatedDeltaNetLayer.swift:168-242,
  GatedDelta.swift:10-59 (`ops`), AttentionLayer.swift:62-147, ModelHead.swift:8-17,
  QwispModel.swift:141-168  (all under swift/Sources/QwispCore/).
It shares no code with oracle/; tests use it to bound the oracle's error and to catch structural
mistakes (a dropped term, a wrong index, a transposed operand) that a bit-exact self-comparison
cannot see.
"""
import numpy as np

H, I, TOPK = 2048, 512, 8
NH, NKV, HD, ROPE = 16, 2, 256, 64
HK, HV, GD, CK = 16, 32, 128, 4
EPS = 1e-6


def deq(t, name):
    w, s, b = t[name + ".weight"], t[name + ".scales"], t[name + ".biases"]
    n, wpr = w.shape
    nib = (w[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))[None, None, :]) & 15
    q = nib.reshape(n, wpr * 8).astype(np.float64)
    return q * np.repeat(s.astype(np.float64), 64, axis=1) + np.repeat(b.astype(np.float64), 64, axis=1)


def rms(x, w=None):
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + EPS)
    return y if w is None else y * w.astype(np.float64)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigmoid(x)


class RefModel:
    def __init__(self, cfg, tensors, max_seq=256):
        self.cfg, self.t = cfg, tensors
        self.pos = 0
        self.cache = {}
        for i in range(cfg.n_layers):
            if cfg.is_linear(i):
                self.cache[i] = dict(conv=np.zeros((CK - 1, 8192)), state=np.zeros((HV, GD, GD)))
            else:
                self.cache[i] = dict(k=np.zeros((NKV, 0, HD)), v=np.zeros((NKV, 0, HD)))
        self._w = {}
        self.route = {}

    def W(self, name):
        if name not in self._w:
            self._w[name] = deq(self.t, name)
        return self._w[name]

    # -- MoEBlock.swift:69-97
    def moe(self, i, x):
        p = f"layers.{i}.mlp."
        E = self.cfg.n_experts
        logits = self.t[p + "gate.weight"].astype(np.float64) @ x
        gates = np.exp(logits - logits.max())
        gates /= gates.sum()
        inds = np.argsort(-gates, kind="stable")[:TOPK]
        sc = gates[inds] / gates[inds].sum()
        self.route[i] = (inds, sc, logits)
        Wg = self.W(p + "switch_mlp.gate_proj").reshape(E, I, H)
        Wu = self.W(p + "switch_mlp.up_proj").reshape(E, I, H)
        Wd = self.W(p + "switch_mlp.down_proj").reshape(E, H, I)
        y = np.zeros(H)
        for e, s in zip(inds, sc):
            y += s * (Wd[e] @ (silu(Wg[e] @ x) * (Wu[e] @ x)))
        sh = self.W(p + "shared_expert.down_proj") @ (silu(self.W(p + "shared_expert.gate_proj") @ x)
                                                      * (self.W(p + "shared_expert.up_proj") @ x))
        g = sigmoid(self.t[p + "shared_expert_gate.weight"].astype(np.float64) @ x)
        return y + g * sh

    # -- GatedDeltaNetLayer.swift:168-242 with GatedDelta.ops (GatedDelta.swift:21-47)
    def gdn(self, i, x):
        p = f"layers.{i}.linear_attn."
        c = self.cache[i]
        qkv = self.W(p + "in_proj_qkv") @ x
        z = (self.W(p + "in_proj_z") @ x).reshape(HV, GD)
        b = self.W(p + "in_proj_b") @ x
        a = self.W(p + "in_proj_a") @ x
        win = np.concatenate([c["conv"], qkv[None, :]], axis=0)          # [4, 8192]
        c["conv"] = win[1:]
        cw = self.t[p + "conv1d.weight"].astype(np.float64)              # [8192, 4]
        conv = silu(np.einsum("kc,ck->c", win, cw))
        q = conv[:HK * GD].reshape(HK, GD)
        k = conv[HK * GD:2 * HK * GD].reshape(HK, GD)
        v = conv[2 * HK * GD:].reshape(HV, GD)
        inv = GD ** -0.5
        q = (inv * inv) * rms(q)
        k = inv * rms(k)
        q = np.repeat(q, HV // HK, axis=0)
        k = np.repeat(k, HV // HK, axis=0)
        beta = sigmoid(b)
        xa = a + self.t[p + "dt_bias"].astype(np.float64)
        g = np.exp(-np.exp(self.t[p + "A_log"].astype(np.float64)) * np.log1p(np.exp(xa)))
        S = c["state"] * g[:, None, None]                                # [hv, dv, dk]
        kv = np.einsum("hvk,hk->hv", S, k)
        delta = (v - kv) * beta[:, None]
        S = S + k[:, None, :] * delta[:, :, None]
        c["state"] = S
        y = np.einsum("hvk,hk->hv", S, q)
        out = silu(z) * rms(y, self.t[p + "norm.weight"])
        return self.W(p + "out_proj") @ out.reshape(-1)

    # -- AttentionLayer.swift:62-147 (decode branch: L = 1, no mask)
    def attn(self, i, x):
        p = f"layers.{i}.self_attn."
        c = self.cache[i]
        qo = (self.W(p + "q_proj") @ x).reshape(NH, 2 * HD)
        q, gate = qo[:, :HD], qo[:, HD:]
        k = (self.W(p + "k_proj") @ x).reshape(NKV, HD)
        v = (self.W(p + "v_proj") @ x).reshape(NKV, HD)
        q = rms(q, self.t[p + "q_norm.weight"])
        k = rms(k, self.t[p + "k_norm.weight"])
        pos = c["k"].shape[1]

        def rope(t):
            half = ROPE // 2
            freq = 1e7 ** (-np.arange(half) / half)
            ang = pos * freq
            x0, x1 = t[:, :half], t[:, half:ROPE]
            out = t.copy()
            out[:, :half] = x0 * np.cos(ang) - x1 * np.sin(ang)
            out[:, half:ROPE] = x0 * np.sin(ang) + x1 * np.cos(ang)
            return out
        q, k = rope(q), rope(k)
        c["k"] = np.concatenate([c["k"], k[:, None, :]], axis=1)
        c["v"] = np.concatenate([c["v"], v[:, None, :]], axis=1)
        out = np.zeros((NH, HD))
        for h in range(NH):
            kh, vh = c["k"][h // (NH // NKV)], c["v"][h // (NH // NKV)]
            s = (kh @ q[h]) * HD ** -0.5
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            out[h] = pr @ vh
        return self.W(p + "o_proj") @ (out * sigmoid(gate)).reshape(-1)

    # -- DecoderLayer.swift:26-36
    def layer(self, i, h):
        p = f"layers.{i}."
        n = rms(h, self.t[p + "input_layernorm.weight"])
        h = h + (self.gdn(i, n) if self.cfg.is_linear(i) else self.attn(i, n))
        n = rms(h, self.t[p + "post_attention_layernorm.weight"])
        return h + self.moe(i, n)

    def embed(self, tok):
        w = self.t["embed_tokens.weight"][tok:tok + 1]
        s = self.t["embed_tokens.scales"][tok:tok + 1]
        b = self.t["embed_tokens.biases"][tok:tok + 1]
        nib = (w[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))[None, None, :]) & 15
        return (nib.reshape(-1).astype(np.float64) * np.repeat(s.astype(np.float64), 64)
                + np.repeat(b.astype(np.float64), 64))

    def forward_hidden(self, h):
        for i in range(self.cfg.n_layers):
            h = self.layer(i, h)
        self.pos += 1
        return h

    def step(self, tok):
        """Returns (hidden, normed, logits)."""
        h = self.forward_hidden(self.embed(tok))
        n = rms(h, self.t["norm.weight"])
        return h, n, self.W("lm_head") @ n
