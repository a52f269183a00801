"""ctypes mirror of include/seedless_hip.h: status codes, the model-description structs and a
builder that fills them from named tensors (numpy arrays or torch tensors).

Tensor names follow the checkpoint naming the reference reads in SeedlessEngine.swift:33-144
(`language_model.model.layers.{i}.linear_attn.in_proj_qkv.weight`, ...), shortened to the part
after `layers.{i}.` for per-layer tensors.
"""
import ctypes as C

H = 2048
MOE_I = 512
TOPK = 8
ATT_HEADS, ATT_KV, ATT_D = 16, 2, 256
GDN_HK, GDN_HV, GDN_D = 16, 32, 128
CONV_K, CONV_DIM = 4, 8192

SL_OK, SL_ERR_ARG, SL_ERR_POISONED, SL_ERR_DEVICE, SL_ERR_UNSUPPORTED, SL_ERR_FORMAT, SL_ERR_TOO_LARGE = 0, -1, -2, -3, -4, -5, -6
SL_LOC_HOST, SL_LOC_DEVICE = 0, 1


class Q4(C.Structure):
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
                ("n", C.c_int32), ("k", C.c_int32)]


class GdnW(C.Structure):
    _fields_ = [("in_proj_qkv", Q4), ("in_proj_z", Q4), ("in_proj_b", Q4), ("in_proj_a", Q4),
                ("out_proj", Q4), ("conv1d_w", C.c_void_p), ("norm_w", C.c_void_p),
                ("a_log", C.c_void_p), ("dt_bias", C.c_void_p), ("norm_w_f32", C.c_void_p)]


class AttnW(C.Structure):
    _fields_ = [("q_proj", Q4), ("k_proj", Q4), ("v_proj", Q4), ("o_proj", Q4),
                ("q_norm", C.c_void_p), ("k_norm", C.c_void_p)]


class MoeW(C.Structure):
    _fields_ = [("router_w", C.c_void_p), ("shared_gate_w", C.c_void_p), ("router_q8", Q4), ("shared_gate_q8", Q4),
                ("sw_gate", Q4), ("sw_up", Q4), ("sw_down", Q4),
                ("sh_gate", Q4), ("sh_up", Q4), ("sh_down", Q4)]


class LayerDesc(C.Structure):
    _fields_ = [("is_linear", C.c_int32), ("input_ln", C.c_void_p), ("post_ln", C.c_void_p),
                ("gdn", GdnW), ("attn", AttnW), ("moe", MoeW)]


class ModelDesc(C.Structure):
    _fields_ = [("n_layers", C.c_int32), ("n_experts", C.c_int32), ("vocab", C.c_int32),
                ("location", C.c_int32), ("layers", C.POINTER(LayerDesc)),
                ("embed", Q4), ("lm_head", Q4), ("final_norm", C.c_void_p)]


class Snap(C.Structure):
    _fields_ = [("kv_len", C.c_int32), ("reserved", C.c_int32)]


class SpecOptions(C.Structure):
    _fields_ = [("max_draft", C.c_int32), ("chain_k", C.c_int32), ("min_match", C.c_int32), ("gate", C.c_int32),
                ("gate_reprobe", C.c_int32), ("pending_prefix", C.c_int32)]


class SpecStats(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("steps", "drafted", "accepted", "draftless", "rejects", "chain_calls",
                                         "gate_suspensions", "pending_flushes")]


STEP_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.c_int, C.POINTER(C.c_int32))
CHAIN_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int32, C.c_int, C.POINTER(C.c_int32))
FORWARD_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.c_int)
FIRST_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32))
VOID_FN = C.CFUNCTYPE(C.c_int, C.c_void_p)


class SpecBackend(C.Structure):
    _fields_ = [("ctx", C.c_void_p), ("max_rows", C.c_int32), ("step_argmax", STEP_FN), ("chained_step_argmax", CHAIN_FN),
                ("forward_tokens", FORWARD_FN), ("first_token", FIRST_FN), ("snapshot", VOID_FN), ("rollback", VOID_FN)]


ADMIT_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.c_int, C.c_int, C.c_int, C.c_int,
                       C.POINTER(C.c_int32), C.POINTER(C.c_int32))
SLOT_STEP_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_int32))
RELEASE_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_int)
CAN_ADMIT_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_int)
TOKEN_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_int, C.c_int32)
FINISH_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_int)


class BatchSlots(C.Structure):
    _fields_ = [("ctx", C.c_void_p), ("slot_count", C.c_int32), ("admit_step", ADMIT_FN), ("step", SLOT_STEP_FN),
                ("release", RELEASE_FN), ("can_admit", CAN_ADMIT_FN)]


def _ptr(t):
    """Address of a numpy array or a torch tensor."""
    if t is None:
        return None
    if hasattr(t, "data_ptr"):
        return t.data_ptr()
    return t.ctypes.data


def _is_f32(t):
    return "float32" in str(t.dtype)


def _q4(tensors, name, n, k):
    w, s, b = tensors[name + ".weight"], tensors[name + ".scales"], tensors[name + ".biases"]
    return Q4(_ptr(w), _ptr(s), _ptr(b), n, k)


def build_desc(cfg, tensors, location):
    """cfg: qwisp_amd.synth.ModelConfig-like (n_layers, n_experts, vocab, is_linear(i));
    tensors: dict name -> array.  Returns (ModelDesc, keepalive) — keepalive must outlive the
    desc's use."""
    E = cfg.n_experts
    layers = (LayerDesc * cfg.n_layers)()
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        L = layers[i]
        L.is_linear = 1 if cfg.is_linear(i) else 0
        L.input_ln = _ptr(tensors[p + "input_layernorm.weight"])
        L.post_ln = _ptr(tensors[p + "post_attention_layernorm.weight"])
        if L.is_linear:
            la = p + "linear_attn."
            L.gdn = GdnW(_q4(tensors, la + "in_proj_qkv", CONV_DIM, H),
                         _q4(tensors, la + "in_proj_z", GDN_HV * GDN_D, H),
                         _q4(tensors, la + "in_proj_b", GDN_HV, H),
                         _q4(tensors, la + "in_proj_a", GDN_HV, H),
                         _q4(tensors, la + "out_proj", H, GDN_HV * GDN_D),
                         _ptr(tensors[la + "conv1d.weight"]), None if _is_f32(tensors[la + "norm.weight"]) else _ptr(tensors[la + "norm.weight"]),
                         _ptr(tensors[la + "A_log"]), _ptr(tensors[la + "dt_bias"]),
                         _ptr(tensors[la + "norm.weight"]) if _is_f32(tensors[la + "norm.weight"]) else None)
        else:
            sa = p + "self_attn."
            L.attn = AttnW(_q4(tensors, sa + "q_proj", ATT_HEADS * 2 * ATT_D, H),
                           _q4(tensors, sa + "k_proj", ATT_KV * ATT_D, H),
                           _q4(tensors, sa + "v_proj", ATT_KV * ATT_D, H),
                           _q4(tensors, sa + "o_proj", H, ATT_HEADS * ATT_D),
                           _ptr(tensors[sa + "q_norm.weight"]), _ptr(tensors[sa + "k_norm.weight"]))
        mp = p + "mlp."
        if mp + "gate.scales" in tensors:      # 8-bit gates, as the released checkpoint stores them
            gates = (None, None, _q4(tensors, mp + "gate", E, H), _q4(tensors, mp + "shared_expert_gate", 1, H))
        else:                                  # fp16 gates (the benchmark configuration)
            gates = (_ptr(tensors[mp + "gate.weight"]), _ptr(tensors[mp + "shared_expert_gate.weight"]), Q4(), Q4())
        L.moe = MoeW(*gates,
                     _q4(tensors, mp + "switch_mlp.gate_proj", E * MOE_I, H),
                     _q4(tensors, mp + "switch_mlp.up_proj", E * MOE_I, H),
                     _q4(tensors, mp + "switch_mlp.down_proj", E * H, MOE_I),
                     _q4(tensors, mp + "shared_expert.gate_proj", MOE_I, H),
                     _q4(tensors, mp + "shared_expert.up_proj", MOE_I, H),
                     _q4(tensors, mp + "shared_expert.down_proj", H, MOE_I))
    d = ModelDesc()
    d.n_layers, d.n_experts, d.vocab, d.location = cfg.n_layers, E, cfg.vocab, location
    d.layers = C.cast(layers, C.POINTER(LayerDesc))
    if cfg.vocab > 0:
        d.embed = _q4(tensors, "embed_tokens", cfg.vocab, H)
        d.lm_head = _q4(tensors, "lm_head", cfg.vocab, H)
        d.final_norm = _ptr(tensors["norm.weight"])
    return d, (layers, tensors)
