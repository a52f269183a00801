"""GPU parity at the sizes the benchmark configurations name, and the arg-max tie rule.

Configuration 1: one Gated-DeltaNet layer over 1024 sequential steps.  Configuration 2: one attention layer
over a pre-filled key/value arena of 4K, 8K and 32K tokens, and a single-launch decode chain at 32K.
Configuration 3: the whole 40-layer model, 256 greedy tokens after a 512-token prompt.  Configuration 4:
32 lanes stepped together, each against its own CPU oracle; the matrix-core (hybrid) rows against the oracle
with a stated bound; at full size, lanes at 1K-16K contexts against the same lanes stepped alone.
Everything goes through the C ABI; the CPU oracle is the checker.
"""
import numpy as np
import pytest

from qwisp_amd import abi
from qwisp_amd.synth import ModelConfig
from tests.gpu_util import device_and_host_model, first_diff, same_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from oracle import orc
    from qwisp_amd import lib
    from qwisp_amd.engine import SeedlessFusedForward
    return dict(torch=torch, orc=orc, lib=lib.get(), Engine=SeedlessFusedForward)


def xrows(m, seed, scale=1.0):
    return (np.random.default_rng(seed).normal(0, scale, (m, abi.H))).astype(np.float16)


# ---- arg-max: the first of several equal maxima wins (argmax_rows, SeedlessFusedVerify.swift:583-590;
#      the reference's own test with a deliberate tie: SeedlessVerifyTests.swift:1161-1186) -------------------
def with_copies_of_row(tensors, src, dst_rows, torch=None):
    """The model's tensors with lm_head row `src` copied over rows `dst_rows` (words, scales and biases), so that
    those logits are equal bit for bit whatever the hidden state."""
    out = dict(tensors)
    for suffix in (".weight", ".scales", ".biases"):
        t = tensors["lm_head" + suffix]
        t = t.clone() if torch is not None else t.copy()
        for d in dst_rows:
            t[d] = t[src]
        out["lm_head" + suffix] = t
    return out


def tie_placements(a, vocab):
    """Rows that share the winner's four-row group of a wave, its wave, its workgroup, and none of these."""
    g = a - a % 4
    same_group = g + (a % 4 + 1) % 4
    same_wave = (a // 64) * 64 + (a % 64 + 4) % 64
    c = a // 64
    next_wave = ((c // 16) * 16 + (c % 16 + 1) % 16) * 64 + a % 64
    other_wg = (a + 3 * 1024) % vocab
    far = (a + vocab // 2 + 17) % vocab
    low = 3 if a > 3 else vocab - 5
    # the single-launch head deals groups of four rows out to its 4096 waves in turn (group g to wave g % 4096, the
    # groups left over one each to the first waves of every workgroup): a later group of the winner's wave, the wave
    # after it, and a row of the left-over groups
    turn = 4 * 4096
    later_group = (a + turn) % (vocab - vocab % turn) if vocab >= 2 * turn else far
    wave_after = (a + 4) % vocab
    left_over = vocab - 7
    return [[same_group], [same_wave], [next_wave], [other_wg], [far], [low, far], [same_group, other_wg, low],
            [later_group], [wave_after], [left_over], [later_group, left_over]]


def test_argmax_ties_go_to_the_lowest_index_on_every_path(env):
    torch, Engine, orc = env["torch"], env["Engine"], env["orc"]
    cfg = ModelConfig(n_layers=1, n_experts=8, vocab=4 * (3 * 4096 + 640), layer_types=("gdn",))   # three turns of the waves + left-over groups
    dev, host = device_and_host_model(cfg)
    eng0 = Engine(cfg, dev, max_m=32, max_seq_len=64)
    tok = 5
    a = int(eng0.step_argmax([tok])[0])
    normed = eng0.hidden_rows(1)
    top = eng0.logits_row(0)[a]
    eng0.close()
    for planted in tie_placements(a, cfg.vocab):
        want = min(planted + [a])
        d2, h2 = with_copies_of_row(dev, a, planted, torch), with_copies_of_row(host, a, planted)
        ora = orc.Oracle(cfg, h2, max_m=4, max_seq_len=8)
        assert int(ora.step_argmax([tok])[0]) == want, planted
        ol = ora.logits_row(0)
        assert all(ol[p].view(np.uint16) == top.view(np.uint16) for p in planted)
        for persistent in (True, False):                      # single-launch step / kernel-per-stage head
            e = Engine(cfg, d2, max_m=32, max_seq_len=64)
            assert e.set_persistent(persistent)
            got = e.step_argmax([tok])
            assert got is not None, e.gpu_fault
            assert int(got[0]) == want, (planted, persistent, int(got[0]), a)
            assert same_bits(e.logits_row(0), ol)
            chain = e.chained_step_argmax(tok, 2)             # the tie inside a chain: the token handed on is the same one
            assert chain is not None
            if persistent:
                for m in (1, 3, 9):                           # lm_head + arg-max over M equal rows (row-tiled kernel for M >= 2)
                    got = e.head_argmax(np.repeat(normed, m, axis=0))
                    assert got.tolist() == [want] * m, (planted, m, got.tolist())
                e.set_hybrid(True)                            # 16 rows: lm_head on the matrix cores, arg-max over the logits rows
                got = e.head_argmax(np.repeat(normed, 16, axis=0))
                lg = e.logits_row(0)
                if all(lg[p].view(np.uint16) == lg[a].view(np.uint16) for p in planted) and int(np.argmax(lg.astype(np.float32))) in planted + [a]:
                    assert got.tolist() == [want] * 16, (planted, got.tolist())
            e.close()
        ora.close()


# ---- configuration 1: 1024 sequential steps of one GDN layer ---------------------------------------------
def test_gdn_layer_1024_sequential_steps(env):
    cfg = ModelConfig(n_layers=1, n_experts=8, vocab=0, layer_types=("gdn",))
    dev, host = device_and_host_model(cfg)
    eng = env["Engine"](cfg, dev, max_m=4, max_seq_len=16)
    ora = env["orc"].Oracle(cfg, host, max_m=4, max_seq_len=16)
    state0 = env["orc"].synth_f32((abi.GDN_HV, abi.GDN_D, abi.GDN_D), 1110, 0.0, 0.1)
    hist0 = np.zeros((abi.CONV_K - 1, abi.CONV_DIM), np.float16)
    assert eng.load_layer_cache(0, hist0, state0)
    ora.load_layer_cache(0, hist0, state0)
    for t in range(1024):
        x = xrows(1, 1200 + t)
        got, want = eng.gdn_layer_rows(0, x), ora.gdn_layer_rows(0, x)
        assert got is not None, eng.gpu_fault
        assert same_bits(got, want), (t, first_diff(got, want))
    (gh, gs), (wh, ws) = eng.read_layer_cache(0), ora.read_layer_cache(0)
    assert same_bits(gh, wh), first_diff(gh, wh)
    assert same_bits(gs, ws), first_diff(gs, ws)
    assert np.isfinite(gs).all() and np.abs(gs).max() > 0


# ---- configuration 2: attention over 8K and 32K tokens of pre-filled keys and values --------------------------
# (66000 tokens, beyond the benchmark's contexts: more than 1024 key tiles, where the single-launch path merges the
# tiles on 32 workgroups again instead of on all of them)
@pytest.mark.parametrize("S", [8192, 32768, 66000])
def test_attention_layer_decode_long_arena(env, S):
    cfg = ModelConfig(n_layers=1, n_experts=8, vocab=0, layer_types=("attn",))
    dev, host = device_and_host_model(cfg)
    eng = env["Engine"](cfg, dev, max_m=4, max_seq_len=S + 16)
    ora = env["orc"].Oracle(cfg, host, max_m=4, max_seq_len=S + 16)
    k = env["orc"].synth_f16((abi.ATT_KV, S, abi.ATT_D), 1310, 0.0, 1.0)
    v = env["orc"].synth_f16((abi.ATT_KV, S, abi.ATT_D), 1311, 0.0, 1.0)
    assert eng.load_layer_cache(0, k, v)
    ora.load_layer_cache(0, k, v)
    assert eng.position == S == ora.position
    for step, m in enumerate([1, 1, 3, 4]):
        x = xrows(m, 1320 + step)
        got, want = eng.attn_layer_rows(0, x), ora.attn_layer_rows(0, x)
        assert got is not None, eng.gpu_fault
        assert same_bits(got, want), (S, step, first_diff(got, want))
    (gk, gv), (wk, wv) = eng.read_layer_cache(0), ora.read_layer_cache(0)
    assert gk.shape == (2, S + 9, 256)
    assert same_bits(gk, wk) and same_bits(gv, wv)


def test_single_launch_chain_at_32k_context_matches_oracle(env):
    """The single-launch step with 513 key tiles per head (two-pass tile units, blocked merge): a chain of 8 tokens
    on an 8-layer stack whose two attention layers start from 32768 pre-filled keys and values."""
    cfg = ModelConfig(n_layers=8, n_experts=32, vocab=8192)
    dev, host = device_and_host_model(cfg)
    S = 32768
    eng = env["Engine"](cfg, dev, max_m=1, max_seq_len=S + 32)
    ora = env["orc"].Oracle(cfg, host, max_m=1, max_seq_len=S + 32)
    for li in range(cfg.n_layers):
        if cfg.is_linear(li):
            continue
        k = env["orc"].synth_f16((abi.ATT_KV, S, abi.ATT_D), 1310 + li, 0.0, 1.0)
        v = env["orc"].synth_f16((abi.ATT_KV, S, abi.ATT_D), 1410 + li, 0.0, 1.0)
        assert eng.load_layer_cache(li, k, v)
        ora.load_layer_cache(li, k, v)
    assert eng.position == S == ora.position
    got = eng.chained_step_argmax(77, 8)
    want = ora.chained_step_argmax(77, 8)
    assert got is not None, eng.gpu_fault
    assert got.tolist() == want.tolist()
    assert same_bits(eng.logits_row(0), ora.logits_row(0))
    for li in range(cfg.n_layers):
        if not cfg.is_linear(li):
            (gk, gv), (wk, wv) = eng.read_layer_cache(li), ora.read_layer_cache(li)
            assert same_bits(gk[:, S:], wk[:, S:]) and same_bits(gv[:, S:], wv[:, S:])


# ---- configuration 3 at its stated length: 512-token prompt, 256 greedy tokens, 40 layers ------------------
def test_full_size_256_tokens_after_512_token_prompt(env):
    from qwisp_amd.synth import FULL_35B_A3B as cfg
    dev, host = device_and_host_model(cfg)
    eng = env["Engine"](cfg, dev, max_m=64, max_seq_len=800)
    del dev
    env["torch"].cuda.empty_cache()
    ora = env["orc"].Oracle(cfg, host, max_m=64, max_seq_len=800)
    prompt = np.random.default_rng(3000).integers(0, cfg.vocab, 512).astype(np.int32)
    got = eng.greedy_generate(prompt, 256, chain_k=8)
    assert got is not None, eng.gpu_fault
    want = ora.greedy_generate(prompt, 256)
    diff = np.nonzero(got != want)[0]
    assert diff.size == 0, f"streams part at token {int(diff[0])}: {got[diff[0]]} vs {want[diff[0]]}"
    assert same_bits(eng.logits_row(0), ora.logits_row(0))
    assert eng.position == ora.position == 512 + 255
    # how close the stream came to a flip: replay the last 64 tokens as single steps and look at the two best logits
    eng2 = eng.new_lane(max_m=64, max_seq_len=800)        # a second sequence on the same weights
    assert eng2.greedy_generate(prompt, 256 - 64, chain_k=8).tolist() == got[:192].tolist()
    margins, ties, cur = [], 0, int(got[191])
    for i in range(64):
        t = eng2.step_argmax([cur])
        lg = eng2.logits_row(0).astype(np.float32)
        top2 = np.partition(lg, -2)[-2:]
        margins.append(float(top2[1] - top2[0]))
        ties += int(top2[1] == top2[0])
        assert int(t[0]) == int(got[192 + i])
        cur = int(t[0])
    eng2.close()
    print(f"config 3: 256 tokens equal to the oracle's; over the last 64 steps min top-1/top-2 margin {min(margins):.4f}, "
          f"median {np.median(margins):.4f}, exact ties {ties}")


# ---- configuration 4: lanes against the oracle, hybrid rows against the oracle ----------------------------
@pytest.fixture(scope="module")
def small_model(env):
    cfg = ModelConfig(n_layers=8, n_experts=32, vocab=8192)
    dev, host = device_and_host_model(cfg)
    return cfg, dev, host


def test_32_lanes_each_equal_to_its_own_oracle(env, small_model):
    """lane_batch_bitexact / lane_batch_argmax_bitexact (SeedlessVerifyTests.swift:5429, 5543) with the CPU oracle as
    the yardstick: 32 lanes at different contexts stepped together; tokens, logits and caches of every lane."""
    cfg, dev, host = small_model
    B = 32
    base = env["Engine"](cfg, dev, max_m=B, max_seq_len=160)
    lanes = [base.new_lane(max_m=B, max_seq_len=160) for _ in range(B)]
    oras = [env["orc"].Oracle(cfg, host, max_m=B, max_seq_len=160) for _ in range(B)]
    rng = np.random.default_rng(4000)
    cur = []
    for i, (lane, ora) in enumerate(zip(lanes, oras)):
        pr = rng.integers(0, cfg.vocab, 1 + (37 * i) % 120).astype(np.int32)
        tl = tw = None
        for j in range(0, len(pr), B):
            tl, tw = lane.step_argmax(pr[j:j + B]), ora.step_argmax(pr[j:j + B])
        assert tl.tolist() == tw.tolist(), i
        cur.append(int(tl[-1]))
    for step in range(3):
        got = type(base).lane_step_argmax(lanes, cur)
        assert got is not None, [l.gpu_fault for l in lanes]
        want = [int(ora.step_argmax([t])[0]) for ora, t in zip(oras, cur)]
        assert got.tolist() == want, step
        cur = want
    for i, (lane, ora) in enumerate(zip(lanes, oras)):
        assert same_bits(lane.logits_row(0), ora.logits_row(0)), i
        assert lane.position == ora.position
        for li in range(cfg.n_layers):
            for x, y in zip(lane.read_layer_cache(li), ora.read_layer_cache(li)):
                assert same_bits(x, y), (i, li, first_diff(x, y))
    for lane in lanes:
        lane.close()
    base.close()


# The reference bounds one matrix-unit GEMM against a float64 reference by |delta| <= 2e-2 per element
# (SeedlessVerifyTests.swift:5795-5899; here: test_mfma_qmm4_against_the_oracle_rows).  Through 8 whole layers the
# deviations compound and a row whose routing flips an expert at a near-tie moves by a few per cent, so the bound on
# final-normed rows (rms about 1) is stated per row: median relative rms error 2 %, worst row 10 %.
HYBRID_REL_RMS_MEDIAN = 0.02
HYBRID_REL_RMS_WORST = 0.10
# The same after the 40 layers of the full-size model (first 64 rows of a 2048-row chunk): the random-init stack keeps
# amplifying what the first layers differ by (and with 256 experts more rows sit near a routing tie), measured 15 %
# median and 32 % worst relative rms; the bound leaves half as much again.
FULL_HYBRID_REL_RMS_MEDIAN = 0.23
FULL_HYBRID_REL_RMS_WORST = 0.50


def test_hybrid_rows_and_hybrid_lane_step_against_the_oracle(env, small_model):
    cfg, dev, host = small_model
    toks = np.random.default_rng(12).integers(0, cfg.vocab, 96).astype(np.int32)
    ora = env["orc"].Oracle(cfg, host, max_m=96, max_seq_len=128)
    want = ora.forward_tokens(toks).astype(np.float64)
    hyb = env["Engine"](cfg, dev, max_m=96, max_seq_len=128)
    hyb.set_hybrid(True)
    got = hyb.forward_tokens(toks)
    assert got is not None, hyb.gpu_fault
    got = got.astype(np.float64)
    rel = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert np.median(rel) < HYBRID_REL_RMS_MEDIAN and rel.max() < HYBRID_REL_RMS_WORST, (np.median(rel), rel.max())
    hyb.close()
    # 16 lanes stepped together with the driver in hybrid mode, each against its own oracle's logits
    B = 16
    base = env["Engine"](cfg, dev, max_m=B, max_seq_len=320)
    lanes = [base.new_lane(max_m=B, max_seq_len=320) for _ in range(B)]
    oras = [env["orc"].Oracle(cfg, host, max_m=B, max_seq_len=320) for _ in range(B)]
    rng = np.random.default_rng(4001)
    cur = []
    for i, (lane, o) in enumerate(zip(lanes, oras)):
        pr = rng.integers(0, cfg.vocab, 2 + (11 * i) % 60).astype(np.int32)
        tl = tw = None
        for j in range(0, len(pr), B):
            tl, tw = lane.step_argmax(pr[j:j + B]), o.step_argmax(pr[j:j + B])
        assert tl.tolist() == tw.tolist()
        cur.append(int(tl[-1]))
    lanes[0].set_hybrid(True)
    got = type(base).lane_step_argmax(lanes, cur)
    assert got is not None, [l.gpu_fault for l in lanes]
    agree = 0
    for i, (lane, o) in enumerate(zip(lanes, oras)):
        w = int(o.step_argmax([cur[i]])[0])
        lg, lw = lane.logits_row(0).astype(np.float64), o.logits_row(0).astype(np.float64)
        assert np.linalg.norm(lg - lw) / np.linalg.norm(lw) < 0.05, i
        agree += int(got[i]) == w
    assert agree >= B - 2, agree          # greedy tokens may differ only at near-ties
    # the matrix-core attention of a lane batch over several key tiles (k_sdpa_lane_mfma walks four tiles per workgroup
    # and the partial sums of the workgroups are merged): three of the lanes go on to contexts of 150, 220 and 300
    # tokens, their oracles with them, and the next batched step is held against the oracles' logits again
    # (the lanes' caches hold one token written by the matrix-core step above, so from here on they follow their oracles
    # to tolerance, not bit for bit: the same tokens are fed to both, the predictions may part at near-ties)
    long_ctx = {3: 150, 8: 220, 13: 300}
    for i, n in long_ctx.items():
        more = rng.integers(0, cfg.vocab, n - lanes[i].position - 1).astype(np.int32)
        same = 0
        for j in range(0, len(more), B):
            tl, tw = lanes[i].step_argmax(more[j:j + B]), oras[i].step_argmax(more[j:j + B])
            assert tl is not None, lanes[i].gpu_fault
            same += int((tl == tw).sum())
        assert same >= 0.9 * len(more), (i, same, len(more))
    cur = [int(t) for t in got]
    for i in long_ctx:
        cur[i] = 7 + i
    assert [lanes[i].position for i in sorted(long_ctx)] == [149, 219, 299]
    got = type(base).lane_step_argmax(lanes, cur)
    assert got is not None, [l.gpu_fault for l in lanes]
    agree = 0
    for i, (lane, o) in enumerate(zip(lanes, oras)):
        w = int(o.step_argmax([cur[i]])[0])
        lg, lw = lane.logits_row(0).astype(np.float64), o.logits_row(0).astype(np.float64)
        assert np.linalg.norm(lg - lw) / np.linalg.norm(lw) < 0.05, (i, lane.position)
        agree += int(got[i]) == w
    assert agree >= B - 2, agree
    for lane in lanes:
        lane.close()
    base.close()


def test_full_size_32_lanes_at_1k_to_16k_contexts_equal_solo_steps(env):
    """Configuration 4 at its stated size: 32 concurrent sequences at contexts of 1K to 16K tokens on the 40-layer
    model, prompts prefilled on the matrix cores (chunks of 256 rows; one 2048-token prompt also as a single chunk of
    2048 rows against two of 1024), a 4-row verify step on one lane.  The CPU
    oracle cannot prefill 278K tokens of the full model, so the check is the size-independent property the reference
    tests (SeedlessVerifyTests.swift:5429): a lane of the batch equals the same lane stepped alone, bit for bit; the
    oracle anchors one short lane."""
    from qwisp_amd.synth import FULL_35B_A3B as cfg
    dev, host = device_and_host_model(cfg)
    B = 32
    base = env["Engine"](cfg, dev, max_m=B, max_seq_len=64)
    del dev
    env["torch"].cuda.empty_cache()
    ctxs = [1024 + (15 * 1024 * i) // (B - 1) for i in range(B)]
    ctxs[5] = 24                                           # one short lane that the oracle can follow
    lanes = [base.new_lane(max_m=256, max_seq_len=max(ctxs) + 64) for _ in range(B)]
    twins = [base.new_lane(max_m=256, max_seq_len=max(ctxs) + 64) for _ in range(B)]
    rng = np.random.default_rng(4000)
    cur = []
    for i in range(B):
        pr = rng.integers(0, cfg.vocab, ctxs[i]).astype(np.int32)
        outs = []
        for e in (lanes[i], twins[i]):
            if ctxs[i] >= 1024:
                e.set_hybrid(True)                         # chunks on the matrix cores (deterministic: both copies get the same bits)
            o = e.greedy_generate(pr, 1, chain_k=1)
            assert o is not None, e.gpu_fault
            e.set_hybrid(False)
            outs.append(int(o[0]))
        assert outs[0] == outs[1]
        cur.append(outs[0])
        if i == 5:
            ora = env["orc"].Oracle(cfg, host, max_m=24, max_seq_len=64)
            assert int(ora.greedy_generate(pr, 1)[0]) == outs[0]
    for step in range(2):
        got = type(base).lane_step_argmax(lanes, cur)
        assert got is not None, [l.gpu_fault for l in lanes]
        want = [int(t.step_argmax([c])[0]) for t, c in zip(twins, cur)]      # alone: the single-launch step
        assert got.tolist() == want, step
        if step == 0:
            assert int(ora.step_argmax([cur[5]])[0]) == want[5]
            assert same_bits(lanes[5].logits_row(0), ora.logits_row(0))
        cur = want
    for i in (0, 5, 17, 31):
        assert same_bits(lanes[i].logits_row(0), twins[i].logits_row(0)), i
    # a 4-row verify step on a long lane equals four single steps of its twin
    rows = np.array([cur[31], 11, 222, 3333], np.int32)
    a = lanes[31].step_argmax(rows)
    b = [int(twins[31].step_argmax([int(t)])[0]) for t in rows]
    assert a is not None and a.tolist() == b
    assert same_bits(lanes[31].logits_row(3), twins[31].logits_row(0))
    for e in lanes + twins:
        e.close()
    # the 2048-token prefill chunk: one chunk of 2048 rows gives the rows of two chunks of 1024, bit for bit
    pr = np.random.default_rng(3000).integers(0, cfg.vocab, 2048).astype(np.int32)
    one, two = base.new_lane(max_m=2048, max_seq_len=2112), base.new_lane(max_m=1024, max_seq_len=2112)
    one.set_hybrid(True); two.set_hybrid(True)
    r1 = one.forward_tokens(pr)
    r2 = np.concatenate([two.forward_tokens(pr[:1024]), two.forward_tokens(pr[1024:])])
    assert r1 is not None, one.gpu_fault
    assert same_bits(r1, r2) and np.isfinite(r1.astype(np.float32)).all()
    # and the chunk's first 64 rows against the oracle's exact rows of the same 64 tokens (a row only sees the rows
    # before it, so the oracle need not follow the other 1984): 40 layers compound what 8 layers do in the bound above
    ora64 = env["orc"].Oracle(cfg, host, max_m=64, max_seq_len=64)
    w64 = ora64.forward_tokens(pr[:64]).astype(np.float64)
    rel = np.linalg.norm(r1[:64].astype(np.float64) - w64, axis=1) / np.linalg.norm(w64, axis=1)
    print("full-size hybrid chunk, first 64 rows against the oracle: median rel rms %.4f worst %.4f" % (np.median(rel), rel.max()))
    assert np.median(rel) < FULL_HYBRID_REL_RMS_MEDIAN and rel.max() < FULL_HYBRID_REL_RMS_WORST, (np.median(rel), rel.max())
    t1, t2 = one.head_argmax(r1[-1:]), two.head_argmax(r2[-1:])
    assert t1.tolist() == t2.tolist()
    assert one.chained_step_argmax(int(t1[0]), 4).tolist() == two.chained_step_argmax(int(t2[0]), 4).tolist()
    one.close(); two.close()
    base.close()


# ---- the chunked (WY) form of the gated delta rule on the matrix cores (hybrid chunks of multiples of 64 rows) -------
def test_chunked_gated_delta_rule_against_the_oracle(env):
    """Hybrid calls whose row count and start are multiples of 64 run the recurrence block-wise (k_gdn_chunk_prep /
    k_gdn_chunk_scan).  Against the oracle's sequential recurrence (GatedDelta.swift:63-124): layer output rows within
    2 % relative rms, the recurrent state within 1 %; the same rows in one call of 256
    and in calls of 64 + 192 give the same bits; a ragged call falls back to the sequential scan."""
    cfg = ModelConfig(n_layers=1, n_experts=8, vocab=0, layer_types=("gdn",))
    dev, host = device_and_host_model(cfg)
    orc = env["orc"]
    state0 = orc.synth_f32((abi.GDN_HV, abi.GDN_D, abi.GDN_D), 1110, 0.0, 0.1)
    hist0 = np.zeros((abi.CONV_K - 1, abi.CONV_DIM), np.float16)
    x = xrows(256, 4242)

    def fresh(hybrid):
        e = env["Engine"](cfg, dev, max_m=256, max_seq_len=16)
        e.set_hybrid(hybrid)
        assert e.load_layer_cache(0, hist0, state0)
        return e
    ora = orc.Oracle(cfg, host, max_m=256, max_seq_len=16)
    ora.load_layer_cache(0, hist0, state0)
    want = ora.gdn_layer_rows(0, x).astype(np.float64)
    wh, ws = ora.read_layer_cache(0)
    one = fresh(True)
    got = one.gdn_layer_rows(0, x)
    assert got is not None, one.gpu_fault
    rel = np.linalg.norm(got.astype(np.float64) - want, axis=1) / np.linalg.norm(want, axis=1)
    assert np.isfinite(got.astype(np.float32)).all() and np.median(rel) < 0.01 and rel.max() < 0.02, (np.median(rel), rel.max())
    gh, gs = one.read_layer_cache(0)
    assert np.abs(gh.astype(np.float32) - wh.astype(np.float32)).max() < 0.05     # the history holds projection rows of the matrix-core GEMM
    assert np.linalg.norm(gs.astype(np.float64) - ws) / np.linalg.norm(ws) < 0.01
    exact = fresh(False)
    ex = exact.gdn_layer_rows(0, x)
    assert not same_bits(ex, got)                       # the chunked form really ran (the exact rows equal the oracle's bits)
    two = fresh(True)
    parts = np.concatenate([two.gdn_layer_rows(0, x[:64]), two.gdn_layer_rows(0, x[64:])])
    assert same_bits(parts, got)
    for a, b in zip(two.read_layer_cache(0), one.read_layer_cache(0)):
        assert same_bits(a, b)
    rag = fresh(True)
    r1 = rag.gdn_layer_rows(0, x[:100])                 # not a multiple of 64: the sequential scan, tolerance-level GEMMs only
    relr = np.linalg.norm(r1.astype(np.float64) - want[:100], axis=1) / np.linalg.norm(want[:100], axis=1)
    assert relr.max() < 0.02
    for e in (one, exact, two, rag):
        e.close()
