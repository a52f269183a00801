"""The entry point that allocates nothing, sl_head_argmax_noalloc, against sl_head_argmax: two calls in a row through
the C ABI, the second with fewer rows (the fixed scratch array keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest

from qwisp_amd import abi
from qwisp_amd.synth import ModelConfig
from tests.gpu_util import device_and_host_model

pytestmark = pytest.mark.gpu


def test_head_argmax_without_allocation_equals_head_argmax():
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from qwisp_amd import lib
    from qwisp_amd.engine import SeedlessFusedForward
    L = lib.get()
    cfg = ModelConfig(n_layers=1, n_experts=8, vocab=8192, layer_types=("gdn",))
    dev, _ = device_and_host_model(cfg)
    eng = SeedlessFusedForward(cfg, dev, max_m=8, max_seq_len=16)
    rng = np.random.default_rng(99)
    stream = torch.cuda.current_stream().cuda_stream

    def both(m, seed):
        x = np.random.default_rng(seed).normal(0, 1, (m, abi.H)).astype(np.float16)
        want = eng.head_argmax(x)
        assert want is not None, eng.gpu_fault
        want_logits = [eng.logits_row(i).copy() for i in range(m)]
        xd = torch.from_numpy(x).cuda()
        od = torch.full((8,), -1, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        st = L.dll.sl_head_argmax_noalloc(eng.h, C.c_void_p(xd.data_ptr()), m, C.c_void_p(od.data_ptr()), C.c_void_p(stream))
        assert st == abi.SL_OK, (st, eng.gpu_fault)
        torch.cuda.synchronize()
        got = od.cpu().numpy()
        assert got[:m].tolist() == want.tolist(), (m, got.tolist(), want.tolist())
        assert (got[m:] == -1).all()                       # nothing written beyond the m results
        return want, want_logits

    first, _ = both(5, 1)                                  # five rows: the row-tiled lm_head with the arg-max in its epilogue
    second, _ = both(1, 2)                                 # then one row: the single-row kernel, over the scratch the first call left
    third, _ = both(8, 3)
    assert len(set(first.tolist() + second.tolist() + third.tolist())) > 3
    # limits: rows beyond the fixed capacity are refused, nothing is poisoned
    xd = torch.zeros((9, abi.H), dtype=torch.float16, device="cuda")
    od = torch.zeros(9, dtype=torch.int32, device="cuda")
    assert L.dll.sl_head_argmax_noalloc(eng.h, C.c_void_p(xd.data_ptr()), 9, C.c_void_p(od.data_ptr()), C.c_void_p(stream)) == abi.SL_ERR_TOO_LARGE
    assert L.dll.sl_head_argmax_noalloc(eng.h, None, 1, C.c_void_p(od.data_ptr()), C.c_void_p(stream)) == abi.SL_ERR_ARG
    assert eng.gpu_fault is None and eng.head_argmax(np.zeros((1, abi.H), np.float16)) is not None

    # It allocates nothing: the device's free memory is the same before and after a series of calls ...
    x = np.random.default_rng(7).normal(0, 1, (6, abi.H)).astype(np.float16)
    want = eng.head_argmax(x)
    xd = torch.from_numpy(x).cuda()
    od = torch.full((8,), -1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for m in (6, 2, 1, 6):
        assert L.dll.sl_head_argmax_noalloc(eng.h, C.c_void_p(xd.data_ptr()), m, C.c_void_p(od.data_ptr()), C.c_void_p(stream)) == abi.SL_OK
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert od.cpu().numpy()[:6].tolist() == want.tolist()
    # ... and it neither allocates, copies nor synchronises: a stream capture, which fails on any of those, records it,
    # and every replay of the graph (with eager work and synchronisations between the replays) gives the eager result
    g = torch.cuda.CUDAGraph()
    od.fill_(-1)
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        cap = torch.cuda.current_stream().cuda_stream
        st = L.dll.sl_head_argmax_noalloc(eng.h, C.c_void_p(xd.data_ptr()), 6, C.c_void_p(od.data_ptr()), C.c_void_p(cap))
    assert st == abi.SL_OK
    for rep in range(3):
        xr = np.random.default_rng(100 + rep).normal(0, 1, (6, abi.H)).astype(np.float16)
        want = eng.head_argmax(xr)                         # eager work of the library between the replays
        xd.copy_(torch.from_numpy(xr))
        od.fill_(-1)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert od.cpu().numpy()[:6].tolist() == want.tolist(), rep
    assert eng.gpu_fault is None
    eng.close()
