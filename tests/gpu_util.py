"""Helpers for the GPU parity tests: build a synthetic model in HBM with the library's generator,
copy the same bytes to the host for the CPU oracle."""
import numpy as np


def device_and_host_model(cfg):
    import torch
    from qwisp_amd import lib, synth
    dev = synth.generate_device(cfg, lib.get())
    host = {}
    for k, v in dev.items():
        a = v.cpu().numpy()
        if a.dtype == np.int32:
            a = a.view(np.uint32)
        host[k] = a
    torch.cuda.synchronize()
    return dev, host


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


def first_diff(a, b):
    a, b = np.asarray(a).reshape(-1), np.asarray(b).reshape(-1)
    idx = np.nonzero(a.view(np.uint16 if a.dtype == np.float16 else a.dtype) !=
                     b.view(np.uint16 if b.dtype == np.float16 else b.dtype))[0]
    if len(idx) == 0:
        return "identical"
    i = int(idx[0])
    return f"{len(idx)} of {a.size} differ; first at {i}: {a[i]!r} vs {b[i]!r}"
