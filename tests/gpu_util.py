"""Helpers shared by the GPU parity tests: tolerance check and tensor upload."""
import sys

import numpy as np
import torch

MAX_ABS, MEAN_ABS = 2e-2, 2e-3     # fp16-compute tolerance of the benchmark definition


def announce(msg):
    """Name the case before it touches the GPU (a faulting run returns only its last output)."""
    print("[gpu-case] " + msg, flush=True)
    sys.stdout.flush()


def dev(a, dtype=torch.float16):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda:0", dtype=dtype).contiguous()


def dev_weights(w):
    return {k: dev(v) for k, v in w.items()}


def assert_close(name, got, ref, max_abs=MAX_ABS, mean_abs=MEAN_ABS):
    g = got.detach().float().cpu().numpy().reshape(-1) if isinstance(got, torch.Tensor) else np.asarray(got, np.float32).reshape(-1)
    r = np.asarray(ref, dtype=np.float32).reshape(-1)
    assert g.shape == r.shape, "%s: shape %s vs %s" % (name, g.shape, r.shape)
    assert np.isfinite(g).all(), "%s: non-finite values" % name
    d = np.abs(g - r)
    assert d.max() <= max_abs and d.mean() <= mean_abs, \
        "%s: max-abs %.4g (limit %.3g) mean-abs %.4g (limit %.3g)" % (name, d.max(), max_abs, d.mean(), mean_abs)
    return float(d.max()), float(d.mean())
