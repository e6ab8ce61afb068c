"""Swin patch merging (2x2 gather + LayerNorm over 4C + reduction to 2C).

CPU part: pins oracle_swin_patch_merge_f32 against the reference's own torch statement of the
module (python/models/swin_transformer/swin_patch_merge.py:3-13) in float64 and against its
tensor-expression index formula (:49-63) evaluated by brute force.  GPU part: the HIP kernel through
the C ABI against the oracle; max-abs <= 2e-2, mean-abs <= 2e-3; with identity LayerNorm statistics
removed (unit weights) the gather itself is checked bit-exactly through a selection matrix.
"""
import numpy as np
import pytest
import torch

import oracle
import synth
from gpu_util import announce, assert_close, dev


def rnd(seed, shape, std=1.0):
    return synth.f16(synth.normal(synth.seed_of(43, seed), shape, std))


def torch_patch_merge(x, H, W, g, b, w, eps):
    t = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float64))
    Cc = x.shape[-1]
    v = t(x).view(1, H, W, Cc)
    x0, x1, x2, x3 = v[:, 0::2, 0::2, :], v[:, 1::2, 0::2, :], v[:, 0::2, 1::2, :], v[:, 1::2, 1::2, :]
    v = torch.cat([x0, x1, x2, x3], -1).view(1, -1, 4 * Cc)
    v = torch.nn.functional.layer_norm(v, (4 * Cc,), None if g is None else t(g), None if b is None else t(b), eps)
    return (v @ t(w))[0].numpy()


@pytest.mark.parametrize("H,W,Cc,affine", [(8, 6, 32, True), (4, 10, 64, False), (2, 2, 32, True)])
def test_oracle_against_the_reference_torch_statement(H, W, Cc, affine):
    x, w = rnd(1, (H * W, Cc)), rnd(2, (4 * Cc, 2 * Cc), 0.05)
    g = (1.0 + 0.2 * rnd(3, (4 * Cc,))).astype(np.float16) if affine else None
    b = rnd(4, (4 * Cc,), 0.2) if affine else None
    got = oracle.swin_patch_merge(x, H, W, g, b, w, 1e-5)
    ref = torch_patch_merge(x, H, W, g, b, w, 1e-5)
    assert got.shape == ref.shape == ((H // 2) * (W // 2), 2 * Cc)
    assert np.abs(got - ref).max() < 2e-5


def test_oracle_gather_against_the_tensor_expression_indices():
    """With w = a selection of single merged channels and the LayerNorm undone (affine chosen per row
    is impossible, so compare normalised values): merged[m][c'] must be x[2i + (c'//C)%2][2j + (c'//C)//2][c'%C]."""
    H, W, Cc = 6, 4, 32
    x = rnd(5, (H * W, Cc)).astype(np.float64)
    K = 4 * Cc
    sel = np.zeros((K, 2 * Cc))
    cols = [0, 1, Cc - 1, Cc, 2 * Cc + 3, 3 * Cc + 5, 4 * Cc - 1]
    for n, c in enumerate(cols):
        sel[c, n] = 1.0
    got = oracle.swin_patch_merge(x, H, W, None, None, sel, 0.0)
    W2 = W // 2
    for m in range((H // 2) * W2):
        i, j = m // W2, m % W2
        row = np.array([x[(2 * i + (c // Cc) % 2) * W + 2 * j + (c // Cc) // 2, c % Cc] for c in range(K)])
        z = (row - row.mean()) / np.sqrt(row.var())
        for n, c in enumerate(cols):
            assert abs(got[m, n] - z[c]) < 1e-4


def test_patch_merge_argument_validation_without_gpu():
    import souffle_hip as sh
    lib = sh.lib()
    assert lib.souffle_swin_patch_merge(None, None, None, None, None, 56, 56, 128, 1e-5, None) == -1
    assert lib.souffle_swin_patch_merge(4096, None, None, 4096, 4096, 55, 56, 128, 1e-5, None) == -2 and "even" in sh.last_error()
    assert lib.souffle_swin_patch_merge(4096, None, None, 4096, 4096, 56, 56, 100, 1e-5, None) == -2 and "multiple of 32" in sh.last_error()


@pytest.mark.gpu
@pytest.mark.parametrize("H,W,Cc,affine", [(56, 56, 128, True), (28, 28, 256, True), (14, 14, 512, False), (6, 10, 32, True),
                                            (2, 2, 64, True)])
def test_patch_merge_matches_oracle(H, W, Cc, affine):
    announce("swin patch merge %dx%dx%d affine=%s" % (H, W, Cc, affine))
    import swin_transformer_binding as sb
    x, w = rnd(6, (H * W, Cc)), rnd(7, (4 * Cc, 2 * Cc), 0.02)
    g = (1.0 + 0.1 * rnd(8, (4 * Cc,))).astype(np.float16) if affine else None
    b = rnd(9, (4 * Cc,), 0.1) if affine else None
    ref = oracle.swin_patch_merge(x, H, W, g, b, w, 1e-5, threads=8)
    y = sb.patch_merging(dev(x), H, W, None if g is None else dev(g), None if b is None else dev(b), dev(w))
    torch.cuda.synchronize()
    assert tuple(y.shape) == ((H // 2) * (W // 2), 2 * Cc)
    assert_close("patch merge", y, ref)


@pytest.mark.gpu
def test_patch_merge_gather_is_exact():
    """A reduction matrix that selects single merged channels shows the gather alone: the kernel's
    normalised value of merged channel c' must be the fp16 rounding of the oracle's."""
    announce("swin patch merge gather")
    import swin_transformer_binding as sb
    H, W, Cc = 8, 12, 32
    x = rnd(10, (H * W, Cc))
    sel = np.zeros((4 * Cc, 2 * Cc), np.float16)
    cols = [0, 1, Cc - 1, Cc, Cc + 7, 2 * Cc, 2 * Cc + 3, 3 * Cc, 3 * Cc + 5, 4 * Cc - 1]
    for n, c in enumerate(cols):
        sel[c, n] = 1.0
    ref = oracle.swin_patch_merge(x, H, W, None, None, sel, 1e-5)
    y = sb.patch_merging(dev(x), H, W, None, None, dev(sel)).float().cpu().numpy()
    # one rounding of the normalised value to fp16 on the way into the MFMA, exact selection afterwards
    assert np.abs(y[:, :len(cols)] - ref[:, :len(cols)]).max() <= 2.0 ** -9 * max(1.0, np.abs(ref).max())
    assert np.all(y[:, len(cols):] == 0)
