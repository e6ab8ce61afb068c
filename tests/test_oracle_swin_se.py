"""Pins oracle/swin_oracle.c and oracle/se_oracle.c against torch library closed forms,
brute force and permutation laws.  CPU only.  Index maps are checked bit-exactly."""
import numpy as np
import pytest
import torch

import oracle
import synth
import torch_ref


@pytest.mark.parametrize("H,W,ws,shift", [(14, 14, 7, 3), (56, 56, 7, 3), (14, 28, 7, 2), (21, 14, 7, 0), (8, 12, 4, 1)])
def test_index_maps_equal_torch_roll_and_partition(H, W, ws, shift):
    g, s, rel, reg = oracle.swin_index_maps(H, W, ws, shift)
    ids = torch.arange(H * W).view(1, H, W, 1)
    rolled = torch.roll(ids, shifts=(-shift, -shift), dims=(1, 2)) if shift else ids
    want = torch_ref.window_partition(rolled, ws).reshape(-1).numpy()
    np.testing.assert_array_equal(g, want)                          # gather = partition(roll(-s))
    assert sorted(g.tolist()) == list(range(H * W))                 # a permutation
    np.testing.assert_array_equal(s[g], np.arange(H * W))           # scatter is its inverse
    # reverse + roll(+s) of window-ordered data reads exactly scatter_idx
    win = torch.arange(H * W).view(-1, ws, ws, 1)
    back = torch_ref.window_reverse(win, ws, H, W)
    back = torch.roll(back, shifts=(shift, shift), dims=(1, 2)) if shift else back
    np.testing.assert_array_equal(s, back.reshape(-1).numpy())
    # relative-position index: published construction
    coords = torch.stack(torch.meshgrid(torch.arange(ws), torch.arange(ws), indexing="ij")).flatten(1)
    r = (coords[:, :, None] - coords[:, None, :]).permute(1, 2, 0).contiguous()
    r[:, :, 0] += ws - 1
    r[:, :, 1] += ws - 1
    r[:, :, 0] *= 2 * ws - 1
    np.testing.assert_array_equal(rel, r.sum(-1).numpy())
    # region labels: published img_mask construction
    if shift:
        img = torch.zeros(1, H, W, 1)
        cnt = 0
        for hs in (slice(0, -ws), slice(-ws, -shift), slice(-shift, None)):
            for wsl in (slice(0, -ws), slice(-ws, -shift), slice(-shift, None)):
                img[:, hs, wsl, :] = cnt
                cnt += 1
        np.testing.assert_array_equal(reg, torch_ref.window_partition(img, ws).reshape(-1).numpy().astype(np.int32))
    else:
        assert not reg.any()


def test_index_maps_brute_force_tiny():
    H = W = 14
    g, _, _, _ = oracle.swin_index_maps(H, W, 7, 3)
    for w in range(4):
        for n in range(49):
            i, j = (w // 2) * 7 + n // 7, (w % 2) * 7 + n % 7       # position in the rolled image
            assert g[w * 49 + n] == ((i + 3) % H) * W + (j + 3) % W  # roll(-3): rolled[i][j] = x[i+3][j+3]


@pytest.mark.parametrize("shift,mask", [(0, True), (3, True), (3, False)])
def test_swin_block_matches_torch(shift, mask):
    H = W = 14
    w = {k: v.astype(np.float32) for k, v in synth.swin_block_weights(3, 1, with_bias=True).items()}
    x = synth.swin_input(3, H * W).astype(np.float32)
    got = oracle.swin_block(x, w, H, W, 128, 4, 7, shift, 4, mask)
    ref = torch_ref.swin_block(x, w, H, W, 4, 7, shift, mask)
    np.testing.assert_allclose(got, ref, rtol=2e-4, atol=2e-4)


def test_swin_pair_is_two_blocks_and_full_size_runs():
    ws = [{k: v.astype(np.float32) for k, v in synth.swin_block_weights(3, b).items()} for b in range(2)]
    x = synth.swin_input(3).astype(np.float32)
    y = oracle.swin_block_pair(x, ws)
    mid = oracle.swin_block(x, ws[0], shift=0)
    np.testing.assert_array_equal(y, oracle.swin_block(mid, ws[1], shift=3))
    ref = torch_ref.swin_block(torch_ref.swin_block(x, ws[0], 56, 56, 4, 7, 0), ws[1], 56, 56, 4, 7, 3)
    np.testing.assert_allclose(y, ref, rtol=3e-4, atol=3e-4)


def test_swin_ffn_is_two_matmuls():
    rng = np.random.default_rng(1)
    x, w1, w2 = rng.normal(size=(64, 32)), rng.normal(size=(32, 96)), rng.normal(size=(96, 32))
    y1, y2 = oracle.swin_ffn(x, w1, w2)
    np.testing.assert_allclose(y1, x @ w1, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(y2, (x @ w1) @ w2, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("C,H,R,combine", [(32, 112, 8, "add"), (96, 56, 4, "mul"), (1152, 7, 48, "add"), (40, 5, 3, "mul")])
def test_se_module_matches_torch(C, H, R, combine):
    rng = np.random.default_rng(C)
    x = rng.random((C, H * H)).astype(np.float32)
    wr, we = rng.normal(0, 0.3, (R, C)).astype(np.float32), rng.normal(0, 0.3, (C, R)).astype(np.float32)
    br, be = rng.normal(0, 0.1, R).astype(np.float32), rng.normal(0, 0.1, C).astype(np.float32)
    y, p = oracle.se_module(x, wr, we, br, be, combine)
    yr, pr = torch_ref.se_module(x, wr, we, br, be, combine)
    np.testing.assert_allclose(p, pr, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(y, yr, rtol=1e-5, atol=1e-5)
