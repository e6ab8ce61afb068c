"""EfficientNet MBConv operators and stack.

CPU part: pins the oracle (oracle/mbconv_oracle.c) against torch library convolutions in
float64, against brute-force loops on tiny inputs and against the shape lists that the
reference's own tuning tables hold (python/models/efficientnet/efficientnet.py:232-244,370-387).
GPU part: the HIP operators and the fused stack, through the C ABI, against the oracle on the
same fp16-rounded seeded tensors.  Tolerance: max-abs <= 2e-2, mean-abs <= 2e-3.
"""
import ctypes as C

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn

import oracle
import synth
from gpu_util import announce, assert_close, dev

# (H, W, C) of every squeeze-excite input and (C, R) of every squeeze layer that the reference tunes
REF_REDUCE_MEAN = {(112, 112, 32), (56, 56, 96), (56, 56, 144), (28, 28, 144), (28, 28, 240), (14, 14, 240),
                   (14, 14, 480), (14, 14, 672), (7, 7, 672), (7, 7, 1152)}
REF_SE_PAIRS = {(32, 8), (96, 4), (144, 6), (240, 10), (480, 20), (672, 28), (1152, 48)}
# (H, W, C, k, k, stride) of the depthwise convolutions of the blocks (efficientnet.py:210-226)
REF_DEPTHWISE = {(112, 112, 32, 3, 1), (112, 112, 96, 3, 2), (56, 56, 144, 3, 1), (56, 56, 144, 3, 2), (56, 56, 144, 5, 2),
                 (28, 28, 144, 3, 2), (28, 28, 240, 5, 1), (28, 28, 240, 3, 2), (14, 14, 480, 5, 1), (14, 14, 672, 5, 1),
                 (14, 14, 672, 5, 2), (7, 7, 1152, 5, 1)}


def rnd(seed, shape, std=1.0):
    return synth.f16(synth.normal(synth.seed_of(40, seed), shape, std))


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


# ------------------------------------------------------------------ oracle pinning ----
def test_block_table_matches_the_reference_shape_lists():
    shapes = synth.mbconv_block_shapes()
    assert len(shapes) == 16
    se_in, pairs, dws = set(), set(), set()
    for s in shapes:
        oh = (s["in_h"] - 1) // s["stride"] + 1
        se_in.add((oh, oh, s["expand_c"]))
        pairs.add((s["expand_c"], s["se_c"]))
        dws.add((s["in_h"], s["in_w"], s["expand_c"], s["kernel"], s["stride"]))
    assert se_in == REF_REDUCE_MEAN
    assert pairs == REF_SE_PAIRS
    # the reference's depthwise table misses the two 3x3 stride-1 shapes of stages 4 and 7 (and lists
    # two shapes EfficientNet-B0 does not contain); the other ten are there
    assert dws - REF_DEPTHWISE == {(14, 14, 480, 3, 1), (7, 7, 1152, 3, 1)}
    assert shapes[-1]["out_c"] == 320 and shapes[-1]["in_h"] == 7


@pytest.mark.parametrize("P,K,N,act,gate,short", [(37, 16, 24, "swish", False, False), (50, 40, 8, "none", True, True),
                                                   (9, 96, 40, "none", True, False), (64, 8, 16, "swish", False, True)])
def test_oracle_pointwise_against_torch_conv2d(P, K, N, act, gate, short):
    x, w = rnd(1, (P, K)), rnd(2, (N, K), 0.1)
    sc, sh = rnd(3, (N,)).astype(np.float32) + 2, rnd(4, (N,)).astype(np.float32)
    g = np.abs(rnd(5, (K,)).astype(np.float32)) if gate else None
    s = rnd(6, (P, N)) if short else None
    got = oracle.pointwise_conv(x, w, sc, sh, g, s, act)
    xi = t64(x) * (t64(g) if gate else 1.0)
    y = Fn.conv2d(xi.t().reshape(1, K, P, 1), t64(w).reshape(N, K, 1, 1)).reshape(N, P).t()
    y = y * t64(sc) + t64(sh)
    if act == "swish":
        y = y * torch.sigmoid(y)
    if short:
        y = y + t64(s)
    assert np.abs(got - y.numpy()).max() < 2e-5


@pytest.mark.parametrize("H,W,Cc,k,stride", [(9, 7, 8, 3, 1), (10, 8, 16, 3, 2), (7, 7, 8, 5, 1), (12, 9, 8, 5, 2),
                                              (1, 1, 8, 3, 1), (2, 3, 8, 5, 2)])
def test_oracle_depthwise_against_torch_conv2d(H, W, Cc, k, stride):
    x, w = rnd(7, (H, W, Cc)), rnd(8, (k, k, Cc), 0.3)
    sc, sh = rnd(9, (Cc,)).astype(np.float32) + 2, rnd(10, (Cc,)).astype(np.float32)
    got = oracle.depthwise_conv(x, w, sc, sh, stride)
    y = Fn.conv2d(t64(x).permute(2, 0, 1)[None], t64(w).permute(2, 0, 1)[:, None], stride=stride, padding=k // 2, groups=Cc)[0]
    y = y * t64(sc)[:, None, None] + t64(sh)[:, None, None]
    y = (y * torch.sigmoid(y)).permute(1, 2, 0).numpy()
    assert got.shape == y.shape == ((H - 1) // stride + 1, (W - 1) // stride + 1, Cc)
    assert np.abs(got - y).max() < 2e-5


def test_oracle_depthwise_against_brute_force_loops():
    H, W, Cc, k, stride = 5, 4, 8, 3, 2
    x, w = rnd(11, (H, W, Cc)).astype(np.float64), rnd(12, (k, k, Cc)).astype(np.float64)
    got = oracle.depthwise_conv(x, w, None, None, stride, act="none")
    for ho in range(3):
        for wo in range(2):
            for c in range(Cc):
                s = 0.0
                for i in range(k):
                    for j in range(k):
                        hi, wi = ho * stride - 1 + i, wo * stride - 1 + j     # one pixel of padding before the image
                        if 0 <= hi < H and 0 <= wi < W:
                            s += x[hi, wi, c] * w[i, j, c]
                assert abs(got[ho, wo, c] - s) < 1e-5
    # a delta kernel at the centre tap with stride 1 is the identity
    w1 = np.zeros((3, 3, Cc))
    w1[1, 1] = 1.0
    assert np.array_equal(oracle.depthwise_conv(x, w1, None, None, 1, act="none"), x.astype(np.float32))


def test_oracle_se_gate_against_torch():
    P, Cc, R = 49, 24, 6
    x = rnd(13, (P, Cc))
    wr, br, we, be = rnd(14, (R, Cc), 0.3), rnd(15, (R,)), rnd(16, (R, Cc), 0.3), rnd(17, (Cc,))
    got = oracle.se_gate(x, wr, br, we, be)
    p = Fn.adaptive_avg_pool2d(t64(x).t().reshape(1, Cc, 7, 7), 1).reshape(Cc)
    r = t64(wr) @ p + t64(br)
    r = r * torch.sigmoid(r)
    e = torch.sigmoid(t64(we).t() @ r + t64(be))
    assert np.abs(got - e.numpy()).max() < 2e-6


def torch_block(x, b):
    """One MBConv block from torch library ops in float64 (NCHW)."""
    H, W = b["in_h"], b["in_w"]
    v = t64(x).reshape(H, W, b["in_c"]).permute(2, 0, 1)[None]
    inp = v
    if b["expand_w"] is not None:
        v = Fn.conv2d(v, t64(b["expand_w"])[:, :, None, None]) * t64(b["expand_scale"])[None, :, None, None] + \
            t64(b["expand_shift"])[None, :, None, None]
        v = v * torch.sigmoid(v)
    k = b["kernel"]
    v = Fn.conv2d(v, t64(b["dw_w"]).permute(2, 0, 1)[:, None], stride=b["stride"], padding=k // 2, groups=b["expand_c"])
    v = v * t64(b["dw_scale"])[None, :, None, None] + t64(b["dw_shift"])[None, :, None, None]
    v = v * torch.sigmoid(v)
    p = v.mean(dim=(2, 3))[0]
    r = t64(b["se_reduce_w"]) @ p + t64(b["se_reduce_b"])
    r = r * torch.sigmoid(r)
    e = torch.sigmoid(t64(b["se_expand_w"]).t() @ r + t64(b["se_expand_b"]))
    v = v * e[None, :, None, None]
    v = Fn.conv2d(v, t64(b["project_w"])[:, :, None, None]) * t64(b["project_scale"])[None, :, None, None] + \
        t64(b["project_shift"])[None, :, None, None]
    if b["has_shortcut"]:
        v = v + inp
    return v[0].permute(1, 2, 0).reshape(-1, b["out_c"]).numpy()


def small_block(kernel, stride, ratio, shortcut, H=9, W=6, ci=16, co=None):
    co = ci if shortcut else (co or 24)
    shape = {"in_h": H, "in_w": W, "in_c": ci, "expand_c": ci * ratio, "out_c": co, "kernel": kernel, "stride": stride,
             "se_c": max(1, ci // 4), "has_shortcut": int(shortcut), "has_expand": ratio != 1}
    return synth.mbconv_block_weights(shape, 41, kernel * 4 + stride * 2 + ratio % 3)


@pytest.mark.parametrize("kernel,stride,ratio,shortcut", [(3, 1, 6, True), (5, 2, 6, False), (3, 1, 1, False), (5, 1, 2, True),
                                                           (3, 2, 1, False)])
def test_oracle_block_against_torch_composition(kernel, stride, ratio, shortcut):
    b = small_block(kernel, stride, ratio, shortcut)
    x = rnd(18, (b["in_h"] * b["in_w"], b["in_c"]))
    e, d, y = oracle.mbconv_block(x, b, dump=True)
    ref = torch_block(x, b)
    assert y.shape == ref.shape
    assert np.abs(y - ref).max() < 1e-4 * max(1.0, np.abs(ref).max())
    # the fp16-storage variant rounds every operator output to the nearest fp16 value
    e2, d2, y2 = oracle.mbconv_block(x, b, round_fp16=True, dump=True)
    if e is not None:
        assert np.array_equal(e2, e.astype(np.float16).astype(np.float32))
    assert np.array_equal(y2, y2.astype(np.float16).astype(np.float32))
    assert np.abs(y2 - y).max() < 2e-2


def test_oracle_stack_chains_blocks():
    blocks = [small_block(3, 1, 1, False, ci=16, co=16), small_block(5, 2, 6, False, ci=16, co=24)]
    blocks[1]["in_h"], blocks[1]["in_w"] = 9, 6
    x = rnd(19, (54, 16))
    y = oracle.mbconv_stack(x, blocks)
    assert np.abs(y - torch_block(torch_block(x, blocks[0]), blocks[1])).max() < 1e-3


# -------------------------------------------------------- host logic of the C ABI ----
def make_desc(blocks):
    import souffle_hip as sh
    arr = (sh.MbconvBlock * len(blocks))()
    for d, b in zip(arr, blocks):
        for f in sh.MB_INT_FIELDS:
            setattr(d, f, int(b[f]))
        for f in sh.MB_PTR_FIELDS:
            setattr(d, f, 4096 if b.get(f) is not None else None)     # fake, aligned, never dereferenced
    return arr


def test_workspace_bytes_and_block_list_validation():
    import souffle_hip as sh
    lib = sh.lib()
    blocks = synth.mbconv_stack_weights()
    n = lib.souffle_mbconv_workspace_bytes(make_desc(blocks), len(blocks))
    act = sum(b["in_h"] * b["in_w"] * b["expand_c"] * 2 for b in blocks if b["expand_w"] is not None)
    assert n > act and n < 64 << 20
    for field, value, text in [("in_c", 12, "multiples of 8"), ("kernel", 4, "kernel must be 3 or 5"), ("stride", 3, "stride"),
                               ("se_c", 65, "se_c"), ("expand_c", 4096, "expand_c"), ("has_shortcut", 1, "shortcut")]:
        bad = [dict(b) for b in blocks]
        bad[0][field] = value
        assert lib.souffle_mbconv_workspace_bytes(make_desc(bad), len(bad)) == 0
        assert text in sh.last_error(), sh.last_error()
    bad = [dict(b) for b in blocks]
    bad[3]["in_h"] = 28
    assert lib.souffle_mbconv_workspace_bytes(make_desc(bad), len(bad)) == 0 and "does not take" in sh.last_error()
    assert lib.souffle_mbconv_workspace_bytes(None, 0) == 0


# ------------------------------------------------------------------------ GPU ----
def dev_block(b):
    out = {}
    for k, v in b.items():
        if isinstance(v, np.ndarray):
            out[k] = dev(v, torch.float16 if v.dtype == np.float16 else torch.float32)
        else:
            out[k] = v
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("P,K,N,act,gate,short", [(12544, 16, 96, "swish", False, False), (3136, 144, 24, "none", True, True),
                                                   (784, 240, 40, "none", True, False), (196, 672, 112, "none", True, True),
                                                   (49, 1152, 320, "none", True, False), (49, 192, 1152, "swish", False, False),
                                                   (37, 8, 8, "swish", False, False), (1, 2048, 16, "none", True, False),
                                                   (100, 40, 24, "none", False, True)])
def test_pointwise_conv_matches_oracle(P, K, N, act, gate, short):
    announce("pointwise P=%d K=%d N=%d %s gate=%s shortcut=%s" % (P, K, N, act, gate, short))
    import efficientnet_binding as eb
    x, w = rnd(21, (P, K)), rnd(22, (N, K), 1.0 / np.sqrt(K))
    sc = (1.0 + 0.2 * rnd(23, (N,))).astype(np.float32)
    sh_ = rnd(24, (N,), 0.3).astype(np.float32)
    g = (0.2 + np.abs(rnd(25, (K,)))).clip(0, 1).astype(np.float32) if gate else None
    s = rnd(26, (P, N)) if short else None
    ref = oracle.pointwise_conv(x, w, sc, sh_, g, s, act, threads=8)
    xd, wd = dev(x).view(1, 1, P, K), dev(w)
    scd, shd = dev(sc, torch.float32), dev(sh_, torch.float32)
    gd = dev(g, torch.float32) if gate else None
    if short:
        got = eb.pointwise_conv2d_bn_short_cut_add(xd, wd, scd, shd, dev(s).view(1, 1, P, N), gate=gd)
    elif act == "swish":
        got = eb.head_conv1x1_bn_swish(xd, wd.t().contiguous().view(1, 1, K, N), scd, shd)
    else:
        got = eb.pointwise_conv2d_bn(xd, wd, scd, shd, gate=gd)
    torch.cuda.synchronize()
    assert_close("pointwise", got, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("H,W,Cc,k,stride", [(112, 112, 32, 3, 1), (112, 112, 96, 3, 2), (56, 56, 144, 5, 2), (28, 28, 240, 5, 1),
                                              (14, 14, 672, 5, 2), (7, 7, 1152, 3, 1), (9, 7, 8, 5, 2), (1, 1, 2048, 3, 1),
                                              (13, 5, 264, 3, 2)])
def test_depthwise_conv_matches_oracle(H, W, Cc, k, stride):
    announce("depthwise %dx%dx%d k=%d s=%d" % (H, W, Cc, k, stride))
    import efficientnet_binding as eb
    x, w = rnd(27, (H, W, Cc)), rnd(28, (k, k, Cc), 1.0 / k)
    sc = (1.0 + 0.2 * rnd(29, (Cc,))).astype(np.float32)
    sh_ = rnd(30, (Cc,), 0.3).astype(np.float32)
    ref = oracle.depthwise_conv(x, w, sc, sh_, stride, threads=8)
    got = eb.fused_depthwise_conv2d_bn_swish(dev(x)[None], dev(w)[..., None].contiguous(), dev(sc, torch.float32),
                                             dev(sh_, torch.float32), stride)
    torch.cuda.synchronize()
    assert tuple(got.shape[1:]) == ref.shape
    assert_close("depthwise", got, ref)


@pytest.mark.gpu
def test_every_block_of_the_stack_matches_oracle():
    """Each of the 16 block shapes on its own (fused launch and per-operator launches), fed
    N(0,1) inputs, against the unrounded fp32 oracle."""
    import efficientnet_binding as eb
    blocks = synth.mbconv_stack_weights()
    for i, b in enumerate(blocks):
        announce("mbconv block %d: %dx%dx%d -> %d k%d s%d" % (i, b["in_h"], b["in_w"], b["in_c"], b["out_c"], b["kernel"], b["stride"]))
        x = rnd(31 + i, (b["in_h"] * b["in_w"], b["in_c"]))
        ref = oracle.mbconv_block(x, b, threads=8)
        stack = eb.MBConvStack([dev_block(b)])
        y_f = stack(dev(x), fused=True).clone()
        y_u = stack(dev(x), fused=False).clone()
        torch.cuda.synchronize()
        assert stack.ws.status() == 0
        assert_close("block %d fused" % i, y_f, ref)
        assert torch.equal(y_f, y_u), "block %d: fused and per-operator launches run the same arithmetic" % i


@pytest.mark.gpu
def test_full_stack_matches_oracle_and_is_deterministic():
    """Benchmark configuration 4: the 16 MBConv blocks of EfficientNet-B0 behind the stem, 112x112x32 in,
    7x7x320 out.  Against the oracle that stores every operator output as fp16 (what the pipeline
    does) and against the unrounded one, both at the same tolerance."""
    announce("mbconv full stack")
    import efficientnet_binding as eb
    blocks = synth.mbconv_stack_weights()
    x = synth.mbconv_input()
    ref_r = oracle.mbconv_stack(x, blocks, round_fp16=True, threads=8)
    ref = oracle.mbconv_stack(x, blocks, threads=8)
    stack = eb.MBConvStack([dev_block(b) for b in blocks])
    xd = dev(x)
    y1 = stack(xd).clone()
    y2 = stack(xd).clone()
    y3 = stack(xd, fused=False).clone()
    y4 = stack(xd).clone()
    torch.cuda.synchronize()
    assert stack.ws.status() == 0
    assert tuple(y1.shape) == (49, 320)
    assert_close("stack vs fp16-storage oracle", y1, ref_r)
    assert_close("stack vs fp32 oracle", y1, ref)
    assert torch.equal(y1, y2) and torch.equal(y1, y3) and torch.equal(y1, y4)


@pytest.mark.gpu
def test_stack_without_squeeze_excite_and_odd_sizes():
    """Blocks without the squeeze-excite module, odd image sizes and a stride-2 block on an odd image."""
    announce("mbconv odd sizes, no SE")
    import efficientnet_binding as eb
    shapes = [{"in_h": 15, "in_w": 11, "in_c": 24, "expand_c": 72, "out_c": 24, "kernel": 3, "stride": 1, "se_c": 0,
               "has_shortcut": 1, "has_expand": True},
              {"in_h": 15, "in_w": 11, "in_c": 24, "expand_c": 24, "out_c": 40, "kernel": 5, "stride": 2, "se_c": 6,
               "has_shortcut": 0, "has_expand": False}]
    blocks = [synth.mbconv_block_weights(s, 42, i) for i, s in enumerate(shapes)]
    for k in ("se_reduce_w", "se_reduce_b", "se_expand_w", "se_expand_b"):
        blocks[0][k] = None
    x = rnd(60, (15 * 11, 24))
    ref = oracle.mbconv_stack(x, blocks)
    stack = eb.MBConvStack([dev_block(b) for b in blocks])
    y = stack(dev(x)).clone()
    torch.cuda.synchronize()
    assert tuple(y.shape) == (8 * 6, 40)
    assert_close("odd stack", y, ref)


@pytest.mark.gpu
def test_mbconv_argument_errors_are_reported():
    announce("mbconv argument errors")
    import efficientnet_binding as eb
    import souffle_hip as sh
    x = torch.zeros(1, 4, 4, 12, dtype=torch.float16, device="cuda:0")
    w = torch.zeros(16, 12, dtype=torch.float16, device="cuda:0")
    with pytest.raises(sh.SouffleError) as e:
        eb.pointwise_conv2d_bn(x, w)
    assert e.value.code == -2 and "multiples of 8" in str(e.value)
    with pytest.raises(TypeError):
        eb.pointwise_conv2d_bn(x.float(), w)
    xd = torch.zeros(1, 4, 4, 16, dtype=torch.float16, device="cuda:0")
    with pytest.raises(sh.SouffleError) as e:
        eb.fused_depthwise_conv2d_bn_swish(xd, torch.zeros(4, 4, 16, 1, dtype=torch.float16, device="cuda:0"))
    assert "kernel must be 3 or 5" in str(e.value)
