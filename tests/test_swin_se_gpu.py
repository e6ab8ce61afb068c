"""GPU parity of the Swin block pair, the Swin FFN entry points and the SE module (through
the C ABI via the binding modules) against the CPU oracle.  fp16 paths: max-abs <= 2e-2 and
mean-abs <= 2e-3; the fp32 SE module: 1e-4 relative; index maps bit-exact."""
import numpy as np
import pytest
import torch

import oracle
import synth
from gpu_util import announce, assert_close, dev, dev_weights

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("hw,with_bias,mask", [(56, False, True), (14, True, True), (28, True, False)])
def test_block_pair_matches_oracle(hw, with_bias, mask):
    announce("swin pair %dx%d bias=%s mask=%s" % (hw, hw, with_bias, mask))
    import swin_transformer_binding as sb
    ws = [synth.swin_block_weights(3, b, with_bias=with_bias) for b in range(2)]
    x = synth.swin_input(3, hw * hw)
    ref = oracle.swin_block_pair(x, ws, hw, hw, use_shift_mask=mask)
    y = sb.swin_block_pair(dev(x), dev_weights(ws[0]), dev_weights(ws[1]), hw, hw, use_shift_mask=mask)
    torch.cuda.synchronize()
    # residual stream values reach |x| ~ 5: fp16 storage of the stream bounds max-abs
    assert_close("swin y", y, ref)


@pytest.mark.parametrize("hw,with_bias", [(56, True), (28, False), (7, True)])
def test_block_pair_split_and_unsplit_agree_and_repeat(hw, with_bias):
    """Four workgroups per window (default) against one workgroup per window: same result up to the
    order of FC2's fp32 additions, both within tolerance of the oracle, and every launch of a mode gives
    the same bits (the hand-over words of the split kernel grow from launch to launch, nothing is reset)."""
    announce("swin pair split/unsplit %dx%d bias=%s" % (hw, hw, with_bias))
    import souffle_hip as sh
    import swin_transformer_binding as sb
    ws = [synth.swin_block_weights(3, b, with_bias=with_bias) for b in range(2)]
    x = synth.swin_input(3, hw * hw)
    ref = oracle.swin_block_pair(x, ws, hw, hw)
    dx, d0, d1 = dev(x), dev_weights(ws[0]), dev_weights(ws[1])
    try:
        sh.set_swin_split(True)
        a1 = sb.swin_block_pair(dx, d0, d1, hw, hw).clone()
        a2 = sb.swin_block_pair(dx, d0, d1, hw, hw).clone()
        sh.set_swin_split(False)
        b1 = sb.swin_block_pair(dx, d0, d1, hw, hw).clone()
        sh.set_swin_split(True)
        a3 = sb.swin_block_pair(dx, d0, d1, hw, hw).clone()
    finally:
        sh.set_swin_split(True)
    torch.cuda.synchronize()
    assert torch.equal(a1, a2) and torch.equal(a1, a3)
    assert_close("split", a1, ref)
    assert_close("unsplit", b1, ref)
    assert (a1.float() - b1.float()).abs().max().item() <= 2 ** -6


def test_block_pair_one_workspace_for_several_image_sizes():
    """A caller may keep ONE workspace for several image sizes (sized for the largest): the hand-over
    words of the split kernel must stay consistent when the sizes alternate."""
    announce("swin pair shared workspace")
    import ctypes as C
    import souffle_hip as sh
    ws_np = [synth.swin_block_weights(3, b) for b in range(2)]
    dws = [dev_weights(w) for w in ws_np]
    arr = (sh.SwinBlockW * 2)(*[sh.SwinBlockW(*[sh.ptr(w.get(k)) for k in sh.SWIN_W_FIELDS]) for w in dws])
    cfgs = {hw: sh.SwinCfg(hw, hw, 128, 4, 7, 3, 4, 1, 1e-5) for hw in (56, 14, 28)}
    ws = sh.Workspace(max(sh.lib().souffle_swin_workspace_bytes(C.byref(c)) for c in cfgs.values()))
    for hw in (56, 14, 28, 14, 56, 28):
        x = synth.swin_input(3, hw * hw)
        dx = dev(x)
        y = torch.empty_like(dx)
        sh.check(sh.lib().souffle_swin_block_pair_fused(C.byref(cfgs[hw]), arr, dx.data_ptr(), y.data_ptr(), ws.ptr, ws.nbytes,
                                                        sh.current_stream()))
        torch.cuda.synchronize()
        assert ws.status() == 0
        assert_close("swin y %d" % hw, y, oracle.swin_block_pair(x, ws_np, hw, hw))


def test_shift_zero_pair_and_identity_blocks():
    """With zero projection and FC2 weights both blocks are the identity whatever the window
    gather / scatter does: the permutation must be undone exactly (bit-exact on fp16 data)."""
    announce("swin identity blocks")
    import swin_transformer_binding as sb
    ws = [synth.swin_block_weights(3, b) for b in range(2)]
    for w in ws:
        w["w_proj"] = np.zeros_like(w["w_proj"])
        w["w_fc2"] = np.zeros_like(w["w_fc2"])
    x = synth.swin_input(3, 56 * 56)
    y = sb.swin_block_pair(dev(x), dev_weights(ws[0]), dev_weights(ws[1]))
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), torch.from_numpy(x))


def test_index_maps_bit_exact():
    announce("swin index maps")
    import swin_transformer_binding as sb
    for (H, W, ws, s) in [(56, 56, 7, 3), (56, 56, 7, 0), (14, 28, 7, 2), (8, 12, 4, 1)]:
        got, ref = sb.index_maps(H, W, ws, s), oracle.swin_index_maps(H, W, ws, s)
        for a, b in zip(got, ref):
            np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("M,K,F", [(256, 512, 2048), (64, 128, 512), (3136, 128, 512)])
def test_fused_feed_mlp(M, K, F):
    announce("swin ffn M=%d K=%d F=%d" % (M, K, F))
    import swin_transformer_binding as sb
    x = synth.f16(synth.normal(31, (M, K), 1.0))
    w1 = synth.f16(synth.normal(32, (K, F), 0.05))
    w2 = synth.f16(synth.normal(33, (F, K), 0.05))
    y1r, _ = oracle.swin_ffn(x, w1, w2)
    y1, y2 = sb.swin_fused_feed_mlp(dev(x), dev(w1), dev(w2))
    torch.cuda.synchronize()
    assert_close("fc1", y1, y1r)
    # the second GEMM consumes the fp16-rounded first output, as the reference kernel does
    y2r = oracle.gemm(y1.float().cpu().numpy(), w2)
    assert_close("fc2", y2, y2r)


def test_swin_ffn_and_fc2_gemm():
    announce("swin_ffn / swin_trans_fc2")
    import swin_transformer_binding as sb
    import swin_trans_fc2
    M, N, K = 256, 512, 2048
    x, w = synth.f16(synth.normal(41, (M, K), 1.0)), synth.f16(synth.normal(42, (K, N), 0.02))
    ref = oracle.gemm(x, w)
    assert_close("swin_ffn", sb.swin_ffn(dev(x), dev(w), M, N, K), ref)
    assert_close("swin_trans_fc2", swin_trans_fc2.swin_trans_fc2(dev(x).view(1, M, K), dev(w)), ref)
    big = synth.f16(synth.normal(43, (4096, 768), 1.0))
    wb = synth.f16(synth.normal(44, (768, 3072), 0.02))
    assert_close("gemm large tile", sb.swin_ffn(dev(big), dev(wb), 4096, 3072, 768), oracle.gemm(big, wb))
    assert sb.bench_swin_ffn(256, 512, 2048, 2, 2, 5) > 0


SE_SHAPES = [(32, 112, 8), (96, 56, 4), (144, 56, 6), (144, 28, 6), (240, 28, 10), (240, 14, 10), (480, 14, 20),
             (672, 14, 28), (672, 7, 28), (1152, 7, 48)]


@pytest.mark.parametrize("C,H,R", SE_SHAPES + [(40, 5, 3)])
def test_se_module_all_reference_shapes(C, H, R):
    """The ten (C,H,R) of cpp/efficientnet/efficientnet_se_module_binding.cu:176-223 plus a ragged one."""
    announce("se C=%d H=%d R=%d" % (C, H, R))
    import efficientnet_se_module_binding as eb
    x = synth.uniform(50 + C, (C, H * H), 0.0, 1.0).astype(np.float32)
    wr = synth.normal(51 + C, (R, C), 0.3).astype(np.float32)
    we = synth.normal(52 + C, (C, R), 0.3).astype(np.float32)
    for combine in ("add", "mul"):
        yr, pr = oracle.se_module(x, wr, we, combine=combine)
        pooled, y = eb.torch_dispatch_efficientnet_se_module_v2_short_cut_fused(
            dev(x, torch.float32).view(1, C, H, H), dev(wr, torch.float32), dev(we, torch.float32), 2, combine=combine)
        torch.cuda.synchronize()
        np.testing.assert_allclose(pooled.cpu().numpy().reshape(-1), pr, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(y.cpu().numpy().reshape(C, -1), yr, rtol=1e-4, atol=1e-5)
