"""The hand-overs between workgroups in their two forms: acknowledged write-through stores + coherent loads (the
default) and, on top of that, the memory model's agent-scope release fence in front of every flag store and acquire
fence behind every poll (souffle_set_strict_fences).  Both must give the same bits, and the oracle's values, on the
few-rows encoder (flag words; split-K tickets without the packed FC2 weights), the many-rows encoder (row-block
hand-overs, grid barrier), the Swin block pair (window hand-overs), the SE module and the MBConv stack (grid barriers)."""
import numpy as np
import pytest
import torch

import oracle
import synth
from gpu_util import announce, assert_close, dev, dev_weights

pytestmark = pytest.mark.gpu


@pytest.fixture
def strict():
    import souffle_hip as sh

    def switch(on):
        sh.set_strict_fences(on)
    yield switch
    sh.set_strict_fences(False)


@pytest.mark.parametrize("B,S,layers,pack", [(1, 128, 12, True), (1, 384, 2, True), (32, 128, 2, True), (1, 128, 3, False)])
def test_encoder_same_bits_with_and_without_the_fences(strict, B, S, layers, pack):
    announce("strict fences: bert encoder B=%d S=%d L=%d pack=%d" % (B, S, layers, pack))
    import bert_binding
    ws = [synth.bert_layer_weights(2, l, with_bias=True) for l in range(layers)]
    x = synth.bert_input(2, B, S)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S, pack=pack)
    plain = enc(dev(x)).clone()
    strict(True)
    fenced = enc(dev(x)).clone()
    fenced_again = enc(dev(x)).clone()
    fenced_per_op = enc(dev(x), fused=False).clone()
    strict(False)
    plain_again = enc(dev(x)).clone()
    assert enc.ws.status() == 0
    assert torch.equal(fenced, plain) and torch.equal(fenced_again, plain) and torch.equal(plain_again, plain)
    assert torch.equal(fenced_per_op, plain)
    assert_close("encoder with fences", fenced, oracle.bert_encoder(x, ws, B, S))


def test_swin_se_mbconv_same_bits_with_and_without_the_fences(strict):
    announce("strict fences: swin block pair, SE module, MBConv stack")
    import efficientnet_binding as efb
    import efficientnet_se_module_binding as eb
    import swin_transformer_binding as sb
    ws = [synth.swin_block_weights(3, b) for b in range(2)]
    xs = synth.swin_input(3)
    dw = [{k: dev(v) for k, v in w.items()} for w in ws]
    blocks = synth.mbconv_stack_weights()
    up = lambda v: torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v
    stack = efb.MBConvStack([{k: up(v) for k, v in b.items()} for b in blocks])
    xm = torch.from_numpy(synth.mbconv_input()).cuda()
    g = torch.Generator(device="cpu").manual_seed(11)
    xse = torch.rand((1, 144, 28, 28), generator=g).cuda()
    wr, we = (torch.randn((6, 144), generator=g) * 0.3).cuda(), (torch.randn((144, 6), generator=g) * 0.3).cuda()

    def run_all():
        y_swin = sb.swin_block_pair(dev(xs), dw[0], dw[1]).clone()
        y_se = eb.torch_dispatch_efficientnet_se_module_v2_short_cut_fused(xse, wr, we, 1)[1].clone()
        y_mb = stack(xm).clone()
        torch.cuda.synchronize()
        return y_swin, y_se, y_mb

    plain = run_all()
    strict(True)
    fenced = run_all()
    strict(False)
    for name, a, b in zip(("swin", "se", "mbconv"), plain, fenced):
        assert torch.equal(a, b), name
    assert_close("swin pair with fences", fenced[0], oracle.swin_block_pair(xs, ws))
