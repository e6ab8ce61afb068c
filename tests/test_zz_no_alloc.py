"""The encoder entry point that allocates nothing (souffle_bert_encoder_fused_static), called through the C ABI:
its output must equal, bit for bit, that of souffle_bert_encoder_fused with a caller's workspace, on two calls in
a row of which the second has the smaller input (both use the library's one static scratch array, which keeps the
first call's contents), and a configuration that does not fit the array must be refused with a message."""
import ctypes as C

import pytest
import torch

import souffle_hip as sh
import synth
from gpu_util import announce, dev, dev_weights

pytestmark = pytest.mark.gpu


def _layer_array(dws):
    import bert_binding
    structs = [bert_binding.make_layer_w(**w) for w in dws]
    arr = (sh.BertLayerW * len(dws))(*structs)
    arr._keep = structs
    return arr


def _both(B, S, layers, seed):
    lib = sh.lib()
    ws = [synth.bert_layer_weights(seed, l, with_bias=True) for l in range(layers)]
    dws = [dev_weights(w) for w in ws]
    arr = _layer_array(dws)
    x = dev(synth.bert_input(seed, B, S))
    cfg = sh.BertCfg(B, S, 768, 12, 3072, sh.ACT_GELU_TANH, 0.125, 1e-12, layers, 0)
    y_ws = torch.empty((B * S, 768), dtype=torch.float16, device="cuda:0")
    y_st = torch.full((B * S, 768), float("nan"), dtype=torch.float16, device="cuda:0")
    work = sh.Workspace(lib.souffle_bert_workspace_bytes(C.byref(cfg)))
    sh.check(lib.souffle_bert_encoder_fused(C.byref(cfg), arr, x.data_ptr(), None, y_ws.data_ptr(), work.ptr, work.nbytes, sh.current_stream()))
    sh.check(lib.souffle_bert_encoder_fused_static(C.byref(cfg), arr, x.data_ptr(), None, y_st.data_ptr(), sh.current_stream()))
    torch.cuda.synchronize()
    assert work.status() == 0
    flags = C.c_uint(99)
    sh.check(lib.souffle_bert_static_status(sh.current_stream(), C.byref(flags), 0))
    assert flags.value == 0          # no bounded wait gave up in the static array either
    return y_ws, y_st


def test_static_scratch_entry_point_equals_the_workspace_entry_point():
    # (nothing is cleared between the calls: other shapes, other layer counts and the many-rows kernel in between)
    announce("bert encoder without allocation: B=1 S=128 L=3, the smaller B=1 S=64 L=2, B=1 S=128 L=3 again, B=16 S=128 L=1, B=1 S=384 L=2")
    for B, S, layers, seed in [(1, 128, 3, 2), (1, 64, 2, 3), (1, 128, 3, 2), (16, 128, 1, 4), (1, 384, 2, 5)]:
        y_ws, y_st = _both(B, S, layers, seed)
        assert torch.isfinite(y_st.float()).all()
        assert torch.equal(y_ws, y_st), "B=%d S=%d L=%d: max diff %g" % (B, S, layers, (y_ws.float() - y_st.float()).abs().max().item())


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    announce("bert encoder without allocation: a configuration beyond the static scratch")
    lib = sh.lib()
    cfg = sh.BertCfg(2, 384, 768, 12, 3072, sh.ACT_GELU_TANH, 0.125, 1e-12, 12, 0)
    w = (sh.BertLayerW * 12)()
    rc = lib.souffle_bert_encoder_fused_static(C.byref(cfg), w, C.c_void_p(256), None, C.c_void_p(256), None)
    assert rc == -4 and "static scratch holds" in sh.last_error(), (rc, sh.last_error())
    assert lib.souffle_bert_encoder_fused_static(None, w, None, None, None, None) == -1
