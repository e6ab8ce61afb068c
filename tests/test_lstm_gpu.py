"""GPU parity of the stacked LSTM (through the C ABI via lstm_binding) against the CPU oracle.
Tolerance: max-abs <= 2e-2, mean-abs <= 2e-3 (fp16 weights, fp32 state)."""
import numpy as np
import pytest
import torch

import oracle
import synth
from gpu_util import announce, assert_close, dev

pytestmark = pytest.mark.gpu


def run(x, w_ih, w_hh, **kw):
    import lstm_binding
    y = lstm_binding.fused_lstm(dev(x, torch.float32).view(1, -1, 256), dev(w_ih), dev(w_hh), **kw)
    torch.cuda.synchronize()
    return y[0]


def test_config1_matches_oracle():
    """Benchmark config 1: 10 layers x 256, T=100, U(-1/16,1/16) fp16 weights, gates i,f,g,o."""
    announce("lstm cfg1 L=10 T=100")
    w_ih, w_hh, x = synth.lstm_tensors(1)
    ref = oracle.lstm(x, w_ih, w_hh)
    assert_close("lstm y", run(x, w_ih, w_hh), ref)


def test_reference_variant_with_bias():
    """Gate slots i,g,f,o and forget bias 1.0 as in cpp/lstm/lstm_reuse_shared_memory.cu:309-318, plus a bias."""
    announce("lstm igfo fb=1 bias")
    w_ih, w_hh, x = synth.lstm_tensors(5, layers=10, timesteps=37)
    bias = synth.normal(synth.seed_of(5, 9), (10, 4, 256), 0.2).astype(np.float32)
    ref = oracle.lstm(x, w_ih, w_hh, bias, "igfo", 1.0)
    got = run(x, w_ih, w_hh, bias=dev(bias, torch.float32), gate_order="igfo", forget_bias=1.0)
    assert_close("lstm y", got, ref)


@pytest.mark.parametrize("L,T", [(1, 1), (3, 5), (10, 256)])
def test_ragged_sizes_and_repeat_calls(L, T):
    announce("lstm L=%d T=%d" % (L, T))
    w_ih, w_hh, x = synth.lstm_tensors(6, layers=L, timesteps=T)
    ref = oracle.lstm(x, w_ih, w_hh)
    a = run(x, w_ih, w_hh)
    b = run(x, w_ih, w_hh)      # the workspace tags must be clean again after a call
    assert_close("lstm y", a, ref)
    assert torch.equal(a, b)


def test_all_ones_smoke_of_reference():
    """cpp/lstm/test_lstm.py:4-13: all-ones inputs and weights; saturated gates give h_t = tanh(t+1)."""
    announce("lstm all ones")
    one = np.ones((40, 256, 256), np.float32)
    y = run(np.ones((100, 256), np.float32), one, one).cpu().numpy()
    np.testing.assert_allclose(y[:, 0], np.tanh(np.arange(1, 101)), atol=1e-3)
    assert np.all(y == y[:, :1])


def test_workspace_of_unknown_content_is_usable_after_init():
    """A C caller's workspace comes from hipMalloc with whatever the memory held: souffle_workspace_init
    zeroes all of it (step tags, hand-over words), after which any entry point may use it, one after the
    other.  Here the workspace is filled with ones first, and serves the LSTM and the Swin block pair."""
    announce("dirty workspace -> init -> lstm, swin")
    import ctypes as C
    import souffle_hip as sh
    w_ih, w_hh, x = synth.lstm_tensors(5, layers=3, timesteps=9)
    lcfg = sh.LstmCfg(3, 256, 9, 1, sh.GATES_IFGO, 0.0)
    scfg = sh.SwinCfg(14, 14, 128, 4, 7, 3, 4, 1, 1e-5)
    nbytes = max(sh.lib().souffle_lstm_workspace_bytes(C.byref(lcfg)), sh.lib().souffle_swin_workspace_bytes(C.byref(scfg)))
    buf = torch.full(((nbytes + 15) // 16 * 4,), 0x3F800001, dtype=torch.int32, device="cuda:0")
    sh.check(sh.lib().souffle_workspace_init(buf.data_ptr(), buf.numel() * 4, sh.current_stream()))
    assert int(buf.abs().max().item()) == 0
    dx, dwi, dwh = dev(x, torch.float32), dev(w_ih), dev(w_hh)
    y = torch.empty((9, 256), dtype=torch.float32, device="cuda:0")
    ws_np = [synth.swin_block_weights(3, b) for b in range(2)]
    dws = [{k: dev(v) for k, v in w.items()} for w in ws_np]
    arr = (sh.SwinBlockW * 2)(*[sh.SwinBlockW(*[sh.ptr(w.get(k)) for k in sh.SWIN_W_FIELDS]) for w in dws])
    xs = synth.swin_input(3, 14 * 14)
    dxs = dev(xs)
    ys = torch.empty_like(dxs)
    for _ in range(2):
        sh.check(sh.lib().souffle_lstm_fused(C.byref(lcfg), dwi.data_ptr(), dwh.data_ptr(), None, dx.data_ptr(), y.data_ptr(),
                                            buf.data_ptr(), buf.numel() * 4, sh.current_stream()))
        sh.check(sh.lib().souffle_swin_block_pair_fused(C.byref(scfg), arr, dxs.data_ptr(), ys.data_ptr(), buf.data_ptr(),
                                                        buf.numel() * 4, sh.current_stream()))
        torch.cuda.synchronize()
        assert_close("lstm y", y, oracle.lstm(x, w_ih, w_hh))
        assert_close("swin y", ys, oracle.swin_block_pair(xs, ws_np, 14, 14))
