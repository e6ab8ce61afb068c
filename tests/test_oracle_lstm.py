"""Pins oracle/lstm_oracle.c against torch.nn.LSTMCell and analytic special cases.  CPU only."""
import numpy as np

import oracle
import torch_ref


def rand(seed, L, Hd, T):
    rng = np.random.default_rng(seed)
    return (rng.uniform(-0.3, 0.3, (4 * L, Hd, Hd)).astype(np.float32), rng.uniform(-0.3, 0.3, (4 * L, Hd, Hd)).astype(np.float32),
            rng.normal(size=(T, Hd)).astype(np.float32), rng.normal(0, 0.2, (L, 4, Hd)).astype(np.float32))


def test_matches_lstmcell_stack():
    w_ih, w_hh, x, b = rand(1, 3, 24, 9)
    np.testing.assert_allclose(oracle.lstm(x, w_ih, w_hh), torch_ref.lstm_stack(x, w_ih, w_hh), atol=2e-6)
    np.testing.assert_allclose(oracle.lstm(x, w_ih, w_hh, b), torch_ref.lstm_stack(x, w_ih, w_hh, b), atol=2e-6)


def test_benchmark_shape_matches_lstmcell():
    import synth
    w_ih, w_hh, x = synth.lstm_tensors(1, layers=10, hidden=256, timesteps=12)
    np.testing.assert_allclose(oracle.lstm(x, w_ih, w_hh), torch_ref.lstm_stack(x, w_ih.astype(np.float32), w_hh.astype(np.float32)), atol=5e-6)


def test_gate_order_and_forget_bias():
    """igfo + forget bias (the reference kernel's variant) equals ifgo on slot-swapped
    matrices with the bias folded into the forget gate."""
    w_ih, w_hh, x, b = rand(2, 2, 16, 7)
    L, Hd = 2, 16
    swap = lambda w: np.concatenate([w[4 * l:4 * l + 4][[0, 2, 1, 3]] for l in range(L)])
    b2 = b.copy()
    b2[:, 1, :] += 1.0
    want = oracle.lstm(x, w_ih, w_hh, b2, "ifgo", 0.0)
    got = oracle.lstm(x, swap(w_ih), swap(w_hh), b[:, [0, 2, 1, 3], :], "igfo", 1.0)
    np.testing.assert_allclose(got, want, atol=1e-6)


def test_special_cases():
    L, Hd, T = 3, 8, 5
    z = np.zeros((4 * L, Hd, Hd), np.float32)
    x = np.random.default_rng(3).normal(size=(T, Hd)).astype(np.float32)
    assert np.all(oracle.lstm(x, z, z) == 0)          # zero weights: g = tanh(0) = 0, so c = h = 0
    # the reference's smoke test (all-ones weights and inputs, cpp/lstm/test_lstm.py:4-13) saturates every gate:
    # c_t = c_{t-1} + 1, h_t = tanh(c_t)
    one = np.full((4 * L, Hd, Hd), 10.0, np.float32)
    y = oracle.lstm(np.ones((T, Hd), np.float32), one, one)
    np.testing.assert_allclose(y[:, 0], np.tanh(np.arange(1, T + 1)), atol=1e-3)
    # layer l at step t depends on x_t (no one-step lag): y_0 is already non-zero
    w_ih, w_hh, x, _ = rand(4, 1, 8, 3)
    assert np.abs(oracle.lstm(x, w_ih, w_hh)[0]).max() > 1e-3
