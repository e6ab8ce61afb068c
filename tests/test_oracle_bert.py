"""Pins the BERT part of the CPU oracle (oracle/bert_oracle.c) against independent
library routines, closed forms and committed golden vectors.  CPU only."""
import os

import numpy as np
import pytest
import torch

import oracle
import synth
import torch_ref

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def small_weights(H, F, seed, with_bias=True):
    rng = np.random.default_rng(seed)
    w = {"qkv_weight": rng.normal(0, 0.2, (3, H, H)), "attn_fc_weight": rng.normal(0, 0.2, (H, H)),
         "fc1_weight": rng.normal(0, 0.2, (H, F)), "fc2_weight": rng.normal(0, 0.2, (F, H))}
    if with_bias:
        w.update({"qkv_bias": rng.normal(0, 0.3, (3 * H,)), "attn_fc_bias": rng.normal(0, 0.3, (H,)),
                  "ln1_gamma": 1 + rng.normal(0, 0.2, (H,)), "ln1_beta": rng.normal(0, 0.2, (H,)),
                  "fc1_bias": rng.normal(0, 0.3, (F,)), "fc2_bias": rng.normal(0, 0.3, (H,)),
                  "ln2_gamma": 1 + rng.normal(0, 0.2, (H,)), "ln2_beta": rng.normal(0, 0.2, (H,))})
    return {k: v.astype(np.float32) for k, v in w.items()}


def test_gemm_matches_matmul_and_layout():
    rng = np.random.default_rng(1)
    x, w, b = rng.normal(size=(37, 53)), rng.normal(size=(53, 29)), rng.normal(size=29)
    y = oracle.gemm(x, w, b)
    ref = (torch.from_numpy(x) @ torch.from_numpy(w) + torch.from_numpy(b)).numpy()
    np.testing.assert_allclose(y, ref, rtol=2e-5, atol=2e-5)
    # a transposed-operand mistake must fail: W is [K][N], not [N][K]
    e = np.zeros((53, 29)); e[5, 7] = 1.0
    y = oracle.gemm(x, e)
    assert np.allclose(y[:, 7], x[:, 5].astype(np.float32)) and np.count_nonzero(np.delete(y, 7, axis=1)) == 0


def test_layernorm_matches_torch_and_invariants():
    rng = np.random.default_rng(2)
    z = rng.normal(3.0, 5.0, size=(11, 768))
    g, b = rng.normal(1, 0.2, 768), rng.normal(0, 0.2, 768)
    for eps in (1e-12, 1e-5):
        y = oracle.layernorm(z, g, b, eps)
        ref = torch.nn.functional.layer_norm(torch.from_numpy(z), (768,), torch.from_numpy(g), torch.from_numpy(b), eps).numpy()
        np.testing.assert_allclose(y, ref, rtol=1e-4, atol=1e-4)
    y = oracle.layernorm(z, None, None, 1e-12)
    assert np.abs(y.mean(axis=1)).max() < 1e-5 and np.abs(y.var(axis=1) - 1).max() < 1e-4   # biased variance
    # eps sits inside the square root: a constant row maps to exactly 0, and a huge eps damps
    assert np.all(oracle.layernorm(np.full((2, 8), 3.0), None, None, 1e-5) == 0)
    y_big = oracle.layernorm(z[:1, :8], None, None, 1e6)
    assert np.abs(y_big).max() < 0.05


def test_gelu_tanh_closed_form():
    xs = np.array([-6.0, -1.0, -0.5, 0.0, 0.5, 1.0, 3.0, 8.0])
    ref = torch.nn.functional.gelu(torch.from_numpy(xs), approximate="tanh").numpy()
    np.testing.assert_allclose(oracle.gelu_tanh(xs), ref, rtol=1e-5, atol=1e-6)
    assert oracle.gelu_tanh([0.0])[0] == 0.0
    assert abs(oracle.gelu_tanh([10.0])[0] - 10.0) < 1e-5 and abs(oracle.gelu_tanh([-10.0])[0]) < 1e-5


def test_gelu_erf_closed_form():
    """The exact GELU against torch's library routine in float64, against math.erf at points whose erf is known to many
    digits, and apart from the tanh form where the two differ most."""
    import math
    xs = np.array([-6.0, -2.0, -1.0, -0.5, 0.0, 0.5, 1.0, 2.0, 3.0, 8.0])
    ref = torch.nn.functional.gelu(torch.from_numpy(xs)).numpy()
    np.testing.assert_allclose(oracle.gelu_erf(xs), ref, rtol=1e-6, atol=1e-7)
    for x in (0.3, 1.0, 1.7, -0.9):
        assert abs(oracle.gelu_erf([x])[0] - 0.5 * x * (1.0 + math.erf(x / math.sqrt(2.0)))) < 1e-6
    assert abs(oracle.gelu_erf([math.sqrt(2.0)])[0] - 0.5 * math.sqrt(2.0) * (1.0 + 0.8427007929497149)) < 1e-6      # erf(1)
    assert oracle.gelu_erf([0.0])[0] == 0.0
    assert abs(oracle.gelu_erf([10.0])[0] - 10.0) < 1e-6 and abs(oracle.gelu_erf([-10.0])[0]) < 1e-6
    d = np.abs(oracle.gelu_erf(np.linspace(-4, 4, 801)) - oracle.gelu_tanh(np.linspace(-4, 4, 801)))
    assert 1e-4 < d.max() < 1e-3                      # two different functions, up to about 5e-4 apart


@pytest.mark.parametrize("act,scale,eps", [("gelu_tanh", 0.25, 1e-12), ("relu", 1 / 64 ** 0.5, 1e-5), ("gelu", 0.125, 1e-12)])
def test_small_layer_matches_torch_all_stages(act, scale, eps):
    B, S, H, nh, F = 2, 16, 64, 4, 128
    rng = np.random.default_rng(3)
    w = small_weights(H, F, 4)
    x = rng.normal(size=(B * S, H)).astype(np.float32)
    mask = np.where(rng.random((B, S, S)) < 0.2, -1e4, 0.0).astype(np.float32)
    got = oracle.bert_layer(x, w, B, S, H, nh, F, act, scale, eps, mask=mask, dump=True)
    ref = torch_ref.bert_layer(x, w, B, S, nh, act, scale, eps, mask=mask)
    names = ["qkv", "probs", "ctx", "ln1", "fc1", "out"]
    for n, a, r in zip(names, got, ref):
        assert a.shape == r.shape, n
        np.testing.assert_allclose(a, r, rtol=2e-4, atol=2e-4, err_msg=n)


def test_bert_base_layer_matches_torch():
    """BASELINE config 0 shapes (B=1,S=128,H=768): the oracle at the size the GPU tests use."""
    w = synth.bert_layer_weights(0, 0, with_bias=True)
    x = synth.bert_input(0, 1, 128)
    got = oracle.bert_layer(x, w, 1, 128, dump=True)
    ref = torch_ref.bert_layer(x.astype(np.float32), {k: v.astype(np.float32) for k, v in w.items()}, 1, 128, 12)
    for a, r in zip(got, ref):
        np.testing.assert_allclose(a, r, rtol=3e-4, atol=3e-4)


def test_special_cases():
    B, S, H, nh, F = 1, 8, 32, 2, 64
    rng = np.random.default_rng(5)
    x = rng.normal(size=(S, H)).astype(np.float32)
    zero = {"qkv_weight": np.zeros((3, H, H)), "attn_fc_weight": np.zeros((H, H)), "fc1_weight": np.zeros((H, F)),
            "fc2_weight": np.zeros((F, H))}
    outs = oracle.bert_layer(x, zero, B, S, H, nh, F, dump=True)
    # zero weights: uniform attention, zero context, y = LN(LN(x)) = LN(x) up to rounding
    np.testing.assert_allclose(outs[1], 1.0 / S, atol=1e-7)
    assert np.all(outs[2] == 0)
    np.testing.assert_allclose(outs[5], oracle.layernorm(x), atol=1e-5)
    # softmax rows sum to one and are shift invariant in the mask
    w = small_weights(H, F, 6, with_bias=False)
    p0 = oracle.bert_layer(x, w, B, S, H, nh, F, dump=True)[1]
    p1 = oracle.bert_layer(x, w, B, S, H, nh, F, mask=np.full((B, S, S), 7.5), dump=True)[1]
    np.testing.assert_allclose(p0.sum(-1), 1.0, atol=1e-6)
    np.testing.assert_allclose(p0, p1, atol=1e-6)
    # value-only identity: with Wv = I and Wo = I, ctx = P.x (pins which of q/k/v slot 2 is, and the head merge)
    ident = dict(w)
    ident["qkv_weight"] = np.stack([w["qkv_weight"][0], w["qkv_weight"][1], np.eye(H)])
    o = oracle.bert_layer(x, ident, B, S, H, nh, F, dump=True)
    hd = H // nh
    for h in range(nh):
        np.testing.assert_allclose(o[2][:, h * hd:(h + 1) * hd], o[1][h] @ x[:, h * hd:(h + 1) * hd], atol=1e-5)


def test_encoder_is_layer_composition():
    B, S, H, nh, F = 1, 8, 32, 2, 64
    x = np.random.default_rng(7).normal(size=(S, H)).astype(np.float32)
    layers = [small_weights(H, F, 10 + i) for i in range(3)]
    y = x
    for l in layers:
        y = oracle.bert_layer(y, l, B, S, H, nh, F)
    np.testing.assert_array_equal(oracle.bert_encoder(x, layers, B, S, H, nh, F), y)


def test_golden_vectors():
    """Small committed vectors produced by tests/golden/make_golden.py from the torch
    float64 restatement."""
    g = np.load(os.path.join(GOLDEN, "bert_layer_small.npz"))
    w = {k[2:]: g[k] for k in g.files if k.startswith("w_")}
    outs = oracle.bert_layer(g["x"], w, int(g["B"]), int(g["S"]), int(g["H"]), int(g["heads"]), int(g["F"]),
                             "gelu_tanh", float(g["scale"]), float(g["eps"]), mask=g["mask"], dump=True)
    for n, a in zip(["qkv", "probs", "ctx", "ln1", "fc1", "out"], outs):
        np.testing.assert_allclose(a, g["out_" + n], rtol=2e-4, atol=2e-4, err_msg=n)
