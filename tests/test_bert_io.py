"""Embedding stage, pooler and the local checkpoint loader.

CPU part: the oracle against torch library routines (float64) and the loader's transposition
rule against torch.nn.functional.linear on the ORIGINAL [out, in] tensors.
GPU part (marked gpu): the HIP kernels through the C ABI against the oracle, fp16 tolerance
max-abs <= 2e-2, mean-abs <= 2e-3."""
import os

import numpy as np
import pytest
import torch

import oracle
import synth


def _tables(vocab=1000, max_pos=512, types=2, seed=40):
    g = lambda i, n, s: (synth.normal(synth.seed_of(seed, i), n) * s).astype(np.float16)
    word = g(0, vocab * 768, 0.05).reshape(vocab, 768)
    pos = g(1, max_pos * 768, 0.05).reshape(max_pos, 768)
    typ = g(2, types * 768, 0.05).reshape(types, 768)
    gam = (1.0 + g(3, 768, 0.1)).astype(np.float16)
    bet = g(4, 768, 0.1)
    return word, pos, typ, gam, bet


def _ids(B, S, vocab, seed=41):
    tok = (synth.uniform01(synth.seed_of(seed, 0), B * S) * vocab).astype(np.int32).reshape(B, S)
    seg = (synth.uniform01(synth.seed_of(seed, 1), B * S) < 0.5).astype(np.int32).reshape(B, S)
    return np.minimum(tok, vocab - 1), seg


def test_oracle_embed_matches_torch_embedding_and_layer_norm():
    word, pos, typ, gam, bet = _tables()
    tok, seg = _ids(3, 40, word.shape[0])
    got = oracle.bert_embed(tok, word, pos, typ, seg, gam, bet, eps=1e-12)
    F = torch.nn.functional
    d = lambda a: torch.from_numpy(a.astype(np.float64))
    tt, ss = torch.from_numpy(tok.astype(np.int64)), torch.from_numpy(seg.astype(np.int64))
    e = F.embedding(tt, d(word)) + d(pos)[:40].unsqueeze(0) + F.embedding(ss, d(typ))
    ref = F.layer_norm(e, (768,), d(gam), d(bet), 1e-12).reshape(-1, 768).numpy()
    assert np.abs(got - ref).max() < 2e-5
    # a swapped position / token-type table, or positions that run across sequences, must show
    wrong = F.embedding(tt, d(word)) + d(pos)[:120].reshape(3, 40, 768) + F.embedding(ss, d(typ))
    assert np.abs(got - F.layer_norm(wrong, (768,), d(gam), d(bet), 1e-12).reshape(-1, 768).numpy()).max() > 1e-2
    # no token types, no affine: plain normalisation with zero mean and unit variance per row
    plain = oracle.bert_embed(tok, word, pos)
    assert np.abs(plain.mean(axis=1)).max() < 1e-5 and np.abs(plain.var(axis=1) - 1).max() < 1e-3


def test_oracle_pooler_matches_torch_and_uses_first_token():
    B, S = 4, 16
    x = synth.bert_input(5, B, S)
    w = (synth.normal(synth.seed_of(42, 0), 768 * 768) * 0.02).astype(np.float16).reshape(768, 768)
    b = (synth.normal(synth.seed_of(42, 1), 768) * 0.02).astype(np.float16)
    got = oracle.bert_pooler(x, w, b, B, S)
    xt = torch.from_numpy(x.astype(np.float64)).reshape(B, S, 768)
    ref = torch.tanh(xt[:, 0] @ torch.from_numpy(w.astype(np.float64)) + torch.from_numpy(b.astype(np.float64))).numpy()
    assert np.abs(got - ref).max() < 2e-5
    assert np.abs(got - torch.tanh(xt[:, 1] @ torch.from_numpy(w.astype(np.float64))).numpy()).max() > 1e-2   # not token 1
    assert np.abs(got - torch.tanh(xt[:, 0] @ torch.from_numpy(w.astype(np.float64)).t()).numpy()).max() > 1e-2   # not W^T


def test_checkpoint_loader_applies_the_reference_transposition_rule(tmp_path):
    """A one-layer checkpoint with HuggingFace tensor names: the loaded [K][N] weights run through the
    oracle must give what torch computes from the original [out, in] tensors."""
    from safetensors.torch import save_file
    import bert_binding
    g = torch.Generator().manual_seed(7)
    rnd = lambda *s: (torch.randn(*s, generator=g) * 0.02)
    p = "encoder.layer.0."
    ck = {}
    for name, shape in [("attention.self.query", (768, 768)), ("attention.self.key", (768, 768)), ("attention.self.value", (768, 768)),
                        ("attention.output.dense", (768, 768)), ("intermediate.dense", (3072, 768)), ("output.dense", (768, 3072))]:
        ck[p + name + ".weight"] = rnd(*shape).half()
        ck[p + name + ".bias"] = rnd(shape[0]).half()
    for name in ("attention.output.LayerNorm", "output.LayerNorm"):
        ck[p + name + ".weight"] = (1 + rnd(768)).half()
        ck[p + name + ".bias"] = rnd(768).half()
    ck["pooler.dense.weight"], ck["pooler.dense.bias"] = rnd(768, 768).half(), rnd(768).half()
    path = os.path.join(tmp_path, "tiny.safetensors")
    save_file(ck, path)
    loaded = bert_binding.load_hf_bert(path)
    assert len(loaded["layers"]) == 1 and loaded["embeddings"] is None and loaded["pooler"] is not None
    lw = {k: v.numpy() for k, v in loaded["layers"][0].items()}
    assert lw["qkv_weight"].shape == (3, 768, 768) and lw["fc1_weight"].shape == (768, 3072) and lw["fc2_weight"].shape == (3072, 768)
    B, S = 1, 64
    x = synth.bert_input(9, B, S)
    got = oracle.bert_layer(x, lw, B, S)
    # the same layer with torch library ops on the checkpoint's own tensors (nn.Linear convention)
    F = torch.nn.functional
    d = lambda k: ck[k].double()
    xt = torch.from_numpy(x.astype(np.float64))
    q, k, v = (F.linear(xt, d(p + "attention.self.%s.weight" % n), d(p + "attention.self.%s.bias" % n)).reshape(S, 12, 64).transpose(0, 1)
               for n in ("query", "key", "value"))
    ctx = (torch.softmax(q @ k.transpose(1, 2) * 0.125, dim=-1) @ v).transpose(0, 1).reshape(S, 768)
    y1 = F.layer_norm(F.linear(ctx, d(p + "attention.output.dense.weight"), d(p + "attention.output.dense.bias")) + xt, (768,),
                      d(p + "attention.output.LayerNorm.weight"), d(p + "attention.output.LayerNorm.bias"), 1e-12)
    hmid = F.gelu(F.linear(y1, d(p + "intermediate.dense.weight"), d(p + "intermediate.dense.bias")), approximate="tanh")
    ref = F.layer_norm(F.linear(hmid, d(p + "output.dense.weight"), d(p + "output.dense.bias")) + y1, (768,),
                       d(p + "output.LayerNorm.weight"), d(p + "output.LayerNorm.bias"), 1e-12).numpy()
    assert np.abs(got - ref).max() < 5e-4
    pooled = oracle.bert_pooler(x, loaded["pooler"]["weight"].numpy(), loaded["pooler"]["bias"].numpy(), B, S)
    assert np.abs(pooled - torch.tanh(F.linear(xt[0], d("pooler.dense.weight"), d("pooler.dense.bias"))).numpy()).max() < 2e-5


def test_embed_and_pooler_reject_bad_arguments_without_gpu():
    import ctypes as C
    import souffle_hip as sh
    lib = sh.lib()
    P = C.c_void_p
    assert lib.souffle_bert_embed(None, None, None, 30522, None, 512, None, 2, None, None, 1e-12, 1, 128, 768, None, None, None) == -1
    assert lib.souffle_bert_embed(P(16), None, P(16), 30522, P(16), 512, None, 0, None, None, 1e-12, 1, 128, 512,
                                  P(16), None, None) == -2 and "hidden=768" in sh.last_error()
    assert lib.souffle_bert_embed(P(16), None, P(24), 30522, P(16), 512, None, 0, None, None, 1e-12, 1, 128, 768,
                                  P(16), None, None) == -3
    # table sizes the host can judge: a position table shorter than the sequence, empty tables
    assert lib.souffle_bert_embed(P(16), None, P(16), 30522, P(16), 64, None, 0, None, None, 1e-12, 1, 128, 768,
                                  P(16), None, None) == -2 and "pos_emb has 64 rows" in sh.last_error()
    assert lib.souffle_bert_embed(P(16), None, P(16), 0, P(16), 512, None, 0, None, None, 1e-12, 1, 128, 768,
                                  P(16), None, None) == -2 and "vocab_size" in sh.last_error()
    assert lib.souffle_bert_embed(P(16), P(16), P(16), 30522, P(16), 512, P(16), 0, None, None, 1e-12, 1, 128, 768,
                                  P(16), None, None) == -2 and "type_vocab_size" in sh.last_error()
    assert lib.souffle_bert_embed(P(16), None, P(16), 30522, P(16), 512, None, 0, None, None, 1e-12, 1, 128, 768,
                                  P(16), P(18), None) == -3
    assert lib.souffle_bert_pooler(None, None, None, 1, 128, 768, None, None) == -1
    assert lib.souffle_bert_pooler(C.c_void_p(16), C.c_void_p(16), None, 0, 128, 768, C.c_void_p(16), None) == -2


@pytest.mark.gpu
@pytest.mark.parametrize("B,S,with_types", [(1, 128, True), (3, 40, False), (32, 128, True)])
def test_embed_gpu_matches_oracle(B, S, with_types):
    import bert_binding
    from gpu_util import announce, assert_close, dev
    announce("bert embed B=%d S=%d types=%s" % (B, S, with_types))
    word, pos, typ, gam, bet = _tables()
    tok, seg = _ids(B, S, word.shape[0])
    ref = oracle.bert_embed(tok, word, pos, typ if with_types else None, seg if with_types else None, gam, bet)
    di = lambda a: torch.from_numpy(a).to("cuda:0")
    got = bert_binding.embed(di(tok), dev(word), dev(pos), dev(typ) if with_types else None, di(seg) if with_types else None,
                             dev(gam), dev(bet))
    torch.cuda.synchronize()
    assert_close("embeddings", got, ref)


@pytest.mark.gpu
def test_embed_gpu_clamps_and_counts_ids_outside_the_tables():
    """Ids that a tokenizer for another vocabulary would produce: no row outside the tables is read (the kernel
    clamps), the rows with good ids are unaffected, and the binding raises like host-side indexing would."""
    import bert_binding
    from gpu_util import announce, assert_close, dev
    announce("bert embed with out-of-range ids")
    B, S = 2, 64
    word, pos, typ, gam, bet = _tables()
    tok, seg = _ids(B, S, word.shape[0])
    ref = oracle.bert_embed(tok, word, pos, typ, seg, gam, bet)
    bad_tok, bad_seg = tok.copy(), seg.copy()
    bad_tok[0, 3] = word.shape[0]
    bad_tok[1, 7] = -5
    bad_tok[1, 9] = 2 ** 31 - 1
    bad_seg[0, 11] = typ.shape[0] + 4
    di = lambda a: torch.from_numpy(a).to("cuda:0")
    with pytest.raises(IndexError, match="4 token or segment ids"):
        bert_binding.embed(di(bad_tok), dev(word), dev(pos), dev(typ), di(bad_seg), dev(gam), dev(bet))
    got = bert_binding.embed(di(bad_tok), dev(word), dev(pos), dev(typ), di(bad_seg), dev(gam), dev(bet), check_ids=False)
    torch.cuda.synchronize()
    good = np.ones(B * S, dtype=bool)
    good[[0 * S + 3, 1 * S + 7, 1 * S + 9, 0 * S + 11]] = False
    assert_close("rows with ids inside the tables", got[torch.from_numpy(good).to("cuda:0")], ref.reshape(B * S, -1)[good])
    assert torch.isfinite(got.float()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("B,S", [(1, 128), (32, 128)])
def test_pooler_gpu_matches_oracle(B, S):
    import bert_binding
    from gpu_util import announce, assert_close, dev
    announce("bert pooler B=%d S=%d" % (B, S))
    x = synth.bert_input(6, B, S)
    w = (synth.normal(synth.seed_of(43, 0), 768 * 768) * 0.02).astype(np.float16).reshape(768, 768)
    b = (synth.normal(synth.seed_of(43, 1), 768) * 0.02).astype(np.float16)
    got = bert_binding.pooler(dev(x), dev(w), dev(b), B, S)
    torch.cuda.synchronize()
    assert_close("pooled", got, oracle.bert_pooler(x, w, b, B, S))


@pytest.mark.gpu
def test_embed_encoder_pooler_chain_gpu():
    """Token ids in, pooled vector out: embedding stage -> 2-layer fused encoder -> pooler, against the
    oracle chain on the same fp16 tables and weights."""
    import bert_binding
    from gpu_util import announce, assert_close, dev, dev_weights
    announce("bert embed -> encoder -> pooler chain")
    B, S, L = 1, 128, 2
    word, pos, typ, gam, bet = _tables()
    tok, seg = _ids(B, S, word.shape[0])
    ws = [synth.bert_layer_weights(2, l, with_bias=True) for l in range(L)]
    pw = (synth.normal(synth.seed_of(44, 0), 768 * 768) * 0.02).astype(np.float16).reshape(768, 768)
    di = lambda a: torch.from_numpy(a).to("cuda:0")
    e = bert_binding.embed(di(tok), dev(word), dev(pos), dev(typ), di(seg), dev(gam), dev(bet))
    y = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)(e)
    pooled = bert_binding.pooler(y, dev(pw), None, B, S)
    torch.cuda.synchronize()
    e_ref = oracle.bert_embed(tok, word, pos, typ, seg, gam, bet).astype(np.float16).astype(np.float32)
    y_ref = oracle.bert_encoder(e_ref, ws, B, S)
    assert_close("chain encoder output", y, y_ref)
    assert_close("chain pooled", pooled, oracle.bert_pooler(y_ref, pw, None, B, S))


def test_erf_gelu_is_not_taken_for_the_tanh_form():
    """HuggingFace's "gelu" is the erf form and has a configuration value of its own; the default stays the tanh form
    that the reference's kernels compute."""
    import bert_binding
    import souffle_hip as sh
    assert bert_binding.make_cfg(1, 128, act="gelu").act == sh.ACT_GELU_ERF != sh.ACT_GELU_TANH
    assert bert_binding.make_cfg(1, 128, act="gelu_tanh").act == bert_binding.make_cfg(1, 128).act == sh.ACT_GELU_TANH
    with pytest.raises(ValueError):
        bert_binding.make_cfg(1, 128, act="swish")
