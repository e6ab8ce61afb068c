"""GPU parity of the BERT encoder layer / encoder (through the C ABI via bert_binding)
against the CPU oracle on identical fp16-rounded seeded inputs.
Tolerance: max-abs <= 2e-2 and mean-abs <= 2e-3 on every tensor the reference returns."""
import numpy as np
import pytest
import torch

import oracle
import synth
from gpu_util import announce, assert_close, dev, dev_weights

pytestmark = pytest.mark.gpu
NAMES = ["output_qkv", "query_key_output", "attn_value_output", "attn_fc_output", "feed_forward_fc1_output",
         "feed_forward_fc2_output"]


def run_layer(w, x, B, S, opt_level, **kw):
    import bert_binding
    dw = dev_weights(w)
    extra = {k: dw[k] for k in dw if k not in ("qkv_weight", "attn_fc_weight", "fc1_weight", "fc2_weight")}
    outs = bert_binding.souffle_bert_layer(dev(x).view(B, S, 768), dw["qkv_weight"], dw["attn_fc_weight"],
                                           dw["fc1_weight"], dw["fc2_weight"], opt_level, **extra, **kw)
    torch.cuda.synchronize()
    return outs


@pytest.mark.parametrize("pack", [True, False])
@pytest.mark.parametrize("opt_level", [4, 1])
@pytest.mark.parametrize("B,S", [(1, 128), (1, 384), (1, 64), (2, 256)])
def test_layer_config0_all_stages(B, S, opt_level, pack):
    """Benchmark config 0 (zero biases, gamma 1, beta 0, tanh-GELU, scale 1/8, eps 1e-12, no mask), with the packed
    copy of the FC2 weights (whole-K FC2 items) and with the [K][N] matrix alone (split-K FC2)."""
    announce("bert layer cfg0 B=%d S=%d opt=%d pack=%d" % (B, S, opt_level, pack))
    w, x = synth.bert_layer_weights(0, 0), synth.bert_input(0, B, S)
    ref = oracle.bert_layer(x, w, B, S, dump=True)
    got = run_layer(w, x, B, S, opt_level, pack=pack)
    for n, g, r in zip(NAMES, got, ref):
        assert_close(n, g, r)


@pytest.mark.parametrize("pack", [True, False])
@pytest.mark.parametrize("opt_level", [3, 2])
def test_layer_bias_affine_mask(opt_level, pack):
    announce("bert layer bias+affine+mask opt=%d pack=%d" % (opt_level, pack))
    B, S = 2, 128
    w, x = synth.bert_layer_weights(0, 1, with_bias=True), synth.bert_input(7, B, S)
    keep = synth.uniform01(synth.seed_of(0, 99), B * S * S).reshape(B, S, S) < 0.85
    keep[:, :, 0] = True
    mask = np.where(keep, 0.0, -10000.0).astype(np.float16)
    ref = oracle.bert_layer(x, w, B, S, mask=mask, dump=True)
    got = run_layer(w, x, B, S, opt_level, mask=dev(mask), pack=pack)
    for n, g, r in zip(NAMES, got, ref):
        assert_close(n, g, r)


@pytest.mark.parametrize("B,S,opt_level,pack", [(1, 128, 4, True), (1, 128, 1, False), (2, 256, 4, False), (16, 128, 4, False), (9, 128, 4, True), (13, 128, 4, False)])
def test_layer_erf_gelu(B, S, opt_level, pack):
    """The exact (erf) GELU of HuggingFace checkpoints, on the few-rows kernel and on both tile sizes of the many-rows one."""
    announce("bert layer erf-GELU B=%d S=%d opt=%d pack=%d" % (B, S, opt_level, pack))
    w, x = synth.bert_layer_weights(0, 3, with_bias=True), synth.bert_input(1, B, S)
    ref = oracle.bert_layer(x, w, B, S, act="gelu", dump=True)
    got = run_layer(w, x, B, S, opt_level, act="gelu", pack=pack)
    for n, g, r in zip(NAMES, got, ref):
        assert_close(n, g, r)
    # ... and it is not the tanh form: the FC1 outputs of the two differ where the oracle's do
    tanh_form = run_layer(w, x, B, S, opt_level, pack=pack)[4]
    assert not torch.equal(tanh_form, got[4])


def test_layer_reference_compat_mode():
    """What the reference's fused CUDA path computes: ReLU, scale 1/sqrt(768), eps 1e-5."""
    announce("bert layer reference-compat")
    B, S = 1, 384
    w, x = synth.bert_layer_weights(0, 2), synth.bert_input(0, B, S)
    ref = oracle.bert_layer(x, w, B, S, act="relu", scale=768 ** -0.5, ln_eps=1e-5, dump=True)
    got = run_layer(w, x, B, S, 4, reference_compat=True)
    for n, g, r in zip(NAMES, got, ref):
        assert_close(n, g, r)


def test_layer_mfma_bound_shape():
    """B=32, S=128 (M=4096): the large-tile path."""
    announce("bert layer B=32 S=128")
    B, S = 32, 128
    w, x = synth.bert_layer_weights(2, 0), synth.bert_input(2, B, S)
    ref = oracle.bert_layer(x, w, B, S, dump=True)
    for opt in (4, 1):
        got = run_layer(w, x, B, S, opt)
        for n, g, r in zip(NAMES, got, ref):
            assert_close("%s(opt %d)" % (n, opt), g, r)


def test_fast_path_equals_dump_path_and_is_deterministic():
    announce("bert layer dump=False determinism")
    B, S = 1, 128
    w, x = synth.bert_layer_weights(0, 0), synth.bert_input(0, B, S)
    for pack in (True, False):
        full = run_layer(w, x, B, S, 4, pack=pack)[-1]
        a = run_layer(w, x, B, S, 4, dump=False, pack=pack)
        b = run_layer(w, x, B, S, 4, dump=False, pack=pack)
        c = run_layer(w, x, B, S, 1, dump=False, pack=pack)
        assert torch.equal(a, b) and torch.equal(a, full)
        assert torch.equal(a, c), "fused and per-op paths run the same arithmetic"


# (13 x 128 and 5 x 384: 1664 and 1920 rows, no multiple of 256: the many-rows kernel on its 128 x 128 tiles)
@pytest.mark.parametrize("B,S,layers,pack", [(1, 128, 12, True), (1, 384, 12, True), (32, 128, 12, True), (9, 128, 2, True), (8, 128, 2, True),
                                             (3, 384, 2, True), (1, 128, 12, False), (1, 384, 3, False), (9, 128, 2, False), (2, 512, 2, True),
                                             (13, 128, 2, True), (5, 384, 2, True)])
def test_encoder_matches_oracle(B, S, layers, pack):
    announce("bert encoder B=%d S=%d L=%d pack=%d" % (B, S, layers, pack))
    import bert_binding
    ws = [synth.bert_layer_weights(2, l) for l in range(layers)]
    x = synth.bert_input(2, B, S)
    ref = oracle.bert_encoder(x, ws, B, S)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S, pack=pack)
    y_f = enc(dev(x), fused=True)
    y_u = enc(dev(x), fused=False)
    torch.cuda.synchronize()
    assert enc.ws.status() == 0
    # errors of successive layers do not compound past the tolerance because each layer ends in a LayerNorm
    assert_close("encoder fused", y_f, ref)
    assert_close("encoder unfused", y_u, ref)
    assert torch.equal(y_f, y_u)


@pytest.mark.parametrize("B,S,layers", [(32, 128, 5), (16, 128, 4), (64, 128, 3), (8, 384, 3), (8, 256, 3), (32, 64, 3), (4, 512, 2), (6, 384, 2),
                                        (13, 128, 2), (5, 384, 2)])
def test_many_rows_encoder_reuses_its_buffers(B, S, layers):
    """At many rows all layers of the fused launch share one set of inter-stage buffers (kept coherent
    by a cache invalidation at the barrier that ends a layer) and the LayerNorms are handed over per
    256-row block: results equal the per-op chain bit for bit over several layers, on repeated launches
    and with a different input in between (a line that survived from an earlier layer or launch would
    show), and no bounded wait gives up."""
    announce("bert encoder many rows, shared buffers B=%d S=%d L=%d" % (B, S, layers))
    import bert_binding
    ws = [synth.bert_layer_weights(2, l) for l in range(layers)]
    x0, x1 = synth.bert_input(2, B, S), synth.bert_input(3, B, S)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    y_u0 = enc(dev(x0), fused=False).clone()
    y_u1 = enc(dev(x1), fused=False).clone()
    y_a = enc(dev(x0)).clone()
    y_b = enc(dev(x1)).clone()
    y_c = enc(dev(x0)).clone()
    torch.cuda.synchronize()
    assert enc.ws.status() == 0
    assert torch.equal(y_a, y_u0) and torch.equal(y_c, y_u0) and torch.equal(y_b, y_u1)
    assert_close("encoder many rows", y_a, oracle.bert_encoder(x0, ws, B, S))


def test_many_rows_encoder_large_batch_fused_equals_per_op():
    """16384 rows (four tiles per workgroup and stage): too large for the oracle in a test, so the check is
    the size-independent one: the fused launch and the per-op chain, which synchronise in different ways
    (hand-overs per row block against kernel boundaries), agree bit for bit, twice."""
    announce("bert encoder B=128 S=128 L=2 fused vs per-op")
    import bert_binding
    B, S, layers = 128, 128, 2
    ws = [synth.bert_layer_weights(2, l) for l in range(layers)]
    x = dev(synth.bert_input(6, B, S))
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    y_u = enc(x, fused=False).clone()
    y_a = enc(x).clone()
    y_b = enc(x).clone()
    torch.cuda.synchronize()
    assert enc.ws.status() == 0
    assert torch.isfinite(y_a.float()).all()
    assert torch.equal(y_a, y_u) and torch.equal(y_b, y_u)


def test_many_rows_encoder_in_a_workspace_of_unknown_content():
    """The many-rows path clears its own hand-over words and writes every buffer before it reads it: a
    workspace that held arbitrary bytes and was initialised again gives the same result, and so does one
    that other shapes of the encoder have used in between."""
    announce("bert encoder many rows, dirtied workspace")
    import bert_binding
    import souffle_hip as sh
    B, S, layers = 16, 128, 3
    ws = [synth.bert_layer_weights(2, l) for l in range(layers)]
    x = dev(synth.bert_input(4, B, S))
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    y_u = enc(x, fused=False).clone()
    enc.ws.buf.fill_(-1)
    sh.check(sh.lib().souffle_workspace_init(enc.ws.ptr, enc.ws.nbytes, sh.current_stream()))
    y_a = enc(x).clone()
    small = bert_binding.Encoder([dev_weights(w) for w in ws[:1]], 1, 128)
    small.ws = enc.ws                                    # another shape of the encoder in the same memory
    small(dev(synth.bert_input(4, 1, 128)))
    y_b = enc(x).clone()
    torch.cuda.synchronize()
    assert enc.ws.status() == 0
    assert torch.equal(y_a, y_u) and torch.equal(y_b, y_u)


@pytest.mark.parametrize("B,S,layers", [(1, 128, 12), (1, 384, 2), (2, 64, 3), (1, 128, 1), (3, 256, 2)])
def test_few_rows_handovers_on_repeated_launches(B, S, layers):
    """The flag hand-overs of the few-rows encoder: launch after launch on one workspace, with another input
    in between (a value that survived from an earlier launch, in a cache or in a flag word, would show), fused
    and per-op launches give the same bits, all LayerNorm vectors and biases present, and no bounded wait gives up."""
    announce("bert encoder few rows, repeated launches B=%d S=%d L=%d" % (B, S, layers))
    import bert_binding
    ws = [synth.bert_layer_weights(2, l, with_bias=True) for l in range(layers)]
    x0, x1 = synth.bert_input(2, B, S), synth.bert_input(3, B, S)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    y_u = enc(dev(x0), fused=False).clone()
    y_1 = enc(dev(x0)).clone()
    z_1 = enc(dev(x1)).clone()
    y_2 = enc(dev(x0)).clone()
    z_u = enc(dev(x1), fused=False).clone()
    y_3 = enc(dev(x0)).clone()
    flags = enc.ws.status()
    assert flags == 0, "a bounded wait gave up (flags %d)" % flags
    assert torch.equal(y_1, y_u) and torch.equal(y_2, y_u) and torch.equal(y_3, y_u) and torch.equal(z_1, z_u)
    assert_close("encoder x0", y_1, oracle.bert_encoder(x0, ws, B, S))
    assert_close("encoder x1", z_1, oracle.bert_encoder(x1, ws, B, S))


def test_pack_fc2_layout():
    """souffle_bert_pack_fc2: 48 slices of 16 columns, 96 k-steps of 64 lanes x 8 halves each; lane L of k-step t holds
    W[32 t + 8 (L / 16) + 0..7][16 s + L % 16]."""
    announce("bert pack_fc2 layout")
    import bert_binding
    w = synth.bert_layer_weights(1, 0)["fc2_weight"]
    got = bert_binding.pack_fc2(dev(w)).cpu().numpy().reshape(48, 96, 64, 8)
    s_, t_, L_, j_ = np.meshgrid(np.arange(48), np.arange(96), np.arange(64), np.arange(8), indexing="ij")
    want = w[32 * t_ + 8 * (L_ // 16) + j_, 16 * s_ + L_ % 16]
    assert np.array_equal(got, want)


def test_few_rows_polled_copy_is_voted_in_the_first_launches():
    """Each XCD polls one of two copies of the hand-over words; which one is decided by votes that workgroup x of
    XCD x casts at the end of the first eight launches on a workspace.  A fresh workspace has no votes and polls the
    first copy of every pair; after ten launches every XCD has its eight votes and polls a block of its own pair;
    the output is the same bits whichever copy is polled."""
    announce("bert encoder few rows: votes on the polled copy")
    import ctypes as C
    import bert_binding
    import souffle_hip as sh
    B, S, layers = 1, 128, 2
    dws = [dev_weights(synth.bert_layer_weights(3, l, with_bias=True)) for l in range(layers)]
    enc = bert_binding.Encoder(dws, B, S)
    enc.ws = sh.Workspace(enc.ws.nbytes)                     # (a fresh, zeroed one: the binding shares workspaces between encoders)
    x = dev(synth.bert_input(9, B, S))

    def polled():
        votes, blocks = (C.c_int * 8)(), (C.c_int * 8)()
        sh.check(sh.lib().souffle_bert_polled_copies(enc.ws.ptr, enc.ws.nbytes, votes, blocks, sh.current_stream()))
        return list(votes), list(blocks)

    votes, blocks = polled()
    assert votes == [0] * 8 and blocks == [(x_ >> 1) * 4 + (x_ & 1) for x_ in range(8)]
    first = enc(x).clone()
    for i in range(9):
        assert torch.equal(enc(x), first), "launch %d" % (i + 2)
    votes, blocks = polled()
    assert votes == [8] * 8, votes
    for x_ in range(8):
        base = (x_ >> 1) * 4 + (x_ & 1)
        assert blocks[x_] in (base, base + 2), (x_, blocks)
    assert enc.ws.status() == 0


def test_few_rows_shapes_take_turns_in_one_workspace():
    """Flag words, ticket counters and completion words of the few-rows kernel carry over from launch to launch
    and are indexed by shape-dependent tile numbers: encoders of different shapes and depths, fused and per-op,
    that take turns in ONE workspace must each give what they give in a workspace of their own."""
    announce("bert encoder few rows, several shapes sharing a workspace")
    import bert_binding
    ws = [synth.bert_layer_weights(6, l, with_bias=True) for l in range(4)]
    dws = [dev_weights(w) for w in ws]
    # (with and without the packed copy of the FC2 weights: the two forms of FC2 use different words of the workspace)
    cases = [(1, 128, 4, True), (2, 64, 2, False), (1, 256, 3, True), (3, 128, 1, True), (1, 384, 2, False), (1, 128, 4, False)]
    encs, xs, want = [], [], []
    for B, S, layers, pack in cases:
        enc = bert_binding.Encoder(dws[:layers], B, S, pack=pack)
        x = dev(synth.bert_input(7, B, S))
        want.append(enc(x).clone())
        encs.append(enc)
        xs.append(x)
    shared = max(encs, key=lambda e: e.ws.nbytes).ws
    for e in encs:
        e.ws = shared
    for rnd in range(3):
        for i, (e, x) in enumerate(zip(encs, xs)):
            got = e(x, fused=(rnd + i) % 3 != 2).clone()
            assert torch.equal(got, want[i]), "round %d, case %s" % (rnd, cases[i])
    assert shared.status() == 0


@pytest.mark.parametrize("B,S", [(1, 128), (1, 384), (8, 128), (16, 128)])
def test_layernorm_of_rows_far_from_zero(B, S):
    """Rows whose mean is far larger than their spread, and feature columns of large magnitude: the LayerNorm
    statistics (per-slice mean and squared deviations, combined pairwise) and the normalisation in the operand
    registers must not lose the spread to cancellation.  Checked against the oracle on the few-rows path, at both
    places where a LayerNorm is applied on load (LN1 inside FC1, LN2 inside the next layer's QKV and at the end),
    at 1024 rows (several m-tiles per workgroup), and on the many-rows path (2048 rows), whose LayerNorm stages are
    separate passes over the rows."""
    announce("bert encoder B=%d S=%d, rows with a large mean" % (B, S))
    import bert_binding
    layers = 2
    ws = [synth.bert_layer_weights(2, l, with_bias=True) for l in range(layers)]
    x = synth.bert_input(5, B, S)
    # The biases of both sublayers carry the offsets, so that the pre-LayerNorm sums (not the attention inputs,
    # whose fp16 rounding a near one-hot softmax would amplify) are what is far from zero: every row of z1 has
    # mean 25 and two columns of magnitude 300, every row of z2 mean -30 and a column of magnitude 1000.
    for w in ws:
        b1 = w["attn_fc_bias"].astype(np.float32) + 25.0
        b1[17] += 300.0
        b1[500] -= 250.0
        w["attn_fc_bias"] = b1.astype(np.float16)
        b2 = w["fc2_bias"].astype(np.float32) - 30.0
        b2[3] += 1000.0
        w["fc2_bias"] = b2.astype(np.float16)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    y_f = enc(dev(x))
    y_u = enc(dev(x), fused=False)
    assert enc.ws.status() == 0
    assert torch.equal(y_f, y_u)
    assert_close("encoder, rows far from zero", y_f, oracle.bert_encoder(x, ws, B, S))


def test_cooperative_launch_matches_oracle():
    """The persistent encoder launched with hipLaunchCooperativeKernel (the runtime's co-residency guarantee)
    instead of the plain launch: same results, checked against the oracle, and an encoder of the many-rows path
    built afterwards in memory that the first one has given back works as well."""
    announce("bert encoder, cooperative launch")
    import bert_binding
    import souffle_hip as sh
    B, S, layers = 1, 128, 3
    ws = [synth.bert_layer_weights(2, l) for l in range(layers)]
    x = synth.bert_input(2, B, S)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    y_plain = enc(dev(x)).clone()
    sh.set_cooperative_launch(True)
    try:
        y_coop = enc(dev(x)).clone()
        y_coop2 = enc(dev(x)).clone()
        flags = enc.ws.status()
        big = bert_binding.Encoder([dev_weights(w) for w in ws[:2]], 8, 128)
        xb = synth.bert_input(3, 8, 128)
        y_big_coop = big(dev(xb)).clone()
        flags |= big.ws.status()
    finally:
        sh.set_cooperative_launch(False)
    assert flags == 0
    assert torch.equal(y_coop, y_plain) and torch.equal(y_coop2, y_plain)
    assert_close("encoder cooperative", y_coop, oracle.bert_encoder(x, ws, B, S))
    del enc, y_coop, y_coop2
    again = bert_binding.Encoder([dev_weights(w) for w in ws[:2]], 8, 128)      # (in memory the first encoder used)
    y_big = again(dev(xb))
    assert again.ws.status() == 0
    assert torch.equal(y_big, y_big_coop)
    assert_close("many rows after cooperative launches", y_big, oracle.bert_encoder(xb, ws[:2], 8, 128))


@pytest.mark.parametrize("B,S,layers,masked", [(1, 100, 2, False), (2, 77, 1, True), (1, 200, 1, False), (3, 5, 1, False)])
def test_sequence_lengths_that_are_not_built(B, S, layers, masked):
    """Any length up to 512 runs as the next built one with the surplus keys masked out; the result is
    that of the unpadded computation (oracle at the true length)."""
    announce("bert encoder B=%d S=%d L=%d masked=%s" % (B, S, layers, masked))
    import bert_binding
    ws = [synth.bert_layer_weights(2, l, with_bias=True) for l in range(layers)]
    x = synth.bert_input(5, B, S)
    mask = None
    if masked:
        keep = synth.uniform01(synth.seed_of(0, 98), B * S * S).reshape(B, S, S) < 0.9
        keep[:, :, 0] = True
        mask = np.where(keep, 0.0, -10000.0).astype(np.float16)
    ref = x
    for w in ws:
        ref = oracle.bert_layer(ref, w, B, S, mask=mask)
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    md = None if mask is None else dev(mask)
    y_f = enc(dev(x), fused=True, mask=md).clone()
    y_u = enc(dev(x), fused=False, mask=md).clone()
    torch.cuda.synchronize()
    assert tuple(y_f.shape) == (B * S, 768)
    assert_close("encoder fused", y_f, ref)
    assert torch.equal(y_f, y_u)
    if layers == 1:
        outs = run_layer(ws[0], x, B, S, 4, mask=md, pack=True)      # (the encoder object packs its FC2 weights: same form of FC2)
        full = oracle.bert_layer(x, ws[0], B, S, mask=mask, dump=True)
        for n, g, r in zip(NAMES, outs, full):
            assert_close(n, g, r)
        assert torch.equal(outs[-1], y_f)


@pytest.mark.parametrize("fused", [True, False])
def test_encoder_replays_from_a_hip_graph(fused):
    """The entry points allocate nothing and queue only kernels, so a caller may capture them: a graph
    of the encoder is replayed several times, with eager launches and synchronisations in between, and
    every replay must give the eager result."""
    announce("bert encoder in a HIP graph fused=%s" % fused)
    import bert_binding
    B, S, layers = 1, 128, 3
    ws = [synth.bert_layer_weights(2, l) for l in range(layers)]
    enc = bert_binding.Encoder([dev_weights(w) for w in ws], B, S)
    x1, x2 = dev(synth.bert_input(2, B, S)), dev(synth.bert_input(3, B, S))
    eager1, eager2 = enc(x1, fused=fused).clone(), enc(x2, fused=fused).clone()
    xin = x1.clone()
    out = torch.empty_like(eager1)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        enc(xin, out=out, fused=fused)
    for i, (xs, ref) in enumerate([(x1, eager1), (x2, eager2), (x1, eager1), (x2, eager2)]):
        xin.copy_(xs)
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref), "replay %d differs from the eager result" % i
        assert torch.equal(enc(xs, fused=fused), ref)          # eager work between the replays
    assert enc.ws.status() == 0


def test_souffle_bert_base_module():
    """The reference's zero-weight 12-layer driver (cpp/bert/bert_base_impl.cu:277-308): returns 0."""
    announce("souffle_bert_base")
    import souffle_bert_base
    assert souffle_bert_base.souffle_bert_base() == 0
    assert souffle_bert_base.souffle_bert_base(seq_len=128, fused=True) == 0


def test_layernorm_invariants_at_full_size():
    """Size-independent property: with gamma 1 / beta 0 every output row has mean 0, variance 1."""
    announce("bert LN invariants B=32")
    B, S = 32, 128
    w, x = synth.bert_layer_weights(2, 1), synth.bert_input(3, B, S)
    y = run_layer(w, x, B, S, 4, dump=False).float()
    assert y.mean(dim=1).abs().max().item() < 2e-3
    assert (y.var(dim=1, unbiased=False) - 1).abs().max().item() < 5e-3


def test_argument_errors_are_reported_not_fatal():
    announce("bert argument errors")
    import bert_binding
    import souffle_hip as sh
    w = dev_weights(synth.bert_layer_weights(0, 0))
    x = torch.zeros(1, 600, 768, dtype=torch.float16, device="cuda:0")
    with pytest.raises(sh.SouffleError) as e:
        bert_binding.souffle_bert_layer(x, w["qkv_weight"], w["attn_fc_weight"], w["fc1_weight"], w["fc2_weight"], 4)
    assert e.value.code == -2 and "seq_len" in str(e.value)
    with pytest.raises(ValueError):
        bert_binding.souffle_bert_layer(x, w["qkv_weight"], w["attn_fc_weight"], w["fc1_weight"], w["fc2_weight"], 9)
    with pytest.raises(TypeError):
        bert_binding.souffle_bert_layer(x.float(), w["qkv_weight"], w["attn_fc_weight"], w["fc1_weight"], w["fc2_weight"], 4)
