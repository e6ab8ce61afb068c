"""bert_binding: drop-in for the reference's pybind module of the same name
(cpp/bert/bert_binding.cu:537-540), reduced to a wrapper over the C ABI.

souffle_bert_layer(src, qkv_weight, attn_fc_weight, feed_forward_fc1_weight,
feed_forward_fc2_weight, opt_level) keeps the reference's positional signature and
returns the same six tensors.  Behaviour the reference hard-codes is exposed as keyword
arguments whose defaults are standard BERT-base (tanh-GELU, scale 1/8, eps 1e-12,
runtime batch and sequence length); `reference_compat=True` selects what the
reference's fused CUDA path computes instead (ReLU, scale 1/sqrt(768), eps 1e-5:
cpp/bert/kernels/fused_sqq_feedforward.cu:327-341, fused_sqq_bert.cu:2934, bert_binding.cu:115).
"""
import ctypes as C

import torch

import souffle_hip as sh

HIDDEN, HEADS, FFN = 768, 12, 3072
_workspaces = {}


def _workspace(cfg, device):
    key = (device, cfg.batch, cfg.seq_len)
    nbytes = sh.lib().souffle_bert_workspace_bytes(C.byref(cfg))
    if nbytes == 0:
        raise sh.SouffleError(-2, sh.last_error())
    ws = _workspaces.get(key)
    if ws is None or ws.nbytes < nbytes:          # grows with the number of layers
        ws = _workspaces[key] = sh.Workspace(nbytes, device)
    return ws


def _check_f16_cuda(name, t, shape=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA tensor" % name)      # reference: CHECK_CUDA
    if t.dtype != torch.float16:
        raise TypeError("%s must be float16" % name)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError("%s must have shape %s, got %s" % (name, tuple(shape), tuple(t.shape)))


def make_cfg(batch, seq_len, act="gelu_tanh", scale=0.125, ln_eps=1e-12, num_layers=1):
    # "gelu" is HuggingFace's name for the erf form, which its BERT checkpoints were trained with; the reference's
    # kernels compute the tanh form ("gelu_tanh", the default here) or ReLU.  The two GELUs differ by up to 5e-4 per
    # activation, so neither name is an alias of the other.
    acts = {"gelu_tanh": sh.ACT_GELU_TANH, "relu": sh.ACT_RELU, "gelu": sh.ACT_GELU_ERF}
    if act not in acts:
        raise ValueError("act must be one of %s" % sorted(acts))
    return sh.BertCfg(batch, seq_len, HIDDEN, HEADS, FFN, acts[act], float(scale), float(ln_eps), num_layers, 0)


def pack_fc2(fc2_weight):
    """The one-time copy of a layer's fc2 weight [3072][768] in the order the few-rows encoder reads it
    (souffle_bert_pack_fc2): made once per model, passed as fc2_packed of the layer."""
    _check_f16_cuda("feed_forward_fc2_weight", fc2_weight, (FFN, HIDDEN))
    packed = torch.empty(sh.lib().souffle_bert_fc2_packed_bytes() // 2, dtype=torch.float16, device=fc2_weight.device)
    sh.check(sh.lib().souffle_bert_pack_fc2(fc2_weight.data_ptr(), packed.data_ptr(), sh.current_stream()))
    return packed


def make_layer_w(qkv_weight, attn_fc_weight, fc1_weight, fc2_weight, qkv_bias=None, attn_fc_bias=None,
                 ln1_gamma=None, ln1_beta=None, fc1_bias=None, fc2_bias=None, ln2_gamma=None, ln2_beta=None,
                 fc2_packed=None):
    _check_f16_cuda("qkv_weight", qkv_weight, (3, HIDDEN, HIDDEN))
    _check_f16_cuda("attn_fc_weight", attn_fc_weight, (HIDDEN, HIDDEN))
    _check_f16_cuda("feed_forward_fc1_weight", fc1_weight, (HIDDEN, FFN))
    _check_f16_cuda("feed_forward_fc2_weight", fc2_weight, (FFN, HIDDEN))
    opt = {"qkv_bias": (qkv_bias, 3 * HIDDEN), "attn_fc_bias": (attn_fc_bias, HIDDEN),
           "ln1_gamma": (ln1_gamma, HIDDEN), "ln1_beta": (ln1_beta, HIDDEN), "fc1_bias": (fc1_bias, FFN),
           "fc2_bias": (fc2_bias, HIDDEN), "ln2_gamma": (ln2_gamma, HIDDEN), "ln2_beta": (ln2_beta, HIDDEN)}
    for name, (t, n) in opt.items():
        if t is not None:
            _check_f16_cuda(name, t)
            if t.numel() != n:
                raise ValueError("%s must have %d elements" % (name, n))
    w = sh.BertLayerW(sh.ptr(qkv_weight), sh.ptr(qkv_bias), sh.ptr(attn_fc_weight), sh.ptr(attn_fc_bias),
                      sh.ptr(ln1_gamma), sh.ptr(ln1_beta), sh.ptr(fc1_weight), sh.ptr(fc1_bias),
                      sh.ptr(fc2_weight), sh.ptr(fc2_bias), sh.ptr(ln2_gamma), sh.ptr(ln2_beta), sh.ptr(fc2_packed))
    if fc2_packed is not None:
        _check_f16_cuda("fc2_packed", fc2_packed)
        if fc2_packed.numel() != FFN * HIDDEN:
            raise ValueError("fc2_packed must have %d elements" % (FFN * HIDDEN))
    w._keep = (qkv_weight, attn_fc_weight, fc1_weight, fc2_weight, qkv_bias, attn_fc_bias, ln1_gamma, ln1_beta,
               fc1_bias, fc2_bias, ln2_gamma, ln2_beta, fc2_packed)
    return w


def _batch_seq(src, batch, seq_len):
    if src.dim() == 3:
        return src.shape[0], src.shape[1]
    if src.dim() == 2:
        if seq_len is None:
            return (batch or 1), src.shape[0] // (batch or 1)
        return src.shape[0] // seq_len, seq_len
    raise ValueError("src must be [B,S,768] or [B*S,768]")


def souffle_bert_layer(src, qkv_weight, attn_fc_weight, feed_forward_fc1_weight, feed_forward_fc2_weight,
                       opt_level, *, act="gelu_tanh", scale=0.125, ln_eps=1e-12, reference_compat=False,
                       mask=None, batch=None, seq_len=None, dump=True, pack=False, **biases):
    """One encoder layer.  opt_level 0-2: per-op HIP launches; 3-4: the fused megakernel
    (the reference's levels: cpp/bert/bert_binding.cu:119-531).  Returns
    [output_qkv, query_key_output, attn_value_output, attn_fc_output,
     feed_forward_fc1_output, feed_forward_fc2_output] as cpp/bert/bert_binding.cu:534.
    With dump=False only the final output is produced and returned (fast path).  pack=True makes the packed copy
    of the fc2 weight for this call (a model object makes it once: Encoder), so that FC2 runs in its whole-K form."""
    if opt_level not in (0, 1, 2, 3, 4):
        raise ValueError("opt_level %r is not supported" % (opt_level,))   # reference prints and returns
    _check_f16_cuda("src", src)
    if src.shape[-1] != HIDDEN:
        raise ValueError("src last dimension must be %d" % HIDDEN)
    if reference_compat:
        act, scale, ln_eps = "relu", 1.0 / (HIDDEN ** 0.5), 1e-5
    B, S = _batch_seq(src, batch, seq_len)
    cfg = make_cfg(B, S, act, scale, ln_eps)
    if pack and biases.get("fc2_packed") is None:
        biases = dict(biases, fc2_packed=pack_fc2(feed_forward_fc2_weight))
    w = make_layer_w(qkv_weight, attn_fc_weight, feed_forward_fc1_weight, feed_forward_fc2_weight, **biases)
    if mask is not None:
        _check_f16_cuda("mask", mask, (B, S, S))
    dev = src.device
    ws = _workspace(cfg, dev)
    M = B * S
    out = torch.empty((M, HIDDEN), dtype=torch.float16, device=dev)
    fn = sh.lib().souffle_bert_layer_fused if opt_level >= 3 else sh.lib().souffle_bert_layer_unfused
    if not dump:
        sh.check(fn(C.byref(cfg), C.byref(w), src.data_ptr(), sh.ptr(mask), out.data_ptr(), None, ws.ptr,
                    ws.nbytes, sh.current_stream()))
        return out
    SP = next(v for v in (64, 128, 256, 384, 512) if v >= S) if S <= 512 else S
    if SP != S:
        # per-stage tensors of a sequence length that is not built: run the padded length with the
        # surplus keys masked out and cut the six tensors back to S
        xp = torch.zeros((B, SP, HIDDEN), dtype=torch.float16, device=dev)
        xp[:, :S] = src.view(B, S, HIDDEN)
        mp = torch.zeros((B, SP, SP), dtype=torch.float16, device=dev)
        mp[:, :, S:] = -10000.0
        if mask is not None:
            mp[:, :S, :S] = mask
        outs = souffle_bert_layer(xp, qkv_weight, attn_fc_weight, feed_forward_fc1_weight, feed_forward_fc2_weight, opt_level,
                                  act=act, scale=scale, ln_eps=ln_eps, mask=mp, dump=True, **biases)
        hd = HIDDEN // HEADS
        rows = lambda t: t.view(B, SP, -1)[:, :S].reshape(B * S, -1)
        return [outs[0].view(B * 3, HEADS, SP, hd)[:, :, :S].contiguous(), outs[1].view(B * HEADS, SP, SP)[:, :S, :S].contiguous(),
                rows(outs[2]), rows(outs[3]), rows(outs[4]), rows(outs[5])]
    qkv = torch.empty((B * 3, HEADS, S, HIDDEN // HEADS), dtype=torch.float16, device=dev)
    probs = torch.empty((B * HEADS, S, S), dtype=torch.float16, device=dev)
    ctx = torch.empty((M, HIDDEN), dtype=torch.float16, device=dev)
    ln1 = torch.empty((M, HIDDEN), dtype=torch.float16, device=dev)
    fc1 = torch.empty((M, FFN), dtype=torch.float16, device=dev)
    d = sh.BertDump(qkv.data_ptr(), probs.data_ptr(), ctx.data_ptr(), ln1.data_ptr(), fc1.data_ptr())
    sh.check(fn(C.byref(cfg), C.byref(w), src.data_ptr(), sh.ptr(mask), out.data_ptr(), C.byref(d), ws.ptr,
                ws.nbytes, sh.current_stream()))
    return [qkv, probs, ctx, ln1, fc1, out]


class Encoder:
    """num_layers encoder layers with distinct weights, run as one cooperative launch
    (fused=True) or as per-op launches.  Stands in for the reference's souffle_bert_base()
    (cpp/bert/bert_base_impl.cu:277-308), which allocates its own zero weights."""

    def __init__(self, layers, batch, seq_len, act="gelu_tanh", scale=0.125, ln_eps=1e-12, device="cuda:0", pack=True):
        self.cfg = make_cfg(batch, seq_len, act, scale, ln_eps, num_layers=len(layers))
        # a model object is built once: the place for the one-time packed copy of every fc2 weight (pack=False keeps
        # the [K][N] matrices only, as the per-call entry point souffle_bert_layer does)
        if pack:
            layers = [l if l.get("fc2_packed") is not None else dict(l, fc2_packed=pack_fc2(l["fc2_weight"])) for l in layers]
        self._w = [make_layer_w(**l) for l in layers]
        self.warr = (sh.BertLayerW * len(layers))(*self._w)
        self.ws = _workspace(self.cfg, torch.device(device))
        self.M = batch * seq_len

    def __call__(self, x, out=None, fused=True, mask=None):
        _check_f16_cuda("x", x)
        if x.numel() != self.M * HIDDEN:
            raise ValueError("x must have %d elements" % (self.M * HIDDEN))
        if out is None:
            out = torch.empty((self.M, HIDDEN), dtype=torch.float16, device=x.device)
        fn = sh.lib().souffle_bert_encoder_fused if fused else sh.lib().souffle_bert_encoder_unfused
        sh.check(fn(C.byref(self.cfg), self.warr, x.data_ptr(), sh.ptr(mask), out.data_ptr(), self.ws.ptr,
                    self.ws.nbytes, sh.current_stream()))
        return out


def embed(token_ids, word_emb, pos_emb, type_emb=None, segment_ids=None, ln_gamma=None, ln_beta=None, ln_eps=1e-12,
          check_ids=True):
    """The stage in front of the encoder: LayerNorm(word[token] + pos[position] + type[segment]).
    Stands in for the HuggingFace embedding module the reference feeds its layer with
    (cpp/bert/test_souffle_bert_layer.py:186-189).  token_ids: int32 CUDA tensor [B, S];
    returns fp16 [B*S, 768].  An id outside its table is never read out of bounds (the kernel clamps
    it); with check_ids the call then waits for the kernel and raises IndexError, as indexing the
    table on the host would."""
    if not isinstance(token_ids, torch.Tensor) or not token_ids.is_cuda or token_ids.dtype != torch.int32 or token_ids.dim() != 2:
        raise TypeError("token_ids must be an int32 CUDA tensor [B, S]")
    B, S = token_ids.shape
    if segment_ids is not None and (segment_ids.dtype != torch.int32 or tuple(segment_ids.shape) != (B, S) or not segment_ids.is_cuda):
        raise TypeError("segment_ids must be an int32 CUDA tensor [B, S]")
    for name, t in (("word_emb", word_emb), ("pos_emb", pos_emb), ("type_emb", type_emb), ("ln_gamma", ln_gamma), ("ln_beta", ln_beta)):
        if t is not None:
            _check_f16_cuda(name, t)
            if t.shape[-1] != HIDDEN:
                raise ValueError("%s last dimension must be %d" % (name, HIDDEN))
    if pos_emb.shape[0] < S:
        raise ValueError("pos_emb has %d rows, sequence length is %d" % (pos_emb.shape[0], S))
    tok = token_ids.contiguous()
    seg = None if segment_ids is None else segment_ids.contiguous()
    for name, t in (("word_emb", word_emb), ("pos_emb", pos_emb), ("type_emb", type_emb)):
        if t is not None and (t.dim() != 2 or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous [rows, %d] table" % (name, HIDDEN))
    out = torch.empty((B * S, HIDDEN), dtype=torch.float16, device=token_ids.device)
    bad = torch.zeros(1, dtype=torch.int32, device=token_ids.device) if check_ids else None
    sh.check(sh.lib().souffle_bert_embed(tok.data_ptr(), sh.ptr(seg), word_emb.data_ptr(), word_emb.shape[0], pos_emb.data_ptr(),
                                         pos_emb.shape[0], sh.ptr(type_emb), 0 if type_emb is None else type_emb.shape[0],
                                         sh.ptr(ln_gamma), sh.ptr(ln_beta), float(ln_eps), B, S, HIDDEN, out.data_ptr(),
                                         sh.ptr(bad), sh.current_stream()))
    if check_ids:
        n_bad = int(bad.item())
        if n_bad:
            raise IndexError("%d token or segment ids lie outside their embedding tables (%d / %d rows)"
                             % (n_bad, word_emb.shape[0], 0 if type_emb is None else type_emb.shape[0]))
    return out


def pooler(x, weight, bias, batch, seq_len):
    """tanh(x[b, 0, :] . weight + bias): the standard BERT pooler behind the encoder.
    weight is [K][N] like every weight here; x fp16 [B*S, 768]; returns fp16 [B, 768]."""
    _check_f16_cuda("x", x)
    _check_f16_cuda("weight", weight, (HIDDEN, HIDDEN))
    if bias is not None:
        _check_f16_cuda("bias", bias)
    if x.numel() != batch * seq_len * HIDDEN:
        raise ValueError("x must have %d elements" % (batch * seq_len * HIDDEN))
    out = torch.empty((batch, HIDDEN), dtype=torch.float16, device=x.device)
    sh.check(sh.lib().souffle_bert_pooler(x.data_ptr(), weight.data_ptr(), sh.ptr(bias), batch, seq_len, HIDDEN, out.data_ptr(),
                                          sh.current_stream()))
    return out


def load_hf_bert(path, num_layers=None, prefix=""):
    """Read a local BERT checkpoint in safetensors format (HuggingFace tensor names) into the
    layouts used here: every nn.Linear weight [out, in] is transposed to [K][N], q/k/v are stacked
    to [3][768][768] (the reference's rule: cpp/bert/test_souffle_bert_layer.py:131-143).
    Returns {"layers": [per-layer dicts of fp16 CPU tensors for Encoder(...)], "embeddings": {...},
    "pooler": {...}}.  Nothing is fetched: `path` must be a file on disk."""
    from safetensors.torch import load_file
    raw = load_file(path)
    t = lambda name: raw[prefix + name]
    kn = lambda name: t(name).t().contiguous().to(torch.float16)          # [out, in] -> [K][N]
    vec = lambda name: t(name).contiguous().to(torch.float16)
    n = 0
    while (prefix + "encoder.layer.%d.attention.self.query.weight" % n) in raw:
        n += 1
    if num_layers is not None:
        n = min(n, num_layers)
    layers = []
    for i in range(n):
        p = "encoder.layer.%d." % i
        layers.append({
            "qkv_weight": torch.stack([kn(p + "attention.self.%s.weight" % q) for q in ("query", "key", "value")]).contiguous(),
            "qkv_bias": torch.stack([vec(p + "attention.self.%s.bias" % q) for q in ("query", "key", "value")]).contiguous(),
            "attn_fc_weight": kn(p + "attention.output.dense.weight"), "attn_fc_bias": vec(p + "attention.output.dense.bias"),
            "ln1_gamma": vec(p + "attention.output.LayerNorm.weight"), "ln1_beta": vec(p + "attention.output.LayerNorm.bias"),
            "fc1_weight": kn(p + "intermediate.dense.weight"), "fc1_bias": vec(p + "intermediate.dense.bias"),
            "fc2_weight": kn(p + "output.dense.weight"), "fc2_bias": vec(p + "output.dense.bias"),
            "ln2_gamma": vec(p + "output.LayerNorm.weight"), "ln2_beta": vec(p + "output.LayerNorm.bias"),
        })
    out = {"layers": layers, "embeddings": None, "pooler": None}
    if prefix + "embeddings.word_embeddings.weight" in raw:
        out["embeddings"] = {"word_emb": vec("embeddings.word_embeddings.weight"), "pos_emb": vec("embeddings.position_embeddings.weight"),
                             "type_emb": vec("embeddings.token_type_embeddings.weight"),
                             "ln_gamma": vec("embeddings.LayerNorm.weight"), "ln_beta": vec("embeddings.LayerNorm.bias")}
    if prefix + "pooler.dense.weight" in raw:
        out["pooler"] = {"weight": kn("pooler.dense.weight"), "bias": vec("pooler.dense.bias")}
    return out
