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
    acts = {"gelu_tanh": sh.ACT_GELU_TANH, "gelu": sh.ACT_GELU_TANH, "relu": sh.ACT_RELU}
    if act not in acts:
        raise ValueError("act must be one of %s" % sorted(acts))
    return sh.BertCfg(batch, seq_len, HIDDEN, HEADS, FFN, acts[act], float(scale), float(ln_eps), num_layers, 0)


def make_layer_w(qkv_weight, attn_fc_weight, fc1_weight, fc2_weight, qkv_bias=None, attn_fc_bias=None,
                 ln1_gamma=None, ln1_beta=None, fc1_bias=None, fc2_bias=None, ln2_gamma=None, ln2_beta=None):
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
                      sh.ptr(fc2_weight), sh.ptr(fc2_bias), sh.ptr(ln2_gamma), sh.ptr(ln2_beta))
    w._keep = (qkv_weight, attn_fc_weight, fc1_weight, fc2_weight, qkv_bias, attn_fc_bias, ln1_gamma, ln1_beta,
               fc1_bias, fc2_bias, ln2_gamma, ln2_beta)
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
                       mask=None, batch=None, seq_len=None, dump=True, **biases):
    """One encoder layer.  opt_level 0-2: per-op HIP launches; 3-4: the fused megakernel
    (the reference's levels: cpp/bert/bert_binding.cu:119-531).  Returns
    [output_qkv, query_key_output, attn_value_output, attn_fc_output,
     feed_forward_fc1_output, feed_forward_fc2_output] as cpp/bert/bert_binding.cu:534.
    With dump=False only the final output is produced and returned (fast path)."""
    if opt_level not in (0, 1, 2, 3, 4):
        raise ValueError("opt_level %r is not supported" % (opt_level,))   # reference prints and returns
    _check_f16_cuda("src", src)
    if src.shape[-1] != HIDDEN:
        raise ValueError("src last dimension must be %d" % HIDDEN)
    if reference_compat:
        act, scale, ln_eps = "relu", 1.0 / (HIDDEN ** 0.5), 1e-5
    B, S = _batch_seq(src, batch, seq_len)
    cfg = make_cfg(B, S, act, scale, ln_eps)
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

    def __init__(self, layers, batch, seq_len, act="gelu_tanh", scale=0.125, ln_eps=1e-12, device="cuda:0"):
        self.cfg = make_cfg(batch, seq_len, act, scale, ln_eps, num_layers=len(layers))
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
