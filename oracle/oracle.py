"""numpy/ctypes front end of the CPU oracle (oracle/liboracle.so) -- TEST INFRASTRUCTURE.

Imported only by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py.
Inputs are numpy arrays (any float dtype); they are widened to fp32 exactly and handed
to the C restatement in oracle/*.c.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
ACT = {"gelu_tanh": 0, "relu": 1, "none": 2, "gelu": 3}      # "gelu": the erf form, as in HuggingFace configs
_lib = None


def build(force=False):
    if force or not os.path.exists(LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    return LIB_PATH


class _BertCfg(C.Structure):
    _fields_ = [("batch", C.c_int), ("seq_len", C.c_int), ("hidden", C.c_int), ("heads", C.c_int),
                ("ffn", C.c_int), ("act", C.c_int), ("scale", C.c_float), ("ln_eps", C.c_float)]


_BERT_W = ["w_qkv", "b_qkv", "w_o", "b_o", "ln1_g", "ln1_b", "w_fc1", "b_fc1", "w_fc2", "b_fc2", "ln2_g", "ln2_b"]


class _BertW(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in _BERT_W]


class _BertDump(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ["qkv", "probs", "ctx", "ln1", "fc1"]]


class _LstmCfg(C.Structure):
    _fields_ = [("layers", C.c_int), ("hidden", C.c_int), ("timesteps", C.c_int), ("batch", C.c_int),
                ("gate_order", C.c_int), ("forget_bias", C.c_float)]


class _SwinCfg(C.Structure):
    _fields_ = [("height", C.c_int), ("width", C.c_int), ("channels", C.c_int), ("heads", C.c_int),
                ("window", C.c_int), ("shift", C.c_int), ("mlp_ratio", C.c_int), ("use_shift_mask", C.c_int),
                ("ln_eps", C.c_float)]


_SWIN_W = ["ln1_g", "ln1_b", "w_qkv", "b_qkv", "rel_table", "w_proj", "b_proj", "ln2_g", "ln2_b", "w_fc1",
           "b_fc1", "w_fc2", "b_fc2"]


class _SwinW(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in _SWIN_W]


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(LIB_PATH)
        _lib.oracle_gelu_tanh.restype = C.c_float
        _lib.oracle_gelu_tanh.argtypes = [C.c_float]
        _lib.oracle_gelu_erf.restype = C.c_float
        _lib.oracle_gelu_erf.argtypes = [C.c_float]
    return _lib


def _f32(a):
    return None if a is None else np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


# map of the binding-level weight names to the oracle's
_BERT_NAMES = {"qkv_weight": "w_qkv", "qkv_bias": "b_qkv", "attn_fc_weight": "w_o", "attn_fc_bias": "b_o",
               "ln1_gamma": "ln1_g", "ln1_beta": "ln1_b", "fc1_weight": "w_fc1", "fc1_bias": "b_fc1",
               "fc2_weight": "w_fc2", "fc2_bias": "b_fc2", "ln2_gamma": "ln2_g", "ln2_beta": "ln2_b"}


def _bert_w(weights, keep):
    w = _BertW()
    for k, v in weights.items():
        a = _f32(v)
        keep.append(a)
        setattr(w, _BERT_NAMES.get(k, k), _p(a))
    return w


def gemm(x, w, bias=None, threads=0):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    M, K = x.shape
    N = w.shape[1]
    y = np.empty((M, N), np.float32)
    lib().oracle_gemm_f32(_p(x), _p(w), _p(bias), _p(y), M, N, K, threads)
    return y


def layernorm(z, g=None, b=None, eps=1e-12):
    z, g, b = _f32(z), _f32(g), _f32(b)
    y = np.empty_like(z)
    lib().oracle_layernorm_f32(_p(z), _p(g), _p(b), _p(y), z.shape[0], z.shape[1], C.c_float(eps))
    return y


def gelu_tanh(x):
    return np.array([lib().oracle_gelu_tanh(float(v)) for v in np.asarray(x).ravel()], np.float32).reshape(np.shape(x))


def gelu_erf(x):
    return np.array([lib().oracle_gelu_erf(float(v)) for v in np.asarray(x).ravel()], np.float32).reshape(np.shape(x))


def bert_layer(x, weights, batch, seq_len, hidden=768, heads=12, ffn=3072, act="gelu_tanh", scale=0.125,
               ln_eps=1e-12, mask=None, dump=False, threads=0):
    """Returns y [M,H] (and the five dump tensors in the reference's order when dump)."""
    cfg = _BertCfg(batch, seq_len, hidden, heads, ffn, ACT[act], scale, ln_eps)
    keep = []
    w = _bert_w(weights, keep)
    x, mask = _f32(x).reshape(batch * seq_len, hidden), _f32(mask)
    M, hd = batch * seq_len, hidden // heads
    y = np.empty((M, hidden), np.float32)
    d, outs = None, None
    if dump:
        outs = [np.empty((3 * batch, heads, seq_len, hd), np.float32), np.empty((batch * heads, seq_len, seq_len), np.float32),
                np.empty((M, hidden), np.float32), np.empty((M, hidden), np.float32), np.empty((M, ffn), np.float32)]
        d = _BertDump(*[_p(o) for o in outs])
    rc = lib().oracle_bert_layer_f32(C.byref(cfg), C.byref(w), _p(x), _p(mask), _p(y), C.byref(d) if d else None, threads)
    if rc:
        raise RuntimeError("oracle_bert_layer_f32 failed: %d" % rc)
    return (outs + [y]) if dump else y


def bert_encoder(x, layers, batch, seq_len, hidden=768, heads=12, ffn=3072, act="gelu_tanh", scale=0.125,
                 ln_eps=1e-12, mask=None, threads=0):
    cfg = _BertCfg(batch, seq_len, hidden, heads, ffn, ACT[act], scale, ln_eps)
    keep = []
    arr = (_BertW * len(layers))(*[_bert_w(l, keep) for l in layers])
    x, mask = _f32(x).reshape(batch * seq_len, hidden), _f32(mask)
    y = np.empty_like(x)
    rc = lib().oracle_bert_encoder_f32(C.byref(cfg), arr, len(layers), _p(x), _p(mask), _p(y), threads)
    if rc:
        raise RuntimeError("oracle_bert_encoder_f32 failed: %d" % rc)
    return y


def bert_embed(token_ids, word_emb, pos_emb, type_emb=None, segment_ids=None, ln_g=None, ln_b=None, eps=1e-12):
    """LayerNorm(word[token] + pos[position] + type[segment]); token_ids [B, S] -> [B*S, hidden] fp32."""
    tok = np.ascontiguousarray(token_ids, dtype=np.int32)
    B, S = tok.shape
    seg = None if segment_ids is None else np.ascontiguousarray(segment_ids, dtype=np.int32)
    w, p = _f32(word_emb), _f32(pos_emb)
    t = None if type_emb is None else _f32(type_emb)
    g = None if ln_g is None else _f32(ln_g)
    b = None if ln_b is None else _f32(ln_b)
    hidden = w.shape[1]
    out = np.empty((B * S, hidden), np.float32)
    ip = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
    fn = lib().oracle_bert_embed_f32
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p] * 7 + [C.c_float, C.c_int, C.c_int, C.c_int, C.c_void_p]
    rc = fn(ip(tok), ip(seg), ip(w), ip(p), ip(t), ip(g), ip(b), float(eps), B, S, hidden, ip(out))
    assert rc == 0, rc
    return out


def bert_pooler(x, w, bias, batch, seq_len):
    """tanh(x[b, 0, :] . W + bias), W [K][N]; x [B*S, hidden] -> [B, hidden] fp32."""
    xx, ww = _f32(x), _f32(w)
    bb = None if bias is None else _f32(bias)
    hidden = ww.shape[1]
    out = np.empty((batch, hidden), np.float32)
    ip = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
    fn = lib().oracle_bert_pooler_f32
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p] * 3 + [C.c_int, C.c_int, C.c_int, C.c_void_p]
    rc = fn(ip(xx), ip(ww), ip(bb), batch, seq_len, hidden, ip(out))
    assert rc == 0, rc
    return out


def lstm(x, w_ih, w_hh, bias=None, gate_order="ifgo", forget_bias=0.0):
    """x [T,H] or [B,T,H]; w_* [L*4,H,H]; returns y with x's shape."""
    x = _f32(x)
    shp = x.shape
    x3 = x.reshape((1,) + shp) if x.ndim == 2 else x
    w_ih, w_hh, bias = _f32(w_ih), _f32(w_hh), _f32(bias)
    L, Hd = w_ih.shape[0] // 4, w_ih.shape[1]
    cfg = _LstmCfg(L, Hd, x3.shape[1], x3.shape[0], {"ifgo": 0, "igfo": 1}[gate_order], forget_bias)
    y = np.empty_like(x3)
    rc = lib().oracle_lstm_f32(C.byref(cfg), _p(w_ih), _p(w_hh), _p(bias), _p(x3), _p(y))
    if rc:
        raise RuntimeError("oracle_lstm_f32 failed: %d" % rc)
    return y.reshape(shp)


def swin_index_maps(height, width, window, shift):
    T, N = height * width, window * window
    g, s, r, reg = (np.empty(T, np.int32), np.empty(T, np.int32), np.empty(N * N, np.int32), np.empty(T, np.int32))
    rc = lib().oracle_swin_index_maps(height, width, window, shift, _p(g), _p(s), _p(r), _p(reg))
    if rc:
        raise RuntimeError("oracle_swin_index_maps failed: %d" % rc)
    return g, s, r.reshape(N, N), reg


def _swin_w(weights, keep):
    w = _SwinW()
    for k, v in weights.items():
        a = _f32(v)
        keep.append(a)
        setattr(w, k, _p(a))
    return w


def swin_block(x, weights, height=56, width=56, channels=128, heads=4, window=7, shift=0, mlp_ratio=4,
               use_shift_mask=True, ln_eps=1e-5, threads=0):
    cfg = _SwinCfg(height, width, channels, heads, window, shift, mlp_ratio, int(use_shift_mask), ln_eps)
    keep = []
    w = _swin_w(weights, keep)
    x = _f32(x)
    y = np.empty_like(x)
    rc = lib().oracle_swin_block_f32(C.byref(cfg), C.byref(w), _p(x), _p(y), threads)
    if rc:
        raise RuntimeError("oracle_swin_block_f32 failed: %d" % rc)
    return y


def swin_block_pair(x, weights2, height=56, width=56, channels=128, heads=4, window=7, shift=3, mlp_ratio=4,
                    use_shift_mask=True, ln_eps=1e-5, threads=0):
    cfg = _SwinCfg(height, width, channels, heads, window, shift, mlp_ratio, int(use_shift_mask), ln_eps)
    keep = []
    arr = (_SwinW * 2)(_swin_w(weights2[0], keep), _swin_w(weights2[1], keep))
    x = _f32(x)
    y = np.empty_like(x)
    rc = lib().oracle_swin_block_pair_f32(C.byref(cfg), arr, _p(x), _p(y), threads)
    if rc:
        raise RuntimeError("oracle_swin_block_pair_f32 failed: %d" % rc)
    return y


def swin_ffn(x, w1, w2, threads=0):
    x, w1, w2 = _f32(x), _f32(w1), _f32(w2)
    M, K = x.shape
    Fd = w1.shape[1]
    y1, y2 = np.empty((M, Fd), np.float32), np.empty((M, K), np.float32)
    lib().oracle_swin_ffn_f32(_p(x), _p(w1), _p(w2), _p(y1), _p(y2), M, K, Fd, threads)
    return y1, y2


def swin_patch_merge(x, height, width, ln_g, ln_b, w, ln_eps=1e-5, threads=0):
    """x [H*W, C] -> [(H/2)*(W/2), 2C]."""
    x, ln_g, ln_b, w = _f32(x), _f32(ln_g), _f32(ln_b), _f32(w)
    Cc = x.shape[-1]
    y = np.empty(((height // 2) * (width // 2), 2 * Cc), np.float32)
    rc = lib().oracle_swin_patch_merge_f32(_p(x), _p(ln_g), _p(ln_b), _p(w), _p(y), height, width, Cc, C.c_float(ln_eps), threads)
    if rc:
        raise RuntimeError("oracle_swin_patch_merge_f32 failed: %d" % rc)
    return y


def se_module(x, w_reduce, w_expand, b_reduce=None, b_expand=None, combine="mul"):
    """x [C,HW]; returns (y [C,HW], pooled [C])."""
    x, w_reduce, w_expand, b_reduce, b_expand = _f32(x), _f32(w_reduce), _f32(w_expand), _f32(b_reduce), _f32(b_expand)
    Cc, HW = x.shape
    R = w_reduce.shape[0]
    y, pooled = np.empty_like(x), np.empty(Cc, np.float32)
    rc = lib().oracle_se_module_f32(_p(x), _p(w_reduce), _p(b_reduce), _p(w_expand), _p(b_expand), _p(y), _p(pooled),
                                    Cc, HW, R, {"mul": 0, "add": 1}[combine])
    if rc:
        raise RuntimeError("oracle_se_module_f32 failed: %d" % rc)
    return y, pooled


# ---- EfficientNet MBConv operators (NHWC, batch 1) ----
_MB_INT = ["in_h", "in_w", "in_c", "expand_c", "out_c", "kernel", "stride", "se_c", "has_shortcut"]
_MB_PTR = ["expand_w", "expand_scale", "expand_shift", "dw_w", "dw_scale", "dw_shift", "se_reduce_w", "se_reduce_b",
           "se_expand_w", "se_expand_b", "project_w", "project_scale", "project_shift"]


class _MbBlock(C.Structure):
    _fields_ = [(n, C.c_int) for n in _MB_INT] + [(n, C.c_void_p) for n in _MB_PTR]


def depthwise_out_extent(n, kernel, stride):
    return lib().oracle_depthwise_out_extent(n, kernel, stride)


def pointwise_conv(x, w, scale=None, shift=None, gate=None, shortcut=None, act="none", threads=0):
    """x [pixels, in_c], w [out_c, in_c] -> [pixels, out_c]."""
    x, w, scale, shift, gate, shortcut = _f32(x), _f32(w), _f32(scale), _f32(shift), _f32(gate), _f32(shortcut)
    P, K = x.shape
    N = w.shape[0]
    y = np.empty((P, N), np.float32)
    rc = lib().oracle_pointwise_conv_f32(_p(x), _p(w), _p(scale), _p(shift), _p(gate), _p(shortcut), _p(y), P, K, N,
                                         {"none": 0, "swish": 1}[act], threads)
    if rc:
        raise RuntimeError("oracle_pointwise_conv_f32 failed: %d" % rc)
    return y


def depthwise_conv(x, w, scale=None, shift=None, stride=1, act="swish", threads=0):
    """x [H, W, C], w [k, k, C] -> [oh, ow, C]."""
    x, w, scale, shift = _f32(x), _f32(w), _f32(scale), _f32(shift)
    H, W, Cc = x.shape
    k = w.shape[0]
    oh, ow = depthwise_out_extent(H, k, stride), depthwise_out_extent(W, k, stride)
    y = np.empty((oh, ow, Cc), np.float32)
    rc = lib().oracle_depthwise_conv_f32(_p(x), _p(w), _p(scale), _p(shift), _p(y), H, W, Cc, k, stride,
                                         {"none": 0, "swish": 1}[act], threads)
    if rc:
        raise RuntimeError("oracle_depthwise_conv_f32 failed: %d" % rc)
    return y


def se_gate(x, w_reduce, b_reduce, w_expand, b_expand):
    """x [pixels, C] -> gate [C]."""
    x, w_reduce, b_reduce, w_expand, b_expand = _f32(x), _f32(w_reduce), _f32(b_reduce), _f32(w_expand), _f32(b_expand)
    P, Cc = x.shape
    g = np.empty(Cc, np.float32)
    rc = lib().oracle_se_gate_f32(_p(x), _p(w_reduce), _p(b_reduce), _p(w_expand), _p(b_expand), _p(g), P, Cc,
                                  w_reduce.shape[0])
    if rc:
        raise RuntimeError("oracle_se_gate_f32 failed: %d" % rc)
    return g


def mbconv_block(x, blk, round_fp16=False, dump=False, threads=0):
    """blk: dict with the integer fields and weight arrays of one block (synth.mbconv_block_weights).
    x [in_h*in_w, in_c] -> y [oh*ow, out_c] (and the expanded / depthwise tensors when dump)."""
    keep, b = [], _MbBlock()
    for n in _MB_INT:
        setattr(b, n, int(blk[n]))
    for n in _MB_PTR:
        a = _f32(blk.get(n))
        keep.append(a)
        setattr(b, n, _p(a))
    x = _f32(x).reshape(blk["in_h"] * blk["in_w"], blk["in_c"])
    oh = depthwise_out_extent(blk["in_h"], blk["kernel"], blk["stride"])
    ow = depthwise_out_extent(blk["in_w"], blk["kernel"], blk["stride"])
    y = np.empty((oh * ow, blk["out_c"]), np.float32)
    e = np.empty((x.shape[0], blk["expand_c"]), np.float32) if dump and blk.get("expand_w") is not None else None
    d = np.empty((oh * ow, blk["expand_c"]), np.float32) if dump else None
    rc = lib().oracle_mbconv_block_f32(C.byref(b), _p(x), _p(y), _p(e), _p(d), int(round_fp16), threads)
    if rc:
        raise RuntimeError("oracle_mbconv_block_f32 failed: %d" % rc)
    return (e, d, y) if dump else y


def mbconv_stack(x, blocks, round_fp16=False, threads=0):
    for blk in blocks:
        x = mbconv_block(x, blk, round_fp16=round_fp16, threads=threads)
    return x
