"""swin_transformer_binding: drop-in for the reference's pybind module of the same name
(cpp/swin_transformer/swin_transformer_binding.cu:276-289), reduced to a wrapper over the
C ABI, plus the Swin block pair the reference only has as TVM operator definitions.

Reference functions kept (same positional arguments and return values):
    swin_fused_feed_mlp(src, fc1_weight, fc2_weight) -> [fc1_output, fc2_output]
    bench_swin_fused_feed_mlp(src, fc1_weight, fc2_weight, num_warmup, repeat, num_bench) -> us
    swin_ffn(src, weight, M, N, K) -> Tensor[M,N]
    bench_swin_ffn(M, N, K, num_warmup, num_bench, repeat) -> us
New: swin_block_pair(x, block0, block1, ...) and index_maps(height, width, window, shift).
"""
import ctypes as C

import numpy as np
import torch

import souffle_hip as sh

_workspaces = {}


def _ws(key, nbytes, device):
    ws = _workspaces.get((key, device))
    if ws is None or ws.nbytes < nbytes:
        ws = _workspaces[(key, device)] = sh.Workspace(nbytes, device)
    return ws


def _check(name, t, shape=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA tensor" % name)           # reference: CHECK_CUDA
    if t.dtype != torch.float16 or not t.is_contiguous():
        raise TypeError("%s must be a contiguous float16 tensor" % name)
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError("%s must have shape %s, got %s" % (name, tuple(shape), tuple(t.shape)))


def swin_fused_feed_mlp(src, fc1_weight, fc2_weight):
    """Y1 = src.W1, Y2 = Y1.W2 in one cooperative launch (no bias, no activation), as
    cpp/swin_transformer/swin_transformer_binding.cu:154-209 (there fixed to 256x512x2048)."""
    _check("src", src)
    M, K = src.shape[-2], src.shape[-1]
    _check("fc1_weight", fc1_weight)
    Fd = fc1_weight.shape[1]
    _check("fc1_weight", fc1_weight, (K, Fd))
    _check("fc2_weight", fc2_weight, (Fd, K))
    ws = _ws("ffn", 16384 + 32 * M * K, src.device)
    y1 = torch.empty((M, Fd), dtype=torch.float16, device=src.device)
    y2 = torch.empty((M, K), dtype=torch.float16, device=src.device)
    sh.check(sh.lib().souffle_swin_ffn_fused(src.data_ptr(), fc1_weight.data_ptr(), fc2_weight.data_ptr(),
                                             y1.data_ptr(), y2.data_ptr(), M, K, Fd, ws.ptr, ws.nbytes,
                                             sh.current_stream()))
    return [y1, y2]


def bench_swin_fused_feed_mlp(src, fc1_weight, fc2_weight, num_warmup, repeat, num_bench):
    """Latency in us under the reference's rule (cpp/swin_transformer/swin_transformer_binding.cu:213-219)."""
    mn, _ = sh.bench_us(lambda: swin_fused_feed_mlp(src, fc1_weight, fc2_weight), num_warmup, num_bench, repeat)
    return mn


def swin_ffn(src, weight, M, N, K):
    """Y[M,N] = src[M,K].weight[K,N] (cpp/swin_transformer/swin_transformer_binding.cu:62-100)."""
    _check("src", src)
    _check("weight", weight, (K, N))
    if src.numel() != M * K:
        raise ValueError("src must have M*K elements")
    y = torch.empty((M, N), dtype=torch.float16, device=src.device)
    sh.check(sh.lib().souffle_gemm_f16(src.data_ptr(), weight.data_ptr(), y.data_ptr(), M, N, K, sh.current_stream()))
    return y


def bench_swin_ffn(M, N, K, num_warmup, num_bench, repeat):
    src = torch.randn((M, K), device="cuda:0").half()
    weight = (torch.randn((K, N), device="cuda:0") * 0.02).half()
    mn, _ = sh.bench_us(lambda: swin_ffn(src, weight, M, N, K), num_warmup, num_bench, repeat)
    return mn


BLOCK_KEYS = sh.SWIN_W_FIELDS


def _block_w(w):
    for k in ("w_qkv", "w_proj", "w_fc1", "w_fc2"):
        _check(k, w[k])
    for k, v in w.items():
        if k not in BLOCK_KEYS:
            raise KeyError("unknown block weight %r" % k)
        _check(k, v)
    s = sh.SwinBlockW(*[sh.ptr(w.get(k)) for k in BLOCK_KEYS])
    s._keep = w
    return s


# grid-wide stages of the block-pair kernel that depend on one another (one grid barrier between the two blocks)
BLOCK_PAIR_GRID_STAGES = 2


def block_pair_launcher(x, block0, block1, out, height=56, width=56, heads=4, window=7, shift=3, mlp_ratio=4,
                        use_shift_mask=True, ln_eps=1e-5):
    """A closure that launches the block pair on preallocated buffers (x -> out) with one bare C-ABI call on the
    current stream and raises on a non-zero status: for callers that time or replay the launch."""
    _check("x", x, (height * width, x.shape[-1]))
    _check("out", out, tuple(x.shape))
    cfg = sh.SwinCfg(height, width, x.shape[-1], heads, window, shift, mlp_ratio, int(use_shift_mask), float(ln_eps))
    nbytes = sh.lib().souffle_swin_workspace_bytes(C.byref(cfg))
    if nbytes == 0:
        raise sh.SouffleError(-2, sh.last_error())
    ws = _ws(("pair", height, width), nbytes, x.device)
    arr = (sh.SwinBlockW * 2)(_block_w(block0), _block_w(block1))
    fn, cfg_ref, xp, yp = sh.lib().souffle_swin_block_pair_fused, C.byref(cfg), x.data_ptr(), out.data_ptr()

    def launch():
        sh.check(fn(cfg_ref, arr, xp, yp, ws.ptr, ws.nbytes, sh.current_stream()))
    launch._keep = (cfg, arr, ws, x, out)
    return launch


def swin_block_pair(x, block0, block1, height=56, width=56, heads=4, window=7, shift=3, mlp_ratio=4,
                    use_shift_mask=True, ln_eps=1e-5, out=None):
    """Regular-window block followed by shifted-window block (Swin-Base stage 1 by default).
    x: [H*W, C] fp16.  block0/block1: dicts with the keys of souffle_swin_block_w."""
    y = torch.empty_like(x) if out is None else out
    block_pair_launcher(x, block0, block1, y, height, width, heads, window, shift, mlp_ratio, use_shift_mask, ln_eps)()
    return y


def index_maps(height, width, window, shift):
    """(gather_idx, scatter_idx, relpos_idx[N,N], region_id) as int32 numpy arrays (host computation)."""
    T, N = height * width, window * window
    g, s, r, reg = (np.empty(T, np.int32), np.empty(T, np.int32), np.empty(N * N, np.int32), np.empty(T, np.int32))
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    sh.check(sh.lib().souffle_swin_index_maps(height, width, window, shift, p(g), p(s), p(r), p(reg)))
    return g, s, r.reshape(N, N), reg


def patch_merge_launcher(x, height, width, norm_weight, norm_bias, reduction_weight, out, ln_eps=1e-5):
    """A closure that launches patch merging on preallocated buffers with one bare C-ABI call on the current stream."""
    Cc = x.shape[-1]
    _check("x", x, (height * width, Cc))
    _check("reduction_weight", reduction_weight, (4 * Cc, 2 * Cc))
    _check("out", out, ((height // 2) * (width // 2), 2 * Cc))
    for n, t in (("norm_weight", norm_weight), ("norm_bias", norm_bias)):
        if t is not None:
            _check(n, t, (4 * Cc,))
    fn = sh.lib().souffle_swin_patch_merge
    a = (x.data_ptr(), sh.ptr(norm_weight), sh.ptr(norm_bias), reduction_weight.data_ptr(), out.data_ptr(), height, width, Cc, float(ln_eps))

    def launch():
        sh.check(fn(*a, sh.current_stream()))
    launch._keep = (x, norm_weight, norm_bias, reduction_weight, out)
    return launch


def patch_merging(x, height, width, norm_weight, norm_bias, reduction_weight, ln_eps=1e-5, out=None):
    """Patch merging between two stages (python/models/swin_transformer/swin_patch_merge.py:3-13):
    x [H*W, C] fp16 -> [(H/2)*(W/2), 2C]; norm_weight / norm_bias [4C] (None = 1 / 0),
    reduction_weight [4C, 2C] (the transpose of torch's Linear weight, like every weight here)."""
    y = torch.empty(((height // 2) * (width // 2), 2 * x.shape[-1]), dtype=torch.float16, device=x.device) if out is None else out
    patch_merge_launcher(x, height, width, norm_weight, norm_bias, reduction_weight, y, ln_eps)()
    return y
