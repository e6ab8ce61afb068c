"""Library restatements (torch CPU, float64) used to pin the CPU oracle.

These are written from the op lists of the reference (cited per function), not
imported from it; torch supplies matmul / softmax / layer_norm / gelu / LSTMCell /
roll / view+permute as independent library routines.
"""
import math

import numpy as np
import torch
import torch.nn.functional as Fn


def _t(a):
    return None if a is None else torch.from_numpy(np.asarray(a, dtype=np.float64))


def bert_layer(x, w, batch, seq_len, heads, act="gelu_tanh", scale=0.125, ln_eps=1e-12, mask=None):
    """Op order of cpp/bert/test_souffle_bert_layer.py:78-110 (post-LN encoder layer), with
    weights [K][N] used as X @ W (:139-143).  Returns the reference's six tensors
    (cpp/bert/bert_binding.cu:534) as float64 numpy arrays."""
    x = _t(x)
    M, H = x.shape
    hd = H // heads
    g = lambda k: _t(w.get(k))
    wqkv = g("qkv_weight")
    qkv = torch.stack([x @ wqkv[j] for j in range(3)])                     # [3][M][H]
    if g("qkv_bias") is not None:
        qkv = qkv + g("qkv_bias").reshape(3, 1, H)
    qkv_h = qkv.reshape(3, batch, seq_len, heads, hd).permute(0, 1, 3, 2, 4)  # [3][B][nh][S][hd]
    q, k, v = qkv_h[0], qkv_h[1], qkv_h[2]
    s = (q @ k.transpose(-1, -2)) * scale
    if mask is not None:
        s = s + _t(mask).reshape(batch, 1, seq_len, seq_len)
    p = torch.softmax(s, dim=-1)
    ctx = (p @ v).permute(0, 2, 1, 3).reshape(M, H)
    z = ctx @ g("attn_fc_weight")
    if g("attn_fc_bias") is not None:
        z = z + g("attn_fc_bias")
    y1 = Fn.layer_norm(z + x, (H,), g("ln1_gamma"), g("ln1_beta"), ln_eps)
    h = y1 @ g("fc1_weight")
    if g("fc1_bias") is not None:
        h = h + g("fc1_bias")
    h = Fn.gelu(h, approximate="tanh") if act == "gelu_tanh" else (Fn.gelu(h) if act == "gelu" else torch.relu(h))
    z2 = h @ g("fc2_weight")
    if g("fc2_bias") is not None:
        z2 = z2 + g("fc2_bias")
    y = Fn.layer_norm(z2 + y1, (H,), g("ln2_gamma"), g("ln2_beta"), ln_eps)
    outs = [qkv_h.reshape(3 * batch, heads, seq_len, hd), p.reshape(batch * heads, seq_len, seq_len), ctx, y1, h, y]
    return [o.numpy() for o in outs]


def lstm_stack(x, w_ih, w_hh, bias=None):
    """Stack of torch.nn.LSTMCell (gate order i,f,g,o, no forget bias); layer l at step t
    consumes layer l-1 at step t (python/models/lstm/tf_lstm.py:94-99)."""
    x = _t(x)
    T, Hd = x.shape
    L = w_ih.shape[0] // 4
    cells = []
    for l in range(L):
        c = torch.nn.LSTMCell(Hd, Hd, bias=True, dtype=torch.float64)
        with torch.no_grad():
            c.weight_ih.copy_(_t(w_ih[4 * l:4 * l + 4]).reshape(4 * Hd, Hd))
            c.weight_hh.copy_(_t(w_hh[4 * l:4 * l + 4]).reshape(4 * Hd, Hd))
            c.bias_hh.zero_()
            if bias is None:
                c.bias_ih.zero_()
            else:
                c.bias_ih.copy_(_t(bias[l]).reshape(4 * Hd))
        cells.append(c)
    h = [torch.zeros(1, Hd, dtype=torch.float64) for _ in range(L)]
    cs = [torch.zeros(1, Hd, dtype=torch.float64) for _ in range(L)]
    ys = []
    with torch.no_grad():
        for t in range(T):
            inp = x[t:t + 1]
            for l in range(L):
                h[l], cs[l] = cells[l](inp, (h[l], cs[l]))
                inp = h[l]
            ys.append(inp[0].clone())
    return torch.stack(ys).numpy()


def window_partition(x, ws):
    """The published Swin window_partition (view + permute), the closed form the reference's
    CPU test compares against (test_swin_tensor_transformer_ops.py:32-65)."""
    B, H, W, C = x.shape
    x = x.view(B, H // ws, ws, W // ws, ws, C)
    return x.permute(0, 1, 3, 2, 4, 5).contiguous().view(-1, ws, ws, C)


def window_reverse(windows, ws, H, W):
    B = int(windows.shape[0] / (H * W / ws / ws))
    x = windows.view(B, H // ws, W // ws, ws, ws, -1)
    return x.permute(0, 1, 3, 2, 4, 5).contiguous().view(B, H, W, -1)


def swin_block(x, w, H, W, heads, ws, shift, use_shift_mask=True, ln_eps=1e-5):
    """python/models/swin_transformer/swin_transformer_main.py:11-61 (Part-1..8) with the
    published relative-position bias and shifted-window mask."""
    x = _t(x)
    T, C = x.shape
    hd = C // heads
    g = lambda k: _t(w.get(k))
    shortcut = x
    z = Fn.layer_norm(x, (C,), g("ln1_g"), g("ln1_b"), ln_eps).view(1, H, W, C)
    if shift > 0:
        z = torch.roll(z, shifts=(-shift, -shift), dims=(1, 2))
    xw = window_partition(z, ws).view(-1, ws * ws, C)
    B_, N, _ = xw.shape
    qkv = xw @ g("w_qkv")
    if g("b_qkv") is not None:
        qkv = qkv + g("b_qkv")
    qkv = qkv.reshape(B_, N, 3, heads, hd).permute(2, 0, 3, 1, 4)
    q, k, v = qkv[0] * hd ** -0.5, qkv[1], qkv[2]
    attn = q @ k.transpose(-2, -1)
    if g("rel_table") is not None:
        coords = torch.stack(torch.meshgrid(torch.arange(ws), torch.arange(ws), indexing="ij")).flatten(1)
        rel = (coords[:, :, None] - coords[:, None, :]).permute(1, 2, 0).contiguous()
        rel[:, :, 0] += ws - 1
        rel[:, :, 1] += ws - 1
        rel[:, :, 0] *= 2 * ws - 1
        idx = rel.sum(-1)
        bias = g("rel_table")[idx.view(-1)].view(N, N, heads).permute(2, 0, 1)
        attn = attn + bias.unsqueeze(0)
    if shift > 0 and use_shift_mask:
        img = torch.zeros(1, H, W, 1, dtype=torch.float64)
        cnt = 0
        for hs in (slice(0, -ws), slice(-ws, -shift), slice(-shift, None)):
            for wsl in (slice(0, -ws), slice(-ws, -shift), slice(-shift, None)):
                img[:, hs, wsl, :] = cnt
                cnt += 1
        mw = window_partition(img, ws).view(-1, N)
        am = mw.unsqueeze(1) - mw.unsqueeze(2)
        am = am.masked_fill(am != 0, -100.0).masked_fill(am == 0, 0.0)
        attn = attn + am.unsqueeze(1)
    attn = torch.softmax(attn, dim=-1)
    o = (attn @ v).transpose(1, 2).reshape(B_, N, C)
    o = o @ g("w_proj")
    if g("b_proj") is not None:
        o = o + g("b_proj")
    o = window_reverse(o.view(-1, ws, ws, C), ws, H, W)
    if shift > 0:
        o = torch.roll(o, shifts=(shift, shift), dims=(1, 2))
    x1 = shortcut + o.view(T, C)
    z = Fn.layer_norm(x1, (C,), g("ln2_g"), g("ln2_b"), ln_eps)
    h = z @ g("w_fc1")
    if g("b_fc1") is not None:
        h = h + g("b_fc1")
    h = Fn.gelu(h, approximate="tanh")
    o = h @ g("w_fc2")
    if g("b_fc2") is not None:
        o = o + g("b_fc2")
    return (x1 + o).numpy()


def se_module(x, w_reduce, w_expand, b_reduce=None, b_expand=None, combine="mul", hw=None):
    """avg_pool2d -> conv2d 1x1 -> swish -> conv2d 1x1 -> sigmoid -> combine, as composed in
    cpp/efficientnet/efficientnet_se_module_unittest_binding.cu:123-130."""
    x = _t(x)
    C, HW = x.shape
    side = int(math.isqrt(HW))
    xi = x.view(1, C, side, HW // side)
    p = Fn.avg_pool2d(xi, (side, HW // side))
    r = Fn.conv2d(p, _t(w_reduce).view(-1, C, 1, 1), _t(b_reduce))
    r = r * torch.sigmoid(r)
    e = torch.sigmoid(Fn.conv2d(r, _t(w_expand).view(C, -1, 1, 1), _t(b_expand)))
    y = xi + e if combine == "add" else xi * e
    return y.view(C, HW).numpy(), p.view(C).numpy()
