"""Seeded synthetic tensors for the benchmark configurations (no dataset, no checkpoint).

A counter-based generator (splitmix64 -> uniform / Box-Muller) so that the same
(config, tensor) id always yields the same values on any machine.  Everything is rounded
to fp16 first; the fp32 copies handed to a CPU checker are exact widenings of the fp16
values the GPU sees.  Seed convention: 0x5EED0000 + config_id*256 + tensor_id.
Weight distributions are the benchmark's (N(0,0.02) BERT/Swin weights, U(-1/16,1/16)
LSTM weights, N(0,1) activations); the reference's own smoke tests draw N(0,1) weights
(cpp/bert/test_bert_binding.py:7-15, python/models/bert/souffle_bert.py:9-17).
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    with np.errstate(over="ignore"):
        z = x + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform01(seed, n):
    """n doubles in [0,1), element i depends only on (seed, i)."""
    with np.errstate(over="ignore"):
        ctr = np.arange(n, dtype=np.uint64) + _splitmix64(np.uint64(seed)) * np.uint64(2)
    return (_splitmix64(ctr) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def uniform(seed, shape, lo, hi):
    n = int(np.prod(shape))
    return (lo + (hi - lo) * uniform01(seed, n)).reshape(shape)


def normal(seed, shape, std=1.0):
    n = int(np.prod(shape))
    m = (n + 1) // 2
    u = uniform01(seed, 2 * m)
    r = np.sqrt(-2.0 * np.log(1.0 - u[:m]))
    th = 2.0 * np.pi * u[m:]
    z = np.concatenate([r * np.cos(th), r * np.sin(th)])[:n]
    return (std * z).reshape(shape)


def seed_of(config_id, tensor_id):
    return 0x5EED0000 + config_id * 256 + tensor_id


def f16(a):
    return np.ascontiguousarray(a, dtype=np.float64).astype(np.float16)


# ---------------------------------------------------------------- BERT ----
H, NH, F = 768, 12, 3072


def bert_layer_weights(config_id=0, layer=0, with_bias=False):
    """fp16 numpy weights of one encoder layer; biases 0 and LN gamma 1 / beta 0 in the
    benchmark configs, random when with_bias (to exercise those code paths)."""
    t = layer * 16
    w = {
        "qkv_weight": f16(normal(seed_of(config_id, t + 1), (3, H, H), 0.02)),
        "attn_fc_weight": f16(normal(seed_of(config_id, t + 2), (H, H), 0.02)),
        "fc1_weight": f16(normal(seed_of(config_id, t + 3), (H, F), 0.02)),
        "fc2_weight": f16(normal(seed_of(config_id, t + 4), (F, H), 0.02)),
    }
    if with_bias:
        w.update({
            "qkv_bias": f16(normal(seed_of(config_id, t + 5), (3 * H,), 0.1)),
            "attn_fc_bias": f16(normal(seed_of(config_id, t + 6), (H,), 0.1)),
            "ln1_gamma": f16(1.0 + normal(seed_of(config_id, t + 7), (H,), 0.1)),
            "ln1_beta": f16(normal(seed_of(config_id, t + 8), (H,), 0.1)),
            "fc1_bias": f16(normal(seed_of(config_id, t + 9), (F,), 0.1)),
            "fc2_bias": f16(normal(seed_of(config_id, t + 10), (H,), 0.1)),
            "ln2_gamma": f16(1.0 + normal(seed_of(config_id, t + 11), (H,), 0.1)),
            "ln2_beta": f16(normal(seed_of(config_id, t + 12), (H,), 0.1)),
        })
    return w


def bert_input(config_id, batch, seq_len):
    return f16(normal(seed_of(config_id, 0), (batch * seq_len, H), 1.0))


# ---------------------------------------------------------------- LSTM ----
def lstm_tensors(config_id=1, layers=10, hidden=256, timesteps=100):
    w_ih = f16(uniform(seed_of(config_id, 1), (layers * 4, hidden, hidden), -1 / 16, 1 / 16))
    w_hh = f16(uniform(seed_of(config_id, 2), (layers * 4, hidden, hidden), -1 / 16, 1 / 16))
    x = normal(seed_of(config_id, 0), (timesteps, hidden), 1.0).astype(np.float32)
    return w_ih, w_hh, x


# ---------------------------------------------------------------- Swin ----
def swin_block_weights(config_id=3, block=0, C=128, heads=4, window=7, mlp_ratio=4, with_bias=False):
    t = block * 16
    w = {
        "w_qkv": f16(normal(seed_of(config_id, t + 1), (C, 3 * C), 0.02)),
        "w_proj": f16(normal(seed_of(config_id, t + 2), (C, C), 0.02)),
        "w_fc1": f16(normal(seed_of(config_id, t + 3), (C, mlp_ratio * C), 0.02)),
        "w_fc2": f16(normal(seed_of(config_id, t + 4), (mlp_ratio * C, C), 0.02)),
        "rel_table": f16(normal(seed_of(config_id, t + 5), ((2 * window - 1) ** 2, heads), 0.02)),
    }
    if with_bias:
        w.update({
            "b_qkv": f16(normal(seed_of(config_id, t + 6), (3 * C,), 0.1)),
            "b_proj": f16(normal(seed_of(config_id, t + 7), (C,), 0.1)),
            "b_fc1": f16(normal(seed_of(config_id, t + 8), (mlp_ratio * C,), 0.1)),
            "b_fc2": f16(normal(seed_of(config_id, t + 9), (C,), 0.1)),
            "ln1_g": f16(1.0 + normal(seed_of(config_id, t + 10), (C,), 0.1)),
            "ln1_b": f16(normal(seed_of(config_id, t + 11), (C,), 0.1)),
            "ln2_g": f16(1.0 + normal(seed_of(config_id, t + 12), (C,), 0.1)),
            "ln2_b": f16(normal(seed_of(config_id, t + 13), (C,), 0.1)),
        })
    return w


def swin_input(config_id=3, tokens=56 * 56, C=128):
    return f16(normal(seed_of(config_id, 0), (tokens, C), 1.0))


# --------------------------------------------------------- EfficientNet ----
# (kernel, stride, in_c, out_c, expand_ratio, repeats) of EfficientNet-B0's seven stages; the
# reference builds the same list from efficientnet_pytorch's block arguments
# (python/models/efficientnet/tvm_efficientnet.py:138-158).  SE ratio 0.25 of the block input.
EFFICIENTNET_B0_STAGES = [(3, 1, 32, 16, 1, 1), (3, 2, 16, 24, 6, 2), (5, 2, 24, 40, 6, 2), (3, 2, 40, 80, 6, 3),
                          (5, 1, 80, 112, 6, 3), (5, 2, 112, 192, 6, 4), (3, 1, 192, 320, 6, 1)]


def mbconv_block_shapes(stages=EFFICIENTNET_B0_STAGES, image=112):
    """The integer fields of every MBConv block of the stack, in order (the stem has already
    halved a 224x224 image to `image`)."""
    out, h = [], image
    for kernel, stride, cin, cout, ratio, repeats in stages:
        for r in range(repeats):
            s, ci = (stride, cin) if r == 0 else (1, cout)
            out.append({"in_h": h, "in_w": h, "in_c": ci, "expand_c": ci * ratio, "out_c": cout, "kernel": kernel,
                        "stride": s, "se_c": max(1, int(ci * 0.25)), "has_shortcut": int(s == 1 and ci == cout),
                        "has_expand": ratio != 1})
            h = (h - 1) // s + 1
    return out


def mbconv_block_weights(shape, config_id=4, block=0, in_rms=1.0):
    """fp16 N(0,0.02) convolution weights and fp32 folded batch-norm scale/shift of one block.
    The folded scales are about those a batch norm would have on this data (they undo the 0.02
    of the weights, the fan-in and the expected magnitude `in_rms` of the block input), so
    activations stay of order one through the stack."""
    t, b = block * 16, dict(shape)
    ci, ce, co, k, r = b["in_c"], b["expand_c"], b["out_c"], b["kernel"], b["se_c"]

    def fold(idx, n, fan_in, rms_in):
        u = uniform(seed_of(config_id, t + idx), (n,), 0.75, 1.25)
        return (u / (0.02 * np.sqrt(fan_in) * rms_in)).astype(np.float32), \
            normal(seed_of(config_id, t + idx + 1), (n,), 0.1).astype(np.float32)

    if b.pop("has_expand"):
        b["expand_w"] = f16(normal(seed_of(config_id, t + 1), (ce, ci), 0.02))
        b["expand_scale"], b["expand_shift"] = fold(2, ce, ci, in_rms)
    else:
        b["expand_w"] = b["expand_scale"] = b["expand_shift"] = None
    b["dw_w"] = f16(normal(seed_of(config_id, t + 4), (k, k, ce), 0.02))
    b["dw_scale"], b["dw_shift"] = fold(5, ce, k * k, 0.6)
    b["se_reduce_w"] = f16(normal(seed_of(config_id, t + 7), (r, ce), 0.02))
    b["se_reduce_b"] = normal(seed_of(config_id, t + 8), (r,), 0.1).astype(np.float32)
    b["se_expand_w"] = f16(normal(seed_of(config_id, t + 9), (r, ce), 0.02))
    b["se_expand_b"] = normal(seed_of(config_id, t + 10), (ce,), 0.5).astype(np.float32)
    b["project_w"] = f16(normal(seed_of(config_id, t + 11), (co, ce), 0.02))
    b["project_scale"], b["project_shift"] = fold(12, co, ce, 0.52)
    return b


def mbconv_stack_weights(config_id=4, stages=EFFICIENTNET_B0_STAGES, image=112):
    out, rms = [], 1.0
    for i, s in enumerate(mbconv_block_shapes(stages, image)):
        out.append(mbconv_block_weights(s, config_id, i, rms))
        rms = float(np.sqrt(1.0 + rms * rms)) if s["has_shortcut"] else 1.0   # the shortcut adds the input back
    return out


def mbconv_input(config_id=4, pixels=112 * 112, channels=32):
    return f16(normal(seed_of(config_id, 0), (pixels, channels), 1.0))
