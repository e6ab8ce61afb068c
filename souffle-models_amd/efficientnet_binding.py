"""efficientnet_binding: the EfficientNet MBConv operators of the reference's
python/models/efficientnet/efficientnet.py as wrappers over the C ABI (the reference has them
as TVM tensor expressions, tuned and timed one by one by tvm_efficientnet.py:62-118; it has no
compiled binding for them besides the squeeze-excite module).

Same operator names and NHWC tensor shapes (batch 1), fp16 data:
  pointwise_conv2d_bn(input[1,H,W,Ci], weight[Co,Ci], bnw1[1,Co], bnw2[1,Co])          :41-57
  pointwise_conv2d_bn_short_cut_add(input, weight, bnw1, bnw2, short_cut[1,H,W,Co])     :83-101
  head_conv1x1_bn_swish(input, weight[1,1,Ci,Co], bnw1, bnw2)                           :502-518
  fused_depthwise_conv2d_bn_swish(input[1,H,W,C], weight[k,k,C,1], mul[1,C], bias_add[1,C], stride) :173-195
and MBConvStack, the fused chain of blocks in one persistent launch.
"""
import ctypes as C

import torch

import souffle_hip as sh


def _half(name, t, dims):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA tensor" % name)
    if t.dtype != torch.float16 or not t.is_contiguous():
        raise TypeError("%s must be a contiguous float16 tensor" % name)
    if t.dim() != dims:
        raise ValueError("%s must have %d dimensions" % (name, dims))
    return t


def _vec(name, t, n):
    if t is None:
        return None
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous():
        raise TypeError("%s must be a contiguous float32 CUDA tensor" % name)
    if t.numel() != n:
        raise ValueError("%s must have %d elements" % (name, n))
    return t


def _pointwise(input, weight, bnw1, bnw2, short_cut, act, gate=None):
    _half("input", input, 4)
    _half("weight", weight, 2)
    if input.shape[0] != 1:
        raise ValueError("batch must be 1")
    _, Hh, Ww, ci = input.shape
    co = weight.shape[0]
    if weight.shape[1] != ci:
        raise ValueError("weight must be [out_channels, in_channels]")
    bnw1, bnw2, gate = _vec("bnw1", bnw1, co), _vec("bnw2", bnw2, co), _vec("gate", gate, ci)
    if short_cut is not None:
        _half("short_cut", short_cut, 4)
        if tuple(short_cut.shape) != (1, Hh, Ww, co):
            raise ValueError("short_cut must be [1, H, W, out_channels]")
    y = torch.empty((1, Hh, Ww, co), dtype=torch.float16, device=input.device)
    sh.check(sh.lib().souffle_pointwise_conv2d_bn(input.data_ptr(), weight.data_ptr(), sh.ptr(bnw1), sh.ptr(bnw2), sh.ptr(gate),
                                                  sh.ptr(short_cut), y.data_ptr(), Hh * Ww, ci, co, act, sh.current_stream()))
    return y


def pointwise_conv2d_bn(input, weight, bnw1=None, bnw2=None, *, gate=None):
    return _pointwise(input, weight, bnw1, bnw2, None, sh.MB_NONE, gate)


def pointwise_conv2d_bn_short_cut_add(input, weight, bnw1, bnw2, short_cut, *, gate=None):
    return _pointwise(input, weight, bnw1, bnw2, short_cut, sh.MB_NONE, gate)


def head_conv1x1_bn_swish(input, weight, bnw1=None, bnw2=None):
    """weight [1, 1, in, out] as the reference declares it; the kernel wants [out][in]."""
    _half("weight", weight, 4)
    return _pointwise(input, weight[0, 0].t().contiguous(), bnw1, bnw2, None, sh.MB_SWISH)


def fused_depthwise_conv2d_bn_swish(input, weight, mul=None, bias_add=None, stride=1):
    _half("input", input, 4)
    _half("weight", weight, 4)
    if input.shape[0] != 1:
        raise ValueError("batch must be 1")
    _, Hh, Ww, c = input.shape
    k = weight.shape[0]
    if tuple(weight.shape) != (k, k, c, 1):
        raise ValueError("weight must be [k, k, channels, 1]")
    mul, bias_add = _vec("mul", mul, c), _vec("bias_add", bias_add, c)
    oh, ow = (Hh - 1) // stride + 1, (Ww - 1) // stride + 1
    y = torch.empty((1, oh, ow, c), dtype=torch.float16, device=input.device)
    sh.check(sh.lib().souffle_depthwise_conv2d_bn_swish(input.data_ptr(), weight.data_ptr(), sh.ptr(mul), sh.ptr(bias_add),
                                                        y.data_ptr(), Hh, Ww, c, k, stride, sh.current_stream()))
    return y


class MBConvStack:
    """A chain of MBConv blocks held on the device.  `blocks`: dicts with the integer fields
    (in_h, in_w, in_c, expand_c, out_c, kernel, stride, se_c, has_shortcut) and the CUDA weight
    tensors (fp16 convolution weights, fp32 folded batch-norm vectors and biases; absent or None
    where the block has none) under the names of souffle_mbconv_block."""

    def __init__(self, blocks, device="cuda:0"):
        self.n = len(blocks)
        self.keep = []
        self.desc = (sh.MbconvBlock * self.n)()
        for d, b in zip(self.desc, blocks):
            for f in sh.MB_INT_FIELDS:
                setattr(d, f, int(b[f]))
            for f in sh.MB_PTR_FIELDS:
                t = b.get(f)
                if t is not None:
                    want = torch.float16 if f.endswith("_w") else torch.float32
                    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != want or not t.is_contiguous():
                        raise TypeError("%s must be a contiguous %s CUDA tensor" % (f, want))
                    self.keep.append(t)
                setattr(d, f, sh.ptr(t))
        nbytes = sh.lib().souffle_mbconv_workspace_bytes(self.desc, self.n)
        if nbytes == 0:
            raise sh.SouffleError(-2, sh.last_error())
        self.ws = sh.Workspace(nbytes, device)
        last = blocks[-1]
        oh, ow = (last["in_h"] - 1) // last["stride"] + 1, (last["in_w"] - 1) // last["stride"] + 1
        self.in_shape = (blocks[0]["in_h"] * blocks[0]["in_w"], blocks[0]["in_c"])
        self.out = torch.empty((oh * ow, last["out_c"]), dtype=torch.float16, device=device)

    def __call__(self, x, fused=True):
        """x [in_h*in_w, in_c] fp16 -> [oh*ow, out_c] fp16 (a buffer owned by the stack)."""
        if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float16 or not x.is_contiguous():
            raise TypeError("x must be a contiguous float16 CUDA tensor")
        if x.numel() != self.in_shape[0] * self.in_shape[1]:
            raise ValueError("x must have %d x %d elements" % self.in_shape)
        sh.check(sh.lib().souffle_mbconv_stack(self.desc, self.n, x.data_ptr(), self.out.data_ptr(), 1 if fused else 0,
                                               self.ws.ptr, self.ws.nbytes, sh.current_stream()))
        return self.out
