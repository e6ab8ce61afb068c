"""efficientnet_se_module_binding: drop-in for the reference's pybind module of the same name
(cpp/efficientnet/efficientnet_se_module_binding.cu:229-233), reduced to a wrapper over the C ABI.

torch_dispatch_efficientnet_se_module_v2_short_cut_fused(input[1,C,H,W] f32, se_reduce_weight[R,C],
se_expand_weight[C,R], opt_level) -> [reduce_output[1,C], se_short_cut_add[1,C,H,W]].
Any (C,H,W,R) within the library's limits, not only the reference's ten shapes.  The
reference combines with add (efficientnet_se_module_unittest_binding.cu:124-130) and labels
its NCHW-ordered output buffer as NHWC (efficientnet_se_module_binding.cu:37-40,160); here
the output is NCHW and says so, and combine defaults to the textbook multiply.
"""
import torch

import souffle_hip as sh

_ws = {}


def torch_dispatch_efficientnet_se_module_v2_short_cut_fused(input, se_reduce_weight, se_expand_weight, opt_level=2,
                                                             *, combine="mul", reduce_bias=None, expand_bias=None):
    for n, t in (("input", input), ("se_reduce_weight", se_reduce_weight), ("se_expand_weight", se_expand_weight)):
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise TypeError("%s must be a CUDA tensor" % n)
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise TypeError("%s must be a contiguous float32 tensor" % n)
    if input.dim() != 4 or input.shape[0] != 1:
        raise ValueError("input must be [1, C, H, W]")
    _, Cc, Hh, Ww = input.shape
    R = se_reduce_weight.shape[0]
    if tuple(se_reduce_weight.shape[:2]) != (R, Cc) or tuple(se_expand_weight.shape[:2]) != (Cc, R):
        raise ValueError("weights must be [R,C] and [C,R]")
    dev = input.device
    nbytes = sh.lib().souffle_se_workspace_bytes(Cc, Hh * Ww, R)
    if nbytes == 0:
        raise sh.SouffleError(-2, sh.last_error())
    ws = _ws.get(dev)
    if ws is None:
        ws = _ws[dev] = sh.Workspace(nbytes, dev)
    y = torch.empty_like(input)
    pooled = torch.empty((1, Cc), dtype=torch.float32, device=dev)
    sh.check(sh.lib().souffle_se_module_fused(input.data_ptr(), se_reduce_weight.data_ptr(), sh.ptr(reduce_bias),
                                              se_expand_weight.data_ptr(), sh.ptr(expand_bias), y.data_ptr(),
                                              pooled.data_ptr(), Cc, Hh * Ww, R,
                                              {"mul": sh.SE_MUL, "add": sh.SE_ADD}[combine], ws.ptr, ws.nbytes,
                                              sh.current_stream()))
    return [pooled, y]
