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


def se_launcher(input, se_reduce_weight, se_expand_weight, out, pooled, *, combine="mul", reduce_bias=None, expand_bias=None):
    """A closure that launches the SE module on preallocated buffers (out like input, pooled [1, C]) with one bare
    C-ABI call on the current stream and raises on a non-zero status: for callers that time or replay the launch."""
    for n, t in (("input", input), ("se_reduce_weight", se_reduce_weight), ("se_expand_weight", se_expand_weight), ("out", out), ("pooled", pooled)):
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
    if tuple(out.shape) != tuple(input.shape) or pooled.numel() != Cc:
        raise ValueError("out must have the input's shape and pooled C elements")
    dev = input.device
    nbytes = sh.lib().souffle_se_workspace_bytes(Cc, Hh * Ww, R)
    if nbytes == 0:
        raise sh.SouffleError(-2, sh.last_error())
    ws = _ws.get(dev)
    if ws is None or ws.nbytes < nbytes:
        ws = _ws[dev] = sh.Workspace(nbytes, dev)
    fn = sh.lib().souffle_se_module_fused
    a = (input.data_ptr(), se_reduce_weight.data_ptr(), sh.ptr(reduce_bias), se_expand_weight.data_ptr(), sh.ptr(expand_bias),
         out.data_ptr(), pooled.data_ptr(), Cc, Hh * Ww, R, {"mul": sh.SE_MUL, "add": sh.SE_ADD}[combine], ws.ptr, ws.nbytes)

    def launch():
        sh.check(fn(*a, sh.current_stream()))
    launch._keep = (input, se_reduce_weight, se_expand_weight, reduce_bias, expand_bias, out, pooled, ws)
    return launch


def torch_dispatch_efficientnet_se_module_v2_short_cut_fused(input, se_reduce_weight, se_expand_weight, opt_level=2,
                                                             *, combine="mul", reduce_bias=None, expand_bias=None):
    if not isinstance(input, torch.Tensor) or not input.is_cuda or input.dtype != torch.float32 or input.dim() != 4:
        raise TypeError("input must be a float32 CUDA tensor [1, C, H, W]")
    y = torch.empty_like(input)
    pooled = torch.empty((1, input.shape[1]), dtype=torch.float32, device=input.device)
    se_launcher(input, se_reduce_weight, se_expand_weight, y, pooled, combine=combine, reduce_bias=reduce_bias, expand_bias=expand_bias)()
    return [pooled, y]
