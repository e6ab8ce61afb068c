"""lstm_binding: drop-in for the reference's pybind module of the same name
(cpp/lstm/lstm_binding.cu:75-78), reduced to a wrapper over the C ABI.

fused_lstm(input_timestep, weight_input_wavefront, weight_state_wavefront) keeps the
reference's positional signature ([1,T,256] fp32 input, two [4*L,256,256] weight tensors,
returns [1,T,256] fp32).  Weights may be fp32 (as the reference passes them; they are
rounded to fp16 once) or fp16.  Keyword defaults follow the benchmark definition (gates
i,f,g,o, no forget bias); the reference kernel's variant is gate_order="igfo",
forget_bias=1.0 (cpp/lstm/lstm_reuse_shared_memory.cu:309-318).
"""
import ctypes as C

import torch

import souffle_hip as sh

_workspaces = {}


def _workspace(cfg, device):
    key = (device, cfg.layers, cfg.timesteps)
    ws = _workspaces.get(key)
    if ws is None:
        nbytes = sh.lib().souffle_lstm_workspace_bytes(C.byref(cfg))
        if nbytes == 0:
            raise sh.SouffleError(-2, sh.last_error())
        ws = _workspaces[key] = sh.Workspace(nbytes, device)
    return ws


def _check_cuda(name, t):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a CUDA tensor" % name)     # reference: CHECK_CUDA (lstm_binding.cu:32-34)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)


def fused_lstm(input_timestep, weight_input_wavefront, weight_state_wavefront, *, bias=None,
               gate_order="ifgo", forget_bias=0.0):
    for n, t in (("input_timestep", input_timestep), ("weight_input_wavefront", weight_input_wavefront),
                 ("weight_state_wavefront", weight_state_wavefront)):
        _check_cuda(n, t)
    if input_timestep.dim() != 3 or input_timestep.shape[0] != 1:
        raise ValueError("input_timestep must be [1, T, hidden]")           # lstm_binding.cu:35
    _, T, Hd = input_timestep.shape
    L4 = weight_input_wavefront.shape[0]
    if L4 % 4 or tuple(weight_input_wavefront.shape) != (L4, Hd, Hd) or \
            tuple(weight_state_wavefront.shape) != (L4, Hd, Hd):
        raise ValueError("weights must be [4*layers, hidden, hidden]")      # lstm_binding.cu:36-37
    x = input_timestep.float().contiguous()
    w_ih = weight_input_wavefront.to(torch.float16).contiguous()
    w_hh = weight_state_wavefront.to(torch.float16).contiguous()
    if bias is not None:
        _check_cuda("bias", bias)
        bias = bias.float().contiguous()
        if bias.numel() != L4 * Hd:
            raise ValueError("bias must be [layers, 4, hidden]")
    cfg = sh.LstmCfg(L4 // 4, Hd, T, 1, {"ifgo": sh.GATES_IFGO, "igfo": sh.GATES_IGFO}[gate_order], float(forget_bias))
    ws = _workspace(cfg, x.device)
    y = torch.empty((1, T, Hd), dtype=torch.float32, device=x.device)
    sh.check(sh.lib().souffle_lstm_fused(C.byref(cfg), w_ih.data_ptr(), w_hh.data_ptr(), sh.ptr(bias), x.data_ptr(),
                                         y.data_ptr(), ws.ptr, ws.nbytes, sh.current_stream()))
    return y
