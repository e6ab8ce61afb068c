"""ctypes view of libsouffle_hip.so (the C ABI declared in include/souffle_hip.h).

The binding modules in this directory (bert_binding, lstm_binding,
swin_transformer_binding, swin_trans_fc2, efficientnet_se_module_binding, efficientnet_binding) are thin
wrappers over this module; torch is used for device memory and streams only.
There is no CPU or eager fallback: if the library is missing, loading fails.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SOUFFLE_HIP_LIB") or os.path.join(_HERE, "libsouffle_hip.so")

ACT_GELU_TANH, ACT_RELU, ACT_GELU_ERF = 0, 1, 2
GATES_IFGO, GATES_IGFO = 0, 1
SE_MUL, SE_ADD = 0, 1


class BertCfg(C.Structure):
    _fields_ = [("batch", C.c_int), ("seq_len", C.c_int), ("hidden", C.c_int), ("heads", C.c_int),
                ("ffn", C.c_int), ("act", C.c_int), ("scale", C.c_float), ("ln_eps", C.c_float),
                ("num_layers", C.c_int), ("reserved", C.c_int)]


BERT_W_FIELDS = ["w_qkv", "b_qkv", "w_o", "b_o", "ln1_g", "ln1_b", "w_fc1", "b_fc1", "w_fc2", "b_fc2",
                 "ln2_g", "ln2_b", "w_fc2_packed"]


class BertLayerW(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in BERT_W_FIELDS]


class BertDump(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ["qkv", "probs", "ctx", "ln1", "fc1"]]


class LstmCfg(C.Structure):
    _fields_ = [("layers", C.c_int), ("hidden", C.c_int), ("timesteps", C.c_int), ("batch", C.c_int),
                ("gate_order", C.c_int), ("forget_bias", C.c_float)]


class SwinCfg(C.Structure):
    _fields_ = [("height", C.c_int), ("width", C.c_int), ("channels", C.c_int), ("heads", C.c_int),
                ("window", C.c_int), ("shift", C.c_int), ("mlp_ratio", C.c_int),
                ("use_shift_mask", C.c_int), ("ln_eps", C.c_float)]


SWIN_W_FIELDS = ["ln1_g", "ln1_b", "w_qkv", "b_qkv", "rel_table", "w_proj", "b_proj", "ln2_g", "ln2_b",
                 "w_fc1", "b_fc1", "w_fc2", "b_fc2"]


class SwinBlockW(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in SWIN_W_FIELDS]


MB_INT_FIELDS = ["in_h", "in_w", "in_c", "expand_c", "out_c", "kernel", "stride", "se_c", "has_shortcut"]
MB_PTR_FIELDS = ["expand_w", "expand_scale", "expand_shift", "dw_w", "dw_scale", "dw_shift", "se_reduce_w", "se_reduce_b",
                 "se_expand_w", "se_expand_b", "project_w", "project_scale", "project_shift"]
MB_NONE, MB_SWISH = 0, 1


class MbconvBlock(C.Structure):
    _fields_ = [(n, C.c_int) for n in MB_INT_FIELDS] + [(n, C.c_void_p) for n in MB_PTR_FIELDS]


class DevInfo(C.Structure):
    _fields_ = [("num_cus", C.c_int), ("lds_bytes_per_cu", C.c_int), ("clock_khz", C.c_int),
                ("mem_clock_khz", C.c_int), ("mem_bus_bits", C.c_int), ("l2_bytes", C.c_int),
                ("cooperative_launch", C.c_int), ("wavefront_size", C.c_int), ("arch", C.c_char * 64)]


BENCH_FN = C.CFUNCTYPE(C.c_int, C.c_void_p)

# name -> (restype, argtypes); every symbol include/souffle_hip.h declares
SIGNATURES = {
    "souffle_last_error": (C.c_char_p, []),
    "souffle_version": (C.c_char_p, []),
    "souffle_device_info": (C.c_int, [C.POINTER(DevInfo)]),
    "souffle_stage_floor_probe": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]),
    "souffle_mfma_probe": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_double), C.c_void_p]),
    "souffle_l2_stream_probe": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_double), C.c_void_p]),
    "souffle_set_stage_trace": (C.c_int, [C.c_void_p, C.c_size_t]),
    "souffle_set_cooperative_launch": (C.c_int, [C.c_int]),
    "souffle_set_strict_fences": (C.c_int, [C.c_int]),
    "souffle_workspace_init": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_workspace_status": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_uint), C.c_int]),
    "souffle_bert_workspace_bytes": (C.c_size_t, [C.POINTER(BertCfg)]),
    "souffle_bert_layer_fused": (C.c_int, [C.POINTER(BertCfg), C.POINTER(BertLayerW), C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.POINTER(BertDump), C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_bert_layer_unfused": (C.c_int, [C.POINTER(BertCfg), C.POINTER(BertLayerW), C.c_void_p, C.c_void_p,
                                             C.c_void_p, C.POINTER(BertDump), C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_bert_encoder_fused": (C.c_int, [C.POINTER(BertCfg), C.POINTER(BertLayerW), C.c_void_p, C.c_void_p,
                                             C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_bert_encoder_unfused": (C.c_int, [C.POINTER(BertCfg), C.POINTER(BertLayerW), C.c_void_p, C.c_void_p,
                                               C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_bert_encoder_fused_static": (C.c_int, [C.POINTER(BertCfg), C.POINTER(BertLayerW), C.c_void_p, C.c_void_p,
                                                    C.c_void_p, C.c_void_p]),
    "souffle_bert_static_status": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint), C.c_int]),
    "souffle_bert_polled_copies": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]),
    "souffle_bert_handover_plan": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "souffle_bert_fc2_packed_bytes": (C.c_size_t, []),
    "souffle_bert_pack_fc2": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "souffle_bert_embed": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                     C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                     C.c_void_p]),
    "souffle_bert_pooler": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]),
    "souffle_lstm_workspace_bytes": (C.c_size_t, [C.POINTER(LstmCfg)]),
    "souffle_lstm_fused": (C.c_int, [C.POINTER(LstmCfg), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                     C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_set_swin_split": (C.c_int, [C.c_int]),
    "souffle_swin_workspace_bytes": (C.c_size_t, [C.POINTER(SwinCfg)]),
    "souffle_swin_block_pair_fused": (C.c_int, [C.POINTER(SwinCfg), C.POINTER(SwinBlockW), C.c_void_p, C.c_void_p,
                                                C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_swin_index_maps": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_void_p]),
    "souffle_swin_ffn_fused": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                         C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]),
    "souffle_gemm_f16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "souffle_swin_patch_merge": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                           C.c_float, C.c_void_p]),
    "souffle_se_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "souffle_se_module_fused": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t,
                                          C.c_void_p]),
    "souffle_mbconv_workspace_bytes": (C.c_size_t, [C.POINTER(MbconvBlock), C.c_int]),
    "souffle_mbconv_stack": (C.c_int, [C.POINTER(MbconvBlock), C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p,
                                       C.c_size_t, C.c_void_p]),
    "souffle_pointwise_conv2d_bn": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                              C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "souffle_depthwise_conv2d_bn_swish": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                                    C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "souffle_bench_us": (C.c_int, [BENCH_FN, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                   C.POINTER(C.c_double), C.POINTER(C.c_double)]),
}

_lib = None


class SouffleError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("souffle_hip error %d: %s" % (code, text))
        self.code = code


def lib():
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libsouffle_hip.so is missing at %s: build it with build.py "
                               "(there is no fallback path)" % LIB_PATH)
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def last_error():
    return lib().souffle_last_error().decode()


def check(rc):
    if rc != 0:
        raise SouffleError(rc, last_error())


def ptr(t):
    """Device pointer of a torch tensor (or None)."""
    return None if t is None else t.data_ptr()


def current_stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


class Workspace:
    """A zero-initialised device workspace, cached by the binding modules."""

    def __init__(self, nbytes, device="cuda:0"):
        import torch
        self.buf = torch.zeros(max(int(nbytes), 16384) // 4 + 4, dtype=torch.int32, device=device)
        self.nbytes = self.buf.numel() * 4
        check(lib().souffle_workspace_init(self.buf.data_ptr(), self.nbytes, current_stream()))

    @property
    def ptr(self):
        return self.buf.data_ptr()

    def status(self, clear=False):
        """Wait for the current stream and return the sticky failure flags (0 = all launches completed)."""
        flags = C.c_uint(0)
        check(lib().souffle_workspace_status(self.buf.data_ptr(), current_stream(), C.byref(flags), 1 if clear else 0))
        return flags.value


def set_stage_trace(tensor):
    """Point the in-kernel stage trace at an int64 CUDA tensor (None = off)."""
    if tensor is None:
        check(lib().souffle_set_stage_trace(None, 0))
    else:
        check(lib().souffle_set_stage_trace(tensor.data_ptr(), tensor.numel() * tensor.element_size()))


def set_swin_split(on):
    """Swin block pair: four workgroups per window (True, the default) or one (False)."""
    check(lib().souffle_set_swin_split(1 if on else 0))


def set_cooperative_launch(on):
    """Launch the persistent kernels cooperatively (True) or plainly (False, the default)."""
    check(lib().souffle_set_cooperative_launch(1 if on else 0))


def set_strict_fences(on):
    """Every hand-over between workgroups also runs the memory model's release / acquire fences (True) or rests on
    acknowledged write-through stores and coherent loads alone (False, the default).  Same results either way."""
    check(lib().souffle_set_strict_fences(1 if on else 0))


def device_info():
    info = DevInfo()
    check(lib().souffle_device_info(C.byref(info)))
    return {n: (getattr(info, n).decode() if n == "arch" else getattr(info, n)) for n, _ in DevInfo._fields_}


def stage_floor_us(stages, device="cuda:0"):
    """(barrier only, barrier + hand-over) time in us of `stages` dependent grid-wide stages without
    arithmetic: the latency floor of a persistent kernel with that many stages.  Synchronises."""
    ws = Workspace(16384, device)
    res = []
    for mode in (0, 1):
        def probe():
            check(lib().souffle_stage_floor_probe(ws.ptr, ws.nbytes, stages, mode, current_stream()))
        mn, _ = bench_us(probe, warmup=3, rounds=3, repeat=10)
        res.append(mn)
    if ws.status() != 0:
        raise SouffleError(-4, "a bounded wait inside the probe gave up")
    return tuple(res)


def measured_ceilings(device="cuda:0"):
    """Empirical ceilings of this device: (device-to-device copy GB/s counting read + written bytes,
    MFMA-only fp16 TFLOP/s).  Synchronises."""
    import torch
    n = 1 << 30
    a = torch.empty(n, dtype=torch.uint8, device=device).fill_(1)
    b = torch.empty_like(a)
    mn, _ = bench_us(lambda: b.copy_(a), warmup=3, rounds=3, repeat=5)
    copy_gbs = 2.0 * n / (mn * 1e-6) / 1e9
    del a, b
    out = torch.empty(device_info()["num_cus"] * 512, dtype=torch.float32, device=device)
    flops = C.c_double()
    iters = 25000

    def probe():
        check(lib().souffle_mfma_probe(out.data_ptr(), out.numel() * 4, iters, C.byref(flops), current_stream()))
    mn, _ = bench_us(probe, warmup=2, rounds=3, repeat=3)
    return copy_gbs, flops.value / (mn * 1e-6) / 1e12


def measured_l2_stream_gbs(region_bytes=1 << 20, device="cuda:0"):
    """Device-wide rate (GB/s) at which all CUs together stream an L2-resident region into LDS.  Synchronises."""
    import torch
    src = torch.ones(region_bytes, dtype=torch.uint8, device=device)
    moved = C.c_double()
    iters = 512

    def probe():
        check(lib().souffle_l2_stream_probe(src.data_ptr(), src.numel(), iters, C.byref(moved), current_stream()))
    mn, _ = bench_us(probe, warmup=2, rounds=3, repeat=3)
    return moved.value / (mn * 1e-6) / 1e9


def bench_us(launch, warmup=20, rounds=10, repeat=100, stream=None):
    """min-of-means and median (us) of `launch()` under the reference's timing rule
    (cpp/souffle_utils/cuda_utils.h:102-136), timed with HIP events on `stream`."""
    def _fn(_):
        launch()
        return 0
    cb = BENCH_FN(_fn)
    mn, med = C.c_double(), C.c_double()
    check(lib().souffle_bench_us(cb, None, current_stream() if stream is None else stream, warmup, rounds,
                                 repeat, C.byref(mn), C.byref(med)))
    return mn.value, med.value
