"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol that
include/souffle_hip.h declares, rejects bad arguments with a status and a message (never
an abort), and computes the Swin index maps bit-exactly."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle
import souffle_hip as sh

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "souffle_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(souffle_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 18
    handle = C.CDLL(sh.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), "libsouffle_hip.so does not export %s" % n
    assert set(names) == set(sh.SIGNATURES), "ctypes table and header disagree: %s" % (set(names) ^ set(sh.SIGNATURES))
    assert b"gfx950" in sh.lib().souffle_version()


def test_bert_validation_without_gpu():
    lib = sh.lib()
    assert lib.souffle_bert_workspace_bytes(None) == 0
    bad = sh.BertCfg(1, 600, 768, 12, 3072, 0, 0.125, 1e-12, 1, 0)
    assert lib.souffle_bert_workspace_bytes(C.byref(bad)) == 0 and "seq_len" in sh.last_error()
    bad = sh.BertCfg(1, 128, 1024, 16, 4096, 0, 0.125, 1e-12, 1, 0)
    assert lib.souffle_bert_workspace_bytes(C.byref(bad)) == 0 and "hidden=768" in sh.last_error()
    ok = sh.BertCfg(1, 128, 768, 12, 3072, 0, 0.125, 1e-12, 1, 0)
    n1 = lib.souffle_bert_workspace_bytes(C.byref(ok))
    big = sh.BertCfg(32, 128, 768, 12, 3072, 0, 0.125, 1e-12, 12, 0)
    n32 = lib.souffle_bert_workspace_bytes(C.byref(big))
    assert 0 < n1 < n32 < (1 << 30)
    # few rows: one set of inter-stage buffers per layer; from 1024 rows (a multiple of 256) up: one set
    # for all layers (plus 16 hand-over words per 256-row block), so the size no longer grows with depth
    bytes_for = lambda b, s, layers: lib.souffle_bert_workspace_bytes(C.byref(sh.BertCfg(b, s, 768, 12, 3072, 0, 0.125, 1e-12, layers, 0)))
    assert bytes_for(1, 128, 12) > 11 * (bytes_for(1, 128, 1) - 4096)
    assert bytes_for(32, 128, 12) == bytes_for(32, 128, 1) == n32
    per_row = 2 * (3 * 768 + 768 + 768 + 768 + 3072 + 768) + 4 * 768 * 2     # qkv, ctx, z1, y1, h, layer output; four fp16 partial sums
    assert 4096 * per_row <= n32 <= 4096 * per_row + (1 << 19)       # (+ control block, flag and completion words, the kept wait masks)
    assert bytes_for(32, 100, 2) > bytes_for(32, 128, 2)                       # padded to 128 inside the call: room for the padded copies
    w = sh.BertLayerW()
    rc = lib.souffle_bert_layer_fused(C.byref(bad), C.byref(w), None, None, None, None, None, 0, None)
    assert rc == -2
    rc = lib.souffle_bert_layer_fused(None, C.byref(w), None, None, None, None, None, 0, None)
    assert rc == -1
    # a valid configuration on a machine without a GPU reports a device error; with one, the NULL pointers
    rc = lib.souffle_bert_layer_fused(C.byref(ok), C.byref(w), None, None, None, None, None, 0, None)
    assert rc in (-5, -1) and sh.last_error()
    bad_act = sh.BertCfg(1, 128, 768, 12, 3072, 7, 0.125, 1e-12, 1, 0)
    assert lib.souffle_bert_layer_unfused(C.byref(bad_act), C.byref(w), None, None, None, None, None, 0, None) == -2


def test_other_families_validate_without_gpu():
    lib = sh.lib()
    assert lib.souffle_lstm_workspace_bytes(C.byref(sh.LstmCfg(10, 256, 100, 1, 0, 0.0))) > 10 * 100 * 256 * 8
    assert lib.souffle_lstm_workspace_bytes(C.byref(sh.LstmCfg(10, 128, 100, 1, 0, 0.0))) == 0
    assert lib.souffle_lstm_fused(C.byref(sh.LstmCfg(10, 256, 100, 2, 0, 0.0)), None, None, None, None, None, None, 0, None) == -2
    assert lib.souffle_lstm_fused(C.byref(sh.LstmCfg(10, 256, 100, 1, 0, 0.0)), None, None, None, None, None, None, 0, None) == -1
    assert lib.souffle_swin_workspace_bytes(C.byref(sh.SwinCfg(56, 56, 128, 4, 7, 3, 4, 1, 1e-5))) >= 56 * 56 * 128 * 2
    assert lib.souffle_swin_workspace_bytes(C.byref(sh.SwinCfg(56, 50, 128, 4, 7, 3, 4, 1, 1e-5))) == 0
    assert lib.souffle_swin_workspace_bytes(C.byref(sh.SwinCfg(56, 56, 96, 3, 7, 3, 4, 1, 1e-5))) == 0
    assert lib.souffle_se_workspace_bytes(32, 112 * 112, 8) > 0
    assert lib.souffle_se_workspace_bytes(4096, 49, 8) == 0
    assert lib.souffle_gemm_f16(None, None, None, 64, 64, 64, None) == -1
    assert lib.souffle_workspace_init(None, 0, None) == -4
    assert lib.souffle_bench_us(sh.BENCH_FN(lambda _: 0), None, None, 1, 0, 1, None, None) == -2


@pytest.mark.parametrize("H,W,ws,shift", [(56, 56, 7, 3), (56, 56, 7, 0), (14, 28, 7, 2), (8, 12, 4, 1), (7, 7, 7, 6)])
def test_swin_index_maps_bit_exact(H, W, ws, shift):
    import swin_transformer_binding as sb
    for a, b in zip(sb.index_maps(H, W, ws, shift), oracle.swin_index_maps(H, W, ws, shift)):
        np.testing.assert_array_equal(a, b)
    with pytest.raises(sh.SouffleError):
        sb.index_maps(10, 14, 7, 3)
    with pytest.raises(sh.SouffleError):
        sb.index_maps(14, 14, 7, 7)


def test_product_does_not_reach_the_oracle():
    """The shipped library and wrappers never link, import or call anything under oracle/."""
    pkg = os.path.join(ROOT, "souffle-models_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".sh")):
                assert "oracle" not in open(os.path.join(dirpath, f)).read().lower(), f
    import subprocess
    out = subprocess.run(["nm", "-D", sh.LIB_PATH], capture_output=True, text=True).stdout
    assert "oracle_" not in out
