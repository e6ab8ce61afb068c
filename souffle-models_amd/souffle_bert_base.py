"""souffle_bert_base: drop-in for the reference's pybind module of the same name
(cpp/bert/bert_base_impl.cu:277-308,1785-1788; caller python/models/bert/souffle_bert.py:31).

souffle_bert_base() -> 0.  Like the reference it allocates an all-zero model and an all-zero
[384, 768] input itself, runs the 12-layer encoder with ONE layer's weights used by every layer
(Bert::Solve, cpp/bert/bert_base_impl.cu:590-678) as per-operator launches (the reference's
unfused O0 baseline: 288 launches there, 72 here), waits for the result and returns 0.
Keyword arguments reach what the reference hard-codes.
"""
import torch

import bert_binding
import souffle_hip as sh


def souffle_bert_base(*, batch=1, seq_len=384, num_layers=12, fused=False, device="cuda:0"):
    z = lambda *shape: torch.zeros(shape, dtype=torch.float16, device=device)
    layer = {"qkv_weight": z(3, bert_binding.HIDDEN, bert_binding.HIDDEN), "attn_fc_weight": z(bert_binding.HIDDEN, bert_binding.HIDDEN),
             "fc1_weight": z(bert_binding.HIDDEN, bert_binding.FFN), "fc2_weight": z(bert_binding.FFN, bert_binding.HIDDEN)}
    enc = bert_binding.Encoder([layer] * num_layers, batch, seq_len, device=device)
    out = enc(z(batch * seq_len, bert_binding.HIDDEN), fused=fused)
    torch.cuda.synchronize()
    if enc.ws.status() != 0:
        raise sh.SouffleError(-4, "a bounded wait inside the launch gave up")
    if not bool(torch.isfinite(out).all()):
        raise sh.SouffleError(-4, "non-finite output")
    return 0
