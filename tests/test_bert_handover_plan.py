"""Host-side check of the few-rows encoder's work split and hand-over plan (no GPU): the plan comes from the library
(souffle_bert_handover_plan evaluates the functions the kernel itself uses), the dependences come from a model, written
here, of which rows and columns of which tensor every item reads and writes.  Every pair of a consumer workgroup and a
producer workgroup whose items touch the same data must be in the plan, every (m-tile, slice) must belong to exactly
one workgroup, and what the consumer waits for must have been published by a phase that precedes it."""
import ctypes as C

import numpy as np
import pytest

import souffle_hip as sh

QKV, ATT, OUT, FC1, FC2, FIN = 0, 1, 2, 3, 4, 6
H, HD = 768, 64


def plan(B, S, G, packed, phase, b):
    items = (C.c_int * 64)()
    n = C.c_int(0)
    needs = (C.c_ubyte * G)()
    sh.check(sh.lib().souffle_bert_handover_plan(B, S, G, packed, phase, b, items, 32, C.byref(n), needs))
    assert n.value <= 32, n.value
    return [(items[2 * i], items[2 * i + 1]) for i in range(n.value)], np.frombuffer(needs, dtype=np.uint8).copy()


def writes(phase, item, B, S, packed):
    """(tensor, row range, column range) written by an item."""
    a, b = item
    if phase == FC2:                       # whole-K form only: (m-tile, 16 columns) of the sum z2 (and their statistics)
        assert packed
        return ("z2", range(32 * a, 32 * a + 32), range(16 * b, 16 * b + 16))
    if phase == QKV:                       # (m-tile, which * 12 + head) -> rows of q, k or v of one head
        return ("qkv%d" % (b // 12), range(32 * a, 32 * a + 32), range((b % 12) * HD, (b % 12 + 1) * HD))
    if phase == ATT:                       # (query block, batch * 12 + head) -> 16 rows of ctx, the head's columns
        r0 = (b // 12) * S + 16 * a
        return ("ctx", range(r0, r0 + 16), range((b % 12) * HD, (b % 12 + 1) * HD))
    if phase == OUT:
        return ("z1", range(32 * a, 32 * a + 32), range(64 * b, 64 * b + 64))
    if phase == FC1:
        return ("h", range(32 * a, 32 * a + 32), range(64 * b, 64 * b + 64))
    raise AssertionError(phase)


def reads(phase, item, B, S, packed):
    """What an item reads of the phase before it: a list of (tensor, rows, columns)."""
    a, b = item
    if phase in (QKV, FIN):                # whole-K form: whole rows of z2 (QKV of a later layer: LayerNorm over the row; FIN: the
        assert packed                      # row statistics)
        return [("z2", range(32 * a, 32 * a + 32), range(0, H))]
    if phase == FC2 and packed:            # the whole K of h
        return [("h", range(32 * a, 32 * a + 32), range(0, 4 * H))]
    if phase == ATT:
        batch, head = b // 12, b % 12
        cols = range(head * HD, (head + 1) * HD)
        q0 = batch * S + 16 * a
        return [("qkv0", range(q0, q0 + 16), cols), ("qkv1", range(batch * S, (batch + 1) * S), cols),
                ("qkv2", range(batch * S, (batch + 1) * S), cols)]
    if phase == OUT:
        return [("ctx", range(32 * a, 32 * a + 32), range(0, H))]
    if phase == FC1:                       # whole rows of z1 (and their statistics: LayerNorm over the row)
        return [("z1", range(32 * a, 32 * a + 32), range(0, H))]
    if phase == FC2:                       # K quarter ks of h
        ks = b & 3
        return [("h", range(32 * a, 32 * a + 32), range(768 * ks, 768 * ks + 768))]
    raise AssertionError(phase)


def overlap(r, w):
    return r[0] == w[0] and max(r[1].start, w[1].start) < min(r[1].stop, w[1].stop) and \
        max(r[2].start, w[2].start) < min(r[2].stop, w[2].stop)


SHAPES = [(1, 64), (1, 128), (2, 128), (1, 256), (3, 256), (1, 384), (2, 384), (1, 512), (7, 128), (15, 64), (8, 128), (2, 512), (11, 128)]


# (the kernel runs grids that are multiples of 8 up to 256; the plan functions are also defined, and checked, for other grids)
@pytest.mark.parametrize("B,S", SHAPES)
@pytest.mark.parametrize("G", [256, 304, 100])
@pytest.mark.parametrize("packed", [1, 0])
def test_every_dependence_is_waited_for_and_every_item_has_one_owner(B, S, G, packed):
    M = B * S
    owned = {ph: [plan(B, S, G, packed, ph, b) for b in range(G)] for ph in (QKV, ATT, OUT, FC1, FC2, FIN)}
    # partition: every item of a phase exactly once
    expect = {QKV: {(mt, ws) for mt in range(M // 32) for ws in range(36)},
              ATT: {(qb, bh) for qb in range(S // 16) for bh in range(B * 12)},
              OUT: {(mt, ws) for mt in range(M // 32) for ws in range(12)},
              FC1: {(mt, ws) for mt in range(M // 32) for ws in range(48)},
              FC2: {(mt, ws) for mt in range(M // 32) for ws in range(48)},
              FIN: {(mt, ws) for mt in range(M // 32) for ws in range(12)}}
    for ph, per_wg in owned.items():
        flat = [it for items, _ in per_wg for it in items]
        assert len(flat) == len(set(flat)), "phase %d: an item has two owners" % ph
        assert set(flat) == expect[ph], "phase %d: items missing or surplus" % ph
    # coverage: consumer workgroup b must wait for every producer workgroup pb whose items write what b's items read
    pairs = ((ATT, QKV), (OUT, ATT), (FC1, OUT), (FC2, FC1)) + (((QKV, FC2), (FIN, FC2)) if packed else ())
    for cph, pph in pairs:
        prod = [[writes(pph, it, B, S, packed) for it in items] for items, _ in owned[pph]]
        for b in range(G):
            items, needs = owned[cph][b]
            if not items:
                continue
            rd = [r for it in items for r in reads(cph, it, B, S, packed)]
            for pb in range(G):
                if prod[pb] and any(overlap(r, w) for r in rd for w in prod[pb]):
                    assert needs[pb], "B=%d S=%d G=%d: workgroup %d phase %d reads what workgroup %d writes and does not wait for it" % (B, S, G, b, cph, pb)
                elif needs[pb]:
                    assert prod[pb], "waits for a workgroup that publishes nothing in the phase before"


def test_plan_rejects_what_the_few_rows_path_does_not_run():
    n = C.c_int(0)
    lib = sh.lib()
    assert lib.souffle_bert_handover_plan(12, 128, 256, 1, 0, 0, None, 0, C.byref(n), None) == -2     # 1536 rows: the many-rows path
    assert lib.souffle_bert_handover_plan(10, 128, 256, 0, 0, 0, None, 0, C.byref(n), None) == -2     # 1280 rows, a multiple of 256: likewise
    assert lib.souffle_bert_handover_plan(1, 100, 256, 1, 0, 0, None, 0, C.byref(n), None) == -2
    assert lib.souffle_bert_handover_plan(1, 128, 256, 1, 5, 0, None, 0, C.byref(n), None) == -2
    assert lib.souffle_bert_handover_plan(1, 128, 256, 0, 0, 256, None, 0, C.byref(n), None) == -2
    assert lib.souffle_bert_handover_plan(1, 128, 256, 1, 0, 0, None, 0, None, None) == -1
