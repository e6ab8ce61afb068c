"""The measurement helpers of the library (device ceilings, latency floor of a chain of grid-wide
stages), which bench.py prints next to the published peaks.  Collected last: they measure the device,
no product path depends on them."""
import pytest

from gpu_util import announce

pytestmark = pytest.mark.gpu


def test_device_probes_report_plausible_ceilings():
    """The measurement helpers behind the bench line's measured ceilings and latency floor."""
    announce("device probes")
    import souffle_hip as sh
    copy_gbs, mfma_tflops = sh.measured_ceilings()
    assert 500 < copy_gbs < 8000 and 200 < mfma_tflops < 2600
    l2_gbs = sh.measured_l2_stream_gbs()
    assert 1000 < l2_gbs < 40000
    with pytest.raises(sh.SouffleError):
        sh.check(sh.lib().souffle_l2_stream_probe(None, 1 << 20, 10, None, None))
    bar_us, floor_us = sh.stage_floor_us(24)
    assert 5 < bar_us < floor_us < 400
    with pytest.raises(sh.SouffleError):
        sh.check(sh.lib().souffle_stage_floor_probe(None, 0, 10, 0, None))


@pytest.mark.gpu
def test_grid_barrier_control_words_after_many_launches():
    """Every word of the grid barrier's control block has a place of its own: after many launches of a kernel with
    three barriers each, every arrival counter equals the value carried over for the next launch, every done flag
    holds the number of the last barrier (a done flag that shared its word with a carried counter value would hold
    that far larger value and let every waiter through), and no bounded wait gave up."""
    import souffle_hip as sh
    from gpu_util import announce
    announce("grid barrier control words")
    ws = sh.Workspace(16384)
    launches, stages = 300, 3
    for _ in range(launches):
        sh.check(sh.lib().souffle_stage_floor_probe(ws.ptr, ws.nbytes, stages, 1, sh.current_stream()))
    assert ws.status() == 0
    c = ws.buf[:512].cpu().numpy().astype("uint32")
    n_cus = sh.device_info()["num_cus"]
    barriers = int(c[24])
    assert barriers > 0 and barriers % launches == 0
    for x in range(8):
        wgs = (n_cus + 7 - x) // 8
        assert int(c[32 * x]) == barriers * wgs == int(c[16 + 32 * x]), (x, int(c[32 * x]), int(c[16 + 32 * x]))
        assert int(c[256 + 32 * x]) == barriers, (x, int(c[256 + 32 * x]))
