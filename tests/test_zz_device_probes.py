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
