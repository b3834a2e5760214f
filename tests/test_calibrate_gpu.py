"""The measuring aid behind bench.py's roofline.sustained_peak: the calibration kernel runs, every workgroup
reports its MFMA loop's time, the streaming wavefronts read while the MFMAs run and stop with them."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mfma_stream_alone_and_beside_an_hbm_stream(capi, dev):
    alone, streamed, ms = capi.calibrate_mfma(0.05, 0, False)
    assert streamed == 0 and ms > 0
    assert 1.0 < alone < 5.1            # PFLOP/s: below the data-sheet peak, above a fifth of it
    beside, tbs, _ = capi.calibrate_mfma(0.05, 1 << 30, False)
    assert 0.5 < beside <= alone * 1.05 and 1.0 < tbs < 8.1
    alone_bf16, _, _ = capi.calibrate_mfma(0.05, 0, True)
    assert 0.5 < alone_bf16 < 2.6


def test_rejects_a_stream_buffer_too_small_to_share(capi, dev):
    lib = capi.library()
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)
    res = torch.zeros(256, 2, dtype=torch.int64, device=dev)
    sink = torch.zeros(2, device=dev)
    lib.calibrate_mfma_launcher(buf.data_ptr(), buf.data_ptr(), 1 << 20, res.data_ptr(), sink.data_ptr(), 256, 8, 0, None)
    assert lib.cuda_agent_amd_last_status() == 2
    torch.cuda.synchronize()
    assert int(res.sum()) == 0          # nothing was launched
