"""The measurement aids that give bench.py its in-run ceilings: they must run, return plausible
figures and refuse bad arguments.  (The attention kernel's load-only twin is covered with the
attention tests.)"""

import ctypes

import pytest
import torch

from pypto_amd import _lib
from pypto_amd.runtime import hbm_read_probe, mfma_only_probe

pytestmark = pytest.mark.gpu


def test_read_probe_both_patterns(worker):
    buf = torch.zeros(512 << 20, dtype=torch.uint8, device="cuda")
    sweep = hbm_read_probe(worker, buf, waves_per_cu=4, warm_rounds=2, rounds=5)
    streams = hbm_read_probe(worker, buf, streams=True, waves_per_cu=4, warm_rounds=2, rounds=5)
    print("read probe GB/s: one sweep", round(sweep["gbps"]), "a stream per wavefront", round(streams["gbps"]), flush=True)
    # far above anything but HBM, not above the published peak
    for r in (sweep, streams):
        assert 1000 < r["gbps"] < 8000, r
    # a buffer that is not a multiple of anything: the tails are read too, nothing faults
    odd = buf[: (3 << 20) + 48]
    for flag in (False, True):
        assert hbm_read_probe(worker, odd, streams=flag, waves_per_cu=3, warm_rounds=0, rounds=1)["us"] > 0
    lib = worker._lib
    us = ctypes.c_double(0.0)
    for args, what in (((buf.data_ptr(), 1 << 20, 2, 4, 0, 1), "pattern"), ((buf.data_ptr(), 1 << 20, 0, 17, 0, 1), "waves_per_cu"),
                       ((buf.data_ptr() + 8, 1 << 20, 0, 4, 0, 1), "aligned"), ((buf.data_ptr(), 1 << 20, 0, 4, 0, 0), "rounds")):
        with pytest.raises(ValueError, match=what):
            _lib.check(lib.pto_hip_hbm_read_probe(*args, 0, ctypes.byref(us)))
    with pytest.raises(ValueError, match="device tensor"):
        hbm_read_probe(worker, torch.zeros(1024))


def test_mfma_probe(worker):
    g = torch.Generator(device="cuda").manual_seed(0)
    a = torch.randn(256, 512, generator=g, device="cuda").to(torch.bfloat16)
    b = torch.randn(512, 256, generator=g, device="cuda").to(torch.bfloat16)
    r = mfma_only_probe(worker, a, b, iters=200, warm_rounds=20, rounds=10)
    print("mfma-only TFLOP/s", round(r["tflops"]), flush=True)
    assert 500 < r["tflops"] < 2600, r  # below the published dense peak, far above any non-MFMA rate
    with pytest.raises(ValueError, match="same dtype"):
        mfma_only_probe(worker, a, b.to(torch.float16))
    with pytest.raises(ValueError, match="16-bit device tensor"):
        mfma_only_probe(worker, a.float(), b)
