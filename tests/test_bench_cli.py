"""bench.py command line: this build measures one GPU; a request for more must end with a message, not a run."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_and_shares_come_from_the_tracked_profile():
    sys.path.insert(0, ROOT)
    import bench
    traffic = bench.measured_traffic()
    shares = bench.measured_simd_shares()
    for k in ("gca_fwd_mfma_kernel", "gca_bwd_dq_mfma_kernel", "gca_bwd_dkdv2_mfma_kernel"):
        assert 0.1 < traffic[k] < 100.0                     # GB per launch
        mfma, valu = shares[k]
        assert 0.0 < mfma < 1.0 and 0.0 < valu < 1.0 and mfma + valu <= 1.0
    assert bench.measured_traffic("profiles/does_not_exist.txt") == {}
