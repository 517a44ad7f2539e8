"""Host-side checks of bench.py: the byte and flop counts it divides by are the algorithmic ones of
the measurement plan, and a run on more than one GPU is refused with a message (this build is for
one GPU)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_algorithmic_bytes():
    import bench
    # 2*R*K + R*Kp/2 + (Kp/64)*Rp*4 + 4, input counted once
    assert bench.quant_bytes((4096, 4096), "nvfp4") == 42_991_620
    assert bench.quant_bytes((8192, 4096), "nvfp4") == 85_983_236
    # 2*R*K + R*align_up(K,16) + 4*Rp
    assert bench.quant_bytes((8192, 4096), "fp8e4m3") == 100_696_064
    assert bench.quant_bytes((8192, 4096), "int8") == 100_696_064
    # ragged sizes pad K to 64 (nvfp4) / 16 (per-row) and the rows to 16
    assert bench.quant_bytes((5, 70), "nvfp4") == 2 * 5 * 70 + 5 * 128 // 2 + 2 * 16 * 4 + 4
    assert bench.quant_bytes((5, 70), "int8") == 2 * 5 * 70 + 5 * 80 + 4 * 16
    # (M+N)*K/2 + (Mp+Np)*K/16 + 2*M*N + 8
    m = n = k = 8192
    assert bench.linear_bytes(m, n, k) == (m + n) * k // 2 + (m + n) * k // 16 + 2 * m * n + 8
    assert bench.MFMA_PEAK_TFLOPS == 2500.0 and bench.HBM_PEAK_GBS == 8000.0


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
