"""Host-side logic of bench.py that needs no GPU: the refusal of more than one GPU, the composite bound, and the
HBM-traffic figure read from the committed profile summary."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode == 2 and "one GPU" in p.stderr and p.stdout.strip() == ""
    env = dict(os.environ, WORLD_SIZE="2")
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, env=env)
    assert p.returncode == 2 and "one GPU" in p.stderr


def test_composite_bound():
    """Half of the FLOPs are P.V at the 16-bit peak, half are scores at the 4-bit peak except for the diagonal share
    2 / (nt + 1) of the visited tiles (1 / nt without the causal mask) at the 8-bit peak."""
    b = _bench()
    for nt, causal in ((64, True), (1024, True), (256, False)):
        d = 2.0 / (nt + 1) if causal else 1.0 / nt
        want = 1.0 / (0.5 * ((1 - d) / b.PEAK_FP4_TFLOPS + d / b.PEAK_FP8_TFLOPS) + 0.5 / b.PEAK_BF16_TFLOPS)
        assert abs(b.composite_peak_tflops(nt, causal) - want) < 1e-6 * want
    assert 3950 < b.composite_peak_tflops(64) < 4000                 # the C3 figure quoted next to the MXFP4 peak


def test_traffic_comes_from_the_profile_summary():
    b = _bench()
    total, commit = b.measured_traffic("c3", "diag")
    assert total is not None and commit
    # read + written bytes of one C3 launch: above the algorithmic 97 + 67 MB, below twice that
    assert 164e6 <= total <= 330e6
    assert b.measured_traffic("c3", "no-such-mode") == (None, None)
    lines = [l for l in open(b.TRAFFIC_FILE) if l.startswith("#@ traffic")]
    assert len(lines) >= 1 and all("commit=" in l for l in lines)


def test_benchmark_inputs_are_the_parity_tests_tensors():
    """bench.py::make_inputs draws on the CPU from one seeded generator: bit for bit what tests/conftest.py::make_qkv (and,
    for the video-DiT workload, tests/test_gpu_route.py::_frames on top of it) hands to the oracle and the kernels."""
    import torch
    from conftest import make_qkv
    b = _bench()
    for seed in (2, 3):                                                  # C3 / C4 scheme: outlier channels
        q, k, v = b.make_inputs(1, 8, 2, 384, 128, seed, "cpu")
        q2, k2, v2 = make_qkv(1, 8, 2, 384, 128, seed=seed, outliers=True)
        assert torch.equal(q, q2) and torch.equal(k, k2) and torch.equal(v, v2)
    q, k, v = b.make_inputs(1, 8, 8, 1024, 64, 0, "cpu", outliers=False)   # C1: plain N(0,1) draws
    q2, k2, v2 = make_qkv(1, 8, 8, 1024, 64, seed=0)
    assert torch.equal(q, q2) and torch.equal(k, k2) and torch.equal(v, v2)
    # C5 scheme: sigma 0.5 and per-frame offsets (21 frames) from a second generator seeded seed + 1
    N, frames = 21 * 20, 21
    q, k, v = b.make_inputs(1, 4, 4, N, 128, 4, "cpu", frames)
    q2, k2, v2 = make_qkv(1, 4, 4, N, 128, seed=4, sigma=0.5)
    g = torch.Generator().manual_seed(5)
    for t in (q2, k2):
        off = 0.5 * torch.randn(frames, 1, 128, generator=g)
        t += off[torch.arange(N) // (N // frames)].reshape(1, 1, N, 128).to(t.dtype)
    assert torch.equal(q, q2) and torch.equal(k, k2) and torch.equal(v, v2)
