"""bench.py's host-side helpers (no GPU): the traffic figures are only taken from a profile summary that was
measured on the current kernel sources, and --gpus above 1 is refused."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_traffic_is_read_per_kernel_instance_and_dropped_when_stale(tmp_path, monkeypatch):
    import bench
    fp = bench.kernel_source_fingerprint()
    assert len(fp) == 16 and int(fp, 16) >= 0
    lines = [
        "et::tile_linear_resident_kernel<2, false, 12, false, 64>   n= 95  fetch avg     17.95 MiB  write avg     36.01 MiB   (fetch min/max 17.95/17.96)",
        "et::tile_linear_resident_kernel<1, false, 8, false, 32>    n=220  fetch avg      9.56 MiB  write avg      0.38 MiB   (fetch min/max 5.02/14.10)",
        "et::attention_kernel<64, 2, 4, false, false, true, 64, false>  n= 35  fetch avg     36.08 MiB  write avg     12.00 MiB   (fetch min/max 36.08/36.08)",
        "et::tile_ffn_fused_kernel<3, true>   n= 95  fetch avg     43.45 MiB  write avg     14.00 MiB   (fetch min/max 43.45/43.45)",
    ]
    p = tmp_path / "traffic.txt"
    monkeypatch.setattr(bench, "TRAFFIC_PROFILE", str(p))
    p.write_text("\n".join(lines) + f"\n\nkernel sources fingerprint: {fp}\n")
    t = bench.measured_traffic_mib()
    assert abs(t["et::tile_linear_resident_kernel<2, false, 12, false, 64>"] - 53.96) < 1e-6   # not the 128-row instance
    assert abs(t["et::tile_ffn_fused_kernel<3, true>"] - 57.45) < 1e-6
    for name in bench.TRAFFIC_KERNELS.values():
        assert name in t
    p.write_text("\n".join(lines) + "\n\nkernel sources fingerprint: 0123456789abcdef\n")
    assert bench.measured_traffic_mib() == {}          # measured on other sources: no figure rather than a stale one
    p.write_text("\n".join(lines) + "\n")
    assert bench.measured_traffic_mib() == {}          # no fingerprint at all
    monkeypatch.setattr(bench, "TRAFFIC_PROFILE", str(tmp_path / "absent.txt"))
    assert bench.measured_traffic_mib() == {}


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one gpu" in (r.stdout + r.stderr).lower()
