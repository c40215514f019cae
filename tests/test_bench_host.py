"""Host-side pieces of bench.py that need no GPU: the arithmetic that turns the two rocprofv3 counter files of
`bench.py --pmc-workload` into HBM bytes per launch (roofline.traffic), and the refusal of more than one GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402

KERNEL = ("void xfthip::(anonymous namespace)::qgemm_skinny_kernel<0, %d, 1, 4, false, false, %s, %s, false, false>"
          "(xfthip::SkinnyParams)")


def _write(path, counter, copy_units, forms):
    rows = ["Counter_Name,Kernel_Name,Counter_Value"]
    for _ in range(3):
        rows.append('%s,"xfthip::stream_copy_kernel(unsigned int const*, unsigned int*, unsigned long)",%r' % (counter, copy_units))
    for (nt, norm, rope), units in forms.items():
        for _ in range(2):
            rows.append('%s,"%s",%r' % (counter, KERNEL % (nt, norm, rope), units))
    with open(path, "w") as f:
        f.write("\n".join(rows) + "\n")


def test_traffic_from_counters_scales_by_the_copy_kernel(tmp_path):
    copy_kib = bench.PMC_COPY_BYTES / 1024.0
    # FETCH_SIZE counts in units of 2 KiB on this machine, WRITE_SIZE in KiB: the copy kernel fixes both factors
    fetch = {(2, "true", "true"): 1000.0, (1, "false", "false"): 500.0, (2, "true", "false"): 2000.0}
    write = {(2, "true", "true"): 10.0, (1, "false", "false"): 4.0, (2, "true", "false"): 20.0}
    f, w = str(tmp_path / "f.csv"), str(tmp_path / "w.csv")
    _write(f, "FETCH_SIZE", copy_kib / 2.0, fetch)
    _write(w, "WRITE_SIZE", copy_kib, write)
    got = bench.traffic_from_counters(f, w)
    assert got == {"qkv": (1000 * 2 + 10) * 1024, "narrow": (500 * 2 + 4) * 1024, "wide": (2000 * 2 + 20) * 1024}


def test_live_traffic_gives_up_without_the_profiler(monkeypatch):
    import shutil
    monkeypatch.setattr(shutil, "which", lambda name: None)
    assert bench.live_traffic() is None


def test_more_than_one_gpu_is_refused():
    pr = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert pr.returncode == 2 and "one GPU" in pr.stderr
