"""Host-side checks of the measurement helpers: counter files -> HBM bytes per launch, keyed by the source hash."""
import json
import os
import subprocess
import sys

import pytest

from mindspeed_amd import build, profile_tools

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = "Dispatch_Id,Kernel_Name,Counter_Name,Counter_Value\n"
FWD = "void ms::(anonymous namespace)::gmm16_fast_kernel<0, true, false, 0, true>(ms::GmmArgs)"
COPY = "ms::(anonymous namespace)::copy_bytes_kernel(char const*, char*, unsigned long)"


def _write(path, counter, rows):
    with open(path, "w") as fh:
        fh.write(HEADER)
        for i, (kernel, value) in enumerate(rows):
            fh.write(f'{i},"{kernel}",{counter},{value}\n')


def test_short_name_strips_namespace_and_arguments():
    assert profile_tools.short_name(FWD) == "gmm16_fast_kernel<0, true, false, 0, true>"


def test_traffic_scales_counters_by_the_copy_and_records_the_build(tmp_path):
    """FETCH_SIZE reads half of what the copy moved (scale 2), WRITE_SIZE all of it (scale 1): a kernel that reads
    1000 and 3000 counter units in two launches and writes 500 twice moves (2000 * 2 + 500) KiB per launch."""
    fetch, write, out = tmp_path / "f.csv", tmp_path / "w.csv", tmp_path / "traffic.json"
    _write(fetch, "FETCH_SIZE", [(COPY, 512 * 1024), (COPY, 4), (FWD, 1000), (FWD, 3000)])
    _write(write, "WRITE_SIZE", [(COPY, 1024 * 1024), (COPY, 8), (FWD, 500), (FWD, 500)])
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "traffic", "--fetch", str(fetch),
                          "--write", str(write), "--copy-mib", "1024", "--out", str(out)],
                         cwd=ROOT, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    data = json.loads(out.read_text())
    assert data["build"] == build.source_hash()
    assert data["bytes_per_launch"]["mixtral"] == {"gmm_fwd": (2000 * 2 + 500) * 1024}


def test_traffic_needs_the_calibration_copy(tmp_path):
    fetch, write = tmp_path / "f.csv", tmp_path / "w.csv"
    _write(fetch, "FETCH_SIZE", [(FWD, 1000)])
    _write(write, "WRITE_SIZE", [(FWD, 500)])
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "traffic", "--fetch", str(fetch),
                          "--write", str(write)], cwd=ROOT, capture_output=True, text=True)
    assert res.returncode != 0 and "copy_bytes_kernel" in res.stderr


def test_source_hash_follows_the_kernel_sources(tmp_path, monkeypatch):
    """The hash that ties measured traffic to a build changes when a kernel source changes."""
    before = build.source_hash()
    assert len(before) == 16 and before == build.source_hash()
    csrc = tmp_path / "csrc"
    csrc.mkdir()
    for name in os.listdir(build.CSRC):
        if name.endswith((".hip", ".h")):
            (csrc / name).write_bytes(open(os.path.join(build.CSRC, name), "rb").read())
    (tmp_path / "include").mkdir()
    (tmp_path / "include" / "mindspeed_amd.h").write_bytes(open(os.path.join(ROOT, "include", "mindspeed_amd.h"), "rb").read())
    monkeypatch.setattr(build, "CSRC", str(csrc))
    monkeypatch.setattr(build, "HERE", str(csrc))       # "<HERE>/../include" resolves inside tmp_path
    assert build.source_hash() == before
    with open(csrc / "gmm_common.h", "a") as fh:
        fh.write("// changed\n")
    assert build.source_hash() != before


@pytest.mark.gpu
def test_tile_timeline_on_the_diagnostic_build():
    """The diagnostic build records one time-stamp record per tile: 14336 tiles of the weight-gradient product, each
    with its phases in order."""
    if not os.path.exists(build.TRACE_LIB_PATH):
        pytest.skip("diagnostic library not built (python -m mindspeed_amd.build --trace)")
    env = dict(os.environ, MINDSPEED_AMD_LIB=build.TRACE_LIB_PATH, PYTHONPATH=ROOT)
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "timeline", "--modes", "dw1", "--data", "zeros"],
                         cwd=ROOT, env=env, capture_output=True, text=True, timeout=240)
    assert res.returncode == 0, res.stderr[-2000:]
    line = [l for l in res.stdout.splitlines() if l.startswith("dw1")][0].split()
    assert line[2] == "14336"
    find, first, loop, epilogue, total = (float(v) for v in line[3:8])
    assert 0 < find and 0 < first and 0 < loop and 0 < epilogue
    assert abs(find + first + loop + epilogue - total) < 0.05 * total


def test_tracked_traffic_profile_belongs_to_these_sources():
    """bench.py reports roofline.traffic only from a profile measured on the kernel sources as they are now; a
    profile left behind by an older build would make it report null."""
    path = os.path.join(ROOT, "profiles", "gmm_hbm_traffic.json")
    data = json.loads(open(path).read())
    assert data["build"] == build.source_hash(), \
        "profiles/gmm_hbm_traffic.json was measured on other kernel sources: re-run the two rocprofv3 --pmc passes " \
        "named in profiles/moe_layer_mixtral_hbm_traffic.txt and `python -m mindspeed_amd.profile_tools traffic --out` it"
    sys.path.insert(0, ROOT)
    import bench
    for kernel in ("gmm_fwd", "gmm_dx", "gmm_dw"):
        assert bench.measured_traffic("mixtral", kernel) == data["bytes_per_launch"]["mixtral"][kernel] > 1e9
