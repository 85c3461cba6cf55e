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


DW = "void ms::(anonymous namespace)::gmm16_fast_kernel<0, false, false, 0, false>(ms::GmmArgs)"


def test_counters_prints_the_derived_ratios(tmp_path):
    """MFMA busy = busy clocks / (4 x wave cycles), L2 hit rate = hits / (hits + misses); torch's own kernels are left out."""
    sq, tcc = tmp_path / "q.csv", tmp_path / "t.csv"
    with open(sq, "w") as fh:
        fh.write(HEADER)
        for i, (k, c, v) in enumerate([(FWD, "SQ_WAVE_CYCLES", 1000), (FWD, "SQ_VALU_MFMA_BUSY_CYCLES", 2680),
                                       (FWD, "SQ_WAIT_INST_LDS", 400), ("at::native::fill", "SQ_WAVE_CYCLES", 5)]):
            fh.write(f'{i},"{k}",{c},{v}\n')
    with open(tcc, "w") as fh:
        fh.write(HEADER)
        for i, (k, c, v) in enumerate([(FWD, "TCC_HIT_sum", 750), (FWD, "TCC_MISS_sum", 250)]):
            fh.write(f'{i},"{k}",{c},{v}\n')
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "counters", str(sq), str(tcc)],
                         cwd=ROOT, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    assert "at::native" not in res.stdout
    derived = [l for l in res.stdout.split("# derived")[1].splitlines() if l.startswith("gmm16_fast_kernel")][0].split()
    assert derived[-5:] == ["0.670", "0.100", "-", "-", "0.750"]


def test_products_reads_the_dispatches_in_launch_order(tmp_path):
    """Six products, two launches each, the first of each left out: 128-byte read requests, 64-byte write requests."""
    path = tmp_path / "c.csv"
    with open(path, "w") as fh:
        fh.write(HEADER)
        d = 0
        for prod in range(6):
            for rep in range(2):
                for c, v in (("TCC_EA0_RDREQ_sum", (prod + 1) * 1e7 * (3 if rep == 0 else 1)), ("TCC_EA0_WRREQ_sum", 1e7),
                             ("TCC_HIT_sum", 3e6), ("TCC_MISS_sum", 1e6)):
                    fh.write(f'{d},"{DW if prod > 3 else FWD}",{c},{v}\n')
                d += 1
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "products", "--csv", str(path), "--iters", "2"],
                         cwd=ROOT, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    rows = {l.split()[0]: l.split()[1:] for l in res.stdout.splitlines()[1:]}
    assert rows["fwd1"] == ["1.28", "0.64", "0.750"] and rows["dw2"] == ["7.68", "0.64", "0.750"]
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "products", "--csv", str(path), "--iters", "3"],
                         cwd=ROOT, capture_output=True, text=True)
    assert res.returncode != 0 and "expected 18" in res.stderr


def test_in_layer_durations_are_recorded_with_the_build(tmp_path):
    stats, out = tmp_path / "s.csv", tmp_path / "in_layer.json"
    with open(stats, "w") as fh:
        fh.write('"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n')
        fh.write('"void ms::(anonymous namespace)::permute_fused_kernel<long, unsigned int __vector(4)>(int)",50,1000000,20000.0,1,1,1,1\n')
        fh.write('"void ms::(anonymous namespace)::swiglu_kernel<ms::BF16, 8>(int)",50,5000000,100000.0,1,1,1,1\n')
        fh.write('"void ms::(anonymous namespace)::gmm16_fast_kernel<0, true, false, 0, true>(ms::GmmArgs)",100,1,1300000.0,1,1,1,1\n')
    res = subprocess.run([sys.executable, "-m", "mindspeed_amd.profile_tools", "in-layer", "--stats", str(stats), "--out", str(out)],
                         cwd=ROOT, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    data = json.loads(out.read_text())
    assert data["build"] == build.source_hash()
    k = data["kernels"]["mixtral"]
    assert set(k) == {"permute_fused_kernel", "swiglu_kernel"}
    # 100,794,368 bytes in 20 us = 5039.7 GB/s = 0.63 of 8 TB/s
    assert k["permute_fused_kernel"]["bytes_per_launch"] == 100794368 and k["permute_fused_kernel"]["frac_of_hbm_peak"] == 0.63
    sys.path.insert(0, ROOT)
    import bench
    saved = bench.IN_LAYER_FILE
    try:
        bench.IN_LAYER_FILE = str(out)
        assert bench.measured_in_layer_durations("mixtral") == k
        data["build"] = "0" * 16
        out.write_text(json.dumps(data))
        assert bench.measured_in_layer_durations("mixtral") is None       # measured on other sources: not reported
    finally:
        bench.IN_LAYER_FILE = saved
