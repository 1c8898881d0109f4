"""CPU-only checks of the C-ABI library: it loads, it exports every function the
header declares, and argument errors are reported without touching a GPU."""
import ctypes
import os
import subprocess

import pytest

from vkop_amd import capi


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(capi.LIB_PATH):
        capi.build()
    return capi.lib()


def test_exports_every_declared_symbol(lib):
    declared = capi.declared_symbols()
    assert len(declared) >= 25
    for name in declared:
        assert hasattr(lib, name), name
    # and the binding knows a signature for each of them, and beyond them only for the
    # measurement hooks of the internal header
    internal = capi.internal_symbols()
    assert internal and not set(internal) & set(declared)
    shipped = [name for name in internal if name not in capi.BENCH_ONLY]
    assert sorted(lib._signatures) == sorted(declared + shipped)
    for name in shipped:
        assert hasattr(lib, name), name

    def exported(path):
        out = subprocess.check_output(["nm", "-D", "--defined-only", path]).decode()
        return {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert set(declared) <= exported(capi.LIB_PATH)
    # the hook that changes what a call launches is not in the shipped library, only in the benchmark's build of it
    assert not set(capi.BENCH_ONLY) & exported(capi.LIB_PATH)
    assert set(capi.BENCH_ONLY) <= set(internal)
    assert set(declared) | set(internal) <= exported(capi.BENCH_LIB_PATH)


def test_no_oracle_or_torch_linked_into_product():
    out = subprocess.check_output(["ldd", capi.LIB_PATH]).decode()
    assert "oracle" not in out and "torch" not in out
    assert "amdhip64" in out


def test_argument_errors_need_no_gpu(lib):
    shape = (ctypes.c_int * 2)(4, 1000)
    dummy = ctypes.c_void_p(256)
    f = lib.vkop_hip_softmax
    assert f(dummy, dummy, 7, shape, 2, 1, 0, 0.0, None, 0, None) == capi.ERR_INVALID
    assert "dtype" in capi.last_error()
    assert f(dummy, dummy, capi.F32, shape, 5, 1, 0, 0.0, None, 0, None) == capi.ERR_INVALID
    assert f(dummy, dummy, capi.F32, shape, 2, 2, 0, 0.0, None, 0, None) == capi.ERR_INVALID
    assert f(dummy, dummy, capi.F32, shape, 2, -3, 0, 0.0, None, 0, None) == capi.ERR_INVALID
    assert f(None, dummy, capi.F32, shape, 2, 1, 0, 0.0, None, 0, None) == capi.ERR_INVALID
    assert f(dummy, dummy, capi.F32, None, 2, 1, 0, 0.0, None, 0, None) == capi.ERR_INVALID
    t = lib.vkop_hip_topk
    assert t(dummy, dummy, dummy, capi.F32, shape, 2, -1, 0, 1, 1, None, 0, None) == capi.ERR_INVALID
    assert t(dummy, dummy, dummy, capi.F32, shape, 2, -1, 1001, 1, 1, None, 0, None) == capi.ERR_INVALID
    assert "exceeds" in capi.last_error()
    big = (ctypes.c_int * 2)(1, 100000)
    assert t(dummy, dummy, dummy, capi.F32, big, 2, -1, capi.MAX_K + 1, 1, 1, None, 0, None) == capi.ERR_UNSUPPORTED
    s = lib.vkop_hip_softmax_topk
    need = lib.vkop_hip_softmax_topk_workspace_bytes(capi.F32, shape, 2, -1, 5)
    assert need > 0
    assert s(dummy, None, dummy, dummy, capi.F32, shape, 2, -1, 5, 1, None, 0, None) == capi.ERR_WORKSPACE
    assert s(dummy, None, dummy, dummy, capi.F32, shape, 2, -1, 5, 1, dummy, need - 1, None) == capi.ERR_WORKSPACE
    assert lib.vkop_hip_reduce_max(dummy, dummy, capi.F32, (ctypes.c_int * 2)(3, 0), 2, 1, None) == capi.ERR_INVALID
    # empty tensors are a no-op, not an error
    empty = (ctypes.c_int * 2)(0, 1000)
    assert f(None, None, capi.F32, empty, 2, 1, 0, 0.0, None, 0, None) == capi.OK


def test_workspace_queries_are_pure(lib):
    shape = (ctypes.c_int * 2)(64, 128256)
    a = lib.vkop_hip_softmax_topk_workspace_bytes(capi.F32, shape, 2, -1, 50)
    b = lib.vkop_hip_softmax_topk_workspace_bytes(capi.F32, shape, 2, -1, 50)
    assert a == b and a % 256 == 0
    assert lib.vkop_hip_softmax_topk_workspace_bytes(9, shape, 2, -1, 50) == 0


def test_timeline_summary_reads_a_log_of_two_lanes():
    """bench.py --timeline: the summary of a log made up here -- two lanes, each scan 8 us and pick 6 us with 2 us
    between them, the lanes half a call apart -- gives back those durations, gaps and the overlap."""
    import importlib.util
    import numpy as np
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    recs = []
    period = 18000  # ns per call of a lane: 8 + 2 + 6 + 2
    for lane, ws in enumerate((0x1000, 0x2000)):
        for call in range(40):
            s0 = 5_000_000 + lane * period // 2 + call * period
            for wg in (0, 16, 500):        # scan workgroups: enter together, the last leaves after 8 us
                recs.append(((wg << 40) | ws, (s0 + wg) // 10, (s0 + 7000 + 2 * wg) // 10))
            p0 = s0 + 8000 + 2000
            for wg in range(4):            # pick workgroups
                recs.append(((1 << 63) | (wg << 40) | ws, (p0 + wg) // 10, (p0 + 5000 + 250 * wg + (250 if wg == 3 else 0)) // 10))
    # (a warm-up stretch long before, which the summary leaves out)
    recs.append((0x1000, 100, 200))
    out = bench.timeline_summary(np.array(recs, dtype=np.uint64), 0.009, 2, 8)
    assert out["lanes_seen"] == 2
    assert abs(out["scan_kernel_us_first_entry_to_last_exit"]["mean"] - 8.0) < 0.05
    assert abs(out["pick_kernel_us_first_entry_to_last_exit"]["mean"] - 6.0) < 0.05
    assert abs(out["gap_us_scan_exit_to_pick_entry_same_lane"] - 2.0) < 0.05
    assert abs(out["gap_us_pick_exit_to_next_scan_entry_same_lane"] - 2.0) < 0.05
    assert abs(out["us_per_call_from_the_log"] - 9.0) < 0.05            # two lanes, 18 us a call each
    assert abs(out["mean_kernels_running"] - 2 * 14.0 / 18.0) < 0.05     # each lane busy 14 of 18 us


def test_route_planner_without_a_gpu(lib):
    """Which kernels a last-axis top-k / fused call takes is decided on the host (vkop_hip_measure_path: 4 one wave
    per row, 2 scan + pick, 3 scan + gather + rank, 1 chunk (+ merge), 0 radix select or general kernels;
    vkop_hip_rows_plan: threads, loads, chunks of the chunk kernel).  The five workloads' routes, the shape that a
    limit of 8192 blocks had left to the radix select, and the rule that no shape takes chunk + merge over SEVERAL
    chunks unless vkop_hip_tune asks for it."""
    F32, F16 = capi.F32, capi.F16
    assert capi.measure_path(F32, (1, 1000), -1, 5) == 4            # C1
    assert capi.measure_path(F32, (256, 1000), -1, 5) == 4          # C2
    assert capi.measure_path(F16, (256, 1000), -1, 5) == 4
    assert capi.measure_path(F32, (64, 128256), -1, 50) == 2        # C3
    assert capi.measure_path(F16, (64, 128256), -1, 50) == 2
    assert capi.measure_path(F32, (8, 262144), -1, 1024) == 3       # C4
    assert capi.measure_path(F32, (16, 8400), -1, 300) == 1         # C5's select: one workgroup a row
    assert capi.rows_plan(F32, (16, 8400), -1, 300)[2] == 1
    assert capi.measure_path(F32, (4, 1048576), -1, 100) == 2       # 16384 blocks a row
    assert capi.measure_path(F32, (1, 128256), -1, 50) == 2         # a single sequence's logits
    several = []
    for dt in (F32, F16):
        for rows in (1, 8, 16, 17, 64, 1024):
            for n in list(range(256, 40000, 997)) + [8192, 8193, 8320, 8321, 16384, 32768, 32769, 65536, 131072, 300000, 1 << 20]:
                for k in (1, 5, 32, 33, 64, 65, 100, 255, 256, 408, 511):
                    if k > n:
                        continue
                    if capi.measure_path(dt, (rows, n), -1, k) == 1 and capi.rows_plan(dt, (rows, n), -1, k)[2] > 1:
                        several.append((dt, rows, n, k))
    assert not several, several[:10]
    try:
        capi.tune("rows.path", 1)
        assert capi.measure_path(F32, (64, 128256), -1, 50) == 1 and capi.rows_plan(F32, (64, 128256), -1, 50)[2] > 1
    finally:
        capi.tune("rows.path", 0)
    # the workspace a call is told to bring covers the headline shape with room in the static scratch's 4 MiB
    need = capi.softmax_topk_workspace_bytes(F32, (64, 128256), -1, 50)
    assert 64 * 1024 < need <= 4 << 20
