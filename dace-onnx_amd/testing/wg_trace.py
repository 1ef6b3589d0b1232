"""Where a contraction kernel's time goes, workgroup by workgroup.

``make -C dace-onnx_amd/csrc trace`` builds ``libmi355x_onnx_trace.so``: the library with wall-clock stamps compiled
into the convolution, k-contiguous GEMM and MatMulInteger kernels (start of a workgroup, first and last step of its
main loop, end of the workgroup, hardware id of its CU). This script runs one of the benchmark shapes through that
build and prints the phases; the package itself never loads the trace build.

    python -m dace_onnx_amd.testing.wg_trace conv4 | mmi5 | qkv | out | ffn1 | ffn2 | out_ksplit | ffn2_ksplit

What the stamps mean per kernel (microseconds; the wall clock ticks at 100 MHz):

* slot 0 start, slot 1 main loop entered (first operands arrived), slot 2 main loop left (by the first wave),
  slot 3 last store issued -- for MatMulInteger: last store acknowledged; the shader cycle counter at the same two
  points of the loop gives the clock the loop ran at (the part lowers it under load: 2.3-2.4 GHz in the fp32 loops,
  1.6 GHz in MatMulInteger's);
* workgroups are grouped by CU through the hardware id register to show which of them share a CU and when each of
  them was in its loop;
* the convolution adds six more, printed after the workgroup's number in the per-CU list: set-up done (first
  barrier), first six steps' loads issued, their first two stored to LDS; after the loop: partial sums of the
  second k-split group exchanged, added, bias arrived (-1 where a kernel has no such stamp).
"""
import ctypes
import os
import sys

import numpy as np

from .. import _lib

TRACE_LIBRARY = os.path.join(os.path.dirname(_lib.LIBRARY_PATH), "libmi355x_onnx_trace.so")
WORDS = 16   # 64-bit words per workgroup in the trace buffer


def load_trace_library():
    if not os.path.exists(TRACE_LIBRARY):
        raise _lib.LibraryNotBuilt(f"{TRACE_LIBRARY} is missing: run `make -C dace-onnx_amd/csrc trace`")
    lib = ctypes.CDLL(TRACE_LIBRARY)
    for name, (restype, argtypes) in _lib.SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    return lib


def _workloads(lib, torch):
    st = _lib.current_stream
    ones, pads = _lib.i64_array([1, 1]), _lib.i64_array([1, 1, 1, 1])

    def conv4():
        x = torch.randn(32, 64, 56, 56, device="cuda")
        w = torch.randn(64, 64, 3, 3, device="cuda") * (2.0 / 576) ** 0.5
        b, y = torch.zeros(64, device="cuda"), torch.empty(32, 64, 56, 56, device="cuda")
        return (lambda: lib.mi355x_conv2d_f32(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 32, 64, 56, 56, 64, 3, 3,
                                              pads, ones, ones, 3, st())), (x, w, b, y)

    def mmi5():
        a = torch.randint(-128, 128, (4096, 768), dtype=torch.int8, device="cuda")
        b = torch.randint(-128, 128, (768, 3072), dtype=torch.int8, device="cuda")
        y = torch.empty(4096, 3072, dtype=torch.int32, device="cuda")
        za, zb = torch.tensor([3], dtype=torch.int8, device="cuda"), torch.tensor([-2], dtype=torch.int8, device="cuda")
        return (lambda: lib.mi355x_matmul_integer_i8(a.data_ptr(), b.data_ptr(), za.data_ptr(), zb.data_ptr(), y.data_ptr(),
                                                     4096, 3072, 768, st())), (a, b, y, za, zb)

    def gemm(M, N, K, epi):
        def make():
            a, w = torch.randn(M, K, device="cuda"), torch.randn(N, K, device="cuda") * 0.05
            bias, res, out = torch.randn(N, device="cuda"), torch.randn(M, N, device="cuda"), torch.empty(M, N, device="cuda")
            return (lambda: lib.mi355x_gemm_f32(a.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(), res.data_ptr(), 1, 1,
                                                M, N, K, _lib.i64_array([0, 0, K, 1]), _lib.i64_array([0, 0, 1, K]),
                                                _lib.i64_array([0, 0, N]), _lib.i64_array([0, 0, N]), 1.0, epi, st())), (a, w, bias, res, out)
        return make

    def ksplit(make):   # the same GEMM through the kernel whose eight waves split K (MI355X_GEMM_KSPLIT=1)
        def wrapped():
            os.environ["MI355X_GEMM_KSPLIT"] = "1"
            lib.mi355x_reload_tuning()
            return make()
        return wrapped

    return {"conv4": conv4, "mmi5": mmi5, "qkv": gemm(1024, 2304, 768, 1), "out": gemm(1024, 768, 768, 9),
            "ffn1": gemm(1024, 3072, 768, 5), "ffn2": gemm(1024, 768, 3072, 9),
            "out_ksplit": ksplit(gemm(1024, 768, 768, 9)), "ffn2_ksplit": ksplit(gemm(1024, 768, 3072, 9))}


def trace(name: str, warm_seconds: float = 0.3, max_workgroups: int = 65536):
    """Runs workload ``name`` once with stamps (after ``warm_seconds`` of launches without) and returns the stamps in
    microseconds relative to the first workgroup's start, ``[workgroups, 4]``, and the CU key of each workgroup."""
    import time
    import torch
    lib = load_trace_library()
    launch, keep = _workloads(lib, torch)[name]()
    os.environ.pop("MI355X_WG_TRACE_BUFFER", None)
    # The shader clock comes up with the time the part has been busy, not with the number of launches: after 500
    # launches of a 13 us kernel (7 ms) its loop still reads 2.0 GHz, after 100 ms 2.3-2.4 GHz.
    deadline = time.perf_counter() + warm_seconds
    while time.perf_counter() < deadline:
        for _ in range(200):
            launch()
        torch.cuda.synchronize()
    buf = torch.zeros(WORDS * max_workgroups, dtype=torch.int64, device="cuda")
    os.environ["MI355X_WG_TRACE_BUFFER"] = str(buf.data_ptr())
    os.environ["MI355X_WG_TRACE_CAPACITY"] = str(max_workgroups)   # workgroups beyond it write no stamps
    try:
        status = launch()
        torch.cuda.synchronize()
    finally:
        os.environ.pop("MI355X_WG_TRACE_BUFFER", None)
        os.environ.pop("MI355X_WG_TRACE_CAPACITY", None)
    if status != 0:
        raise _lib.MI355XError(lib.mi355x_last_error().decode())
    d = buf.cpu().numpy().reshape(-1, WORDS)
    d = d[d[:, 0] != 0]
    t = (d[:, :4] - d[:, 0].min()).astype(np.float64) / 100.0
    extra = np.where(d[:, 5:11] != 0, d[:, 5:11] - d[:, 0].min(), -100).astype(np.float64) / 100.0   # kernel-specific stamps
    trace.extra = extra
    trace.raw = d.astype(np.float64)
    hw, xcc = d[:, 4] & 0xffffffff, d[:, 4] >> 32
    key = (xcc & 0xf) * 1000 + ((hw >> 13) & 7) * 100 + ((hw >> 12) & 1) * 20 + ((hw >> 8) & 0xf)
    del keep
    return t, key


def report(name: str):
    t, key = trace(name)
    pct = lambda v: " / ".join(f"{x:.2f}" for x in np.percentile(v, [10, 50, 90]))
    print(f"{name}: {len(t)} workgroups on {len(set(key.tolist()))} CUs; times in us as p10 / median / p90")
    print(f"  start after the first workgroup's   {pct(t[:, 0])}   (last one: {t[:, 0].max():.2f})")
    print(f"  start -> main loop                  {pct(t[:, 1] - t[:, 0])}")
    print(f"  main loop                           {pct(t[:, 2] - t[:, 1])}")
    print(f"  main loop left -> end               {pct(t[:, 3] - t[:, 2])}")
    print(f"  last workgroup ends at              {t[:, 3].max():.2f}")
    cycles = trace.raw[:, 13] - trace.raw[:, 12]   # the shader cycle counter at the loop's start and end
    print(f"  shader clock inside the loop        {pct(cycles / ((t[:, 2] - t[:, 1]) * 1e3))} GHz")
    by_cu = {}
    for i in range(len(t)):
        by_cu.setdefault(int(key[i]), []).append(tuple(round(float(v), 2) for v in t[i]) + (i,) + tuple(round(float(v), 2) for v in trace.extra[i]))
    first = sorted(by_cu[int(key[0])])
    print(f"  the CU of workgroup 0 ran (start, loop entered, loop left, end, workgroup): {first}")


if __name__ == "__main__":
    report(sys.argv[1] if len(sys.argv) > 1 else "conv4")
