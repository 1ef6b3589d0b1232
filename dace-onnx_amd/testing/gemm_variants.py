"""The k-contiguous fp32 GEMM (activations x [N, K] weights, bias epilogue) through the library's own choice and through
each forced form of the kernel, over a set of shapes.

    python -m dace_onnx_amd.testing.gemm_variants            # the four launches of the BERT-base layer and shapes around them
    python -m dace_onnx_amd.testing.gemm_variants rounds     # 3072-wide outputs of 512 to 3328 tiles of 128 x 48, K = 768 .. 4096

Prints microseconds per launch (HIP events around graph-recorded launches after a warm-up by time, as bench.py measures
its rows), the best of the forced forms and the ratio of the library's choice to it. The forms (``MI355X_GEMM_NT_*``):

* ``48 deep`` / ``48 lean``: 64 x 48 tiles by eight waves, 64-k tiles three deep / 32-k tiles three deep (three workgroups per CU);
* ``48 w16``: 64 x 48 tiles by 16 waves in four k-split groups (where K is a multiple of 64);
* ``64`` / ``96`` / ``144``: 64 x 64, 128 x 96 (16 waves) and 64 x 144 tiles;
* ``128 deep`` / ``128 lean``: 128 x 48 tiles with the six-deep ring (two workgroups per CU) / the three-deep one (three).

Every form is checked against float64 in tests/test_configs_gpu.py::test_k_contiguous_gemm_tiles_and_epilogues.
"""
import os
import sys

from .. import _lib
from .profiling import graph_time_us

VARIABLES = ("MI355X_GEMM_NT_BM", "MI355X_GEMM_NT_BN", "MI355X_GEMM_NT_PER_CU", "MI355X_GEMM_NT_WAVES", "MI355X_GEMM_NT_BK")
FORMS = (("library", {}),
         ("48 deep", {"MI355X_GEMM_NT_BN": "48", "MI355X_GEMM_NT_PER_CU": "2", "MI355X_GEMM_NT_WAVES": "8"}),
         ("48 lean", {"MI355X_GEMM_NT_BN": "48", "MI355X_GEMM_NT_PER_CU": "3", "MI355X_GEMM_NT_WAVES": "8"}),
         ("48 w16", {"MI355X_GEMM_NT_BN": "48", "MI355X_GEMM_NT_WAVES": "16"}),
         ("64", {"MI355X_GEMM_NT_BN": "64"}), ("96", {"MI355X_GEMM_NT_BN": "96"}), ("144", {"MI355X_GEMM_NT_BN": "144"}),
         ("128 deep", {"MI355X_GEMM_NT_BM": "128", "MI355X_GEMM_NT_BN": "48", "MI355X_GEMM_NT_PER_CU": "2"}),
         ("128 lean", {"MI355X_GEMM_NT_BM": "128", "MI355X_GEMM_NT_BN": "48", "MI355X_GEMM_NT_PER_CU": "3"}))


def shapes(which: str):
    if which == "rounds":
        return [(128 * m, 3072, K) for K in (768, 1536, 2048, 3072, 4096) for m in (8, 12, 14, 16, 18, 20, 24, 28, 32, 36, 40, 52)]
    out = []
    for K in (256, 768, 1536, 3072):
        for M, N in ((128, 768), (512, 768), (1024, 768), (1024, 1024), (512, 3072), (1024, 1536), (384, 4096), (2048, 768),
                     (1536, 1152), (1024, 2304), (1024, 3072), (2048, 2304), (4096, 1024), (4096, 4096)):
            out.append((M, N, K))
    return out


def main():
    import torch
    lib = _lib.library()
    st = _lib.current_stream
    which = sys.argv[1] if len(sys.argv) > 1 else "layer"

    def run(M, N, K, variables):
        for name in VARIABLES:
            os.environ.pop(name, None)
        os.environ.update(variables)
        lib.mi355x_reload_tuning()
        a, w = torch.randn(M, K, device="cuda"), torch.randn(N, K, device="cuda") * 0.05
        bias, out = torch.randn(N, device="cuda"), torch.empty(M, N, device="cuda")
        launch = lambda: lib.mi355x_gemm_f32(a.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(), None, 1, 1, M, N, K,
                                             _lib.i64_array([0, 0, K, 1]), _lib.i64_array([0, 0, 1, K]), _lib.i64_array([0, 0, N]),
                                             None, 1.0, _lib.EPI_BIAS, st())
        return min(graph_time_us(launch, reps=20) for _ in range(2))

    print(f"{'M x N x K':>18s} {'tiles 128x48':>12s} " + " ".join(f"{name:>9s}" for name, _ in FORMS) + "   library / best forced form")
    try:
        for M, N, K in shapes(which):
            times = [run(M, N, K, variables) for _, variables in FORMS]
            best = min(times[1:])
            tiles = ((M + 127) // 128) * ((N + 47) // 48)
            print(f"{M:6d}x{N:5d}x{K:5d} {tiles:12d} " + " ".join(f"{t:9.2f}" for t in times) +
                  f"   {times[0] / best:5.3f} ({FORMS[1 + times[1:].index(best)][0]}; {2.0 * M * N * K / times[0] / 1e6:5.1f} TFLOP/s)", flush=True)
    finally:
        for name in VARIABLES:
            os.environ.pop(name, None)
        lib.mi355x_reload_tuning()


if __name__ == "__main__":
    main()
