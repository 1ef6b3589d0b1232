"""The four GEMM launches of the BERT-base encoder layer under different tile walks.

    python -m dace_onnx_amd.testing.gemm_tile_order                 # microseconds per launch and walk
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir> -o p -- python3 -m dace_onnx_amd.testing.gemm_tile_order --dispatch 3
                                                                    # the same launches, three of each in a fixed order, for the counters

``MI355X_GEMM_GROUP_M`` sets the height, in tile rows, of the panels an XCD's slab of tiles is walked in (the library's
own choice makes the block of tiles resident on an XCD about square in operand bytes); ``MI355X_GEMM_CONFIG`` sends the
problem to the generic kernel, which stages both operands through LDS; ``MI355X_GEMM_KSPLIT=1`` to the kernel whose eight
waves split K (``csrc/gemm_f32_ksplit.hip``). With ``--dispatch n`` every combination is
launched ``n`` times back to back, in the order printed, so that a per-dispatch counter file can be read by position.
"""
import argparse
import os

from .. import _lib
from .profiling import graph_time_us

SHAPES = (("qkv", 1024, 2304, 768, 1), ("out", 1024, 768, 768, 9), ("ffn1", 1024, 3072, 768, 5), ("ffn2", 1024, 768, 3072, 9))
WALKS = (("library", {}), ("group_m 1", {"MI355X_GEMM_GROUP_M": "1"}), ("group_m 2", {"MI355X_GEMM_GROUP_M": "2"}),
         ("group_m 3", {"MI355X_GEMM_GROUP_M": "3"}), ("group_m 4", {"MI355X_GEMM_GROUP_M": "4"}),
         ("group_m 6", {"MI355X_GEMM_GROUP_M": "6"}), ("group_m 8", {"MI355X_GEMM_GROUP_M": "8"}),
         ("group_m 16", {"MI355X_GEMM_GROUP_M": "16"}),
         ("k split over 8 waves, 32x96 tiles, 32x32x2 MFMA", {"MI355X_GEMM_KSPLIT": "1"}),
         ("generic 64x48 (both operands through LDS)", {"MI355X_GEMM_CONFIG": "2"}),
         ("generic 128x128 (both operands through LDS)", {"MI355X_GEMM_CONFIG": "0"}))


def main():
    import torch
    ap = argparse.ArgumentParser()
    ap.add_argument("--dispatch", type=int, default=0, help="launch every combination this many times, untimed, in the order printed")
    args = ap.parse_args()
    lib = _lib.library()
    st = _lib.current_stream
    index = 0
    for name, M, N, K, epi in SHAPES:
        a, w = torch.randn(M, K, device="cuda"), torch.randn(N, K, device="cuda") * 0.05
        bias, res, out = torch.randn(N, device="cuda"), torch.randn(M, N, device="cuda"), torch.empty(M, N, device="cuda")
        launch = lambda: lib.mi355x_gemm_f32(a.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(), res.data_ptr(), 1, 1, M, N, K,
                                             _lib.i64_array([0, 0, K, 1]), _lib.i64_array([0, 0, 1, K]), _lib.i64_array([0, 0, N]),
                                             _lib.i64_array([0, 0, N]), 1.0, epi, st())
        for walk, variables in WALKS:
            for key in ("MI355X_GEMM_GROUP_M", "MI355X_GEMM_CONFIG", "MI355X_GEMM_KSPLIT"):
                os.environ.pop(key, None)
            os.environ.update(variables)
            lib.mi355x_reload_tuning()
            if args.dispatch:
                for _ in range(args.dispatch):
                    _lib.check(launch(), "gemm")
                torch.cuda.synchronize()
                print(f"dispatches {index} .. {index + args.dispatch - 1}: {name} {M}x{N}x{K}, {walk}", flush=True)
                index += args.dispatch
            else:
                print(f"{name:5s} {M}x{N}x{K:<5d} {walk:46s} {graph_time_us(launch, reps=20):8.2f} us", flush=True)
    for key in ("MI355X_GEMM_GROUP_M", "MI355X_GEMM_CONFIG", "MI355X_GEMM_KSPLIT"):
        os.environ.pop(key, None)
    lib.mi355x_reload_tuning()


if __name__ == "__main__":
    main()
