"""MatMulInteger on the benchmark shape (4096 x 3072, int8, zero points 3 / -2) through each form of the kernel.

    python -m dace_onnx_amd.testing.mmi_variants

Prints microseconds per launch (HIP events around graph-recorded launches, as bench.py measures its rows) at K = 768 and
K = 3072 and the slope between the two, i.e. the time one 64-k step of the whole problem takes, for

* ``stream``: the persistent kernel, 128 x 128 tiles, three workgroups per CU (``MI355X_MMI_TILE`` unset picks it at K = 768);
* ``tile 128`` / ``tile 256``: one 128 x 128 or 256 x 192 tile per workgroup, both operands through LDS;
* ``tile 128, A direct`` / ``tile 256, A direct``: the same two with A read from global memory straight into the MFMA
  operand registers (only B goes through LDS) -- the layout that halves the LDS bytes per step and loses to the vector
  memory pipe: a load whose neighbouring lanes touch different rows is taken at one row per cycle.

Every variant is bit-exact (tests/test_configs_gpu.py::test_forced_matmul_integer_variants).
"""
import os

from .. import _lib
from .profiling import graph_time_us

VARIANTS = (("stream (3 workgroups per CU)", "1"), ("tile 128", "128"), ("tile 256", "256"),
            ("tile 128, A direct", "129"), ("tile 256, A direct", "257"))


def main():
    import torch
    lib = _lib.library()
    st = _lib.current_stream
    M, N = 4096, 3072
    rows = {}
    for K in (768, 3072):
        a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda")
        b = torch.randint(-128, 128, (K, N), dtype=torch.int8, device="cuda")
        y = torch.empty(M, N, dtype=torch.int32, device="cuda")
        za, zb = torch.tensor([3], dtype=torch.int8, device="cuda"), torch.tensor([-2], dtype=torch.int8, device="cuda")
        with_zp = lambda: lib.mi355x_matmul_integer_i8(a.data_ptr(), b.data_ptr(), za.data_ptr(), zb.data_ptr(), y.data_ptr(), M, N, K, st())
        without = lambda: lib.mi355x_matmul_integer_i8(a.data_ptr(), b.data_ptr(), None, None, y.data_ptr(), M, N, K, st())
        for name, tile in VARIANTS:
            os.environ["MI355X_MMI_TILE"] = tile   # 1: none of the tile kernels, i.e. the persistent one at any K
            lib.mi355x_reload_tuning()
            rows.setdefault(name, {})[K] = (graph_time_us(with_zp, reps=20), graph_time_us(without, reps=20))
    os.environ.pop("MI355X_MMI_TILE", None)
    lib.mi355x_reload_tuning()
    print(f"{'variant':32s} {'K=768 zp':>9s} {'no zp':>7s} {'K=3072 zp':>10s} {'no zp':>7s} {'us per 64-k step (zp)':>22s}")
    for name, _ in VARIANTS:
        (z1, n1), (z2, n2) = rows[name][768], rows[name][3072]
        print(f"{name:32s} {z1:9.2f} {n1:7.2f} {z2:10.2f} {n2:7.2f} {(z2 - z1) / 36.0:22.3f}")


if __name__ == "__main__":
    main()
