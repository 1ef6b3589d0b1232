"""Conv + bias + Relu through the library's own choice and through the other forms of the gather kernel, over the 3 x 3 and
1 x 1 layers of a ResNet-50 at 8 and 32 images.

    python -m dace_onnx_amd.testing.conv_variants

Prints microseconds per launch (HIP events around graph-recorded launches after a warm-up by time, as bench.py measures
its rows) for

* ``library``: 64-position tiles through the lean kernel (three-deep register ring, three workgroups per CU);
* ``six-deep``: the same tiles through the six-deep ring, two workgroups per CU (``MI355X_CONV_PER_CU=2``);
* ``wide``: 128-position tiles, one workgroup per CU (``MI355X_CONV_GATHER_BN=128``).

The three add up the same products in the same order: the results are compared bit for bit here as well.
"""
import os

from .. import _lib
from .profiling import graph_time_us

VARIABLES = ("MI355X_CONV_PER_CU", "MI355X_CONV_GATHER_BN")
FORMS = (("library", {}), ("six-deep", {"MI355X_CONV_PER_CU": "2"}), ("wide", {"MI355X_CONV_GATHER_BN": "128"}))
LAYERS = ((64, 56, 64, 3), (128, 28, 128, 3), (256, 14, 256, 3), (512, 7, 512, 3), (64, 56, 256, 1), (256, 56, 64, 1), (256, 56, 128, 1),
          (512, 28, 128, 1), (1024, 14, 256, 1), (2048, 7, 512, 1), (512, 7, 2048, 1), (128, 28, 512, 1))   # C, H = W, M, k


def main():
    import torch
    lib = _lib.library()
    st = _lib.current_stream
    ones = _lib.i64_array([1, 1])

    def run(N, C, H, M, k, variables):
        for name in VARIABLES:
            os.environ.pop(name, None)
        os.environ.update(variables)
        lib.mi355x_reload_tuning()
        g = torch.Generator(device="cuda").manual_seed(1)
        x = torch.randn(N, C, H, H, device="cuda", generator=g)
        w = torch.randn(M, C, k, k, device="cuda", generator=g) * (2.0 / (C * k * k)) ** 0.5
        b = torch.randn(M, device="cuda", generator=g)
        y = torch.full((N, M, H, H), float("nan"), device="cuda")
        pads = _lib.i64_array([k // 2] * 4)
        launch = lambda: lib.mi355x_conv2d_f32(x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), N, C, H, H, M, k, k, pads, ones, ones,
                                               _lib.EPI_BIAS | _lib.EPI_RELU, st())
        _lib.check(launch(), "conv2d")
        torch.cuda.synchronize()
        return min(graph_time_us(launch, reps=20) for _ in range(2)), y.clone()

    print(f"{'images x C x H x W -> M, filter':>34s} {'tiles':>6s} " + " ".join(f"{name:>9s}" for name, _ in FORMS) + "   TFLOP/s  library / best  same bits")
    try:
        for N in (8, 32):
            for C, H, M, k in LAYERS:
                results = [run(N, C, H, M, k, variables) for _, variables in FORMS]
                times = [t for t, _ in results]
                same = all(bool(torch.equal(results[0][1], y)) for _, y in results[1:])
                tiles = ((M + 63) // 64) * ((N * H * H + 63) // 64)
                flop = 2.0 * N * M * H * H * C * k * k
                print(f"{N:3d} x {C:4d} x {H:2d} x {H:2d} -> {M:4d}, {k} x {k}    {tiles:6d} " + " ".join(f"{t:9.2f}" for t in times) +
                      f"   {flop / times[0] / 1e6:7.1f}  {times[0] / min(times):14.3f}  {same}", flush=True)
    finally:
        for name in VARIABLES:
            os.environ.pop(name, None)
        lib.mi355x_reload_tuning()


if __name__ == "__main__":
    main()
