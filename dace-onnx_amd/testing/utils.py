"""Comparison helpers with the reference's tolerances (``daceml/testing/utils.py:6-37``)."""
import typing

import numpy as np
import torch


def torch_tensors_close(name, torch_v, dace_v, rtol=1e-5, atol=1e-4):
    """Assert that the two torch tensors are close; print the offending elements if not."""
    torch_v, dace_v = torch_v.detach().cpu(), dace_v.detach().cpu()
    if not torch.allclose(torch_v, dace_v, rtol=rtol, atol=atol, equal_nan=True):
        diff = torch.abs(dace_v - torch_v)
        failed = diff > atol + rtol * torch.abs(dace_v)
        print(f"{name} was not close: max |diff| {diff.max().item():.3e}, "
              f"{int(failed.sum())} of {failed.numel()} elements outside atol={atol} rtol={rtol}")
        for x, y, _ in zip(torch_v[failed], dace_v[failed], range(20)):
            print(f"  expected {x.item():.8e} got {y.item():.8e} |diff| {abs(x - y).item():.3e} "
                  f"allowed {atol + rtol * abs(y).item():.3e}")
        assert False, f"{name} was not close"


def max_rel_error(expected, actual) -> float:
    """max |actual - expected| / max |expected| in float64: the "1e-4 relative" of the fp32 kernels."""
    e = np.asarray(expected, dtype=np.float64)
    a = np.asarray(actual, dtype=np.float64)
    scale = np.abs(e).max() if e.size else 1.0
    return float(np.abs(a - e).max() / (scale if scale > 0 else 1.0)) if e.size else 0.0


T = typing.TypeVar("T")


def copy_to_gpu(gpu: bool, tensor: T) -> T:
    return tensor.cuda() if gpu else tensor
