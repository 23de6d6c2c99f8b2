"""Small helpers with the reference's names (src/rten_cpp/utils.py)."""
import contextlib
from typing import Callable, List, Optional

import torch


@contextlib.contextmanager
def no_dispatch():
    guard = torch._C._DisableTorchDispatch()
    try:
        yield
    finally:
        del guard


def _test_memory(func: Callable, _iter: int = 10, quantiles: Optional[List[float]] = None, return_mode="mean"):
    """Peak device memory of ``func`` in MiB over ``_iter`` runs (utils.py:18-40)."""
    assert return_mode in ["min", "max", "mean", "median"]
    total_mem = []
    for _ in range(_iter):
        torch.cuda.reset_peak_memory_stats()
        func()
        total_mem.append(torch.cuda.max_memory_allocated() / 2**20)
    total_mem = torch.tensor(total_mem, dtype=torch.float)
    if quantiles is not None:
        q = torch.quantile(total_mem, torch.tensor(quantiles, dtype=torch.float)).tolist()
        return q[0] if len(q) == 1 else q
    return getattr(torch, return_mode)(total_mem).item()


def _tensor_mem(a: torch.Tensor) -> float:
    return a.element_size() * a.numel() / 2**20
