"""
Helpers shared by the estimator classes (role of python/culsh/utils.py in the reference).

Device arrays come from PyTorch-ROCm (its tensors expose ``__cuda_array_interface__``);
cupy arrays and cupyx CSR matrices are accepted too when cupy is installed, but cupy is
never required.
"""

from __future__ import annotations

import logging
import random
from typing import Any, Optional

import numpy as np
import scipy.sparse


def resolve_seed(seed: Optional[int]) -> int:
    """None -> a fresh random seed in [0, 2^63), anything else is returned as is
    (python/culsh/utils.py:15-19)."""
    return random.randint(0, 2**63 - 1) if seed is None else seed


def _torch():
    import torch

    return torch


def is_torch_tensor(arr: Any) -> bool:
    return type(arr).__module__.split(".")[0] == "torch" and hasattr(arr, "data_ptr")


def _is_cupyx_csr(arr: Any) -> bool:
    return type(arr).__module__.startswith("cupyx") and type(arr).__name__ == "csr_matrix"


_TORCH_TO_NUMPY = {"torch.float32": np.float32, "torch.float64": np.float64, "torch.float16": np.float16,
                   "torch.int32": np.int32, "torch.int64": np.int64}


def get_array_info(arr: Any) -> tuple[int, int, np.dtype]:
    """(rows, cols, numpy dtype) of a 2-D dense or CSR input; ValueError unless 2-D
    (python/culsh/utils.py:22-31)."""
    if arr.ndim != 2:
        raise ValueError(f"Expected 2D array, got {arr.ndim}D")
    dtype = arr.dtype
    if is_torch_tensor(arr):
        dtype = np.dtype(_TORCH_TO_NUMPY.get(str(arr.dtype), np.void))
    return int(arr.shape[0]), int(arr.shape[1]), np.dtype(dtype)


class DeviceCSR:
    """Device-resident CSR structure (column ids and row pointers only; MinHash ignores the
    values)."""

    def __init__(self, indices, indptr, shape):
        self.indices = indices
        self.indptr = indptr
        self.shape = tuple(shape)
        self.ndim = 2

    @property
    def dtype(self):
        return np.dtype(np.float32)


def ensure_device_array(arr: Any):
    """Dense input -> C-contiguous device array; CSR input -> device CSR structure.  Host
    data is copied to the current GPU (python/culsh/utils.py:34-53)."""
    torch = _torch()
    if isinstance(arr, DeviceCSR) or _is_cupyx_csr(arr):
        return arr
    if scipy.sparse.issparse(arr):
        csr = arr.tocsr() if not scipy.sparse.isspmatrix_csr(arr) else arr
        return DeviceCSR(torch.from_numpy(np.ascontiguousarray(csr.indices)).cuda(),
                         torch.from_numpy(np.ascontiguousarray(csr.indptr)).cuda(), csr.shape)
    if is_torch_tensor(arr):
        if not arr.is_cuda:
            arr = arr.cuda()
        return arr if arr.is_contiguous() else arr.contiguous()
    if hasattr(arr, "__cuda_array_interface__"):  # cupy or another device array library
        if not arr.flags.c_contiguous:
            import cupy as cp

            return cp.ascontiguousarray(arr)
        return arr
    return torch.from_numpy(np.ascontiguousarray(arr)).cuda()


def compute_recall(lsh_indices, gt_indices) -> float:
    """|candidates ∩ ground truth| / |ground truth| (python/culsh/utils.py:56-67)."""
    if len(gt_indices) == 0:
        return 0.0
    to_np = lambda a: a.detach().cpu().numpy() if is_torch_tensor(a) else (a.get() if hasattr(a, "get") else np.asarray(a))
    return len(np.intersect1d(to_np(lsh_indices), to_np(gt_indices))) / len(gt_indices)


def get_logger(instance: object) -> logging.Logger:
    """Per-class INFO logger writing to stderr; the handler is attached once per class."""
    logger = logging.getLogger(instance.__class__.__name__)
    logger.setLevel(logging.INFO)
    if not logger.handlers:
        handler = logging.StreamHandler()
        handler.setFormatter(logging.Formatter("%(asctime)s [%(name)s] %(levelname)s: %(message)s",
                                               datefmt="%Y-%m-%d %H:%M:%S"))
        logger.addHandler(handler)
    return logger
