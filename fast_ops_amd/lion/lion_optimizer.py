"""Fused Lion optimizer for MI355X: drop-in for ``fast_ops.lion.lion_optimizer.Lion``.

Same constructor, validation, state key and ``step()`` semantics as the reference class
(fast_ops/lion/lion_optimizer.py:29-76); the arithmetic is that of the reference formula
(fast_ops/lion/lion_optimizer_ref.py:51,64,65,67) under PyTorch's type promotion, for parameters/gradients and
momenta in fp32, fp16 or bf16 (fp32 parameters with a bf16 momentum is the tuned path).

What differs from the reference, on purpose:

* one kernel launch per parameter group instead of one per parameter (lion_optimizer.py:64-76 launches per tensor):
  the tensors of a group are cut into 8192-element chunks whose descriptors live in a device table that is rebuilt
  only when a parameter, gradient or momentum pointer changes;
* the reference kernel requires one half dtype for all three tensors (lion_update.cu:132-135); here parameter and
  momentum dtypes are independent. Freshly created momentum is bf16 for fp32 parameters (the paper's choice) and
  ``zeros_like(param)`` for half parameters (lion_optimizer.py:68-73) unless ``exp_avg_dtype`` says otherwise;
* the six scalar constants are computed here in Python double precision and rounded once to fp32, which is what the
  reference formula's Python expressions do.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Iterable, List, Optional, Tuple

import numpy as np
import torch
from torch import Tensor
from torch.nn import Parameter
from torch.optim.optimizer import Optimizer

from .. import _lib

_CHUNK_DTYPE = np.dtype([("p", "<u8"), ("g", "<u8"), ("m", "<u8"), ("n", "<i4"), ("reserved", "<i4")])
assert _CHUNK_DTYPE.itemsize == ctypes.sizeof(_lib.FoLionChunk) == 32


def _dense_same_layout(a: Tensor, *others: Tensor) -> bool:
    """True when `a` is non-overlapping and dense and the others share its strides exactly (element i of one is
    element i of the others in memory order). The reference checks density only (lion_update.cu:109-112,137-139)."""
    if any(o.shape != a.shape or o.stride() != a.stride() for o in others):
        return False
    if a.is_contiguous():
        return True
    expect = 1
    for size, stride in sorted(((s, st) for s, st in zip(a.shape, a.stride()) if s != 1), key=lambda x: x[1]):
        if stride != expect:
            return False
        expect *= size
    return True


_DTYPE_CODE = {torch.float32: _lib.FO_DTYPE_F32, torch.float16: _lib.FO_DTYPE_F16, torch.bfloat16: _lib.FO_DTYPE_BF16}


def make_consts(lr: float, betas: Tuple[float, float], weight_decay: float,
                p_dtype: torch.dtype = torch.float32, m_dtype: torch.dtype = torch.bfloat16) -> "_lib.FoLionConsts":
    c = _lib.FoLionConsts()
    _lib.check(_lib.load().fo_lion_make_consts_typed(float(lr), float(betas[0]), float(betas[1]), float(weight_decay),
                                                     _DTYPE_CODE[p_dtype], _DTYPE_CODE[m_dtype], ctypes.byref(c)),
               "fo_lion_make_consts_typed")
    return c


def build_chunk_table(ptrs: List[Tuple[int, int, int, int]], p_size: int = 4, m_size: int = 2) -> np.ndarray:
    """(p_ptr, g_ptr, m_ptr, numel) per tensor -> structured array of fo_lion_chunk descriptors; p_size / m_size are
    the element sizes of parameters (and gradients) and of the momentum."""
    C = _lib.FO_LION_CHUNK
    # all tensors at once (a rebuild happens whenever a gradient comes back at another address, and a Python loop over
    # the tensors took 3 ms for the 148 tensors of GPT-2-small)
    arr = np.array([t for t in ptrs if t[3] != 0], dtype=np.uint64).reshape(-1, 4)
    numel = arr[:, 3].astype(np.int64)
    n = (numel + (C - 1)) // C                                  # chunks per tensor
    total = int(n.sum())
    t = np.zeros(total, dtype=_CHUNK_DTYPE)
    if total == 0:
        return t
    first = np.cumsum(n) - n                                    # index of each tensor's first chunk
    off = (np.arange(total, dtype=np.int64) - np.repeat(first, n)) * C      # element offset of the chunk in its tensor
    off_u = off.astype(np.uint64)
    t["p"] = np.repeat(arr[:, 0], n) + off_u * np.uint64(p_size)
    t["g"] = np.repeat(arr[:, 1], n) + off_u * np.uint64(p_size)
    t["m"] = np.repeat(arr[:, 2], n) + off_u * np.uint64(m_size)
    t["n"] = np.minimum(C, np.repeat(numel, n) - off).astype(np.int32)
    return t


def lion_update(param: Tensor, grad: Tensor, exp_avg: Tensor, lr: float, beta1: float, beta2: float, weight_decay: float) -> None:
    """Single-tensor in-place update: the call the reference extension exposes (fast_ops/lion/lion.cpp:4-15)."""
    _check_tensors(param, grad, exp_avg)
    c = make_consts(lr, (beta1, beta2), weight_decay, param.dtype, exp_avg.dtype)
    with torch.cuda.device(param.device):
        stream = torch.cuda.current_stream(param.device).cuda_stream
        _lib.check(
            _lib.load().fo_lion_update_typed(param.data_ptr(), grad.data_ptr(), exp_avg.data_ptr(), param.numel(),
                                             _DTYPE_CODE[param.dtype], _DTYPE_CODE[exp_avg.dtype], ctypes.byref(c), stream),
            "fo_lion_update_typed",
        )


def _check_tensors(param: Tensor, grad: Tensor, exp_avg: Tensor) -> None:
    if not (param.is_cuda and grad.is_cuda and exp_avg.is_cuda):
        raise RuntimeError("fused Lion runs on the GPU only: parameters, gradients and momentum must be device tensors")
    if not (param.device == grad.device == exp_avg.device):
        raise RuntimeError("parameter, gradient and momentum must live on the same device")
    if param.dtype not in _DTYPE_CODE or exp_avg.dtype not in _DTYPE_CODE or grad.dtype != param.dtype:
        raise RuntimeError(
            f"unsupported dtypes (param {param.dtype}, grad {grad.dtype}, exp_avg {exp_avg.dtype}): parameters and momentum "
            "may each be float32, float16 or bfloat16, and the gradient has the parameter's dtype (lion_update.cu:132)"
        )
    if grad.is_sparse:
        raise RuntimeError("Lion does not support sparse gradients")
    if not _dense_same_layout(param, grad, exp_avg):
        raise RuntimeError("expected tensor to be contiguous")   # message of lion_update.cu:109-112


class Lion(Optimizer):
    """Lion optimizer ("Symbolic Discovery of Optimization Algorithms", https://arxiv.org/abs/2302.06675), fused."""

    def __init__(
        self,
        params: Iterable[Parameter],
        lr: float = 1e-4,
        betas: Tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 0.0,
        *,
        exp_avg_dtype: Optional[torch.dtype] = None,
    ) -> None:
        """
        :param params: iterable of parameters to optimize or dicts defining parameter groups
        :param lr: learning rate
        :param betas: coefficients of the update interpolation and of the momentum decay
        :param weight_decay: decoupled weight decay coefficient
        :param exp_avg_dtype: dtype of momentum buffers this optimizer creates (state loaded or seeded by the caller
          keeps its own dtype). None: bfloat16 for float32 parameters, the parameter's dtype otherwise
        """
        # same checks, exception type and messages as lion_optimizer.py:49-52
        if lr <= 0:
            raise RuntimeError(f"expected positive LR, got {lr}")
        if not all(0 <= beta <= 1 for beta in betas):
            raise RuntimeError(f"betas must be between 0 and 1. got {betas}")
        if exp_avg_dtype is not None and exp_avg_dtype not in _DTYPE_CODE:
            raise RuntimeError(f"exp_avg_dtype {exp_avg_dtype} is not implemented: float32, float16 or bfloat16")
        defaults = {"lr": lr, "betas": betas, "weight_decay": weight_decay}
        super().__init__(params, defaults)
        self._exp_avg_dtype = exp_avg_dtype
        # (group index, device, parameter dtype, momentum dtype) -> _Table
        self._tables: Dict[tuple, "_Table"] = {}
        # per parameter: [gradient object, momentum object, (device, parameter dtype, momentum dtype), (p, g, m pointers, numel)]
        # of the last step; a parameter whose gradient and momentum are still those objects needs no checks and no
        # pointer queries (148 tensors: 0.3 ms of host time per step otherwise)
        self._seen: Dict[Parameter, list] = {}
        _lib.load()   # fail at construction, not at the first step, when the library is missing

    def load_state_dict(self, state_dict) -> None:
        """As torch's, except that a loaded momentum keeps the dtype it was saved with. torch casts floating-point
        state to the parameter's dtype, which would silently turn the bf16 momentum of fp32 parameters into fp32
        after a resume: other rounding points (the trajectory would differ from an uninterrupted run) and 20 instead
        of 16 bytes per parameter. A checkpoint written by the reference optimizer (momentum in the parameter's dtype,
        lion_optimizer.py:68-73) loads as it is."""
        super().load_state_dict(state_dict)
        saved_state = state_dict["state"]
        for saved_group, group in zip(state_dict["param_groups"], self.param_groups):
            for pid, param in zip(saved_group["params"], group["params"]):
                saved = saved_state.get(pid)
                if saved is None or "exp_avg" not in saved or param not in self.state:
                    continue
                want = saved["exp_avg"].dtype
                if self.state[param]["exp_avg"].dtype != want:
                    self.state[param]["exp_avg"] = saved["exp_avg"].to(device=param.device, dtype=want, copy=True)
        self._seen.clear()

    @torch.no_grad()
    def step(self) -> None:
        """Parameter and state (momentum) update: one fused launch per parameter group and device."""
        lib = _lib.load()
        seen = self._seen
        for gi, group in enumerate(self.param_groups):
            lr = group["lr"]
            weight_decay = group["weight_decay"]
            beta1, beta2 = group["betas"]
            # one launch per (device, parameter dtype, momentum dtype)
            buckets: Dict[Tuple[torch.device, torch.dtype, torch.dtype], List[Tuple[int, int, int, int]]] = {}
            for param in group["params"]:
                grad: Optional[Tensor] = param.grad
                if grad is None:
                    continue
                rec = seen.get(param)
                same_p_m = (rec is not None and rec[1] is self.state[param].get("exp_avg")
                            and rec[3][0] == param.data_ptr() and rec[3][2] == rec[1].data_ptr())
                if same_p_m and rec[0] is grad and rec[3][1] == grad.data_ptr():
                    # same gradient and momentum objects over the same memory as last step (gradients accumulated in
                    # place): dtypes, devices and layouts cannot have changed, the checks need not be repeated
                    bucket, entry = rec[2], rec[3]
                elif (same_p_m and grad.dtype == param.dtype and grad.device == param.device and not grad.is_sparse
                      and grad.shape == param.shape and grad.stride() == param.stride()):
                    # a new gradient tensor for an unchanged parameter and momentum (zero_grad(set_to_none=True), torch's
                    # default, makes one every step): only the gradient needs looking at, against the parameter it was
                    # checked with before
                    bucket = rec[2]
                    entry = (rec[3][0], grad.data_ptr(), rec[3][2], rec[3][3])
                    rec[0], rec[3] = grad, entry
                else:
                    state = self.state[param]
                    if "exp_avg" not in state:
                        # exponential moving average of the gradient (lion_optimizer.py:68-73)
                        dt = self._exp_avg_dtype or (torch.bfloat16 if param.dtype == torch.float32 else param.dtype)
                        state["exp_avg"] = torch.zeros_like(param, dtype=dt, memory_format=torch.preserve_format)
                    exp_avg: Tensor = state["exp_avg"]
                    _check_tensors(param, grad, exp_avg)
                    bucket = (param.device, param.dtype, exp_avg.dtype)
                    entry = (param.data_ptr(), grad.data_ptr(), exp_avg.data_ptr(), param.numel())
                    seen[param] = [grad, exp_avg, bucket, entry]
                buckets.setdefault(bucket, []).append(entry)
            for (device, p_dtype, m_dtype), ptrs in buckets.items():
                consts = make_consts(lr, (beta1, beta2), weight_decay, p_dtype, m_dtype)
                slot = (gi, device, p_dtype, m_dtype)
                table = self._tables.get(slot)
                if table is None:
                    table = self._tables[slot] = _Table(device)
                with torch.cuda.device(device):
                    table.update(ptrs, p_dtype.itemsize, m_dtype.itemsize)
                    stream = torch.cuda.current_stream(device).cuda_stream
                    _lib.check(lib.fo_lion_step_typed(table.dev.data_ptr(), table.n_chunks, _DTYPE_CODE[p_dtype], _DTYPE_CODE[m_dtype],
                                                      ctypes.byref(consts), stream), "fo_lion_step_typed")


class _Table:
    """The device table of chunk descriptors of one launch, rebuilt only when a pointer changes - with
    zero_grad(set_to_none=True), PyTorch's default, that is whenever the allocator hands the gradients other addresses
    than last time. A rebuild goes through a pinned staging buffer and an asynchronous copy on the current stream (the
    launch that follows on the same stream sees it); the buffer is reused once that copy is known to be done."""

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self.key: Optional[tuple] = None
        self.dev: Optional[Tensor] = None
        self.n_chunks = 0
        self._pinned: Optional[Tensor] = None
        self._copied: Optional[torch.cuda.Event] = None

    def update(self, ptrs: List[Tuple[int, int, int, int]], p_size: int, m_size: int) -> None:
        key = tuple(ptrs)
        if key == self.key:
            return
        table = build_chunk_table(ptrs, p_size, m_size)
        raw = table.view(np.uint8)
        n = raw.shape[0]
        if self._copied is not None:
            self._copied.synchronize()          # the previous copy out of the staging buffer
        if self._pinned is None or self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 1), dtype=torch.uint8, pin_memory=True)
        self._pinned[:n].numpy()[:] = raw
        # a new device tensor per rebuild: a kernel of an earlier step may still be reading the old table (its memory
        # goes back to torch's allocator, which hands it out again in stream order)
        self.dev = torch.empty(max(n, 1), dtype=torch.uint8, device=self.device)
        self.dev[:n].copy_(self._pinned[:n], non_blocking=True)
        if self._copied is None:
            self._copied = torch.cuda.Event()
        self._copied.record()
        self.key, self.n_chunks = key, int(table.shape[0])
