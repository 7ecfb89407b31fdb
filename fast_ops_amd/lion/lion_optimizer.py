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
from operator import attrgetter, is_, itemgetter
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
    arr = np.array(ptrs, dtype=np.uint64).reshape(-1, 4)
    return _chunk_table_of_columns(arr[:, 0], arr[:, 1], arr[:, 2], arr[:, 3], p_size, m_size)


def _chunk_table_of_columns(p_ptrs, g_ptrs, m_ptrs, numels, p_size: int, m_size: int) -> np.ndarray:
    C = _lib.FO_LION_CHUNK
    # all tensors at once (a rebuild happens whenever a gradient comes back at another address, and a Python loop over
    # the tensors took 3 ms for the 148 tensors of GPT-2-small)
    arr = np.array([p_ptrs, g_ptrs, m_ptrs, numels], dtype=np.uint64).T
    arr = arr[arr[:, 3] != 0]
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
        # per parameter group: what the last step learnt about it (_GroupPlan). The optimizer holds no reference to any
        # gradient: like the reference (lion_optimizer.py:57-76) it keeps no tensor alive beyond state["exp_avg"], so
        # zero_grad(set_to_none=True) really frees the gradients and the next backward gets their memory back - usually
        # at the same addresses, which leaves the chunk table valid.
        self._plans: Dict[int, "_GroupPlan"] = {}
        _lib.load()   # fail at construction, not at the first step, when the library is missing

    @property
    def table_rebuilds(self) -> int:
        """How many times a device chunk table was (re)built since construction, over all launches of this optimizer."""
        return sum(t.rebuilds for t in self._tables.values())

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
        self._plans.clear()

    @torch.no_grad()
    def step(self) -> None:
        """Parameter and state (momentum) update: one fused launch per parameter group and device."""
        lib = _lib.load()
        for gi, group in enumerate(self.param_groups):
            plist = group["params"]
            grads = list(map(_GRAD, plist))
            plan = self._plans.get(gi)
            live_grads = None
            if plan is not None and plan.plist is plist and len(plist) == len(plan.params):
                # The usual step: the same parameters have gradients as last time, the parameters and momenta are the
                # same objects over the same memory, and the gradients - new tensors after zero_grad(set_to_none=True),
                # torch's default - are dense like their parameters (torch itself refuses a gradient of another shape,
                # dtype or device when it is assigned). Then only the gradients' addresses are new. Written with map()
                # over the whole group: 148 tensors take 0.1 ms this way and 0.4 ms in a Python loop. (A momentum is
                # recognised as the object it was; storage swapped under that object - exp_avg.data = ... - is not
                # looked for, a parameter's is.)
                live_grads = [g for g in grads if g is not None]
                try:
                    if not (len(live_grads) == len(plan.live)
                            and (plan.all_live or [g is not None for g in grads] == plan.mask)
                            and all(map(is_, plist, plan.params))
                            and all(map(_IS_CONTIGUOUS, live_grads))
                            and list(map(_DATA_PTR, plan.live)) == plan.p_ptrs
                            and all(map(is_, map(_EXP_AVG, plan.states), plan.moms))):
                        live_grads = None
                    else:
                        g_ptrs = list(map(_DATA_PTR, live_grads))
                except (RuntimeError, KeyError):
                    live_grads = None      # e.g. a sparse gradient (no strides, no data pointer): the full checks say so
            if live_grads is None:
                plan, g_ptrs = self._look_at_group(gi, plist, grads)
                self._plans[gi] = plan
            if not plan.live:
                continue
            lr = group["lr"]
            weight_decay = group["weight_decay"]
            betas = group["betas"]
            # one launch per (device, parameter dtype, momentum dtype)
            for (device, p_dtype, m_dtype), idx in plan.buckets:
                consts = make_consts(lr, betas, weight_decay, p_dtype, m_dtype)
                slot = (gi, device, p_dtype, m_dtype)
                table = self._tables.get(slot)
                if table is None:
                    table = self._tables[slot] = _Table(device)
                if idx is None:
                    ptrs = (plan.p_ptrs, g_ptrs, plan.m_ptrs, plan.numels)
                else:
                    ptrs = tuple([col[i] for i in idx] for col in (plan.p_ptrs, g_ptrs, plan.m_ptrs, plan.numels))
                with torch.cuda.device(device):
                    stream = torch.cuda.current_stream(device)
                    table.update(ptrs, p_dtype.itemsize, m_dtype.itemsize, stream)
                    _lib.check(lib.fo_lion_step_typed(table.dev.data_ptr(), table.n_chunks, _DTYPE_CODE[p_dtype], _DTYPE_CODE[m_dtype],
                                                      ctypes.byref(consts), stream.cuda_stream), "fo_lion_step_typed")

    def _look_at_group(self, gi: int, plist: list, grads: list) -> Tuple["_GroupPlan", List[int]]:
        """Every check on every tensor of a group that has a gradient (the first step, and whenever the quick look of
        step() finds something changed); creates missing momenta. Returns the group's plan and the gradients' addresses."""
        plan = _GroupPlan()
        plan.plist, plan.params = plist, tuple(plist)
        plan.mask = [g is not None for g in grads]
        plan.all_live = all(plan.mask)
        plan.live, plan.states, plan.moms, plan.p_ptrs, plan.m_ptrs, plan.numels = [], [], [], [], [], []
        g_ptrs: List[int] = []
        by_bucket: Dict[tuple, List[int]] = {}
        dense = True
        for param, grad in zip(plist, grads):
            if grad is None:
                continue
            state = self.state[param]
            if "exp_avg" not in state:
                # exponential moving average of the gradient (lion_optimizer.py:68-73)
                dt = self._exp_avg_dtype or (torch.bfloat16 if param.dtype == torch.float32 else param.dtype)
                state["exp_avg"] = torch.zeros_like(param, dtype=dt, memory_format=torch.preserve_format)
            exp_avg: Tensor = state["exp_avg"]
            _check_tensors(param, grad, exp_avg)
            dense = dense and param.is_contiguous()
            by_bucket.setdefault((param.device, param.dtype, exp_avg.dtype), []).append(len(plan.live))
            plan.live.append(param)
            plan.states.append(state)
            plan.moms.append(exp_avg)
            plan.p_ptrs.append(param.data_ptr())
            plan.m_ptrs.append(exp_avg.data_ptr())
            plan.numels.append(param.numel())
            g_ptrs.append(grad.data_ptr())
        plan.buckets = [(key, None if len(by_bucket) == 1 else idx) for key, idx in by_bucket.items()]
        # (a group with a parameter that is dense but not contiguous - a transposed weight, channels-last - is looked at
        # in full every step: the quick look only knows "contiguous")
        if not dense:
            plan.plist = None
        return plan, g_ptrs


_GRAD = attrgetter("grad")
_EXP_AVG = itemgetter("exp_avg")
_DATA_PTR = Tensor.data_ptr
_IS_CONTIGUOUS = Tensor.is_contiguous


class _GroupPlan:
    """What Lion.step learnt about a parameter group the last time it looked at every tensor: the group's list of
    parameters (the list object and its elements then), which of them had a gradient (`mask`; `live` = those that had),
    their state dicts, momenta, the addresses of parameters and momenta, element counts, and how the live parameters
    fall into launches (`buckets`: ((device, parameter dtype, momentum dtype), indices into `live` or None for all))."""
    __slots__ = ("plist", "params", "mask", "all_live", "live", "states", "moms", "p_ptrs", "m_ptrs", "numels", "buckets")


class _Table:
    """The device table of chunk descriptors of one launch, rebuilt only when a pointer changes - with
    zero_grad(set_to_none=True), PyTorch's default, that is whenever the allocator hands the gradients other addresses
    than last time (it usually hands out the same ones). A rebuild goes through a pinned staging buffer and an
    asynchronous copy on the current stream (the launch that follows on the same stream sees it); the buffer is reused
    once that copy is known to be done. `rebuilds` counts them.

    A rebuild synchronizes with an event, may allocate and copies from the host: none of that can be recorded into a HIP
    graph, so a rebuild under stream capture raises instead of breaking the capture (capture a step whose parameter,
    gradient and momentum tensors are the ones of the step before). The replaced device table is kept until the rebuild
    after this one, and a table used on another stream than the one it was filled on is recorded there, so that its
    memory is never handed out while a launch of an earlier step may still read it."""

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self.key: Optional[tuple] = None
        self.dev: Optional[Tensor] = None
        self.n_chunks = 0
        self.rebuilds = 0
        self._pinned: Optional[Tensor] = None
        self._copied: Optional[torch.cuda.Event] = None
        self._previous: Optional[Tensor] = None
        self._stream: Optional[int] = None

    def update(self, key: tuple, p_size: int, m_size: int, stream: "torch.cuda.Stream") -> None:
        """`key` = (parameter addresses, gradient addresses, momentum addresses, element counts), four lists."""
        if key == self.key:
            if stream.cuda_stream != self._stream:
                # filled on another stream: wait for the fill, and tell the allocator that this stream reads the table
                stream.wait_event(self._copied)
                self.dev.record_stream(stream)
            return
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                "Lion.step under stream capture: a parameter, gradient or momentum tensor is not where it was at the last "
                "step, so the chunk table would have to be rebuilt (a host copy, which cannot be captured). Run one step "
                "on the same tensors before capturing, and keep the gradients in place (zero_grad(set_to_none=False))."
            )
        table = _chunk_table_of_columns(*key, p_size, m_size)
        raw = table.view(np.uint8)
        n = raw.shape[0]
        if self._copied is not None:
            self._copied.synchronize()          # the previous copy out of the staging buffer
        if self._pinned is None or self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 1), dtype=torch.uint8, pin_memory=True)
        self._pinned[:n].numpy()[:] = raw
        # a new device tensor per rebuild: a kernel of an earlier step may still be reading the old table, which
        # therefore stays referenced for one more rebuild
        self._previous = self.dev
        self.dev = torch.empty(max(n, 1), dtype=torch.uint8, device=self.device)
        self.dev[:n].copy_(self._pinned[:n], non_blocking=True)
        if self._copied is None:
            self._copied = torch.cuda.Event()
        self._copied.record(stream)
        self.key, self.n_chunks, self._stream = tuple(list(col) for col in key), int(table.shape[0]), stream.cuda_stream
        self.rebuilds += 1
