"""MI355X-native implementation of fast-ops' two hot kernels behind the reference's Python surfaces.

* ``fast_ops_amd.flash_attention.flash_attention.multi_head_attention`` - FlashAttention forward
  (reference: fast_ops/flash_attention/flash_attention.py:48-77)
* ``fast_ops_amd.lion.lion_optimizer.Lion`` - fused Lion optimizer (reference: fast_ops/lion/lion_optimizer.py:29-76)

Both call hand-written gfx950 HIP kernels in ``libfastops_hip.so`` through the C ABI of ``include/fastops.h``.
The top-level ``fast_ops`` package re-exports the same modules under the reference's import paths.
"""
__version__ = "0.1.0"
