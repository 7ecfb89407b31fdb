// Entry points of libfastops_hip.so that are not tied to one kernel: status text, version, tuning hook.
#include <string.h>

#include "common.hpp"

namespace fo {
std::atomic<int> g_lion_variant{-1};
std::atomic<int> g_attn_variant{-1};
std::atomic<int> g_attn_bwd_variant{-1};
std::atomic<int> g_attn_order{-1};
std::atomic<int> g_attn_keep_on{-1};
std::atomic<int> g_attn_tail{-1};
std::atomic<int> g_attn_balance{-1};
std::atomic<int> g_attn_bwd_order{-1};
}  // namespace fo

extern "C" const char* fo_strerror(int status) {
  switch (status) {
    case FO_OK: return "ok";
    case FO_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FO_ERR_BAD_DTYPE: return "unsupported dtype: inputs must be half-precision floating point (float16 or bfloat16)";
    case FO_ERR_BAD_HEAD_DIM: return "unsupported head_dim: it must be a multiple of 8 from 8 to 128";
    case FO_ERR_BAD_SHAPE: return "a size is not positive or is too large";
    case FO_ERR_BAD_STRIDE: return "bad stride: rows must be contiguous in head_dim and start on 16-byte boundaries";
    case FO_ERR_MISALIGNED: return "a base pointer is not aligned as required";
    case FO_ERR_LAUNCH: return "the HIP runtime reported a kernel launch failure";
    case FO_ERR_UNSUPPORTED: return "request is valid but not implemented by this build";
    default: return "unknown fastops status";
  }
}

extern "C" int fo_version(void) { return 2000; }

extern "C" int fo_tune_set(const char* key, int value) {
  if (!key) return FO_ERR_NULL_POINTER;
  if (value < -1) return FO_ERR_UNSUPPORTED;
  // Every accepted value selects a kernel (or a workgroup order) that computes the same function; values that stand
  // for timing ablations with wrong results exist only in a library built with FO_ABLATIONS.
  if (strcmp(key, "lion.variant") == 0) {
    if (value >= 32) return FO_ERR_UNSUPPORTED;                       // launch shapes 0..31
    fo::g_lion_variant = value; return FO_OK;
  }
  if (strcmp(key, "attn.variant") == 0) {
    // FO_ATTN_KERNEL_*: 0 / 1 = 128-row kernel with the lazy / the exact rescale, 8 = 128 rows in the pipelined kernel,
    // 16 / 32 = 256-row pipelined kernel with 8 / 4 waves
    bool ok = value == -1 || value == 0 || value == 1 || value == 8 || value == 16 || value == 32;
#if defined(FO_ABLATIONS)
    ok = true;
#endif
    if (!ok) return FO_ERR_UNSUPPORTED;
    fo::g_attn_variant = value; return FO_OK;
  }
  if (strcmp(key, "attn_bwd.variant") == 0) {
    if (value > 1) return FO_ERR_UNSUPPORTED;                         // 0 = plain dK/dV kernel, 1 = pipelined (default)
    fo::g_attn_bwd_variant = value; return FO_OK;
  }
  if (strcmp(key, "attn.order") == 0) { fo::g_attn_order = value; return FO_OK; }
  if (strcmp(key, "attn.keep_on") == 0) {
    if (value > 2) return FO_ERR_UNSUPPORTED;
    fo::g_attn_keep_on = value; return FO_OK;
  }
  if (strcmp(key, "attn.tail") == 0) {
    if (value > 1) return FO_ERR_UNSUPPORTED;                         // 0 = one launch, 1 = a half-empty last round goes to the 128-row form (default)
    fo::g_attn_tail = value; return FO_OK;
  }
  if (strcmp(key, "attn.balance") == 0) {
    if (value > 1) return FO_ERR_UNSUPPORTED;                         // 0 = plain order, 1 = balanced where it applies (default)
    fo::g_attn_balance = value; return FO_OK;
  }
  if (strcmp(key, "attn_bwd.order") == 0) { fo::g_attn_bwd_order = value; return FO_OK; }
  return FO_ERR_UNSUPPORTED;
}

extern "C" int fo_tune_get(const char* key) {
  if (!key) return FO_ERR_NULL_POINTER;
  if (strcmp(key, "lion.variant") == 0) return fo::tune(fo::g_lion_variant);
  if (strcmp(key, "attn.variant") == 0) return fo::tune(fo::g_attn_variant);
  if (strcmp(key, "attn_bwd.variant") == 0) return fo::tune(fo::g_attn_bwd_variant);
  if (strcmp(key, "attn.order") == 0) return fo::tune(fo::g_attn_order);
  if (strcmp(key, "attn.keep_on") == 0) return fo::tune(fo::g_attn_keep_on);
  if (strcmp(key, "attn.tail") == 0) return fo::tune(fo::g_attn_tail);
  if (strcmp(key, "attn.balance") == 0) return fo::tune(fo::g_attn_balance);
  if (strcmp(key, "attn_bwd.order") == 0) return fo::tune(fo::g_attn_bwd_order);
  if (strcmp(key, "build.ablations") == 0) {
#if defined(FO_ABLATIONS)
    return 1;
#else
    return 0;
#endif
  }
  return FO_ERR_UNSUPPORTED;
}
