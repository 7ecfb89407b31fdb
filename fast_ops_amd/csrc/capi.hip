// Entry points of libfastops_hip.so that are not tied to one kernel: status text, version, tuning hook.
#include <string.h>

#include "common.hpp"

namespace fo {
int g_lion_variant = -1;
int g_attn_variant = -1;
int g_attn_bwd_variant = -1;
int g_attn_order = -1;
int g_attn_bwd_order = -1;
}  // namespace fo

extern "C" const char* fo_strerror(int status) {
  switch (status) {
    case FO_OK: return "ok";
    case FO_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FO_ERR_BAD_DTYPE: return "unsupported dtype: inputs must be half-precision floating point (float16 or bfloat16)";
    case FO_ERR_BAD_HEAD_DIM: return "unsupported head_dim: this build implements head_dim 64 and 128";
    case FO_ERR_BAD_SHAPE: return "a size is not positive or is too large";
    case FO_ERR_BAD_STRIDE: return "bad stride: rows must be contiguous in head_dim and start on 16-byte boundaries";
    case FO_ERR_MISALIGNED: return "a base pointer is not aligned as required";
    case FO_ERR_LAUNCH: return "the HIP runtime reported a kernel launch failure";
    case FO_ERR_UNSUPPORTED: return "request is valid but not implemented by this build";
    default: return "unknown fastops status";
  }
}

extern "C" int fo_version(void) { return 1000; }

extern "C" int fo_tune_set(const char* key, int value) {
  if (!key) return FO_ERR_NULL_POINTER;
  if (value < -1) return FO_ERR_UNSUPPORTED;
  if (strcmp(key, "lion.variant") == 0) { fo::g_lion_variant = value; return FO_OK; }
  if (strcmp(key, "attn.variant") == 0) { fo::g_attn_variant = value; return FO_OK; }
  if (strcmp(key, "attn_bwd.variant") == 0) { fo::g_attn_bwd_variant = value; return FO_OK; }
  if (strcmp(key, "attn.order") == 0) { fo::g_attn_order = value; return FO_OK; }
  if (strcmp(key, "attn_bwd.order") == 0) { fo::g_attn_bwd_order = value; return FO_OK; }
  return FO_ERR_UNSUPPORTED;
}

extern "C" int fo_tune_get(const char* key) {
  if (!key) return FO_ERR_NULL_POINTER;
  if (strcmp(key, "lion.variant") == 0) return fo::g_lion_variant;
  if (strcmp(key, "attn.variant") == 0) return fo::g_attn_variant;
  if (strcmp(key, "attn_bwd.variant") == 0) return fo::g_attn_bwd_variant;
  if (strcmp(key, "attn.order") == 0) return fo::g_attn_order;
  if (strcmp(key, "attn_bwd.order") == 0) return fo::g_attn_bwd_order;
  return FO_ERR_UNSUPPORTED;
}
