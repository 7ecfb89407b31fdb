// Shared helpers for the HIP sources of libfastops_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/fastops.h"

namespace fo {

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) uint16_t u16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

// variant selectors set through fo_tune_set (-1 = default). Atomic so that a host thread that sets one while another
// thread launches reads a whole value; an entry point reads each selector once per call.
extern std::atomic<int> g_lion_variant;
extern std::atomic<int> g_attn_variant;
extern std::atomic<int> g_attn_bwd_variant;
extern std::atomic<int> g_attn_bwd_order;   // attention backward: -1 automatic, 0 all heads in one group, n > 0 groups of n heads
extern std::atomic<int> g_attn_balance;   // 128-row attention kernel, causal: 0 plain heaviest-first order also where a launch fits the chip at once, otherwise (default) balanced
extern std::atomic<int> g_attn_tail;      // 256-row attention kernel, non-causal: 0 = never hand the last round to the 128-row form (see launch_rows256_w4_noncausal)
extern std::atomic<int> g_attn_keep_on;   // 256-row attention kernel, four waves: see launch_wide
extern std::atomic<int> g_attn_order;   // 128-row attention kernel, causal: -1 automatic, 0 head by head, n > 0 heaviest query blocks first within groups of n heads per XCD
inline int tune(const std::atomic<int>& v) { return v.load(std::memory_order_relaxed); }

inline int launch_status() { return hipGetLastError() == hipSuccess ? FO_OK : FO_ERR_LAUNCH; }

}  // namespace fo
