// The attention backward kernels for __bf16 operands at head_dim 128 as a translation unit of their own (attn_bwd.hip
// says how the units divide the work; the build compiles them in parallel).
#define FO_ATTN_UNIT 2
#include "attn_bwd.hip"
