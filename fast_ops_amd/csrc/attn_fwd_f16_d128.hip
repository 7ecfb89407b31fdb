// The attention forward kernels for _Float16 operands at head_dim 128 as a translation unit of their own (attn_fwd.hip
// says how the units divide the work; the build compiles them in parallel).
#define FO_ATTN_UNIT 4
#include "attn_fwd.hip"
