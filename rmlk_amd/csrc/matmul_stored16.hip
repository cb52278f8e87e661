// The tiled MFMA products over weights stored as 16-bit values (IEEE half, bfloat16; fp32 arithmetic):
// the second compilation of matmul.hip, which holds the kernels and says how the two parts meet.
#define RMLK_MATMUL_PART 2
#include "matmul.hip"
