// The 16-bit GEMM's kernels for binary16 operands, B row-major: one of the four parts that ko_gemm16.hip is compiled into (see there).
#define KO_GEMM16_BF16 0
#define KO_GEMM16_B_ROW 1
#define KO_GEMM16_ENTRY 0
#include "ko_gemm16.hip"
