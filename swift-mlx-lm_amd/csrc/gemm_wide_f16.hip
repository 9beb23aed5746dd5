// wide-tile prefill GEMM, f16 activations
#define WIDE_XF16 1
#include "gemm_wide.inl"
