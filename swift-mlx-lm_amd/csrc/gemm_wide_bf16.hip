// wide-tile prefill GEMM, bf16 activations
#define WIDE_XF16 0
#include "gemm_wide.inl"
