// Streamed-weight matrix-core kernel for 2-bit codes (see gemm_stream.inl).
#define QBITS 2
#include "gemm_stream.inl"
