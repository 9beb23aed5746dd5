// Streamed-weight matrix-core kernel for 3-bit codes (see gemm_stream.inl).
#define QBITS 3
#include "gemm_stream.inl"
