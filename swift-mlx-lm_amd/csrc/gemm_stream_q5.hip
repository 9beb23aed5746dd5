// Streamed-weight matrix-core kernel for 5-bit codes (see gemm_stream.inl).
#define QBITS 5
#include "gemm_stream.inl"
