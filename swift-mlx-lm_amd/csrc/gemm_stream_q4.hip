// Streamed-weight matrix-core kernel for 4-bit codes (see gemm_stream.inl).
#define QBITS 4
#include "gemm_stream.inl"
