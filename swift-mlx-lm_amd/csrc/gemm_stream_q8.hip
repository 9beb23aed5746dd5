// Streamed-weight matrix-core kernel for 8-bit codes (see gemm_stream.inl).
#define QBITS 8
#include "gemm_stream.inl"
