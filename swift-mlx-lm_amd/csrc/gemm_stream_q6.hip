// Streamed-weight matrix-core kernel for 6-bit codes (see gemm_stream.inl).
#define QBITS 6
#include "gemm_stream.inl"
