// Split-plane GEMV kernels for 2-bit codes (see gemv_planes.inl).
#define QBITS 2
#include "gemv_launch.inl"
