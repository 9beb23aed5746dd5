// Split-plane GEMV kernels for 3-bit codes (see gemv_planes.inl).
#define QBITS 3
#include "gemv_launch.inl"
