// Split-plane GEMV kernels for 5-bit codes (see gemv_planes.inl).
#define QBITS 5
#include "gemv_launch.inl"
