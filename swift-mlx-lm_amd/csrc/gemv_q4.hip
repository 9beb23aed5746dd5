// Split-plane GEMV kernels for 4-bit codes (see gemv_planes.inl).
#define QBITS 4
#include "gemv_launch.inl"
