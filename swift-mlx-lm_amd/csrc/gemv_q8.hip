// Split-plane GEMV kernels for 8-bit codes (see gemv_planes.inl).
#define QBITS 8
#include "gemv_launch.inl"
