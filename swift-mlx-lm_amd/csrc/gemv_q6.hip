// Split-plane GEMV kernels for 6-bit codes (see gemv_planes.inl).
#define QBITS 6
#include "gemv_launch.inl"
