// Backward kernels (stub while the forward is brought up).
#pragma once
#include "sa2_common.hpp"
namespace sa2 {
template <int D> __global__ void delta_kernel(KParams p) {}
template <int D> __global__ void bwd_dq_kernel(KParams p) {}
template <int D> __global__ void bwd_dkv1_kernel(KParams p) {}
template <int D> __global__ void bwd_dkv2_kernel(KParams p) {}
}
