// kernels of the 2x2x2 stride-2 conv / transposed conv with e2m1 compute
#include "conv2_kernel.hpp"
void conv2_launch_f4(int out, int up, int MT, const conv_args &a, dim3 grid, size_t smem) { launch_conv2<4>(out, up, MT, a, grid, smem); }
void conv3s2_launch_f4(int out, int MT, const conv_args &a, dim3 grid, size_t smem) { launch_conv3s2<4>(out, MT, a, grid, smem); }
