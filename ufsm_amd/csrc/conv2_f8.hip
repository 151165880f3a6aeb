// kernels of the 2x2x2 stride-2 conv / transposed conv with e4m3 compute
#include "conv2_kernel.hpp"
void conv2_launch_f8(int out, int up, int MT, const conv_args &a, dim3 grid, size_t smem) { launch_conv2<8>(out, up, MT, a, grid, smem); }
void conv3s2_launch_f8(int out, int MT, const conv_args &a, dim3 grid, size_t smem) { launch_conv3s2<8>(out, MT, a, grid, smem); }
