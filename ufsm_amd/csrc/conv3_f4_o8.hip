// kernels of the 3x3x3 MX convolution with e2m1 compute and MX-fp8 output
#include "conv3_kernel.hpp"
CONV3_LAUNCH_DECL(4, 8) { launch_out<4, 8>(stride, epi, MT, NT, a, smem); }
