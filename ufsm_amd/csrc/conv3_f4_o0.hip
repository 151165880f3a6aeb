// kernels of the 3x3x3 MX convolution with e2m1 compute and fp32 / fp16 plane output
#include "conv3_kernel.hpp"
CONV3_LAUNCH_DECL(4, 0) { launch_out<4, 0>(stride, epi, MT, NT, a, smem); }
