// kernels of the 3x3x3 MX convolution with e4m3 compute and fp32 / fp16 plane output
#include "conv3_kernel.hpp"
CONV3_LAUNCH_DECL(8, 0) { launch_out<8, 0>(stride, epi, MT, NT, a, smem); }
