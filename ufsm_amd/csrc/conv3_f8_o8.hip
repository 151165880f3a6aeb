// kernels of the 3x3x3 MX convolution with e4m3 compute and MX-fp8 output
#include "conv3_kernel.hpp"
CONV3_LAUNCH_DECL(8, 8) { launch_out<8, 8>(stride, epi, MT, NT, a, smem); }
#ifdef DBG_TIMING
extern "C" void mi_dbg_read(long long *out) { MIRT(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_dbg), sizeof(long long) * 64)); }
#endif
