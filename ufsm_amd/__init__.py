"""MI355X (gfx950) MX fp8 / fp4 3-D U-Net forward kernels behind the reference's lp_* C ABI.

The product is the shared library `libufsm_lp.so` (HIP kernels + C ABI, see include/mi_lp.h); this package only loads it
and mirrors the entry points for Python callers. There is no CPU fallback: loading fails loudly when the library is not built.
"""
from .lp import lib, load, LP, shape5, gnp_t, split_t, at_geom, at_dims, at_bp, at_ws, at_rays, DevBuf, MI_GN_SLOT_BYTES  # noqa: F401
