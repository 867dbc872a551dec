"""MI355X (gfx950) evaluation backend for tenncor operator graphs.

``tenncor_amd.capi`` binds the C ABI declared in ``include/tcg.h`` (the HIP
library ``libtcg.so``).  There is no CPU fallback: loading fails loudly when the
library has not been built, and creating a context fails when no GPU is visible.
"""
