"""MI355X (gfx950) implementation of blockwise-int4 x fp16 GEMM/GEMV and its quantize/prepack step.

* ``gemmlib_amd.capi``            -- ctypes view of the C ABI (``include/ms_blkq4gemm.h``)
* ``gemmlib_amd.ms_blkq4linear``  -- ``BlkQ4Linear`` (needs the built ``ms_blkq4linear_ext`` extension)
* ``gemmlib_amd.build``           -- in-tree build of the native parts
"""
