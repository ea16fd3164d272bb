"""Drop-in for the reference's ``python/ms_blkq4linear.py``: ``from ms_blkq4linear import BlkQ4Linear`` works
unchanged (reference: python/ms_blkq4linear.py:10-28).  The implementation is ``gemmlib_amd.ms_blkq4linear``;
the compiled extension is the top-level module ``ms_blkq4linear_ext`` next to this file, as the reference's
``python/setup.py:17-26`` installs it."""

import ms_blkq4linear_ext  # noqa: F401  (fails loudly if the extension is not built: there is no fallback)
from gemmlib_amd.ms_blkq4linear import BlkQ4Linear

__all__ = ["BlkQ4Linear"]
