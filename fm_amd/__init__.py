"""fm_amd: the Factorization-Memory scan of lexionbear/fm for AMD MI355X (gfx950).

`fm_amd.scan.fm_scan` mirrors the reference module `fm/scan/fm_scan.py`
(same names, same signatures); the kernels live in `fm_amd/csrc` and are
reached through the C ABI declared in `include/fmscan.h`.
"""
__version__ = "0.1.0"
