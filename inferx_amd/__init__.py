"""inferx_amd: a single-GPU inference engine for MI355X (gfx950).

Importing the package touches no GPU and builds nothing; the HIP library is
built and loaded on the first call that needs it (`inferx_amd.csrc`).
"""
__version__ = "0.1.0"
