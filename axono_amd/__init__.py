"""axono_amd: the LLM decode path of Axono on MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (include/axhip.h, built into axono_amd/lib/libaxhip.so) and
the host-side mirror of the reference's Python surface for that path.
"""
__version__ = "0.2.0"
