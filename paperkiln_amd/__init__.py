"""paperkiln_amd: the attention hot path of paperkiln, MI355X (gfx950) native.

Importing the package never touches the GPU; the shared library is loaded on
first use and every op raises if it is missing.
"""
__all__ = ["synth"]
