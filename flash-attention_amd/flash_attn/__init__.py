"""FlashAttention for AMD MI355X (gfx950): hand-written HIP kernels behind the reference's Python API."""
__version__ = "0.1.0"
