"""FlashAttention2 / TriangleAttention for AMD MI355X (gfx950): hand-written HIP
kernels behind a C ABI, with the Python operator surface of
mindspore-ai/acctransformer."""
__version__ = "0.1.0"
