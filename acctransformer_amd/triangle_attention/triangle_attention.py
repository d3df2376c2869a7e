"""TriangleAttention layer.

Mirrors train/acctransformer/triangle_attention/triangle_attention.py:28-165 of
the reference: causal attention that leaves the upper-triangle blocks out
instead of masking them, no 1/sqrt(d) scaling, additive -10000 mask, optional
dropout on the probabilities.  The reference unrolls ceil(S / block_size)
StridedSlice -> BatchMatMul -> Softmax -> BatchMatMul -> Concat sub-graphs
(`:137-165`) whose score and probability tensors live in device memory.  Here
the whole layer is ONE launch of the fused forward kernel: `row_block_prefix =
block_size` makes query row i see exactly the keys [0, (i // block_size + 1) *
block_size) of the reference's row-block prefixes, the kernel never visits a
64-wide key tile past that limit, and the mask is only read on the 128x128
blocks that mix masked and unmasked entries.  When block_size is not a
multiple of 128 (the kernel's block granularity) the row blocks are launched
one by one on views of q, k, v, as the reference slices them.

Dropout follows the FlashAttention layer here: training mode only, keep
probability rounded to a multiple of 1/256, one (seed, offset) stream per call
from torch's seed and a per-layer call counter; `dropout_state=(seed, offset)`
fixes the stream of a call (a re-run forward then draws the same mask).
"""
from __future__ import annotations

import torch

from acctransformer_amd.flash_attention.ops.flash_attention.flash_attention_impl import get_flash_attention

__all__ = ["TriangleAttention"]


class TriangleAttention(torch.nn.Module):
    """Triangle Attention Layer (same arguments, checks and error texts as the
    reference Cell).

    Inputs: query, key, value [batch, head_num, seq_len, head_dim] (fp16/bf16),
    attention_mask [batch, seq_len, seq_len] (1 = masked).
    Output: [batch, head_num, seq_len, head_dim].
    """

    def __init__(self, block_size=512, dropout_rate=0., dp=1, mp=1):
        super().__init__()
        if block_size <= 0:
            raise ValueError(f"block size must be positive integer, but got {block_size}")
        if dropout_rate < 0. or dropout_rate >= 1.:
            raise ValueError(f"dropout rate must be between 0 and 1, but got {dropout_rate}")
        if dp <= 0:
            raise ValueError(f"data parallel must be positive integer, but got {dp}")
        if mp <= 0:
            raise ValueError(f"model parallel must be positive integer, but got {mp}")
        self.block_size = block_size
        self.dropout_rate = dropout_rate
        self.enable_dropout = dropout_rate > 0.
        self.keep_prob = 1.0 - dropout_rate
        self.dp, self.mp = dp, mp
        self._fused = block_size % 128 == 0
        self._op = get_flash_attention(scale=1.0, keep_prob=self.keep_prob,
                                       row_block_prefix=block_size if self._fused else 0)
        self._calls = 0                               # one fresh dropout mask per training call

    def forward(self, query, key, value, attention_mask, dropout_state=None):
        bsz, head_num, seq_len, _ = query.shape
        # dropout: no mask tensor, the library draws the keep decisions from a (seed, offset) pair
        dropping = self.enable_dropout and self.training
        if dropout_state is not None:
            seed, call = int(dropout_state[0]) & 0xFFFFFFFFFFFFFFFF, int(dropout_state[1])
        else:
            seed = (torch.initial_seed() ^ 0x7F4A7C15F39CC060) & 0xFFFFFFFFFFFFFFFF
            call = self._calls
            if dropping:
                self._calls += 1
        if self._fused:
            o, _ = self._op(query, key, value, attention_mask, (seed, call & 0xFFFFFFFF) if dropping else None, None)
            return o
        # block_size off the 128 grid: one launch per row block on sliced views (`:137-163`)
        out = torch.empty_like(query)
        for blk, q_begin in enumerate(range(0, seq_len, self.block_size)):
            q_end = min(q_begin + self.block_size, seq_len)
            kv_end = q_end
            cur_mask = attention_mask[:, q_begin:q_end, :kv_end].contiguous()
            cur_drop = (seed, (call * 4096 + blk) & 0xFFFFFFFF) if dropping else None    # every row block its own stream
            o, _ = self._op(query[:, :, q_begin:q_end], key[:, :, :kv_end], value[:, :, :kv_end], cur_mask, cur_drop, None)
            out[:, :, q_begin:q_end] = o
        return out

    construct = forward
