"""FlashAttention layer.

Mirrors train/acctransformer/flash_attention/nn/layer/flash_attention.py:31-207
of the reference (constructor arguments, their checks and error texts, the
call signature and the returned tensor).  The reference multiplies q and k each
by fp16(head_dim ** -0.25) before the op (`:117,188-189`); here the product of
those two factors is handed to the kernel as `scale`, which applies it to
q k^T in fp32 -- two elementwise passes over q and k disappear and the scores
carry one rounding less.  Dropout: the reference materialises an fp16
{0, 1/keep_prob} mask with DropoutGenMask/DropoutDoMask (`:198-203`); here no
mask tensor exists: every training call hands the op a fresh (seed, offset)
pair and the library draws the keep decisions itself (Philox4x32-10), the same
in forward and backward, and applies the 1/keep_prob factor inside the kernel.
The seed follows torch's global seed, so `torch.manual_seed` makes a run
repeatable.

Differences from the reference Cell that a caller can see:
  * Dropout is applied in training mode only (`module.train()`), the torch
    convention; the reference applies it whenever `dropout_rate > 0`
    (`:198-203`).  Call `.train()` to get the reference's behaviour.
  * The keep probability actually used is `round(256 * keep_prob) / 256`
    (the keep decision compares one random byte with a threshold), e.g.
    0.9 -> 230/256 = 0.8984; kept probabilities are scaled by the
    reciprocal of that value, so the expectation is exact.
  * The dropout stream of a call is (seed, offset) = (torch's seed mixed
    with a per-layer id, a per-layer call counter).  The counter is Python
    state: a forward that is re-run (activation checkpointing) would draw a
    new mask.  Pass `dropout_state=(seed, offset)` to `forward` to fix the
    stream of a call explicitly; the same pair reproduces the same mask.
  * Head dims: any multiple of 8 up to 256 (the reference admits multiples
    of 16 up to 256); others raise in the constructor.  Dropout works at
    every head dim; an alibi_mask needs a head_dim of at most 128 other
    than 40 (the op raises otherwise).
"""
from __future__ import annotations

import itertools
import math

import torch

from acctransformer_amd.flash_attention.ops.flash_attention.flash_attention_impl import get_flash_attention

__all__ = ['FlashAttention']
HEAD_DIM_MAX_LIMIT = 256
_layer_ids = itertools.count(1)


class FlashAttention(torch.nn.Module):
    """Flash Attention Layer (same arguments as the reference Cell).

    Inputs: query, key, value [batch, head_num, seq_len, head_dim] (fp16/bf16),
    attn_mask [1 or batch, seq_len, seq_len] or a (1,128,128) causal tile
    (1 = masked), alibi_mask [batch, head_num, 1, seq_len].
    Output: [batch, head_num, seq_len, head_dim].
    """

    def __init__(self,
                 head_dim,
                 dropout_rate=0.0,
                 prev_block_num=65536,
                 next_block_num=65536,
                 tiling_stgy_name="sparse",
                 dp=1,
                 mp=1,
                 have_attention_mask_batch=True,
                 alibi=False
                 ):
        super().__init__()
        if head_dim > HEAD_DIM_MAX_LIMIT:
            raise ValueError("head_dim too large, reduce head_dim and try again.")
        if head_dim <= 0 or head_dim % 8 != 0:
            raise ValueError(f"head_dim must be a positive multiple of 8, but got {head_dim}")
        if alibi:
            raise ValueError("alibi not supported in the current version.")
        s = torch.tensor(1. / math.sqrt(math.sqrt(head_dim)), dtype=torch.float16)   # the reference's fp16 factor
        self.scale = float(s) * float(s)
        self.head_dim = head_dim
        self.dropout_rate = dropout_rate
        self.enable_dropout = self.dropout_rate > 0.0
        self.keep_prob = 1.0 - dropout_rate
        self.have_attention_mask_batch = have_attention_mask_batch
        self.alibi = alibi
        self.dp, self.mp = dp, mp
        self.in_strategy = None
        self._layer_id = next(_layer_ids)             # separates the dropout streams of different layers
        self._calls = 0                               # one fresh mask per training call
        self.flash_attention = get_flash_attention(
            prev_block_num=prev_block_num,
            next_block_num=next_block_num,
            tiling_stgy_name=tiling_stgy_name,
            scale=self.scale,
            keep_prob=self.keep_prob,
        )

    def shard(self, in_strategy=None, out_strategy=None):
        """Records the (dp, mp, 1, 1) strategy the reference writes into the
        primitive (`:132-177`).  Every (batch, head) pair is independent, so a
        caller that splits batch or heads across devices needs no collective;
        nothing here launches one."""
        if in_strategy is None:
            in_strategy = ((1, 1, 1, 1), (1, 1, 1, 1), (1, 1, 1, 1))
        self.in_strategy = in_strategy
        self.dp, self.mp = in_strategy[0][0], in_strategy[0][1]
        return self

    def forward(self, q, k, v, attn_mask=None, alibi_mask=None, dropout_state=None):
        bsz, head_num, seq_len, head_dim = q.shape
        _, k_head_num, _, _ = k.shape
        _, v_head_num, _, _ = v.shape
        if head_num != k_head_num or head_num != v_head_num:
            raise ValueError(
                "the head_num of query, key and value must be the same, "
                "If different head_num are used, users need to change themselves to be same by tile.")
        if self.enable_dropout and self.training:
            if dropout_state is not None:             # the caller fixes the stream (e.g. a checkpointed forward that is re-run)
                drop_mask = (int(dropout_state[0]) & 0xFFFFFFFFFFFFFFFF, int(dropout_state[1]) & 0xFFFFFFFF)
            else:
                seed = (torch.initial_seed() ^ (self._layer_id * 0x9E3779B97F4A7C15)) & 0xFFFFFFFFFFFFFFFF
                drop_mask = (seed, self._calls & 0xFFFFFFFF)
                self._calls += 1
        else:
            drop_mask = None
        o, _ = self.flash_attention(q, k, v, attn_mask, drop_mask, alibi_mask)
        return o

    construct = forward
