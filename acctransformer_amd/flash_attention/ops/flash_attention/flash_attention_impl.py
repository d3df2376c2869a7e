"""Operator binding of the FlashAttention2 forward / backward kernels.

Mirrors train/acctransformer/flash_attention/ops/flash_attention/flash_attention_impl.py:96-154
of the reference: `get_flash_attention(prev_block_num, next_block_num,
tiling_stgy_name)` returns the forward primitive
`(query, key, value, attn_mask, dropout_mask, alibi_mask) -> (output, rowsum)`
with its gradient attached, and `get_flash_attention_grad(...)` returns
`bprop(query, key, value, attn_mask, dropout_mask, alibi_mask, outs, douts)
-> (dq, dk, dv, 0, 0, 0)`.  Where the reference hands tensor descriptors to a
TBE kernel builder, this module hands device pointers to the C ABI of
libacct_fa.so; torch supplies memory, streams and autograd plumbing only.

Differences from the reference that a caller can see:
  * `scale` (default 1.0, the raw op) is applied to q k^T inside the kernel in
    fp32; the reference's layer pre-multiplies q and k instead.
  * masks may be uint8/bool as well as floating; a floating attn_mask is read
    as "nonzero = masked" (the reference multiplies its value by -10000, and
    only ever feeds 0/1).  A floating dropout_mask is the reference's
    {0, 1/keep_prob} form; a uint8/bool one is {0,1} with `keep_prob` given.
    Masks in q's dtype (the reference's form) and uint8 masks are handed to
    the library as they are, without a conversion pass; other dtypes are
    converted to uint8 first.  Without `keep_prob`, a floating dropout mask
    costs one reduction and a host sync to recover keep_prob = 1 / max.
  * `dropout_mask` may also be a `(seed, offset)` pair of ints: the keep mask
    is then drawn inside the library (Philox4x32-10, defined in
    include/acct_fa.h) instead of being read from a [B,N,Sq,Sk] tensor, the
    same way in forward and backward; `keep_prob` must be given.
  * dq, dk, dv come back in q's dtype directly (the reference returns fp32
    and casts to fp16 in bprop, flash_attention_impl.py:121-123).
"""
from __future__ import annotations

import weakref

import torch

from acctransformer_amd import _capi

TILING_BLOCK_SIZE = 128                       # constants.py:19 of the reference ops
_STRATEGIES = ("sparse", "wukong")            # tiling_strategy/sparse_tiling.py, wukong_tiling.py


def _check_strategy(name):
    # tiling_strategy/strategy.py:51-58: unknown names raise at construction
    if name not in _STRATEGIES:
        raise Exception(f"Strategy:{name} not supported")


# ---- attn_mask classification ------------------------------------------------
_mask_cache = {}


def _is_compact_shape(shape):
    """attention.py:279-285 (is_only_causal_mask): (128,128) or (1,128,128)."""
    if len(shape) == 2:
        return shape[0] == TILING_BLOCK_SIZE and shape[1] == TILING_BLOCK_SIZE
    if len(shape) == 3:
        return shape[0] == 1 and shape[1] == TILING_BLOCK_SIZE and shape[2] == TILING_BLOCK_SIZE
    return False


# Off (the default): an attn_mask tensor goes to the library as it is, and the library's own pre-pass finds the
# blocks that are clean, wholly masked or the plain causal diagonal -- on the device, with no host round trip.
# On: the operator compares the mask with the lower-triangular pattern once per tensor (one device compare and
# one host sync) and, on a match, passes ACCT_MASK_CAUSAL, which needs no pre-pass at all.
DETECT_CAUSAL_MASKS = False


def _classify_mask(attn_mask, Sq, Sk, io_dtype):
    """Returns (mask_kind, tensor or None).  A mask in the operands' dtype -- the
    reference's form -- or in uint8 goes to the library as it is; only other
    dtypes are converted.  The outcome is remembered per tensor object and
    version, so a mask reused across steps is inspected once."""
    key = id(attn_mask)
    hit = _mask_cache.get(key)
    if (hit is not None and hit[0]() is attn_mask and hit[1] == attn_mask._version
            and hit[2] == (Sq, Sk, io_dtype, DETECT_CAUSAL_MASKS)):
        return hit[3], hit[4]
    if attn_mask.dtype == torch.bool:
        m = attn_mask.contiguous().view(torch.uint8)
    elif attn_mask.dtype in (torch.uint8, io_dtype):
        m = attn_mask.contiguous()
    else:
        m = attn_mask.ne(0).to(torch.uint8)
    wide = m.dtype != torch.uint8
    compact = _is_compact_shape(tuple(attn_mask.shape)) and not (Sq == TILING_BLOCK_SIZE and Sk == TILING_BLOCK_SIZE
                                                                  and attn_mask.dim() == 3)
    if compact:
        kind, out = (_capi.MASK_TILE_F16 if wide else _capi.MASK_TILE_U8), m.reshape(128, 128)
        if DETECT_CAUSAL_MASKS:
            tri = torch.triu(torch.ones(128, 128, dtype=torch.bool, device=m.device), diagonal=1)
            if torch.equal(m.reshape(128, 128).ne(0), tri):
                kind, out = _capi.MASK_CAUSAL, None      # evaluated by index compare, no loads
        compact_kind = True
    else:
        compact_kind = False
        if m.dim() == 2:
            m = m.unsqueeze(0)
        if m.dim() != 3 or m.shape[1] != Sq or m.shape[2] != Sk:
            raise ValueError(f"attn_mask must be [1|B,{Sq},{Sk}] or a (1,128,128) causal tile, got {tuple(attn_mask.shape)}")
        kind, out = (_capi.MASK_DENSE_F16 if wide else _capi.MASK_DENSE_U8), m
        if DETECT_CAUSAL_MASKS and Sq == Sk:
            rows = torch.arange(Sq, device=m.device)
            tri = rows[None, :] > rows[:, None]
            if torch.equal(m.ne(0), tri.expand_as(m)):
                kind, out = _capi.MASK_CAUSAL, None
    if len(_mask_cache) > 64:
        for k_ in [k_ for k_, v_ in _mask_cache.items() if v_[0]() is None]:
            del _mask_cache[k_]
    _mask_cache[key] = (weakref.ref(attn_mask), attn_mask._version, (Sq, Sk, io_dtype, DETECT_CAUSAL_MASKS), kind, out, compact_kind)
    return kind, out


# ---- what the library's pre-passes derive from a mask tensor, kept per tensor ----
# Block classes and column bitmaps depend on the mask's contents and on the band only, so a mask that is
# reused from step to step (the usual case) is classified once: the buffer is handed to every later call
# with mask_bits_filled = 1.  Entries are dropped with their tensor, on an in-place edit of it (torch's
# version counter), and when a call arrives on another stream (the fill is ordered on the stream that ran it).
_mask_bits_cache = {}


def _attach_mask_bits(p, mask_tensor, device):
    """Points `p` at the pre-pass results of `mask_tensor` (the tensor handed to the library): a filled buffer
    from an earlier call, or a fresh one that `_mask_bits_done(p)` marks as filled once a call has run."""
    if p.mask_kind not in (_capi.MASK_DENSE_U8, _capi.MASK_DENSE_F16, _capi.MASK_TILE_U8, _capi.MASK_TILE_F16):
        return
    stream = torch.cuda.current_stream(device).cuda_stream
    sig = (p.mask_kind, p.B, p.Sq, p.Sk, p.prev_block_num, p.next_block_num, p.row_block_prefix, stream,
           mask_tensor.data_ptr())
    key = id(mask_tensor)
    hit = _mask_bits_cache.get(key)
    if hit is not None and hit[0]() is mask_tensor and hit[1] == mask_tensor._version and hit[2] == sig:
        entry = hit
    else:
        buf = _capi.attach_mask_bits(p, device)
        if buf is None:
            return
        if len(_mask_bits_cache) > 64:
            for k_ in [k_ for k_, v_ in _mask_bits_cache.items() if v_[0]() is None]:
                del _mask_bits_cache[k_]
        entry = (weakref.ref(mask_tensor), mask_tensor._version, sig, buf, [False])
        _mask_bits_cache[key] = entry
    p.mask_bits = entry[3].data_ptr()
    p.mask_bits_filled = 1 if entry[4][0] else 0
    p._keepalive.append(entry[3])
    p._mask_bits_entry = entry


def _mask_bits_done(p):
    """A call with `p` has been enqueued: its mask pre-pass results are in the buffer for every later call."""
    entry = getattr(p, "_mask_bits_entry", None)
    if entry is not None:
        entry[4][0] = True
        p.mask_bits_filled = 1


def _is_seed_pair(x):
    return isinstance(x, (tuple, list)) and len(x) == 2 and all(isinstance(t, int) for t in x)


def _prepare_dropout(dropout_mask, keep_prob, io_dtype):
    """Returns (mask or None, keep_prob, (seed, offset) or None).  The mask goes to the library as uint8 {0,1}
    or, in the operands' dtype, as the reference's {0, 1/keep_prob}."""
    if dropout_mask is None:
        return None, 1.0, None
    if _is_seed_pair(dropout_mask):
        if keep_prob is None:
            raise ValueError("a (seed, offset) dropout_mask needs keep_prob")
        return None, float(keep_prob), (int(dropout_mask[0]), int(dropout_mask[1]))
    if dropout_mask.dtype in (torch.uint8, torch.bool):
        d8 = dropout_mask.contiguous()
        d8 = d8.view(torch.uint8) if d8.dtype == torch.bool else d8
        if keep_prob is None:
            raise ValueError("a uint8/bool dropout_mask needs keep_prob")
        return d8, float(keep_prob), None
    # the reference's form: fp16 {0, 1/keep_prob} (layer/flash_attention.py:198-203)
    if keep_prob is None:
        mx = float(dropout_mask.max())
        keep_prob = 1.0 / mx if mx > 0 else 1.0
    if dropout_mask.dtype == io_dtype:
        return dropout_mask.contiguous(), float(keep_prob), None
    return dropout_mask.ne(0).to(torch.uint8), float(keep_prob), None


def _build_params(q, k, v, attn_mask, dropout_mask, alibi_mask, prev_block_num, next_block_num, scale, keep_prob,
                  row_block_prefix=0):
    Sq, Sk = q.shape[2], k.shape[2]
    kind, m8 = (_capi.MASK_NONE, None) if attn_mask is None else _classify_mask(attn_mask, Sq, Sk, q.dtype)
    if kind == _capi.MASK_CAUSAL and attn_mask is not None and _mask_cache[id(attn_mask)][5] and next_block_num > 0:
        # a compact tile only ever touches diagonal blocks (attention.py:363-365,
        # flash_attention_fwd.py:353-356): blocks right of the diagonal stay visible
        kind, m8 = _capi.MASK_TILE_U8, torch.triu(torch.ones(128, 128, dtype=torch.uint8, device=q.device), diagonal=1)
    d8, keep, seed = _prepare_dropout(dropout_mask, keep_prob, q.dtype)
    if alibi_mask is not None and alibi_mask.dtype != q.dtype:
        alibi_mask = alibi_mask.to(q.dtype)
    p = _capi.make_params(q, k, v, scale=scale, keep_prob=keep, prev_block_num=prev_block_num,
                          next_block_num=next_block_num, mask_kind=kind, attn_mask=m8, drop_mask=d8,
                          alibi=alibi_mask, row_block_prefix=row_block_prefix,
                          drop_seed=None if seed is None else seed[0], drop_offset=0 if seed is None else seed[1])
    if m8 is not None and q.is_cuda:
        # block classes / column bitmaps of the mask: derived once per mask tensor, by the first call that sees it
        _attach_mask_bits(p, m8, q.device)
    return p


def _rows_contiguous(t):
    return t if t.stride(-1) == 1 else t.contiguous()


class _FlashAttentionFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, attn_mask, dropout_mask, alibi_mask, prev_block_num, next_block_num, scale, keep_prob,
                row_block_prefix):
        q, k, v = _rows_contiguous(q), _rows_contiguous(k), _rows_contiguous(v)
        p = _build_params(q, k, v, attn_mask, dropout_mask, alibi_mask, prev_block_num, next_block_num, scale, keep_prob,
                          row_block_prefix)
        # with dropout, the keep bits the forward packs (or draws) are kept for the backward of this step
        needs_grad = any(ctx.needs_input_grad[:3])
        ctx.drop_bits = _capi.attach_drop_bits(p, q.device) if needs_grad else None
        o, lse = _capi.fa_fwd(p, q)
        _mask_bits_done(p)
        if ctx.drop_bits is not None:
            p.drop_bits_filled = 1
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.params = p
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, o, lse = ctx.saved_tensors
        dq, dk, dv = _capi.fa_bwd(ctx.params, q, k, v, o, do, lse)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def get_flash_attention_grad(prev_block_num=65536, next_block_num=65536, tiling_stgy_name='sparse',
                             scale=1.0, keep_prob=None, row_block_prefix=0):
    """flash_attention_impl.py:96-126 of the reference: returns
    bprop(query, key, value, attn_mask, dropout_mask, alibi_mask, outs, douts)
    -> (dq, dk, dv, zeros_like(attn_mask), zeros_like(dropout_mask), zeros_like(alibi_mask))."""
    _check_strategy(tiling_stgy_name)

    def bprop(query, key, value, attn_mask, dropout_mask, alibi_mask, outs, douts):
        output, rowsum = outs
        dout = douts[0]
        q, k, v = _rows_contiguous(query), _rows_contiguous(key), _rows_contiguous(value)
        p = _build_params(q, k, v, attn_mask, dropout_mask, alibi_mask, prev_block_num, next_block_num, scale, keep_prob,
                          row_block_prefix)
        dq, dk, dv = _capi.fa_bwd(p, q, k, v, output, dout, rowsum)
        _mask_bits_done(p)
        zeros = tuple(torch.zeros_like(t) if torch.is_tensor(t) else None for t in (attn_mask, dropout_mask, alibi_mask))
        return (dq, dk, dv) + zeros

    return bprop


def get_flash_attention(prev_block_num=65536, next_block_num=65536, tiling_stgy_name='sparse',
                        scale=1.0, keep_prob=None, row_block_prefix=0):
    """flash_attention_impl.py:129-154 of the reference: returns the forward
    primitive (query, key, value, attn_mask=None, dropout_mask=None,
    alibi_mask=None) -> (output [B,N,Sq,D] in q's dtype, rowsum fp32 [B,N,Sq]),
    differentiable in query, key and value."""
    _check_strategy(tiling_stgy_name)

    def fa_forward(query, key, value, attn_mask=None, dropout_mask=None, alibi_mask=None):
        return _FlashAttentionFn.apply(query, key, value, attn_mask, dropout_mask, alibi_mask,
                                       prev_block_num, next_block_num, scale, keep_prob, row_block_prefix)

    fa_forward.prev_block_num = prev_block_num
    fa_forward.next_block_num = next_block_num
    fa_forward.tiling_stgy_name = tiling_stgy_name
    fa_forward.bprop = get_flash_attention_grad(prev_block_num, next_block_num, tiling_stgy_name, scale, keep_prob,
                                                row_block_prefix)
    return fa_forward
