"""Inference forward operator `flash_attention_tik`.

Mirrors infer/flash_attention/tik/tbe/impl/flash_attention_tik.py:9-16 of the
reference (operator `FlashAttentionTik`: inputs q, k, v, output y) together
with its shape function
(infer/flash_attention/tik/op_proto/flash_attention_tik.cpp:160-193) and the
checks of its kernel builder
(infer/flash_attention/tik/tbe/impl/flash_attention_fwd.py:89-140):
y = softmax(q k^T) v without mask and without scaling
(tests/infer/flash_attention/tik/data_gen.py:32-34), q, k, v fp16
[batch*heads, seq, D] or [batch, heads, seq, D], D in {40, 64, 80, 160}.

The reference builds a separate FlashAttention-1 style kernel for this
operator; here it is the training forward kernel with scale = 1 and no side
inputs, compiled for the two extra head dims as well.  Invalid shapes raise
AcctError with the reason (the reference returns GRAPH_FAILED / marks the
builder invalid).
"""
from __future__ import annotations

import torch

from acctransformer_amd import _capi

__all__ = ["flash_attention_tik"]


def flash_attention_tik(q, k, v, y=None, kernel_name="flash_attention_tik"):
    """y = softmax(q k^T) v.  Returns y (written into `y` when one is given)."""
    del kernel_name                                   # the reference names the generated binary with it
    out_shape = _capi.infer_shape(tuple(q.shape), tuple(k.shape), tuple(v.shape))
    if q.dtype != torch.float16 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k and v must be float16")  # op_info_cfg/ai_core/ascend310p: float16 only
    q4, k4, v4 = (t.unsqueeze(0) if t.dim() == 3 else t for t in (q, k, v))
    q4, k4, v4 = (t if t.stride(-1) == 1 else t.contiguous() for t in (q4, k4, v4))
    p = _capi.make_params(q4, k4, v4, scale=1.0)
    o, _ = _capi.fa_fwd(p, q4)
    o = o.reshape(out_shape)
    if y is not None:
        y.copy_(o)
        return y
    return o
