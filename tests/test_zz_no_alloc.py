"""GPU test of acct_fa_bwd_static, the backward entry point that allocates nothing: its scratch memory is a
buffer inside the library's device image.  Its results must equal those of acct_fa_bwd with a workspace of the
same size bit for bit (and those of acct_fa_bwd with a full-size workspace within the parity gate), on two calls in a
row of which the second is smaller (the buffer keeps the first call's contents), and a problem whose scratch
need exceeds the buffer must be refused."""
import ctypes

import numpy as np
import pytest
import torch

from acctransformer_amd import _capi

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _problem(B, N, Sq, Sk, D, seed, **kw):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, N, Sq, D, generator=g).half().to(DEV)
    k = torch.randn(B, N, Sk, D, generator=g).half().to(DEV)
    v = torch.randn(B, N, Sk, D, generator=g).half().to(DEV)
    dO = torch.randn(B, N, Sq, D, generator=g).half().to(DEV)
    p = _capi.make_params(q, k, v, scale=D ** -0.5, **kw)
    o, lse = _capi.fa_fwd(p, q)
    return p, q, k, v, o, dO, lse


STATIC_BYTES = 8 << 20      # ACCT_FA_STATIC_SCRATCH_BYTES


def _both(p, q, k, v, o, dO, lse):
    # the reference call gets a workspace of the static buffer's size: with more room acct_fa_bwd may split the
    # query range of its dK/dV launch, which sums in another order (checked against the gate below)
    lib = _capi.load()
    ref = _capi.fa_bwd(p, q, k, v, o, dO, lse, workspace_bytes=STATIC_BYTES)
    got = [torch.empty_like(t) for t in (q, k, v)]
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.acct_fa_bwd_static(ctypes.byref(p), o.data_ptr(), dO.data_ptr(), lse.data_ptr(),
                                got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(), st)
    assert rc == 0, lib.acct_last_error().decode()
    torch.cuda.synchronize()
    return ref, got


def test_static_scratch_backward_equals_workspace_backward():
    # first call: a dense padding mask with a causal part (block classes and column bitmaps live in the scratch
    # buffer next to the row statistics); second call: smaller, other mask kind, ragged lengths
    B, N, S, D = 2, 4, 1024, 128
    m = np.triu(np.ones((S, S), np.uint8), 1)[None].repeat(B, 0)
    m[0, :, 900:] = 1
    m[1, :, 333:] = 1
    first = _problem(B, N, S, S, D, 200, mask_kind=_capi.MASK_DENSE_U8, attn_mask=torch.from_numpy(m).to(DEV))
    ref, got = _both(*first)
    assert all(torch.equal(a, b) for a, b in zip(ref, got))
    # and within the parity gate of the call with a full-size workspace (split dK/dV launch)
    full = _capi.fa_bwd(*first)
    for a, b in zip(full, got):
        assert ((a.float() - b.float()).abs() <= 2e-3 + 1e-3 * a.float().abs()).all()
    second = _problem(1, 3, 200, 333, 64, 201, mask_kind=_capi.MASK_CAUSAL)
    ref, got = _both(*second)
    assert all(torch.equal(a, b) for a, b in zip(ref, got))
    # and the first problem again, after the smaller one has written over the front of the buffer
    ref, got = _both(*first)
    assert all(torch.equal(a, b) for a, b in zip(ref, got))


def test_static_scratch_backward_refuses_what_does_not_fit():
    lib = _capi.load()
    # dropout keep bits of B16 N16 S1024 need 4 x the buffer: refused with a message, nothing launched
    B, N, S, D = 16, 16, 1024, 128
    p, q, k, v, o, dO, lse = _problem(B, N, S, S, D, 202, keep_prob=0.9, drop_seed=7)
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p)) > (8 << 20)
    g = [torch.empty_like(t) for t in (q, k, v)]
    rc = lib.acct_fa_bwd_static(ctypes.byref(p), o.data_ptr(), dO.data_ptr(), lse.data_ptr(),
                                g[0].data_ptr(), g[1].data_ptr(), g[2].data_ptr(), None)
    assert rc == -7 and "acct_fa_bwd_static" in lib.acct_last_error().decode()
    # with the caller's drop_bits buffer the rest fits
    bits = _capi.attach_drop_bits(p, q.device)
    o2, lse2 = _capi.fa_fwd(p, q)
    p.drop_bits_filled = 1
    ref, got = _both(p, q, k, v, o2, dO, lse2)
    assert all(torch.equal(a, b) for a, b in zip(ref, got))
    del bits
