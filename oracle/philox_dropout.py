"""CPU restatement of the counter-based dropout mask (TEST INFRASTRUCTURE ONLY).

Only tests, `__graft_entry__.smoke()` and the CPU-baseline leg of `bench.py`
may import this module; the product never does.

The reference draws its dropout mask with MindSpore's DropoutGenMask /
DropoutDoMask on a [B,N,Sq,Sk] tensor
(train/acctransformer/flash_attention/nn/layer/flash_attention.py:198-203);
that generator is a MindSpore/CANN component which is absent from the
reference tree, so its bit stream cannot be pinned ("parity unpinned" for the
random stream itself).  What the operator computes GIVEN a keep mask is pinned
by the masked-attention oracle (oracle/unfused_attention.py).  The mask used
here is defined by the C ABI (include/acct_fa.h, `drop_philox`): Philox4x32-10
(Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
SC'11), restated below from the paper and pinned by the known-answer vectors
of the Random123 distribution (tests/test_oracle_pins.py).
"""
from __future__ import annotations

import numpy as np

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """counter: uint32 [..., 4]; key: (k0, k1) python ints.  Returns uint32 [..., 4]."""
    c = np.asarray(counter, dtype=np.uint32).astype(np.uint64)
    c0, c1, c2, c3 = c[..., 0], c[..., 1], c[..., 2], c[..., 3]
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _M0 * c0                     # 32x32 -> 64, exact in uint64
        p1 = _M1 * c2
        n0 = (p1 >> np.uint64(32)) ^ c1 ^ np.uint64(k0)
        n2 = (p0 >> np.uint64(32)) ^ c3 ^ np.uint64(k1)
        c1 = p1 & _MASK32
        c3 = p0 & _MASK32
        c0, c2 = n0, n2
        k0 = (k0 + _W0) & 0xFFFFFFFF
        k1 = (k1 + _W1) & 0xFFFFFFFF
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def keep_threshold(keep_prob):
    """Bytes below this value keep the element; the probability actually used is threshold / 256."""
    return int(min(256, max(1, np.floor(256.0 * np.float32(keep_prob) + 0.5))))


def dropout_keep_mask(B, N, Sq, Sk, seed, offset, keep_prob):
    """uint8 [B,N,Sq,Sk] keep mask of `drop_philox` mode (include/acct_fa.h):
    counter = (i, 2*(j//32) + (j//4)%2, b*N + h, offset), key = (seed lo, seed hi),
    byte 4*((j//8)%4) + j%4 of the 16 output bytes, keep iff byte < threshold."""
    thr = keep_threshold(keep_prob)
    ngrp = (Sk + 31) // 32
    bh = np.arange(B * N, dtype=np.uint32)[:, None, None]
    i = np.arange(Sq, dtype=np.uint32)[None, :, None]
    c1 = np.arange(2 * ngrp, dtype=np.uint32)[None, None, :]
    ctr = np.empty((B * N, Sq, 2 * ngrp, 4), dtype=np.uint32)
    ctr[..., 0] = i
    ctr[..., 1] = c1
    ctr[..., 2] = bh
    ctr[..., 3] = np.uint32(int(offset) & 0xFFFFFFFF)
    out = philox4x32_10(ctr, (int(seed) & 0xFFFFFFFF, (int(seed) >> 32) & 0xFFFFFFFF))
    by = out.view(np.uint8).reshape(B * N, Sq, 2 * ngrp, 16)          # little endian: byte t of word t//4
    j = np.arange(Sk)
    grp = 2 * (j // 32) + (j // 4) % 2
    t = 4 * ((j // 8) % 4) + j % 4
    keep = by[:, :, grp, t] < thr
    return np.ascontiguousarray(keep.reshape(B, N, Sq, Sk), dtype=np.uint8)
