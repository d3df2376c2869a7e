"""Writes tests/golden/fa_cases.npz: small seeded inputs and the outputs the CPU
oracle (oracle/unfused_attention.py, fp64) gives for them.

The reference ships no golden vectors for this path (its LFS test data is
absent and its tests draw unseeded random inputs), so these fixtures are made
here from the restated oracle, whose functions are pinned independently in
tests/test_oracle_pins.py.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import unfused_attention as orc  # noqa: E402

CASES = {
    # name: (B, N, Sq, Sk, D, options)
    "causal_d128": (1, 1, 256, 256, 128, dict(causal=True, next_block_num=0)),
    "ref_shape_d80": (1, 1, 128, 128, 80, dict(causal=True)),                 # ST/test_fa_fwd_precision.py:16
    "ragged_pad_drop_alibi_d64": (2, 2, 144, 200, 64, dict(pad=True, drop=0.9, alibi=True)),
    "band_d64": (1, 1, 384, 384, 64, dict(prev_block_num=1, next_block_num=0)),
}


def build(name, B, N, Sq, Sk, D, opt):
    rng = np.random.default_rng(sum(map(ord, name)))
    q = rng.standard_normal((B, N, Sq, D)).astype(np.float16)
    k = rng.standard_normal((B, N, Sk, D)).astype(np.float16)
    v = rng.standard_normal((B, N, Sk, D)).astype(np.float16)
    dO = rng.standard_normal((B, N, Sq, D)).astype(np.float16)
    scale = float(D) ** -0.5
    mask = drop = alibi = None
    keep = 1.0
    if opt.get("causal"):
        mask = np.triu(np.ones((1, Sq, Sk), np.uint8), 1)
    if opt.get("pad"):
        lens = rng.integers(Sk // 4, Sk + 1, size=B)
        mask = np.broadcast_to((np.arange(Sk)[None, None, :] >= lens[:, None, None]), (B, Sq, Sk)).astype(np.uint8).copy()
    if opt.get("drop"):
        keep = opt["drop"]
        drop = (rng.random((B, N, Sq, Sk)) < keep).astype(np.uint8)
    if opt.get("alibi"):
        sl = orc.alibi_slopes(N)
        alibi = (sl[None, :, None, None] * np.arange(Sk)[None, None, None, :]).astype(np.float16)
    kw = dict(scale=scale, attn_mask=mask, alibi=None if alibi is None else alibi.astype(np.float32),
              drop_mask=drop, keep_prob=keep,
              prev_block_num=opt.get("prev_block_num", 65536), next_block_num=opt.get("next_block_num", 65536))
    O, L = orc.unfused_fwd(q, k, v, **kw)
    dQ, dK, dV = orc.unfused_bwd(q, k, v, dO, **kw)
    out = dict(q=q, k=k, v=v, dO=dO, O=O.astype(np.float32), L=L.astype(np.float32),
               dQ=dQ.astype(np.float32), dK=dK.astype(np.float32), dV=dV.astype(np.float32),
               scale=np.float32(scale), keep_prob=np.float32(keep),
               prev_block_num=np.int32(kw["prev_block_num"]), next_block_num=np.int32(kw["next_block_num"]))
    if mask is not None:
        out["attn_mask"] = mask
    if drop is not None:
        out["drop_mask"] = np.packbits(drop, axis=-1)      # bit-packed along Sk to keep the file small
    if alibi is not None:
        out["alibi"] = alibi
    return {f"{name}/{key}": val for key, val in out.items()}


def main():
    blob = {}
    for name, (B, N, Sq, Sk, D, opt) in CASES.items():
        blob.update(build(name, B, N, Sq, Sk, D, opt))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fa_cases.npz")
    np.savez_compressed(path, **blob)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
