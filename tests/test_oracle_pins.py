"""Pins of the CPU oracle (oracle/unfused_attention.py).

None of these re-types the oracle's formula: each check fixes a function
through a closed form, an independent library routine, brute force, or an
invariant that a dropped term / wrong sign / transposed operand would break.
The reference ships no golden vectors for this path, so these pins plus the
committed fixtures under tests/golden/ are what anchors parity.
"""
import numpy as np
import pytest
import scipy.special
import torch

from oracle import philox_dropout as phx
from oracle import unfused_attention as orc


def _rand(shape, seed, dtype=np.float16):
    return np.random.default_rng(seed).standard_normal(shape).astype(dtype)


# ---- forward -----------------------------------------------------------------
def test_fwd_all_ones_closed_form():
    # README example of the reference layer: all-ones q,k,v with a causal mask.
    # Every visible score equals D*scale, so P is uniform over the prefix:
    # O == 1 everywhere and L[i] = D*scale + ln(i+1).
    B, N, S, D = 1, 2, 96, 16
    one = np.ones((B, N, S, D), np.float16)
    mask = np.triu(np.ones((1, S, S), np.float32), 1)
    scale = 0.25
    O, L = orc.unfused_fwd(one, one, one, scale=scale, attn_mask=mask)
    assert np.allclose(O, 1.0, atol=1e-12)
    assert np.allclose(L[0, 0], D * scale + np.log(np.arange(S) + 1.0), atol=1e-9)
    O16, mid = orc.np_unfused_fwd_fp16(one, one, one, mask.astype(np.float16))
    assert np.allclose(O16.astype(np.float64), 1.0, atol=2e-3)
    assert np.allclose(orc.np_lse_from_mid(mid[3], mid[2])[0, 0], D + np.log(np.arange(S) + 1.0), atol=2e-2)


def test_fwd_zero_keys_gives_prefix_mean():
    B, N, S, D = 1, 1, 40, 8
    q, v = _rand((B, N, S, D), 0), _rand((B, N, S, D), 1)
    k = np.zeros_like(q)
    mask = np.triu(np.ones((1, S, S), np.float32), 1)
    O, L = orc.unfused_fwd(q, k, v, scale=1.0, attn_mask=mask)
    want = np.cumsum(v[0, 0].astype(np.float64), axis=0) / (np.arange(S)[:, None] + 1.0)
    assert np.allclose(O[0, 0], want, atol=1e-12)
    assert np.allclose(L[0, 0], np.log(np.arange(S) + 1.0), atol=1e-12)


def test_fwd_one_hot_logit_selects_value_row():
    # q = 30*e_0, k_j = e_0 only for j = 5: softmax is a delta at 5 -> O = v[5]
    S, D = 16, 8
    q = np.zeros((1, 1, S, D), np.float16); q[..., 0] = 30.0
    k = np.zeros((1, 1, S, D), np.float16); k[0, 0, 5, 0] = 2.0
    v = _rand((1, 1, S, D), 2)
    O, _ = orc.unfused_fwd(q, k, v)
    assert np.allclose(O[0, 0], np.broadcast_to(v[0, 0, 5].astype(np.float64), (S, D)), atol=1e-10)


def test_fwd_matches_torch_sdpa_and_logsumexp():
    B, N, Sq, Sk, D = 2, 3, 33, 47, 16
    q, k, v = _rand((B, N, Sq, D), 3), _rand((B, N, Sk, D), 4), _rand((B, N, Sk, D), 5)
    mask = (np.random.default_rng(6).random((B, Sq, Sk)) < 0.3).astype(np.float32)
    mask[:, :, 0] = 0
    bias = _rand((B, N, Sq, Sk), 7, np.float32) * 0.5
    scale = 0.3
    O, L = orc.unfused_fwd(q, k, v, scale=scale, attn_mask=mask, alibi=bias)
    add = torch.from_numpy(bias.astype(np.float64) - 10000.0 * mask[:, None].astype(np.float64))
    tq, tk, tv = (torch.from_numpy(x.astype(np.float64)) for x in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=add, scale=scale).numpy()
    assert np.allclose(O, want, atol=1e-10)
    s = scale * np.einsum("bnid,bnjd->bnij", q.astype(np.float64), k.astype(np.float64)) + add.numpy()
    assert np.allclose(L, scipy.special.logsumexp(s, axis=-1), atol=1e-10)


def test_fwd_additive_mask_is_not_minus_inf():
    # a fully masked row is the softmax of the raw scores (the -10000 cancels),
    # not NaN and not uniform: T/attention.py:357-371 adds, it does not select
    S, D = 8, 4
    q, k, v = _rand((1, 1, S, D), 8), _rand((1, 1, S, D), 9), _rand((1, 1, S, D), 10)
    mask = np.zeros((1, S, S), np.float32); mask[0, 3, :] = 1
    O, L = orc.unfused_fwd(q, k, v, attn_mask=mask)
    O0, L0 = orc.unfused_fwd(q, k, v)
    assert np.allclose(O[0, 0, 3], O0[0, 0, 3], atol=1e-9)
    assert np.allclose(L[0, 0, 3], L0[0, 0, 3] - 10000.0, atol=1e-6)


def test_fp16_restatement_tracks_fp64_spec():
    B, N, S, D = 2, 2, 64, 32
    q, k, v = (_rand((B, N, S, D), s) * 0.5 for s in (11, 12, 13))
    q, k, v = q.astype(np.float16), k.astype(np.float16), v.astype(np.float16)
    mask = np.triu(np.ones((1, S, S), np.float16), 1)
    O16, mid = orc.np_unfused_fwd_fp16(q, k, v, mask)
    O, L = orc.unfused_fwd(q, k, v, attn_mask=mask.astype(np.float32))
    assert np.max(np.abs(O16.astype(np.float64) - O)) < 5e-3
    assert np.max(np.abs(orc.np_lse_from_mid(mid[3], mid[2]) - L)) < 2e-2
    t = orc.torch_unfused_fwd_fp32(q, k, v).numpy().astype(np.float64)
    O_nomask, _ = orc.unfused_fwd(q, k, v)
    assert np.max(np.abs(t - O_nomask)) < 2e-3


def test_dropout_semantics_rowsum_before_dropout():
    # V = 1 -> O[i,:] = sum_j P[i,j]*drop[i,j]/keep: equals kept_mass/keep, not 1
    B, N, S, D = 1, 1, 32, 4
    q, k = _rand((B, N, S, D), 14), _rand((B, N, S, D), 15)
    v = np.ones((B, N, S, D), np.float16)
    drop = (np.random.default_rng(16).random((B, N, S, S)) < 0.7).astype(np.uint8)
    keep = 0.7
    O, L = orc.unfused_fwd(q, k, v, drop_mask=drop, keep_prob=keep)
    _, L_nodrop = orc.unfused_fwd(q, k, v)
    assert np.allclose(L, L_nodrop)                      # l and m ignore dropout
    s = q[0, 0].astype(np.float64) @ k[0, 0].astype(np.float64).T
    p = scipy.special.softmax(s, axis=-1)
    assert np.allclose(O[0, 0, :, 0], (p * drop[0, 0]).sum(-1) / keep, atol=1e-12)
    # V = I exposes the dropped positions exactly
    S2 = D2 = 16
    q2, k2 = _rand((1, 1, S2, D2), 17), _rand((1, 1, S2, D2), 18)
    eye = np.eye(S2, dtype=np.float16)[None, None]
    drop2 = (np.random.default_rng(19).random((1, 1, S2, S2)) < 0.5).astype(np.uint8)
    O2, _ = orc.unfused_fwd(q2, k2, eye, drop_mask=drop2, keep_prob=0.5)
    assert np.array_equal(O2[0, 0] == 0.0, drop2[0, 0] == 0)


def test_online_softmax_merge_and_tiling_invariance():
    # closed form of tests/train/flash_attention/ut/test_update_ML.py:68-72
    m, l = np.array([[1.0]]), np.array([[2.0]])
    mb, lb = np.array([[3.0]]), np.array([[0.5]])
    m2, l2 = orc.online_softmax_merge(m, l, mb, lb)
    assert m2[0, 0] == 3.0 and np.isclose(l2[0, 0], np.exp(-2.0) * 2.0 + 0.5)
    S, D = 200, 16
    q, k, v = _rand((S, D), 20), _rand((S, D), 21), _rand((S, D), 22)
    mask = np.triu(np.ones((S, S), np.float32), 1)
    ref_o, ref_l = orc.unfused_fwd(q[None, None], k[None, None], v[None, None], scale=0.2, attn_mask=mask[None])
    for blk in (7, 64, 128, 200):
        o, l = orc.tiled_fwd(q, k, v, scale=0.2, attn_mask=mask, block=blk)
        assert np.allclose(o, ref_o[0, 0], atol=1e-10) and np.allclose(l, ref_l[0, 0], atol=1e-10)


# ---- backward ----------------------------------------------------------------
def _loss_fp64(q, k, v, dO, **kw):
    O, _ = orc.unfused_fwd(q, k, v, **kw)
    return float(np.sum(O * dO))


def test_bwd_matches_finite_differences():
    B, N, Sq, Sk, D = 1, 2, 6, 9, 4
    rng = np.random.default_rng(23)
    q, k, v, dO = (rng.standard_normal(s) for s in ((B, N, Sq, D), (B, N, Sk, D), (B, N, Sk, D), (B, N, Sq, D)))
    mask = (rng.random((1, Sq, Sk)) < 0.3).astype(np.float64); mask[:, :, 0] = 0
    drop = (rng.random((B, N, Sq, Sk)) < 0.8).astype(np.uint8)
    bias = rng.standard_normal((1, N, 1, Sk))
    kw = dict(scale=0.7, attn_mask=mask, alibi=bias, drop_mask=drop, keep_prob=0.8)
    dQ, dK, dV = orc.unfused_bwd(q, k, v, dO, **kw)
    eps = 1e-6
    for name, x, g in (("q", q, dQ), ("k", k, dK), ("v", v, dV)):
        num = np.zeros_like(x)
        it = np.nditer(x, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            old = x[idx]
            x[idx] = old + eps; fp = _loss_fp64(q, k, v, dO, **kw)
            x[idx] = old - eps; fm = _loss_fp64(q, k, v, dO, **kw)
            x[idx] = old
            num[idx] = (fp - fm) / (2 * eps)
        assert np.allclose(g, num, atol=1e-6), name


def test_bwd_matches_torch_autograd_and_fa_identities():
    B, N, S, D = 2, 2, 24, 8
    rng = np.random.default_rng(24)
    q, k, v, dO = (rng.standard_normal((B, N, S, D)) for _ in range(4))
    mask = np.triu(np.ones((1, S, S)), 1)
    scale = 0.4
    dQ, dK, dV = orc.unfused_bwd(q, k, v, dO, scale=scale, attn_mask=mask)
    tq, tk, tv = (torch.tensor(x, requires_grad=True) for x in (q, k, v))
    s = scale * tq @ tk.transpose(-1, -2) - 10000.0 * torch.tensor(mask)[:, None]
    o = torch.softmax(s, -1) @ tv
    o.backward(torch.tensor(dO))
    assert np.allclose(dQ, tq.grad.numpy(), atol=1e-10)
    assert np.allclose(dK, tk.grad.numpy(), atol=1e-10)
    assert np.allclose(dV, tv.grad.numpy(), atol=1e-10)
    # the identity the reference's backward relies on (ST/common.py:156-169):
    # rowsum(P*dP) == rowsum(dO*O), hence rowsum(dS) == 0 without dropout
    p = torch.softmax(s, -1).detach().numpy()
    dP = dO @ np.swapaxes(v, -1, -2)
    O = p @ v
    assert np.allclose((p * dP).sum(-1), (dO * O).sum(-1), atol=1e-10)


def test_bwd_with_saved_output_is_the_same_function_of_exact_output():
    # O_saved = exact O must reproduce the plain gradient; a perturbed O moves dQ, dK only via D
    B, N, S, D = 1, 1, 12, 4
    rng = np.random.default_rng(41)
    q, k, v, dO = (rng.standard_normal((B, N, S, D)) for _ in range(4))
    O, _ = orc.unfused_fwd(q, k, v, scale=0.5)
    g0 = orc.unfused_bwd(q, k, v, dO, scale=0.5)
    g1 = orc.unfused_bwd(q, k, v, dO, scale=0.5, O_saved=O)
    assert all(np.allclose(a, b, atol=1e-12) for a, b in zip(g0, g1))
    g2 = orc.unfused_bwd(q, k, v, dO, scale=0.5, O_saved=O + 0.1)
    assert np.allclose(g2[2], g0[2]) and not np.allclose(g2[0], g0[0])
    # d(dQ)/dD = -scale * P k summed over keys: shift D by c = 0.1 * rowsum(dO)
    s = 0.5 * q[0, 0] @ k[0, 0].T
    p = scipy.special.softmax(s, -1)
    c = 0.1 * dO[0, 0].sum(-1, keepdims=True)
    assert np.allclose(g2[0][0, 0], g0[0][0, 0] - 0.5 * (p * c) @ k[0, 0], atol=1e-12)


def test_fp16_grad_restatement_tracks_fp64():
    B, N, S, D = 1, 2, 48, 16
    q, k, v, dO = (_rand((B, N, S, D), s) * 0.5 for s in (25, 26, 27, 28))
    q, k, v, dO = (x.astype(np.float16) for x in (q, k, v, dO))
    mask = np.triu(np.ones((1, S, S), np.float16), 1)
    O, (_, P, _, _) = orc.np_unfused_fwd_fp16(q, k, v, mask)
    g16 = orc.np_unfused_grad_fp16(q, k, v, P, O, dO)
    g64 = orc.unfused_bwd(q, k, v, dO, attn_mask=mask.astype(np.float32))
    for a, b in zip(g16, g64):
        assert np.max(np.abs(a.astype(np.float64) - b)) < 2e-2


# ---- band, tiling, masks -------------------------------------------------------
def test_band_predicates_brute_force():
    for Sq, Sk, prev, nxt in ((700, 900, 1, 2), (512, 512, 65536, 0), (300, 1000, 0, 0), (1000, 300, 2, 65536)):
        vis = orc.band_visible(Sq, Sk, prev, nxt)
        Tr, Tc = -(-Sq // 128), -(-Sk // 128)
        for qb in range(Tr):
            cnt = 0
            for kb in range(Tc):
                want = orc.band_block_visible(qb, kb, prev, nxt)
                blk = vis[qb * 128:(qb + 1) * 128, kb * 128:(kb + 1) * 128]
                assert blk.all() == want and blk.any() == want
                cnt += want
            if qb < Tc:      # the reference's count formula assumes the diagonal block exists
                assert cnt == orc.band_block_count(qb, Tc, prev, nxt)


def test_sparse_tiling_known_answers():
    assert orc.sparse_tiling(4096, 4096) == (128, 128, 128, 128, 32, 32)
    assert orc.sparse_tiling(200, 333) == (128, 72, 128, 77, 2, 3)
    assert orc.sparse_tiling(64, 100) == (64, 64, 100, 100, 1, 1)


def test_band_equals_explicit_mask():
    S, D = 384, 8
    q, k, v = _rand((1, 1, S, D), 29), _rand((1, 1, S, D), 30), _rand((1, 1, S, D), 31)
    vis = orc.band_visible(S, S, 1, 0)
    # absent keys == a mask so strong it underflows: use a -1e9 bias through alibi
    bias = np.where(vis, 0.0, -1e9)[None, None]
    O1, L1 = orc.unfused_fwd(q, k, v, prev_block_num=1, next_block_num=0)
    O2, L2 = orc.unfused_fwd(q, k, v, alibi=bias)
    assert np.allclose(O1, O2, atol=1e-12) and np.allclose(L1, L2, atol=1e-9)


def test_compact_causal_tile_equals_full_causal_with_block_skip():
    # T/flash_attention_fwd.py:353-356: the tile only ever touches diagonal blocks
    S, D = 300, 8
    q, k, v = _rand((1, 1, S, D), 32), _rand((1, 1, S, D), 33), _rand((1, 1, S, D), 34)
    tile = np.triu(np.ones((128, 128), np.float32), 1)
    dense = orc.expand_compact_causal_mask(tile, S, S)[None]
    full = np.triu(np.ones((1, S, S), np.float32), 1)
    O1, L1 = orc.unfused_fwd(q, k, v, attn_mask=dense, next_block_num=0)
    O2, L2 = orc.unfused_fwd(q, k, v, attn_mask=full)
    assert np.allclose(O1, O2, atol=1e-12) and np.allclose(L1, L2, atol=1e-9)


def test_triangle_attention_equals_dense_causal():
    # design of tests/train/triangle_attention/ut/test_triangle_attention.py:73-121,
    # divisible and non-divisible sequence lengths (scaled down)
    for S, bs in ((256, 64), (288, 64), (200, 128)):
        B, N, D = 2, 2, 8
        q, k, v = _rand((B, N, S, D), 35), _rand((B, N, S, D), 36), _rand((B, N, S, D), 37)
        mask = np.triu(np.ones((B, S, S), np.float32), 1)
        tri = orc.triangle_attention_fwd(q, k, v, mask, block_size=bs)
        dense, _ = orc.unfused_fwd(q, k, v, scale=1.0, attn_mask=mask)
        assert np.allclose(tri, dense, atol=1e-12)


def test_alibi_row_bias_equivalent_to_full_relative_bias():
    # slope*j differs from -slope*(i-j) by a per-row constant, which softmax removes
    B, N, S, D = 1, 4, 64, 8
    q, k, v = _rand((B, N, S, D), 38), _rand((B, N, S, D), 39), _rand((B, N, S, D), 40)
    sl = orc.alibi_slopes(N)
    assert np.isclose(sl[0], 2.0 ** (-8.0 / N)) and np.isclose(sl[-1], 2.0 ** -8.0)
    j = np.arange(S, dtype=np.float64)
    row = (sl[:, None] * j[None, :])[None, :, None, :]
    full = (-sl[:, None, None] * (j[:, None] - j[None, :]))[None]
    mask = np.triu(np.ones((1, S, S), np.float32), 1)
    O1, L1 = orc.unfused_fwd(q, k, v, scale=0.35, attn_mask=mask, alibi=row)
    O2, L2 = orc.unfused_fwd(q, k, v, scale=0.35, attn_mask=mask, alibi=full)
    assert np.allclose(O1, O2, atol=1e-10)
    assert np.allclose(L1 - L2, (sl[:, None] * j[None, :])[None], atol=1e-9)


def test_layer_scale_is_square_of_fp16_factor():
    assert np.isclose(orc.flash_attention_layer_scale(128), float(np.float16(128 ** -0.25)) ** 2)
    assert abs(orc.flash_attention_layer_scale(128) - 128 ** -0.5) < 1e-4


# ---- tolerance functions -----------------------------------------------------
def test_data_compare_hand_counts():
    gt = np.array([1.0, 2.0, 0.0, -4.0])
    pred = np.array([1.0 + 0.0019, 2.0 + 0.0031, 0.0009, -4.0 - 0.5])
    # thresholds rtol*|gt|+atol = .002, .003, .001, .005 -> violations: idx 1 and 3 (2 of 4)
    res, frac, frac_max = orc.data_compare(gt, pred)
    assert res == "Failed" and frac == 0.5
    # max bound 0.1*|gt|+atol = .101,.201,.001,.401 -> idx 3 violates
    assert frac_max == 0.25
    res, frac, frac_max = orc.data_compare(gt, gt + 1e-4)
    assert res == "Pass" and frac == 0.0 and frac_max == 0.0
    ok, ratio, mx = orc.tolerance_gate(gt, gt + np.array([0.0, 0.002, 0.0, 0.0]))
    assert ok and np.isclose(ratio, 0.002 / (2e-3 + 2e-3)) and np.isclose(mx, 0.002)
    ok, _, _ = orc.tolerance_gate(gt, gt + np.array([0.0, 0.0, 0.0021, 0.0]))
    assert not ok


# ---- counter-based dropout mask ---------------------------------------------------
def test_philox4x32_10_known_answers():
    # the known-answer vectors shipped with the Random123 library (kat_vectors, "philox4x32 10")
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        got = phx.philox4x32_10(np.array(ctr, dtype=np.uint32), key)
        assert tuple(int(x) for x in got) == want
    # vectorised over leading dimensions = one call per counter
    ctrs = np.array([k[0] for k in kat[:1]] * 3, dtype=np.uint32).reshape(3, 1, 4)
    assert np.array_equal(phx.philox4x32_10(ctrs, (0, 0))[2, 0], np.array(kat[0][2], dtype=np.uint32))


def test_dropout_keep_mask_layout_and_rate():
    B, N, Sq, Sk = 2, 3, 40, 100
    seed, off = (0xABCD << 32) | 0x1234, 9
    m = phx.dropout_keep_mask(B, N, Sq, Sk, seed, off, 0.75)
    assert m.shape == (B, N, Sq, Sk) and m.dtype == np.uint8 and set(np.unique(m)) <= {0, 1}
    # element by element from the definition in the C header, with scalar calls
    thr = phx.keep_threshold(0.75)
    assert thr == 192
    rng = np.random.default_rng(0)
    for _ in range(50):
        b, h, i, j = (int(rng.integers(n)) for n in (B, N, Sq, Sk))
        out = phx.philox4x32_10(np.array([i, 2 * (j // 32) + (j // 4) % 2, b * N + h, off], dtype=np.uint32),
                                (seed & 0xFFFFFFFF, seed >> 32))
        t = 4 * ((j // 8) % 4) + j % 4
        byte = (int(out[t // 4]) >> (8 * (t % 4))) & 0xFF
        assert m[b, h, i, j] == (1 if byte < thr else 0)
    # a different offset or seed gives a different mask; the keep rate is threshold / 256
    assert not np.array_equal(m, phx.dropout_keep_mask(B, N, Sq, Sk, seed, off + 1, 0.75))
    assert not np.array_equal(m, phx.dropout_keep_mask(B, N, Sq, Sk, seed + 1, off, 0.75))
    big = phx.dropout_keep_mask(1, 4, 256, 256, 42, 0, 0.9)
    assert abs(big.mean() - phx.keep_threshold(0.9) / 256) < 0.004
    assert phx.keep_threshold(1.0) == 256 and phx.keep_threshold(0.001) == 1
