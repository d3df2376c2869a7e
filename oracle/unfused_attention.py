"""CPU oracle for the FlashAttention2 / TriangleAttention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
it exists so that tests, the smoke check and the benchmark's CPU-baseline leg
can compare the HIP kernels with the reference's own *unfused* attention
(BatchMatMul -> Softmax -> BatchMatMul) on identical inputs.

Every function restates, from the reference's text, the algorithm of the file
and lines it cites (paths are relative to the reference tree):

  ST = tests/train/flash_attention/st
  T  = train/acctransformer/flash_attention/ops/flash_attention
  L  = train/acctransformer/flash_attention/nn/layer
  TA = train/acctransformer/triangle_attention

Pinning status (what fixes each function independently of its own formula is
in tests/test_oracle_pins.py):

  np_unfused_fwd_fp16, np_unfused_grad_fp16 ... pinned by closed forms, scipy
      logsumexp / torch SDPA special cases and fp64 finite differences.
  unfused_fwd / unfused_bwd (the fp64 spec oracle) ... pinned the same way plus
      torch.autograd through an independent formulation.
  band_visible, sparse_tiling, band_block_count ... pinned by brute force.
  data_compare ... pinned by hand-computed counts.

What no test here can pin is the reference *device* kernel's rounding
(fp16 scores and running max, fp16 D, cube accumulation order): the reference
ships no golden vectors, so parity is defined against this unfused oracle
("parity unpinned" at the Ascend/CANN boundary only).
"""
from __future__ import annotations

import math

import numpy as np

MASK_FILL_VALUE = -10000.0      # T/constants.py:24 ; additive, not -inf
TILING_BLOCK_SIZE = 128         # T/constants.py:19 ; also the band granularity
BLOCK_NUM_UNBOUNDED = 65536     # L/flash_attention.py:95-96 defaults


# ----------------------------------------------------------------------------
# 1. Faithful restatements of the reference's numpy oracle (fp16 matmuls)
# ----------------------------------------------------------------------------
def np_unfused_fwd_fp16(Q, K, V, attn_mask=None, drop_mask=None):
    """ST/common.py:110-132 (np_impl_sa_fwd), statement by statement.

    Q,K,V fp16 [B,N,S,D]; attn_mask fp16 [1|B,S,S] with 1 = masked;
    drop_mask fp16 [B,N,S,S] holding {0, 1/keep_prob}.  Returns
    (O fp16, (Sim fp32 = exp(S - rowmax), P fp16, row_sum fp32, row_max fp16)).
    """
    sim = np.matmul(Q, np.transpose(K, (0, 1, 3, 2)))            # fp16 matmul
    if attn_mask is not None:
        sim = sim + np.expand_dims(MASK_FILL_VALUE * attn_mask, 1)
    row_max = np.max(sim, axis=-1, keepdims=True)
    sim = sim - row_max
    sim = np.exp(sim.astype("float32"))
    row_sum = np.sum(sim, axis=-1, keepdims=True)
    P = (sim / row_sum).astype("float16")
    if drop_mask is not None:
        P = P * drop_mask
    O = np.matmul(P, V)
    return O, (sim, P, row_sum, row_max)


def np_lse_from_mid(row_max, row_sum):
    """L = rowmax + ln(rowsum), as the reference's grad test builds it
    (ST/test_fa_grad_precision.py:35-36); the kernel-side definition is
    T/flash_attention_fwd.py:302-306."""
    l = row_max.astype("float32") + np.log(row_sum)
    return np.squeeze(l, axis=-1)


def np_unfused_grad_fp16(Q, K, V, P, O, dO, drop_mask=None):
    """ST/common.py:147-175 (np_impl_sa_grad): the FlashAttention form of the
    softmax gradient, D = rowsum(dO*O) rounded to fp16."""
    dV = np.matmul(np.transpose(P, (0, 1, 3, 2)), dO)
    dP = np.matmul(dO, np.transpose(V, (0, 1, 3, 2)))
    if drop_mask is not None:
        dP = dP * drop_mask
    d = np.sum((dO * O).astype("float32"), axis=-1, keepdims=True).astype("float16")
    dS = P * (dP - d)
    dQ = np.matmul(dS, K)
    dK = np.matmul(np.transpose(dS, (0, 1, 3, 2)), Q)
    return dQ, dK, dV


def torch_unfused_fwd_fp32(q, k, v):
    """tests/infer/flash_attention/tik/data_gen.py:32-34: softmax(q k^T) v in
    fp32 on the CPU, result rounded to fp16.  No scale, no mask."""
    import torch
    qf, kf, vf = (torch.as_tensor(x).float() for x in (q, k, v))
    s = torch.matmul(qf, kf.transpose(-1, -2))
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, vf).half()


def data_compare(ground_truth, predict, rtol=0.001, rtol_pct_thd=0.001, atol=0.001, max_rtol=0.1):
    """ST/common.py:178-192: pass iff at most rtol_pct_thd of the elements
    violate |d| <= rtol*|gt| + atol and none violates the max_rtol bound."""
    gt = np.asarray(ground_truth, dtype=np.float64)
    pr = np.asarray(predict, dtype=np.float64)
    diff = np.abs(pr - gt)
    total = gt.size
    over = np.sum(diff > rtol * np.abs(gt) + atol) / total
    over_max = np.sum(diff > max_rtol * np.abs(gt) + atol) / total
    ok = not (over > rtol_pct_thd or over_max > 0)
    return ("Pass" if ok else "Failed"), float(over), float(over_max)


def tolerance_gate(ground_truth, predict, atol=2e-3, rtol=1e-3):
    """The acceptance gate of this build: every element within
    atol + rtol*|gt| (max-abs 2e-3 / rtol 1e-3).  Returns (ok, worst excess
    ratio, max abs diff)."""
    gt = np.asarray(ground_truth, dtype=np.float64)
    pr = np.asarray(predict, dtype=np.float64)
    diff = np.abs(pr - gt)
    ratio = diff / (atol + rtol * np.abs(gt))
    return bool(np.all(ratio <= 1.0)), float(ratio.max(initial=0.0)), float(diff.max(initial=0.0))


# ----------------------------------------------------------------------------
# 2. Integer helpers: tiling and the block band
# ----------------------------------------------------------------------------
def sparse_tiling(Nq, N):
    """T/tiling_strategy/sparse_tiling.py:26-44: Br=min(128,Nq), Bc=min(128,N),
    ragged last tiles.  Returns (Br, last_Br, Bc, last_Bc, Tr, Tc)."""
    Br = min(TILING_BLOCK_SIZE, Nq)
    Bc = min(TILING_BLOCK_SIZE, N)
    Tr, Tc = -(-Nq // Br), -(-N // Bc)
    last_Br = Br if Nq % Br == 0 else Nq % Br
    last_Bc = Bc if N % Bc == 0 else N % Bc
    return Br, last_Br, Bc, last_Bc, Tr, Tc


def band_block_visible(q_blk, kv_blk, prev_block_num, next_block_num):
    """T/flash_attention_fwd.py:444-445 and T/flash_attention_bwd.py:299-300:
    block (q_blk, kv_blk) is computed iff
    kv_blk - next_block_num <= q_blk <= kv_blk + prev_block_num."""
    return kv_blk - next_block_num <= q_blk <= kv_blk + prev_block_num


def band_block_count(tr_idx, Tc, prev_block_num, next_block_num):
    """T/attention.py:162-167 (get_cur_tr_block_num)."""
    return min(tr_idx, prev_block_num) + 1 + min(next_block_num, Tc - tr_idx - 1)


def band_visible(Sq, Sk, prev_block_num, next_block_num):
    """Boolean [Sq,Sk]: True where the 128-row / 128-column block of (i, j)
    lies inside the band."""
    qb = (np.arange(Sq) // TILING_BLOCK_SIZE)[:, None]
    kb = (np.arange(Sk) // TILING_BLOCK_SIZE)[None, :]
    return (kb - next_block_num <= qb) & (qb <= kb + prev_block_num)


def expand_compact_causal_mask(tile, Sq, Sk):
    """The compact mask mode (T/attention.py:279-285,363-365 and
    T/flash_attention_fwd.py:353-356): one 128x128 tile that is applied only
    on blocks with q_blk == kv_blk.  Returns the equivalent dense [Sq,Sk]
    mask (zero away from the diagonal blocks)."""
    tile = np.asarray(tile).reshape(TILING_BLOCK_SIZE, TILING_BLOCK_SIZE)
    out = np.zeros((Sq, Sk), dtype=np.float32)
    for b in range(min(-(-Sq // 128), -(-Sk // 128))):
        r0, c0 = b * 128, b * 128
        r1, c1 = min(r0 + 128, Sq), min(c0 + 128, Sk)
        out[r0:r1, c0:c1] = tile[: r1 - r0, : c1 - c0]
    return out


# ----------------------------------------------------------------------------
# 3. The spec oracle: operator semantics in float64
# ----------------------------------------------------------------------------
def _scores(q, k, b, h, scale, attn_mask, alibi, visible):
    """fp64 scores of one (b,h): scale*q k^T + alibi + (-10000)*mask.
    Mask applied additively (T/attention.py:357-371), mask batch index
    broadcast when its leading dim is 1 (T/attention.py:270-277); alibi is
    [B,N,1,Sk] (L/flash_attention.py:185) or a full [B|1,N,Sq,Sk] bias."""
    s = scale * (q[b, h].astype(np.float64) @ k[b, h].astype(np.float64).T)
    if alibi is not None:
        ab = alibi[b if alibi.shape[0] > 1 else 0, h if alibi.shape[1] > 1 else 0].astype(np.float64)
        s = s + ab                                  # [1,Sk] or [Sq,Sk] broadcasts
    if attn_mask is not None:
        m = attn_mask[b if attn_mask.shape[0] > 1 else 0].astype(np.float64)
        s = s + MASK_FILL_VALUE * m
    if visible is not None:
        s = np.where(visible, s, -np.inf)           # outside the band: absent
    return s


def unfused_fwd(q, k, v, scale=1.0, attn_mask=None, alibi=None, drop_mask=None, keep_prob=1.0,
                prev_block_num=BLOCK_NUM_UNBOUNDED, next_block_num=BLOCK_NUM_UNBOUNDED):
    """Operator semantics of the forward kernel, evaluated unfused in fp64.

      S = scale*q k^T + alibi - 10000*mask          inside the block band
      m = rowmax S ; Pt = exp(S - m) ; l = rowsum Pt      (l BEFORE dropout,
                                                T/flash_attention_fwd.py:143-151)
      L = m + ln l                              (T/flash_attention_fwd.py:302-306)
      O = (Pt / l * drop / keep_prob) v         (T/attention.py:373-395)

    q [B,N,Sq,D]; k,v [B,N,Sk,D]; attn_mask [1|B,Sq,Sk] (nonzero = masked,
    value multiplies -10000); drop_mask [B,N,Sq,Sk] of {0,1}.
    Returns O fp64 [B,N,Sq,D] (unrounded) and L fp64 [B,N,Sq].
    """
    B, N, Sq, D = q.shape
    Sk = k.shape[2]
    dense_band = prev_block_num >= BLOCK_NUM_UNBOUNDED and next_block_num >= BLOCK_NUM_UNBOUNDED
    visible = None if dense_band else band_visible(Sq, Sk, prev_block_num, next_block_num)
    O = np.empty((B, N, Sq, D), dtype=np.float64)
    L = np.empty((B, N, Sq), dtype=np.float64)
    for b in range(B):
        for h in range(N):
            s = _scores(q, k, b, h, scale, attn_mask, alibi, visible)
            m = np.max(s, axis=-1, keepdims=True)
            pt = np.exp(s - m)
            l = np.sum(pt, axis=-1, keepdims=True)
            p = pt / l
            if drop_mask is not None:
                p = p * (drop_mask[b, h].astype(np.float64) / keep_prob)
            O[b, h] = p @ v[b, h].astype(np.float64)
            L[b, h] = (m + np.log(l))[:, 0]
    return O, L


def unfused_bwd(q, k, v, dO, scale=1.0, attn_mask=None, alibi=None, drop_mask=None, keep_prob=1.0,
                prev_block_num=BLOCK_NUM_UNBOUNDED, next_block_num=BLOCK_NUM_UNBOUNDED, O_saved=None):
    """Analytic gradient of unfused_fwd in fp64 (T/flash_attention_bwd.py:88-257):

      P = softmax(S) ; Pd = P*drop/keep ; dV = Pd^T dO ; dP = (dO v^T)*drop/keep
      D = rowsum(dO * O) ; dS = P*(dP - D) ; dQ = scale dS k ; dK = scale dS^T q

    With O_saved (the forward's rounded output) D is taken from it instead of
    the exact O: the "fa version" ground truth of ST/common.py:156-169, which
    the reference adopts because the rounding of the saved O otherwise
    dominates the comparison when the softmax is nearly one-hot.
    """
    B, N, Sq, D = q.shape
    Sk = k.shape[2]
    dense_band = prev_block_num >= BLOCK_NUM_UNBOUNDED and next_block_num >= BLOCK_NUM_UNBOUNDED
    visible = None if dense_band else band_visible(Sq, Sk, prev_block_num, next_block_num)
    dQ = np.empty(q.shape, dtype=np.float64)
    dK = np.empty(k.shape, dtype=np.float64)
    dV = np.empty(v.shape, dtype=np.float64)
    for b in range(B):
        for h in range(N):
            s = _scores(q, k, b, h, scale, attn_mask, alibi, visible)
            m = np.max(s, axis=-1, keepdims=True)
            pt = np.exp(s - m)
            p = pt / np.sum(pt, axis=-1, keepdims=True)
            dr = None if drop_mask is None else drop_mask[b, h].astype(np.float64) / keep_prob
            pd = p if dr is None else p * dr
            do = dO[b, h].astype(np.float64)
            vv = v[b, h].astype(np.float64)
            o = pd @ vv if O_saved is None else np.asarray(O_saved[b, h], dtype=np.float64)
            dV[b, h] = pd.T @ do
            dp = do @ vv.T
            if dr is not None:
                dp = dp * dr
            dd = np.sum(do * o, axis=-1, keepdims=True)
            ds = p * (dp - dd)
            dQ[b, h] = scale * (ds @ k[b, h].astype(np.float64))
            dK[b, h] = scale * (ds.T @ q[b, h].astype(np.float64))
    return dQ, dK, dV


def online_softmax_merge(m, l, m_blk, l_blk):
    """tests/train/flash_attention/ut/test_update_ML.py:68-72:
    m' = max(m, m~);  l' = e^{m-m'} l + e^{m~-m'} l~."""
    m_new = np.maximum(m, m_blk)
    l_new = np.exp(m - m_new) * l + np.exp(m_blk - m_new) * l_blk
    return m_new, l_new


def tiled_fwd(q, k, v, scale=1.0, attn_mask=None, block=128):
    """FlashAttention2 forward written as the reference kernel walks it
    (T/flash_attention_fwd.py:308-457: KV-tile loop with running m, l, O and a
    final O/l, L = m + ln l), in fp64.  Exists to show the merge rule is
    order- and tile-size-independent; single (b,h) slice API: q [Sq,D]."""
    Sq, D = q.shape
    Sk = k.shape[0]
    m = np.full((Sq, 1), -np.inf)
    l = np.zeros((Sq, 1))
    o = np.zeros((Sq, D))
    for j0 in range(0, Sk, block):
        s = scale * (q.astype(np.float64) @ k[j0:j0 + block].astype(np.float64).T)
        if attn_mask is not None:
            s = s + MASK_FILL_VALUE * attn_mask[:, j0:j0 + block].astype(np.float64)
        m_blk = np.max(s, axis=-1, keepdims=True)
        p = np.exp(s - m_blk)
        l_blk = np.sum(p, axis=-1, keepdims=True)
        m_new, l_new = online_softmax_merge(m, l, m_blk, l_blk)
        o = o * np.exp(m - m_new) + np.exp(m_blk - m_new) * (p @ v[j0:j0 + block].astype(np.float64))
        m, l = m_new, l_new
    return o / l, (m + np.log(l))[:, 0]


# ----------------------------------------------------------------------------
# 4. Layer-level compositions
# ----------------------------------------------------------------------------
def flash_attention_layer_scale(head_dim):
    """L/flash_attention.py:117,188-189: q and k are each multiplied by
    fp16(head_dim ** -0.25); the effective score scale is that value squared."""
    s = np.float16(1.0 / math.sqrt(math.sqrt(head_dim)))
    return float(s) * float(s)


def triangle_attention_fwd(q, k, v, attn_mask, block_size=512):
    """TA/triangle_attention.py:105-165: for row block i attend
    q[i*bs:(i+1)*bs] to k,v[0:(i+1)*bs] with mask slice * -10000 added, softmax,
    P v, concatenate; tail block when S % bs != 0.  No 1/sqrt(d) scale.
    fp64; attn_mask [B,S,S]."""
    B, N, S, D = q.shape
    out = np.empty((B, N, S, D), dtype=np.float64)
    groups, tail = divmod(S, block_size)
    spans = [(i * block_size, (i + 1) * block_size) for i in range(groups)]
    if tail > 0:
        spans.append((groups * block_size, S))
    for q0, q1 in spans:
        kv_end = q1
        for b in range(B):
            adder = MASK_FILL_VALUE * attn_mask[b if attn_mask.shape[0] > 1 else 0, q0:q1, 0:kv_end].astype(np.float64)
            for h in range(N):
                s = q[b, h, q0:q1].astype(np.float64) @ k[b, h, 0:kv_end].astype(np.float64).T + adder
                s = s - np.max(s, axis=-1, keepdims=True)
                p = np.exp(s)
                p = p / np.sum(p, axis=-1, keepdims=True)
                out[b, h, q0:q1] = p @ v[b, h, 0:kv_end].astype(np.float64)
    return out


def alibi_slopes(n_heads):
    """slope_h = 2^(-8(h+1)/n_heads) (the ALiBi configuration of the
    benchmark workload; the reference's own alibi path is dead code,
    T/attention.py:347-355)."""
    return np.array([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)], dtype=np.float64)
