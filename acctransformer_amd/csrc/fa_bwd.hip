// FlashAttention2 backward for gfx950 (CDNA4): recompute-based, deterministic.
//
// Replaces the reference's backward kernel builder
// (train/acctransformer/flash_attention/ops/flash_attention/flash_attention_bwd.py:88-426:
// P recomputed from the saved L, D = rowsum(dO*O), dS = P*(dP - D), and
// dQ/dK/dV accumulated with fp32 atomics in global memory).  Here no atomics
// are used; the work is split in two kernels that each keep their
// accumulators in registers:
//
//   fa_bwd_dq_kernel   -- query-tile owner.  Also produces D (delta) for its
//                         rows.  S^T = K Q^T and dP^T = V dO^T put one query
//                         row per lane, dS^T is then directly the B operand of
//                         dQ^T += K^T dS^T (K^T via transposed LDS reads).
//   fa_bwd_dkdv_kernel -- kv-tile owner.  S = Q K^T and dP = dO V^T put one
//                         key row per lane (K, V fragments live in registers),
//                         P and dS are directly the B operands of
//                         dV^T += dO^T P and dK^T += Q^T dS.
#include "fa_common.hpp"
#include "fa_launch.hpp"

#include <type_traits>

namespace acct {
template <typename T>
ACCT_DEV typename Elem<T>::V8 pack8(const float* x) {
  using E = Elem<T>;
  typename E::V2 t0 = E::cvt2(x[0], x[1]), t1 = E::cvt2(x[2], x[3]), t2 = E::cvt2(x[4], x[5]), t3 = E::cvt2(x[6], x[7]);
  typename E::V8 r = {t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
  return r;
}

// ============================================================================
// dQ kernel (and delta): query-tile owner, structure of the forward kernel
// ============================================================================
template <typename T, int D, int QG, int NW, bool BIAS, bool DROP, bool MASKT>
ACCT_DEV void fa_bwd_dq_body(const FaArgs& a) {
  using E = Elem<T>;
  using V8 = typename E::V8;
  using C = SwzCfg<D>;
  constexpr int BM = 32 * QG * NW;
  constexpr int TILEB = 64 * C::PITCH;
  constexpr int FRING = 4, TRING = 3;                     // fragment reads in flight ahead of their MFMA (row-major / transposed)
  constexpr bool RINGS = !(BIAS || DROP);                 // (the side-input variants have no registers for the rings)   // fragment reads in flight ahead of their MFMA (row-major / transposed)
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;   // [2 buffers][K tile | V tile]; reused by the epilogue

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: everything derived from it stays in scalar registers
  const int BH = a.B * a.N;
  int bh, rank;
  wg_map(blockIdx.x, BH, a.n_tiles, bh, rank);
  const int qt = a.n_tiles - 1 - rank;
  const int b = bh / a.N, h = bh % a.N;
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * 32 * QG;
  const int q_end = min(q0 + BM, a.Sq);
  const int wq_end = min(wq0 + 32 * QG, a.Sq);

  const T* qp = (const T*)a.q + b * a.q_sb + h * a.q_sh;
  const T* kp = (const T*)a.k + b * a.k_sb + h * a.k_sh;
  const T* vp = (const T*)a.v + b * a.v_sb + h * a.v_sh;
  const T* op = (const T*)a.o + b * a.o_sb + h * a.o_sh;
  const T* dop = (const T*)a.dout + b * a.o_sb + h * a.o_sh;

  const int qb_lo = q0 / 128, qb_hi = (q_end - 1) / 128;
  const int kvb_lo = max(0, qb_lo - a.prev_blk), kvb_hi = min(a.Tc - 1, qb_hi + a.next_blk);
  int j_lo = kvb_lo * 2, j_hi = min(kvb_hi * 2 + 1, (a.Sk - 1) / 64);
  const bool causal = a.mask_kind == kMaskCausal;
  if (causal) j_hi = min(j_hi, (q_end - 1) / 64);
  if (a.row_prefix) j_hi = min(j_hi, (((q_end - 1) / a.row_prefix + 1) * a.row_prefix - 1) / 64);
  const int wqb = wq0 / 128;
  BlkClassWindow flwin;                                     // block classes of a dense mask: 64 blocks at a time in scalar registers
  bool flwin_ready = false;
  if (MASKT && a.mask_kind == kMaskDense) {
    // tiles at either end whose 128x128 blocks are wholly masked for every row block of this workgroup are
    // not streamed at all (key padding: the padded tail of every sequence).  With at most 64 blocks in the
    // band, one round trip to memory yields both the trimmed range and the wave's class window.
    const uint8_t* fl = a.blkflags + ((int64_t)(a.mask_sb ? b : 0) * a.Tr) * a.Tc;
    int b_lo = j_lo >> 1, b_hi = j_hi >> 1;
    // (the dropout variants have no register to spare for the key tails -- one more spill costs them 5 % on every
    // tile -- and read such blocks as mask bytes)
    const uint8_t* tails = a.blktail ? a.blktail + ((int64_t)(a.mask_sb ? b : 0) * a.Tr) * a.Tc : nullptr;
    if (j_lo <= j_hi && flwin.init_trimmed(fl, 1, a.Tc, qb_lo, qb_hi - qb_lo + 1, min(wqb, qb_hi), b_lo, b_hi, lane, tails)) {
      j_lo = max(j_lo, b_lo * 2);
      j_hi = min(j_hi, b_hi * 2 + 1);
      flwin_ready = true;
    } else {
      auto dead = [&](int j) {
        for (int qb = qb_lo; qb <= qb_hi; qb++)
          if (fl[(int64_t)qb * a.Tc + (j >> 1)] != kBlkSkip) return false;
        return true;
      };
      trim_dead_tiles(j_lo, j_hi, lane, dead);
    }
  }
  const int wkv_limit = a.row_prefix ? (wq0 / a.row_prefix + 1) * a.row_prefix : 0x7fffffff;

  // Q and dO fragments (B operands), delta and L of the lane's query row
  V8 qf[QG][C::KS], dof[QG][C::KS];
  float dl[QG], lq[QG];
#pragma unroll
  for (int gq = 0; gq < QG; gq++) {
    const int row = wq0 + 32 * gq + l32;
    const int row_c = min(row, a.Sq - 1);
    float part = 0.f;
#pragma unroll
    for (int t = 0; t < C::KS; t++) {
      // k-steps (or the upper half of one) past the head dim: zeros there make the products
      // ignore whatever the K / V tiles hold in that slot
      const bool inside = 16 * t + 8 * g < a.hd;
      V8 z;
#pragma unroll
      for (int e = 0; e < 8; e++) z[e] = 0;
      qf[gq][t] = inside ? *reinterpret_cast<const V8*>(qp + (int64_t)row_c * a.q_ss + 16 * t + 8 * g) : z;
      dof[gq][t] = inside ? *reinterpret_cast<const V8*>(dop + (int64_t)row_c * a.o_ss + 16 * t + 8 * g) : z;
      const V8 ov = inside ? *reinterpret_cast<const V8*>(op + (int64_t)row_c * a.o_ss + 16 * t + 8 * g) : z;
#pragma unroll
      for (int e = 0; e < 8; e++) part += (float)dof[gq][t][e] * (float)ov[e];
    }
    dl[gq] = pair_sum(part);
    lq[gq] = INFINITY;                                   // rows past Sq: P = exp2(x - inf) = 0
    if (row < a.Sq) {
      // (minus p_shift: the recomputed probabilities carry a factor 2^p_shift, see FaArgs)
      lq[gq] = a.lse[(int64_t)bh * a.Sq + row] * kLog2e - a.p_shift;
      if (g == 0) {
        a.delta[(int64_t)bh * a.Sq + row] = dl[gq];
        a.nlse[(int64_t)bh * a.Sq + row] = -lq[gq];        // p_shift - LSE*log2(e): the exp2 offset the dK/dV kernel adds
      }
    }
  }

  // per-lane LDS offsets (tile-invariant)
  // row-major fragment of k-step t: row l32, chunk 2t + g.  Chunk c + 8 of a row sits in slot (c ^ swz) ^ 8, so the
  // offsets of the upper parts of a wide head dim are one XOR away from the first four.
  constexpr int NKOFF = (C::CH >= 16 && C::KS > 8) ? 4 : C::KS;
  int koff_[NKOFF];
#pragma unroll
  for (int t = 0; t < NKOFF; t++) koff_[t] = l32 * C::PITCH + swz_off(2 * t + g, C::swz(l32));
  auto koff = [&](int t) { return t < NKOFF ? koff_[t] : (koff_[t & 3] ^ ((t >> 2) * 128)); };
  const int trow = 4 * g + ((lane & 15) >> 2);
  const int tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
  int toff[C::DB];
#pragma unroll
  for (int db = 0; db < C::DB; db++) toff[db] = trow * C::PITCH + swz_off(4 * db + tchunk, C::swz(trow)) + 8 * (lane & 1);

  f32x16 acc[QG][C::DB];
#pragma unroll
  for (int gq = 0; gq < QG; gq++)
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[gq][db][r] = 0.f;

  const int mb = a.mask_sb ? b : 0;
  const uint8_t* maskp = a.mask ? a.mask + (a.mask_kind == kMaskDense ? (int64_t)mb * a.mask_sb * a.mask_es : 0) : nullptr;
  const T* alibip = BIAS ? (const T*)a.alibi + b * a.al_sb + h * a.al_sh : nullptr;
  const bool mask_vec = a.mask_kind == kMaskDense ? ((((uintptr_t)a.mask / a.mask_es) | (uintptr_t)a.Sk | (uintptr_t)a.mask_sb) & 3) == 0
                                                  : ((uintptr_t)a.mask & (4 * a.mask_es - 1)) == 0;
  const bool alibi_vec = BIAS && (((uintptr_t)a.alibi & 7) | ((a.al_sb | a.al_sh | a.al_sq) & 3)) == 0;

  TileDma<T, D, 64, NW> kdma, vdma;
  const int cpr = a.hd >> 3;                                // valid 16-byte chunks per row
  kdma.plan(a.k_ss, cpr);
  vdma.plan(a.v_ss, cpr);
  // bias tiles of this wave's rows are staged through a wave-private LDS region one tile ahead
  ACCT_LDS char* bias_lds = smem + 4 * TILEB + wave * (QG * 4096);
  const bool bias_staged = BIAS && (a.Sk & 7) == 0 && (((uintptr_t)a.alibi & 15) | ((a.al_sb | a.al_sh | a.al_sq) & 7)) == 0;
  const bool row_bias = BIAS && a.al_sq == 0;            // the bias depends on the key only: one 128-byte row per tile
  auto stage_bias = [&](int jn) {
#pragma unroll
    for (int gq = 0; gq < QG; gq++) {
      if (row_bias) bias_row_dma<T>(alibip, jn * 64, a.Sk, bias_lds + gq * 4096);
      else bias_tile_dma<T>(alibip, a.al_sq, wq0 + 32 * gq, a.Sq, jn * 64, a.Sk, bias_lds + gq * 4096);
    }
  };
  // keep bits of this wave's rows and one tile, staged with the tile's DMA (double buffered)
  using DropStage = DropRowStage<DROP, QG, 2>;
  ACCT_LDS char* drop_lds = smem + 4 * TILEB + (BIAS ? NW * QG * 4096 : 0) + wave * (2 * DropStage::BYTES);
  if (j_lo <= j_hi) {
    tile_dma<T, D, 64, NW>(kp, a.k_ss, j_lo * 64, a.Sk, smem, a.hd >> 3);
    tile_dma<T, D, 64, NW>(vp, a.v_ss, j_lo * 64, a.Sk, smem + TILEB, a.hd >> 3);
    if (BIAS && bias_staged && wq0 < a.Sq) stage_bias(j_lo);
    DropStage::issue(a, bh, wq0, j_lo, lane, drop_lds);
    // A full wait the compiler can see: every load issued so far (Q, dO fragments included) is complete,
    // so it places no vmcnt wait inside the loop -- such a wait would also stall on the next tile's DMA.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    // block classes of a dense mask: 64 blocks at a time into scalar registers
    const uint8_t* flrow = (MASKT && a.mask_kind == kMaskDense) ? a.blkflags + ((int64_t)mb * a.Tr + wqb) * a.Tc : nullptr;
    if (!flwin_ready) flwin.init(flrow, 1, j_lo >> 1, j_hi >> 1, lane, (flrow && a.blktail) ? a.blktail + (flrow - a.blkflags) : nullptr);
    for (int j = j_lo; j <= j_hi; j++) {
      const uint32_t fl_cur = flwin.get(j >> 1, lane);
      const int buf = (j - j_lo) & 1;
      ACCT_LDS char* kbuf = smem + buf * 2 * TILEB;
      ACCT_LDS char* vbuf = kbuf + TILEB;
      if (j < j_hi) {
        ACCT_LDS char* nb = smem + (buf ^ 1) * 2 * TILEB;
        if ((j + 2) * 64 <= a.Sk) {
          kdma.issue(kp, a.k_ss, (j + 1) * 64, nb);
          vdma.issue(vp, a.v_ss, (j + 1) * 64, nb + TILEB);
        } else {                                            // ragged last tile: clamped rows
          tile_dma<T, D, 64, NW>(kp, a.k_ss, (j + 1) * 64, a.Sk, nb, a.hd >> 3);
          tile_dma<T, D, 64, NW>(vp, a.v_ss, (j + 1) * 64, a.Sk, nb + TILEB, a.hd >> 3);
        }
        DropStage::issue(a, bh, wq0, j + 1, lane, drop_lds + (buf ^ 1) * DropStage::BYTES);
      }
      const int kv0 = j * 64;
      const int kvb = j >> 1;
      bool act = (kvb - a.next_blk <= wqb) && (wqb <= kvb + a.prev_blk) && (wq0 < a.Sq);
      if (causal) act = act && (kv0 <= wq_end - 1);
      act = act && (kv0 < wkv_limit);
      bool apply_mask = false;
      bool diag = causal;                                   // keys after the query are hidden, by index compare
      int last_key = a.Sk - 1;                              // last key that exists and is not behind a key tail
      if (MASKT && a.mask_kind == kMaskDense && act) {
        act = fl_cur != kBlkSkip;
        apply_mask = fl_cur == kBlkApply;
        if (fl_cur == kBlkTriu) { diag = true; act = kv0 <= wq_end - 1; }
        if (apply_mask) {
          const int tail = (int)flwin.tail(kvb);
          if (tail) {
            // every row of the block hides exactly the keys from its tail-th on: an index compare, no mask loads
            apply_mask = false;
            last_key = min(last_key, kvb * 128 + tail - 1);
            act = kv0 <= last_key;
          }
        }
      } else if (MASKT && a.mask_kind == kMaskTile) {
        apply_mask = wqb == kvb;
      }
      const bool edge = apply_mask || (diag && (kv0 + 63 > wq0)) || (kv0 + 63 > last_key);
      if (act) {
        V8 dsf[QG][2][2];
#pragma unroll
        for (int c = 0; c < 2; c++) {
          f32x16 s[QG], dp[QG];
#pragma unroll
          for (int gq = 0; gq < QG; gq++) {
            if (BIAS && bias_staged) {
              // the bias enters as the initial value of the score accumulators (bias / scale, the MFMAs add
              // q.k): nothing per score afterwards, no bias registers alive next to the scores
              typename E::V4 bv[4];
#pragma unroll
              for (int r4 = 0; r4 < 4; r4++) bv[r4] = bias_tile_read<T>(bias_lds + gq * 4096, row_bias ? 0 : l32, 4 * c + r4, g);
#pragma unroll
              for (int r = 0; r < 16; r++) s[gq][r] = (float)bv[r >> 2][r & 3] * a.inv_scale;
            } else {
#pragma unroll
              for (int r = 0; r < 16; r++) s[gq][r] = 0.f;
            }
#pragma unroll
            for (int r = 0; r < 16; r++) dp[gq][r] = 0.f;
          }
          if constexpr (RINGS) {
            // K and V fragments of the chunk travel through a ring of FRING register sets (FRING reads in
            // flight ahead of the MFMA that consumes the oldest); S and dP MFMAs alternate.  The scheduling
            // barriers keep the compiler from folding the ring back into read-wait-MFMA.
            constexpr int NF = 2 * C::KS;
            auto faddr = [&](int i) { return ((i & 1) ? vbuf : kbuf) + koff(i >> 1) + c * 32 * C::PITCH; };
            V8 ring[FRING];
#pragma unroll
            for (int i = 0; i < FRING; i++) ring[i] = lds_read_frag<T>(faddr(i));
#pragma unroll
            for (int i = 0; i < NF; i++) {
              const int t = i >> 1;
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int gq = 0; gq < QG; gq++) {
                if (i & 1) dp[gq] = E::mfma(ring[i % FRING], dof[gq][t], dp[gq]);
                else s[gq] = E::mfma(ring[i % FRING], qf[gq][t], s[gq]);
              }
              if (i + FRING < NF) ring[i % FRING] = lds_read_frag<T>(faddr(i + FRING));
            }
            __builtin_amdgcn_sched_barrier(0);
          } else {
            V8 kf[C::KS], vf[C::KS];
#pragma unroll
            for (int t = 0; t < C::KS; t++) kf[t] = lds_read_frag<T>(kbuf + koff(t) + c * 32 * C::PITCH);
#pragma unroll
            for (int t = 0; t < C::KS; t++) vf[t] = lds_read_frag<T>(vbuf + koff(t) + c * 32 * C::PITCH);
#pragma unroll
            for (int t = 0; t < C::KS; t++)
#pragma unroll
              for (int gq = 0; gq < QG; gq++) s[gq] = E::mfma(kf[t], qf[gq][t], s[gq]);
#pragma unroll
            for (int t = 0; t < C::KS; t++)
#pragma unroll
              for (int gq = 0; gq < QG; gq++) dp[gq] = E::mfma(vf[t], dof[gq][t], dp[gq]);
          }
          if (BIAS && bias_staged && c == 1) {
            // the whole bias tile has been read and the reads consumed: its LDS region can take the next
            // tile, which has the rest of this step to land (the end-of-step wait covers it)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (j < j_hi) stage_bias(j + 1);
          }
          // element (gq, r): q = wq0 + 32 gq + l32 ; kv = kv0 + 32 c + 8 (r/4) + 4 g + r%4
#pragma unroll
          for (int gq = 0; gq < QG; gq++) {
            const int qrow = wq0 + 32 * gq + l32;
            const int qrow_c = min(qrow, a.Sq - 1);
            float ds[16];
            const bool bias_pending = BIAS && !bias_staged;  // (a staged bias is already inside s)
            if (!edge && !bias_pending && !DROP) {           // interior tile: no side inputs at all
#pragma unroll
              for (int r = 0; r < 16; r++) {
                const float p = fast_exp2(__builtin_fmaf(s[gq][r], a.scale_log2e, -lq[gq]));
                ds[r] = p * (dp[gq][r] - dl[gq]);
              }
            } else if (!apply_mask && !bias_pending && !DROP) {
              // causal diagonal and/or ragged key tail only: P of a hidden key is exactly 0 (with the
              // additive mask it underflows to the same value), one compare and select per element
              int vis = last_key - kv0 - 32 * c - 4 * g;         // last visible key, relative to this lane's first
              if (diag) vis = min(vis, qrow - kv0 - 32 * c - 4 * g);
#pragma unroll
              for (int r = 0; r < 16; r++) {
                float p = fast_exp2(__builtin_fmaf(s[gq][r], a.scale_log2e, -lq[gq]));
                if (8 * (r >> 2) + (r & 3) > vis) p = 0.f;
                ds[r] = p * (dp[gq][r] - dl[gq]);
              }
            } else {
              // side inputs, in short passes over the 16 scores so that few values are live at a time
              float x[16];
#pragma unroll
              for (int r = 0; r < 16; r++) x[r] = __builtin_fmaf(s[gq][r], a.scale_log2e, -lq[gq]);
              if (BIAS && !bias_staged) {                    // a bias the DMA cannot stage (alignment): direct loads
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                  float bias[4];
                  load_bias4<T>(alibip + (int64_t)qrow_c * a.al_sq, kv0 + 32 * c + 8 * r4 + 4 * g, a.Sk, alibi_vec, bias);
#pragma unroll
                  for (int e = 0; e < 4; e++) x[4 * r4 + e] = __builtin_fmaf(bias[e], kLog2e, x[4 * r4 + e]);
                }
              }
              if (apply_mask) {
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                  const int kv = kv0 + 32 * c + 8 * r4 + 4 * g;
                  uint32_t mbits;
                  if (a.mask_kind == kMaskDense) mbits = load_mask4(maskp + (int64_t)qrow_c * a.Sk * a.mask_es, kv, a.Sk, mask_vec, a.mask_es);
                  else mbits = load_mask4(maskp + (qrow_c & 127) * 128 * a.mask_es, kv & 127, 128, mask_vec, a.mask_es);
#pragma unroll
                  for (int e = 0; e < 4; e++)
                    if ((mbits >> (8 * e)) & 0xffu) x[4 * r4 + e] += kMaskFill * kLog2e;
                }
              }
              if ((diag && (kv0 + 63 > wq0)) || (kv0 + 63 > last_key)) {
                // keys after the query (causal), past Sk or behind a key tail: P is exactly 0
                int vis = last_key - kv0 - 32 * c - 4 * g;
                if (diag) vis = min(vis, qrow - kv0 - 32 * c - 4 * g);
#pragma unroll
                for (int r = 0; r < 16; r++)
                  if (8 * (r >> 2) + (r & 3) > vis) x[r] = -INFINITY;
              }
              uint32_t dw = 0xffffffffu;                        // keep bits of this row: keys kv0 + 32c .. +31
              if (DROP) dw = DropStage::word(drop_lds + buf * DropStage::BYTES, 32 * gq + l32, c) >> (4 * g);
#pragma unroll
              for (int r = 0; r < 16; r++) {
                const float p = fast_exp2(x[r]);
                if (DROP) {
                  // dP of a dropped key is 0, of a kept one dP / keep_prob: a one-bit signed field extract gives
                  // the all-ones / all-zeros mask, and the scaling rides on the FMA that subtracts D
                  const float dpk = __uint_as_float(__float_as_uint(dp[gq][r]) & (uint32_t)__builtin_amdgcn_sbfe((int)dw, 8 * (r >> 2) + (r & 3), 1));
                  ds[r] = p * __builtin_fmaf(dpk, a.inv_keep, -dl[gq]);
                } else {
                  ds[r] = p * (dp[gq][r] - dl[gq]);
                }
              }
            }
            dsf[gq][c][0] = pack8<T>(ds);
            dsf[gq][c][1] = pack8<T>(ds + 8);
          }
        }
        // ---- dQ^T += K^T dS^T : transposed K fragments through a ring of TRING register sets ----
        if constexpr (RINGS) {
          constexpr int NT = 4 * C::DB;
          auto tread = [&](int i) {
            const int db = i % C::DB, ch = i / C::DB;           // ch = 2 c + hh: rows 16 ch .. of the tile
            const ACCT_LDS char* kaddr = kbuf + toff[db] + 16 * ch * C::PITCH;
            return join_tr<T>(lds_read_tr(kaddr), lds_read_tr(kaddr + C::tr_hi(db)));
          };
          V8 ring[TRING];
#pragma unroll
          for (int i = 0; i < TRING; i++) ring[i] = tread(i);
#pragma unroll
          for (int i = 0; i < NT; i++) {
            const int db = i % C::DB, ch = i / C::DB;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int gq = 0; gq < QG; gq++) acc[gq][db] = E::mfma(ring[i % TRING], dsf[gq][ch >> 1][ch & 1], acc[gq][db]);
            if (i + TRING < NT) ring[i % TRING] = tread(i + TRING);
          }
          __builtin_amdgcn_sched_barrier(0);
        } else {
#pragma unroll
          for (int c = 0; c < 2; c++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++)
#pragma unroll
              for (int db = 0; db < C::DB; db++) {
                const ACCT_LDS char* kaddr = kbuf + toff[db] + (32 * c + 16 * hh) * C::PITCH;
                const V8 ktf = join_tr<T>(lds_read_tr(kaddr), lds_read_tr(kaddr + C::tr_hi(db)));
#pragma unroll
                for (int gq = 0; gq < QG; gq++) acc[gq][db] = E::mfma(ktf, dsf[gq][c][hh], acc[gq][db]);
              }
        }
      } else if (BIAS && bias_staged && j < j_hi && wq0 < a.Sq) {
        stage_bias(j + 1);                                  // nothing to read in this step: the region is free
      }
      dma_wait();
      __syncthreads();
    }
  }

  // ---- epilogue: dQ = scale * dQ^T, transposed through the wave's own LDS region ----
  const float dq_scale = a.scale * a.p_unshift;
  T* dqp = (T*)a.dq + b * a.q_sb + h * a.q_sh;
  constexpr int OPITCH = C::DB * 64 + 16;
  ACCT_LDS char* obuf = smem + wave * (32 * OPITCH);
#pragma unroll
  for (int gq = 0; gq < QG; gq++) {
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        typename E::V2 t0 = E::cvt2(acc[gq][db][4 * r4 + 0] * dq_scale, acc[gq][db][4 * r4 + 1] * dq_scale);
        typename E::V2 t1 = E::cvt2(acc[gq][db][4 * r4 + 2] * dq_scale, acc[gq][db][4 * r4 + 3] * dq_scale);
        typename E::V4 ov = {t0[0], t0[1], t1[0], t1[1]};
        *reinterpret_cast<ACCT_LDS typename E::V4*>(obuf + l32 * OPITCH + (32 * db + 8 * r4 + 4 * g) * 2) = ov;
      }
    const int nch = a.hd >> 3;                       // valid 16-byte chunks per row
    const uint32_t nch_inv = recip16(nch);
#pragma unroll
    for (int i = 0; i < (32 * C::CPR + 63) / 64; i++) {
      const int idx = lane + 64 * i;
      const int r = div_small(idx, nch_inv), ch = idx - r * nch;
      const int grow = wq0 + 32 * gq + r;
      if (idx < 32 * nch && grow < a.Sq) {
        const u32x4 v = *reinterpret_cast<const ACCT_LDS u32x4*>(obuf + r * OPITCH + ch * 16);
        *reinterpret_cast<u32x4*>(dqp + (int64_t)grow * a.q_ss + ch * 8) = v;
      }
    }
  }
}

// The variant that knows mask tensors but neither a bias nor dropout carries a second body: a workgroup whose
// rows see nothing but the causal pattern in a dense mask (block classes: clean before the diagonal, the
// causal diagonal, skipped after it) runs the code of the variant without side inputs, by index compare.
template <typename T, int D, int QG, int NW, bool BIAS, bool DROP, bool MASKT>
__global__ void __launch_bounds__(64 * NW) fa_bwd_dq_kernel(const FaArgs a) {
  if constexpr (MASKT && !BIAS && !DROP) {
    if (a.mask_kind == kMaskDense) {
      constexpr int BM = 32 * QG * NW;
      int bh, rank;
      wg_map(blockIdx.x, a.B * a.N, a.n_tiles, bh, rank);
      const int q0 = (a.n_tiles - 1 - rank) * BM, q_end = min(q0 + BM, a.Sq);
      const int qb_lo = q0 / 128, qb_hi = (q_end - 1) / 128;
      const int kvb_lo = max(0, qb_lo - a.prev_blk), kvb_hi = min(a.Tc - 1, qb_hi + a.next_blk);
      const uint8_t* fl = a.blkflags + ((int64_t)(a.mask_sb ? bh / a.N : 0) * a.Tr) * a.Tc;
      if (dense_lines_are_causal(fl, 1, a.Tc, qb_lo, qb_hi - qb_lo + 1, kvb_lo, kvb_hi, false, a, threadIdx.x & 63)) {
        FaArgs c = a;
        c.mask_kind = kMaskCausal;
        fa_bwd_dq_body<T, D, QG, NW, false, false, false>(c);
        return;
      }
    }
  }
  fa_bwd_dq_body<T, D, QG, NW, BIAS, DROP, MASKT>(a);
}

// Epilogue of the dK/dV kernel: dV (V role) or dK (K role) of a wave's key rows, scaled, converted and transposed
// through the wave's own LDS region so that the global stores are whole rows.  acc[gk][db] = [d rows of block db,
// key column l32] of key group gk; wk0 = first key row of the wave's pair.
template <typename T, int D, int NGK>
ACCT_DEV void dkdv_store_rows(const f32x16 (&acc)[NGK][SwzCfg<D>::DB], const FaArgs& a, int b, int h, int wk0, bool krole,
                              float oscale, ACCT_LDS char* smem) {
  using E = Elem<T>;
  using C = SwzCfg<D>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, g = lane >> 5;
  T* outp = krole ? (T*)a.dk + b * a.k_sb + h * a.k_sh : (T*)a.dv + b * a.v_sb + h * a.v_sh;
  const int64_t oss = krole ? a.k_ss : a.v_ss;
  constexpr int OPITCH = C::DB * 64 + 16;
  ACCT_LDS char* obuf = smem + wave * (32 * OPITCH);
#pragma unroll
  for (int gk = 0; gk < NGK; gk++) {
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        typename E::V2 t0 = E::cvt2(acc[gk][db][4 * r4 + 0] * oscale, acc[gk][db][4 * r4 + 1] * oscale);
        typename E::V2 t1 = E::cvt2(acc[gk][db][4 * r4 + 2] * oscale, acc[gk][db][4 * r4 + 3] * oscale);
        typename E::V4 ov = {t0[0], t0[1], t1[0], t1[1]};
        *reinterpret_cast<ACCT_LDS typename E::V4*>(obuf + l32 * OPITCH + (32 * db + 8 * r4 + 4 * g) * 2) = ov;
      }
    const int nch = a.hd >> 3;                       // valid 16-byte chunks per row
    const uint32_t nch_inv = recip16(nch);
#pragma unroll
    for (int i = 0; i < (32 * C::CPR + 63) / 64; i++) {
      const int idx = lane + 64 * i;
      const int r = div_small(idx, nch_inv), ch = idx - r * nch;
      const int grow = wk0 + 32 * gk + r;
      if (idx < 32 * nch && grow < a.Sk) {
        const u32x4 v = *reinterpret_cast<const ACCT_LDS u32x4*>(obuf + r * OPITCH + ch * 16);
        *reinterpret_cast<u32x4*>(outp + (int64_t)grow * oss + ch * 8) = v;
      }
    }
  }
}

// Second half of a dK/dV launch whose query range was cut into a.q_split slices (few heads and a short key
// sequence would otherwise leave most of the chip idle): one workgroup per key tile, the same wave and lane
// roles as the dK/dV kernel; every lane adds up its accumulators over the slices in ascending order (a fixed
// order: the result does not depend on which slice finished first) and stores the rows.
template <typename T, int D, int NGK>
__global__ void __launch_bounds__(512) fa_bwd_dkdv_reduce_kernel(const FaArgs a, float drop_scale) {
  using C = SwzCfg<D>;
  constexpr int NW = 8, WK = 32 * NGK, BNK = 4 * WK;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool krole = wave >= 4;
  const int BH = a.B * a.N, n_wg = BH * a.n_tiles, wg = blockIdx.x;
  int bh, kt;
  wg_map(wg, BH, a.n_tiles, bh, kt);
  const int b = bh / a.N, h = bh % a.N;
  const int wk0 = kt * BNK + (wave & 3) * WK;
  f32x16 acc[NGK][C::DB];
#pragma unroll
  for (int gk = 0; gk < NGK; gk++)
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[gk][db][r] = 0.f;
  for (int slice = 0; slice < a.q_split; slice++) {
    const float* part = a.dkdv_part + ((((int64_t)slice * n_wg + wg) * NW + wave) * (NGK * C::DB) << 10) + lane * 16;
#pragma unroll
    for (int gk = 0; gk < NGK; gk++)
#pragma unroll
      for (int db = 0; db < C::DB; db++) {
        const f32x16 v = *reinterpret_cast<const f32x16*>(part + ((gk * C::DB + db) << 10));
#pragma unroll
        for (int r = 0; r < 16; r++) acc[gk][db][r] += v[r];
      }
  }
  const float oscale = (krole ? a.scale : drop_scale) * a.p_unshift;
  dkdv_store_rows<T, D, NGK>(acc, a, b, h, wk0, krole, oscale, smem);
}

// ============================================================================
// dK/dV kernel: kv-tile owner, 8 waves in 4 pairs.  A pair owns 64 key rows.
// Its first wave (V role) keeps the K fragments of those rows in registers,
// recomputes S = Q K^T and P, hands P (fp16) to its partner through LDS and
// accumulates dV^T += dO^T P.  The partner (K role) keeps the V fragments,
// computes dP = dO V^T, forms dS = P*(dP - D) and accumulates dK^T += Q^T dS.
// Splitting the two accumulators over two waves halves the registers per wave
// (two waves fit on each SIMD and overlap each other's MFMA and exp/convert
// phases) while every Q / dO fragment read from LDS still feeds two MFMAs.
// ============================================================================
constexpr int kPark = 6;        // stationary fragments parked in LDS per wave (D = 128)
constexpr int kParkHot = 4;     // the variant without side inputs has registers for two more fragments
// stationary fragments parked in LDS per wave: the bias variants give one up for the bias tiles' LDS
template <int D, bool BIAS, bool MASKT>
constexpr int dkdv_park() { return D == 128 ? (BIAS ? kPark - 1 : (MASKT ? kPark : kParkHot)) : 0; }
// key groups of 32 rows per wave: head dims above 128 leave registers for the accumulators of one only
template <int D> constexpr int dkdv_groups() { return D > 128 ? 1 : 2; }

// MASKT = false compiles the mask-tensor handling out (no mask, or the causal mask by index compare):
// the hot variant must not carry that code's register pressure.
template <typename T, int D, bool BIAS, bool DROP, bool MASKT, int NGK = 2>
ACCT_DEV void fa_bwd_dkdv_body(const FaArgs& a) {
  static_assert(NGK == 2 || (NGK == 1 && !BIAS), "one key group per wave: no bias variants");
  using E = Elem<T>;
  using V8 = typename E::V8;
  using C = SwzCfg<D>;
  constexpr int NW = 8;
  constexpr int WK = 32 * NGK;                      // key rows per wave pair
  constexpr int BNK = 4 * WK;                       // key rows per workgroup
  constexpr int TILEB = 64 * C::PITCH;
  constexpr int STATB = 2 * 64 * 4;                 // -LSE*log2(e) and D of the 64 rows of a tile
  constexpr int DROPB = DROP ? 2048 : 0;            // keep bits of the tile's 64 rows for the workgroup's 256 keys: [key][2 chunks] words
  constexpr int STAGEB = 2 * TILEB + STATB + DROPB; // one buffer: Q tile | dO tile | -LSE*log2(e) | D | keep bits
  constexpr int PXB = 2048 * NGK;                   // P of one pair and chunk: 64 lanes x 32 bytes per key group
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;   // [2 stage buffers][2 x 4 pair P buffers]
  ACCT_LDS char* pexch = smem + 2 * STAGEB;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, g = lane >> 5;
  const int pair = __builtin_amdgcn_readfirstlane(wave & 3);   // wave-uniform: the pair's key range stays in scalar registers
  const bool krole = wave >= 4;                     // false: V role (S, P, dV); true: K role (dP, dS, dK)
  const int BH = a.B * a.N, n_wg = BH * a.n_tiles;
  int wg = blockIdx.x, slice = 0;                   // q_split > 1: the grid holds every key tile once per query slice
  if (a.q_split > 1) {
    slice = wg / n_wg;
    wg -= slice * n_wg;
  }
  int bh, kt;                                       // causal: the first key tiles are the heaviest
  wg_map(wg, BH, a.n_tiles, bh, kt);
  const int b = bh / a.N, h = bh % a.N;
  const int k0 = kt * BNK;
  const int wk0 = k0 + pair * WK;                   // first key row of this pair
  const int k_end = min(k0 + BNK, a.Sk);

  const T* qp = (const T*)a.q + b * a.q_sb + h * a.q_sh;
  const T* kp = (const T*)a.k + b * a.k_sb + h * a.k_sh;
  const T* vp = (const T*)a.v + b * a.v_sb + h * a.v_sh;
  const T* dop = (const T*)a.dout + b * a.o_sb + h * a.o_sh;
  // visible query tiles (64 rows) of this workgroup
  const int kb_lo = k0 / 128, kb_hi = (k_end - 1) / 128;
  const int qb_lo = max(0, kb_lo - a.next_blk), qb_hi = min(a.Tr - 1, kb_hi + a.prev_blk);
  int i_lo = qb_lo * 2, i_hi = min(qb_hi * 2 + 1, (a.Sq - 1) / 64);
  const bool causal = a.mask_kind == kMaskCausal;
  if (causal) i_lo = max(i_lo, k0 / 64);            // query tiles wholly above the diagonal contribute 0
  if (a.q_split > 1) {                              // this workgroup's slice of the 64-row query tiles
    const int per = ((a.Sq + 63) / 64 + a.q_split - 1) / a.q_split;
    i_lo = max(i_lo, slice * per);
    i_hi = min(i_hi, (slice + 1) * per - 1);
  }
  const int wkb = wk0 / 128;
  BlkClassWindowLaneTails flwin;                      // block classes of a dense mask: 64 blocks at a time in scalar registers
  bool flwin_ready = false;
  if (MASKT && a.mask_kind == kMaskDense) {
    // query tiles at either end whose blocks are wholly masked for every key block of this workgroup are
    // not streamed at all (key padding: a workgroup of padded keys has nothing to do).  With at most 64 query
    // blocks, one round trip to memory yields both the trimmed range and the pair's class window.
    const uint8_t* fl = a.blkflags + ((int64_t)(a.mask_sb ? b : 0) * a.Tr) * a.Tc;
    int b_lo = i_lo >> 1, b_hi = i_hi >> 1;
    // (the bias variants have no register to spare for the key tails: they read such blocks through the bitmaps)
    const uint8_t* tails = (!BIAS && a.blktail) ? a.blktail + ((int64_t)(a.mask_sb ? b : 0) * a.Tr) * a.Tc : nullptr;
    if (i_lo <= i_hi && flwin.init_trimmed(fl, a.Tc, 1, kb_lo, kb_hi - kb_lo + 1, min(wkb, kb_hi), b_lo, b_hi, lane, tails)) {
      i_lo = max(i_lo, b_lo * 2);
      i_hi = min(i_hi, b_hi * 2 + 1);
      flwin_ready = true;
    } else {
      auto dead = [&](int i) {
        for (int kb = kb_lo; kb <= kb_hi; kb++)
          if (fl[(int64_t)(i >> 1) * a.Tc + kb] != kBlkSkip) return false;
        return true;
      };
      trim_dead_tiles(i_lo, i_hi, lane, dead);
    }
  }

  // stationary B operands: K fragments (V role) or V fragments (K role) of the pair's 64 key rows;
  // lane holds key row 32 gk + l32, d = 16t + 8g ..
  // The last PARK k-steps of the second key group live in a wave-private LDS slab instead of
  // registers (16 VGPRs at D = 128): that is what lets two waves share a SIMD without spilling.
  constexpr int PARK = dkdv_park<D, BIAS, MASKT>();
  V8 bf[NGK][C::KS];
  ACCT_LDS char* park = pexch + 8 * PXB + wave * (PARK * 1024) + lane * 16;
  // bias tile (32 query rows x the pair's 64 keys) of the V-role wave, staged one chunk ahead by DMA
  ACCT_LDS char* bias_lds = pexch + 8 * PXB + 8 * (PARK * 1024) + pair * 4096;
  {
    const T* src = krole ? vp : kp;
    const int64_t ss = krole ? a.v_ss : a.k_ss;
#pragma unroll
    for (int gk = 0; gk < NGK; gk++) {
      const int row = min(wk0 + 32 * gk + l32, a.Sk - 1);
#pragma unroll
      for (int t = 0; t < C::KS; t++) {
        // k-steps (or the upper half of one) past the head dim: zeros there make the products
        // ignore whatever the Q / dO tiles hold in that slot
        const bool inside = 16 * t + 8 * g < a.hd;
        V8 v;
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0;
        if (inside) v = *reinterpret_cast<const V8*>(src + (int64_t)row * ss + 16 * t + 8 * g);
        if (gk == 1 && t >= C::KS - PARK) *reinterpret_cast<ACCT_LDS V8*>(park + (t - (C::KS - PARK)) * 1024) = v;
        else bf[gk][t] = v;
      }
    }
  }
  f32x16 acc[NGK][C::DB];                             // dV^T (V role) or dK^T (K role): [d rows, key column l32]
#pragma unroll
  for (int gk = 0; gk < NGK; gk++)
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[gk][db][r] = 0.f;

  // per-lane LDS offsets (tile-invariant)
#define FOFF(t) (foff4[(t) & 3] ^ (((t) >> 2) * 128))
#define TOFF(db) (toff2[(db) & 1] + ((db) >> 1) * 128)

  const int mb = a.mask_sb ? b : 0;
  const uint8_t* maskp = a.mask ? a.mask + (a.mask_kind == kMaskDense ? (int64_t)mb * a.mask_sb * a.mask_es : 0) : nullptr;
  const T* alibip = BIAS ? (const T*)a.alibi + b * a.al_sb + h * a.al_sh : nullptr;

  // stage q tile i into buffer `sb`: Q and dO by 16-byte DMA (2 instructions per wave each),
  // LSE (wave 0) and D (wave 1) by 4-byte DMA; rows past Sq repeat the last row
  // (addresses are re-derived per call here: this kernel has no registers to spare for a TileDma plan)
  auto stage = [&](int i, ACCT_LDS char* sb) {
    if ((i + 1) * 64 <= a.Sq) {
      TileDma<T, D, 64, NW>::issue_direct(qp, a.q_ss, i * 64, sb, a.hd >> 3);
      TileDma<T, D, 64, NW>::issue_direct(dop, a.o_ss, i * 64, sb + TILEB, a.hd >> 3);
    } else {                                         // ragged last tile: clamped rows
      tile_dma<T, D, 64, NW>(qp, a.q_ss, i * 64, a.Sq, sb, a.hd >> 3);
      tile_dma<T, D, 64, NW>(dop, a.o_ss, i * 64, a.Sq, sb + TILEB, a.hd >> 3);
    }
    if (wave < 2) {                                  // (pointers rebuilt from the kernel arguments: nothing to keep live)
      const int r = min(i * 64 + lane, a.Sq - 1);
      dma4((wave == 0 ? a.nlse : a.delta) + (int64_t)bh * a.Sq + r, sb + 2 * TILEB + wave * 256);
    }
    if (DROP) {
      // word c of key k (LDS dword 2k + c) = rows 64i + 32c .. +31 of that key's column entry; one dword per lane.
      // Read from LDS in the loop, the words cost no wait on the vector-memory counter, which would also wait
      // for the tile DMA in flight.
      const int idx = wave * 64 + lane, key = min(k0 + (idx >> 1), a.Sk - 1);
      dma4(a.dropcol + ((((int64_t)bh * a.Tr + (i >> 1)) * a.Sk + key) << 2) + 2 * (i & 1) + (idx & 1),
           sb + 2 * TILEB + STATB + wave * 256);
    }
  };

  // A bias with row stride 0 (the reference's ALiBi form [B, N, 1, Sk]) depends on the key only: a lane of this
  // kernel owns a key column, so the bias is one value per lane and key group for the whole query loop
  // (in units of the raw scores; 0 for the K role, whose accumulators hold dP)
  const bool row_bias = BIAS && a.al_sq == 0;
  float brow[NGK];
#pragma unroll
  for (int gk = 0; gk < NGK; gk++)
    brow[gk] = (row_bias && !krole) ? (float)alibip[min(wk0 + 32 * gk + l32, a.Sk - 1)] * a.inv_scale : 0.f;
  const bool bias_staged = BIAS && !row_bias && !krole && wk0 < a.Sk && (a.Sk & 7) == 0 &&
                           (((uintptr_t)a.alibi & 15) | ((a.al_sb | a.al_sh | a.al_sq) & 7)) == 0;
  auto stage_bias = [&](int cn) { bias_tile_dma<T, false>(alibip, a.al_sq, cn * 32, a.Sq, wk0, a.Sk, bias_lds); };

  // per-chunk predicates of this pair (chunk = 32 query rows; two per staged tile), as bits of one value
  // so that they live in a register: 1 act, 2 apply_mask, 4 limits (some (row, key) of the chunk is
  // absent), 8 diag (keys after the query are hidden, by index compare); bits 8..15: key tail of the block (the
  // block's keys from that one on are hidden from every row: a limit like the end of the keys), 0 for none
  auto classify = [&](int cidx, uint32_t fl, uint32_t tail) -> uint32_t {
    const int qc0 = cidx * 32, qt0 = (cidx >> 1) * 64, qb = cidx >> 2;
    bool act = (wkb - a.next_blk <= qb) && (qb <= wkb + a.prev_blk) && (wk0 < a.Sk);
    if (causal) act = act && (qt0 + 63 >= wk0);
    if (a.row_prefix) act = act && (wk0 < (qt0 / a.row_prefix + 1) * a.row_prefix);
    bool apply_mask = false, diag = causal;
    if (MASKT && a.mask_kind == kMaskDense) {
      if (act) {
        act = fl != kBlkSkip;                          // class of block (qb, wkb)
        apply_mask = fl == kBlkApply;
        if (fl == kBlkTriu) { diag = true; act = qt0 + 63 >= wk0; }
        if (apply_mask && tail) {
          apply_mask = false;
          act = wk0 < wkb * 128 + (int)tail;            // (else every key of the pair is hidden)
        } else {
          tail = 0;
        }
      } else {
        tail = 0;
      }
    } else {
      tail = 0;
      if (MASKT && a.mask_kind == kMaskTile) apply_mask = wkb == qb;
    }
    const bool limits = (diag && (wk0 + WK - 1 > qc0)) || (wk0 + WK > a.Sk) || (qc0 + 32 > a.Sq);
    return (act ? 1u : 0u) | (apply_mask ? 2u : 0u) | (limits ? 4u : 0u) | (diag ? 8u : 0u) | (tail << 8);
  };

  if (i_lo <= i_hi) {
    // The query tiles are walked from the last one down: with a causal mask the key tiles of a head start at
    // different rows (their diagonals) but all END at the last row, so walking down keeps the workgroups of a head
    // -- they run side by side on one XCD -- on the same Q / dO tile at the same time, and one fetch from memory
    // serves them all.  (Walking up, they stay four tiles apart and the XCD's L2 holds the tiles in between only
    // just.)  Position p of the walk is tile i_hi - p; the two 32-row chunks of a tile keep their order.
    const int ntile = i_hi - i_lo + 1, npos = 2 * ntile;
    auto chunk_at = [&](int pos) { return 2 * (i_hi - (pos >> 1)) + (pos & 1); };
    stage(i_hi, smem);
    if (BIAS && bias_staged) stage_bias(chunk_at(0));
    // A full wait the compiler can see: the stationary fragments loaded above are complete, so it places
    // no vmcnt wait inside the loop -- such a wait would also stall on the next tile's DMA.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    // The K role runs one chunk behind the V role: in step n the V role recomputes P of chunk n,
    // publishes it and accumulates dV; the K role picks up P of chunk n-1.  One barrier per step,
    // nothing is carried across it in registers.
    const int c_lo = 2 * i_lo, c_hi = 2 * i_hi + 1;
    (void)c_lo;
    // offsets of the transposed fragments of d block db: kept across the steps where the registers allow
    // (a fifth of the step's vector instructions otherwise), re-derived in every step in the bias + dropout variant
    constexpr bool KEEP_TOFF = !(BIAS && DROP);
    int toff2_kept[2] = {0, 0};
    if (KEEP_TOFF) {
      const int trow = 4 * g + ((lane & 15) >> 2);
      const int tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
#pragma unroll
      for (int db = 0; db < 2; db++) toff2_kept[db] = trow * C::PITCH + swz_off(4 * db + tchunk, C::swz(trow)) + 8 * (lane & 1);
    }
    constexpr bool KEEP_FOFF = !BIAS;   // the variants without a bias have the registers for the row-major offsets too
    int foff4_kept[4] = {0, 0, 0, 0};
    if (KEEP_FOFF) {
#pragma unroll
      for (int t = 0; t < 4; t++) foff4_kept[t] = l32 * C::PITCH + swz_off(2 * t + g, C::swz(l32));
    }
    const uint8_t* flcol = (MASKT && a.mask_kind == kMaskDense) ? a.blkflags + (int64_t)mb * a.Tr * a.Tc + wkb : nullptr;
    if (!flwin_ready) flwin.init_descending(flcol, a.Tc, c_lo >> 2, c_hi >> 2, lane, (!BIAS && flcol && a.blktail) ? a.blktail + (flcol - a.blkflags) : nullptr);
    for (int n = 0; n <= npos; n++) {
      if ((n & 1) && (n >> 1) + 1 < ntile) stage(i_hi - ((n >> 1) + 1), smem + ((((n >> 1) + 1) & 1) * STAGEB));
      const int cpos = __builtin_amdgcn_readfirstlane(krole ? n - 1 : n);   // position of the chunk this wave works on in this step (wave-uniform: scalar)
      if (cpos >= 0 && cpos < npos) {
        const int cidx = chunk_at(cpos);
        const uint32_t fl_cur = flwin.get(cidx >> 2, lane);
        const uint32_t cls = classify(cidx, fl_cur, (MASKT && !BIAS) ? flwin.tail(cidx >> 2) : 0u);
        const bool act = cls & 1u, apply_mask = cls & 2u, limits = cls & 4u, diag = cls & 8u;
        // keys from key_end on are hidden from every row of the chunk (a key tail): a lane owns a key, so its whole
        // column of P is zeroed after the probabilities are packed (one AND per packed word)
        const int key_end = (cls >> 8) ? wkb * 128 + (int)(cls >> 8) : 0x7fffffff;
        const bool ktail = wk0 + WK > key_end;
        const bool edge = (BIAS && !bias_staged && !row_bias) || apply_mask || limits;   // (a staged or per-key bias is already inside the scores)
        if (act) {
          const int c = cidx & 1, qc0 = cidx * 32;
          // Where the registers do not allow keeping them (see above), the per-lane LDS offsets are
          // re-derived in every step (a handful of VALU ops).  Chunk c + 8 of a row sits in slot (c ^ swz) ^ 8: the row-major
          // fragments of the upper half of the head dim are one XOR away from the lower four, and the
          // transposed ones (row % 16 < 8, swizzle bit 3 clear) 128 bytes after them.
          int ln = lane;
          asm volatile("" : "+v"(ln));
          int foff4[4];                               // row-major fragment of k-step t: row l32, chunk 2t + g
#pragma unroll
          for (int t = 0; t < 4; t++) foff4[t] = KEEP_FOFF ? foff4_kept[t] : (ln & 31) * C::PITCH + swz_off(2 * t + (ln >> 5), C::swz(ln & 31));
          int toff2[2];
          if (KEEP_TOFF) {
            toff2[0] = toff2_kept[0];
            toff2[1] = toff2_kept[1];
          } else {
            const int trow = 4 * (ln >> 5) + ((ln & 15) >> 2);
            const int tchunk = 2 * ((ln >> 4) & 1) + ((ln & 3) >> 1);
#pragma unroll
            for (int db = 0; db < 2; db++) toff2[db] = trow * C::PITCH + swz_off(4 * db + tchunk, C::swz(trow)) + 8 * (ln & 1);
          }
          ACCT_LDS char* qbuf = smem + ((cpos >> 1) & 1) * STAGEB;
          ACCT_LDS char* dobuf = qbuf + TILEB;
          const ACCT_LDS float* lbuf = (const ACCT_LDS float*)(qbuf + 2 * TILEB);
          const ACCT_LDS float* dbuf = lbuf + 64;
          ACCT_LDS char* px = pexch + ((cidx & 1) * 4 + pair) * PXB + ln * 16;
          // rows of this lane's C registers: q = qc0 + 8 (r/4) + 4 g + r%4 ; key = wk0 + 32 gk + l32
          f32x16 t0[NGK];                              // S (V role) or dP (K role) of the two key groups
          if (BIAS && bias_staged) {
            // V role: the bias enters as the initial value of the score accumulators (bias / scale, the MFMAs
            // add q.k): no bias registers alive next to the scores.  Transposed reads of the row-major tile:
            // each hands a lane the four consecutive rows 8i + 4g .. +3 of its key column (a 16-lane group
            // covers 4 rows x 16 keys and supplies the addresses of that block's 8-byte pieces)
            const ACCT_LDS char* bl = bias_lds + (4 * g + ((lane & 15) >> 2)) * 128 + ((lane >> 4) & 1) * 32 + (lane & 3) * 8;
#pragma unroll
            for (int gk = 0; gk < NGK; gk++)
#pragma unroll
              for (int i = 0; i < 4; i++) {
                const typename E::V4 bv = __builtin_bit_cast(typename E::V4, lds_read_tr(bl + i * 8 * 128 + gk * 64));
#pragma unroll
                for (int e = 0; e < 4; e++) t0[gk][4 * i + e] = (float)bv[e] * a.inv_scale;
              }
          } else {
#pragma unroll
            for (int gk = 0; gk < NGK; gk++)
#pragma unroll
              for (int r = 0; r < 16; r++) t0[gk][r] = BIAS ? brow[gk] : 0.f;
          }
          {
            // software pipeline: the A fragments travel through a ring of ARING register sets (ARING reads in
            // flight ahead of the MFMAs that consume the oldest), the parked B fragment is requested one
            // k-step ahead
            constexpr int ARING = 2;
            const ACCT_LDS char* abuf = (krole ? dobuf : qbuf) + c * 32 * C::PITCH;
            V8 ar[ARING];
#pragma unroll
            for (int t = 0; t < ARING; t++) ar[t] = lds_read_frag<T>(abuf + FOFF(t));
            V8 b1 = (0 >= C::KS - PARK) ? *reinterpret_cast<const ACCT_LDS V8*>(park) : bf[NGK - 1][0];
#pragma unroll
            for (int t = 0; t < C::KS; t++) {
              V8 b1n = b1;
              if (t + 1 < C::KS)
                b1n = (t + 1 >= C::KS - PARK) ? *reinterpret_cast<const ACCT_LDS V8*>(park + (t + 1 - (C::KS - PARK)) * 1024) : bf[NGK - 1][t + 1];
              __builtin_amdgcn_sched_barrier(0);
              t0[0] = E::mfma(ar[t % ARING], bf[0][t], t0[0]);                              // S[q, key] or dP[q, key]
              if (NGK == 2) t0[NGK - 1] = E::mfma(ar[t % ARING], b1, t0[NGK - 1]);
              __builtin_amdgcn_sched_barrier(0);
              if (t + ARING < C::KS) ar[t % ARING] = lds_read_frag<T>(abuf + FOFF(t + ARING));
              b1 = b1n;
            }
          }
          if (BIAS && bias_staged) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // bias tile consumed: stage the next chunk's
            if (cpos + 1 < npos) stage_bias(chunk_at(cpos + 1));
          }
          uint32_t dcw[NGK] = {};                       // keep bits of the chunk's 32 rows for this lane's two key columns
          if (DROP) {
            const ACCT_LDS uint32_t* dc = (const ACCT_LDS uint32_t*)(qbuf + 2 * TILEB + STATB) + 2 * (pair * WK + l32) + c;
#pragma unroll
            for (int gk = 0; gk < NGK; gk++) dcw[gk] = dc[64 * gk] >> (4 * g);
          }
          V8 bfr[NGK][2];                              // B fragments of the second product: P (V role) or dS (K role)
          if (!krole) {
            if (edge) {
              // Side inputs and range limits are folded into the raw scores in place, in three short
              // passes that each keep few values live: + bias/scale (unstaged bias only); - 10000/scale where the mask bit of
              // (row, key) is set; -inf where the key comes after the query (causal) or where the key
              // or the query row does not exist (the probability is exactly 0 either way).
              if (BIAS && !bias_staged && !row_bias) {      // a bias the DMA cannot stage (alignment): direct loads
                const int qlast = a.Sq - 1 - qc0;               // last valid row, relative to the chunk
                const T* brow0 = alibip + (int64_t)qc0 * a.al_sq;
#pragma unroll
                for (int gk = 0; gk < NGK; gk++) {
                  const int kv_c = min(wk0 + 32 * gk + l32, a.Sk - 1);
#pragma unroll
                  for (int r = 0; r < 16; r++) {
                    const int qr_c = min(8 * (r >> 2) + 4 * g + (r & 3), qlast);
                    t0[gk][r] += (float)brow0[qr_c * (int)a.al_sq + kv_c] * a.inv_scale;
                    if ((r & 3) == 3) asm volatile("" ::: "memory");   // keep the loads in small batches
                  }
                }
              }
              if (MASKT && apply_mask) {
                // one 32-bit word of the key column's bitmap covers the 32 rows of the chunk
                const uint32_t* cb = a.mask_kind == kMaskDense
                                         ? a.colbits + ((((int64_t)mb * a.Tr + (qc0 >> 7)) * a.Sk) << 2) + ((qc0 >> 5) & 3)
                                         : a.colbits + ((qc0 >> 5) & 3);
                const uint32_t addbits = __float_as_uint(a.mask_add_raw);
#pragma unroll
                for (int gk = 0; gk < NGK; gk++) {
                  const int kv_c = min(wk0 + 32 * gk + l32, a.Sk - 1);
                  const uint32_t w = cb[(a.mask_kind == kMaskDense ? kv_c : (kv_c & 127)) * 4] >> (4 * g);
#pragma unroll
                  for (int r = 0; r < 16; r++) {
                    // (bit ? -1 : 0) & bits(-10000/scale), added
                    const int32_t sel = (int32_t)(w << (31 - (8 * (r >> 2) + (r & 3)))) >> 31;
                    t0[gk][r] += __uint_as_float((uint32_t)sel & addbits);
                  }
                }
              }
              if (limits)
#pragma unroll
              for (int gk = 0; gk < NGK; gk++) {
                const int kv = wk0 + 32 * gk + l32;
                int lo = diag ? kv - qc0 - 4 * g : -64;         // chunk rows below it come before the key
                int hi = a.Sq - 1 - qc0 - 4 * g;                // last query row that exists
                if (kv >= a.Sk) hi = -64;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                  const int cr = 8 * (r >> 2) + (r & 3);
                  if (cr < lo || cr > hi) t0[gk][r] = -INFINITY;
                }
              }
            }
#pragma unroll
            for (int gk = 0; gk < NGK; gk++) {
              const int kv_c = min(wk0 + 32 * gk + l32, a.Sk - 1);
#pragma unroll
              for (int hh = 0; hh < 2; hh++) {
                float p[8], pd[8];
#pragma unroll
                for (int r4 = 0; r4 < 2; r4++) {
                  const f32x4 lv = *reinterpret_cast<const ACCT_LDS f32x4*>(lbuf + 32 * c + 16 * hh + 8 * r4 + 4 * g);
#pragma unroll
                  for (int e = 0; e < 4; e++) {
                    p[4 * r4 + e] = fast_exp2(__builtin_fmaf(t0[gk][8 * hh + 4 * r4 + e], a.scale_log2e, lv[e]));
                    pd[4 * r4 + e] = p[4 * r4 + e];
                    // dropped: 0; kept: P (the 1 / keep_prob is applied to dV once, at the end)
                    if (DROP) pd[4 * r4 + e] = __uint_as_float(__float_as_uint(p[4 * r4 + e]) & (uint32_t)__builtin_amdgcn_sbfe((int)dcw[gk], 16 * hh + 8 * r4 + e, 1));
                  }
                }
                V8 pv = pack8<T>(pd);
                f16x8 ph = pack8<f16>(p);                  // un-dropped P for the partner, always fp16 (P <= 1: finer than bf16)
                if (ktail) {
                  const uint32_t km = wk0 + 32 * gk + l32 < key_end ? 0xffffffffu : 0u;
                  u32x4 w0 = __builtin_bit_cast(u32x4, pv), w1 = __builtin_bit_cast(u32x4, ph);
#pragma unroll
                  for (int e = 0; e < 4; e++) { w0[e] &= km; w1[e] &= km; }
                  pv = __builtin_bit_cast(V8, w0);
                  ph = __builtin_bit_cast(f16x8, w1);
                }
                bfr[gk][hh] = pv;
                *reinterpret_cast<ACCT_LDS f16x8*>(px + (2 * gk + hh) * 1024) = ph;
              }
            }
          } else {
#pragma unroll
            for (int gk = 0; gk < NGK; gk++) {
              const int kv_c = min(wk0 + 32 * gk + l32, a.Sk - 1);
#pragma unroll
              for (int hh = 0; hh < 2; hh++) {
                const f16x8 ph = *reinterpret_cast<const ACCT_LDS f16x8*>(px + (2 * gk + hh) * 1024);
                float ds[8];
#pragma unroll
                for (int r4 = 0; r4 < 2; r4++) {
                  const f32x4 dv4 = *reinterpret_cast<const ACCT_LDS f32x4*>(dbuf + 32 * c + 16 * hh + 8 * r4 + 4 * g);
#pragma unroll
                  for (int e = 0; e < 4; e++) {
                    float dpv = t0[gk][8 * hh + 4 * r4 + e];
                    float dpd = dpv - dv4[e];
                    // dropped: dP = 0; kept: dP / keep_prob, scaled by the FMA that subtracts D
                    if (DROP) dpd = __builtin_fmaf(__uint_as_float(__float_as_uint(dpv) & (uint32_t)__builtin_amdgcn_sbfe((int)dcw[gk], 16 * hh + 8 * r4 + e, 1)), a.inv_keep, -dv4[e]);
                    // (an FMA with a zero addend keeps the fp16 -> fp32 conversion inside one mixed-precision instruction)
                    ds[4 * r4 + e] = __builtin_fmaf((float)ph[4 * r4 + e], dpd, 0.0f);
                  }
                }
                bfr[gk][hh] = pack8<T>(ds);
              }
            }
          }
          // dV^T += dO^T P (V role) ; dK^T += Q^T dS (K role): contract over the 32 query rows of the chunk
          const ACCT_LDS char* tb = (krole ? qbuf : dobuf) + c * 32 * C::PITCH;
          {
            // transposed fragments through a ring of BRING register sets, as above
            constexpr int BRING = 2, NT = 2 * C::DB;
            auto tread = [&](int i) {
              const int db = i % C::DB, hh = i / C::DB;
              const ACCT_LDS char* ta = tb + TOFF(db) + 16 * hh * C::PITCH;
              return join_tr<T>(lds_read_tr(ta), lds_read_tr(ta + C::tr_hi(db)));
            };
            V8 tr[BRING];
#pragma unroll
            for (int i = 0; i < BRING; i++) tr[i] = tread(i);
#pragma unroll
            for (int i = 0; i < NT; i++) {
              const int db = i % C::DB, hh = i / C::DB;
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int gk = 0; gk < NGK; gk++) acc[gk][db] = E::mfma(tr[i % BRING], bfr[gk][hh], acc[gk][db]);
              __builtin_amdgcn_sched_barrier(0);
              if (i + BRING < NT) tr[i % BRING] = tread(i + BRING);
            }
          }
        } else if (BIAS && bias_staged && cpos + 1 < npos) {
          stage_bias(chunk_at(cpos + 1));               // nothing to read in this step: the region is free
        }
      }
      dma_wait();                                     // a tile requested at the top of this step has landed
      __syncthreads();
    }
  }

  if (a.q_split > 1) {
    // this workgroup saw one slice of the query range: its sums go to the workspace as they sit in the registers
    // (fa_bwd_dkdv_reduce_kernel adds the slices up in a fixed order and stores the rows)
    float* part = a.dkdv_part + ((((int64_t)slice * n_wg + wg) * NW + wave) * (NGK * C::DB) << 10) + lane * 16;
#pragma unroll
    for (int gk = 0; gk < NGK; gk++)
#pragma unroll
      for (int db = 0; db < C::DB; db++) *reinterpret_cast<f32x16*>(part + ((gk * C::DB + db) << 10)) = acc[gk][db];
    return;
  }
  const float oscale = (krole ? a.scale : (DROP ? a.inv_keep : 1.0f)) * a.p_unshift;
  dkdv_store_rows<T, D, NGK>(acc, a, b, h, wk0, krole, oscale, smem);
}

#undef FOFF
#undef TOFF

// (two bodies in the variant that knows mask tensors only, as in the dQ kernel: a workgroup whose key blocks
// see nothing but the causal pattern runs the code of the variant without side inputs)
template <typename T, int D, bool BIAS, bool DROP, bool MASKT, int NGK = 2>
__global__ void __launch_bounds__(512) fa_bwd_dkdv_kernel(const FaArgs a) {
  if constexpr (MASKT && !BIAS && !DROP) {
    if (a.mask_kind == kMaskDense) {
      constexpr int BNK = 4 * 32 * NGK;
      const int BH = a.B * a.N, n_wg = BH * a.n_tiles;
      int wg = blockIdx.x;
      if (a.q_split > 1) wg -= (wg / n_wg) * n_wg;
      int bh, kt;
      wg_map(wg, BH, a.n_tiles, bh, kt);
      const int k0 = kt * BNK, k_end = min(k0 + BNK, a.Sk);
      const int kb_lo = k0 / 128, kb_hi = (k_end - 1) / 128;
      const int qb_lo = max(0, kb_lo - a.next_blk), qb_hi = min(a.Tr - 1, kb_hi + a.prev_blk);
      const uint8_t* fl = a.blkflags + ((int64_t)(a.mask_sb ? bh / a.N : 0) * a.Tr) * a.Tc;
      if (dense_lines_are_causal(fl, a.Tc, 1, kb_lo, kb_hi - kb_lo + 1, qb_lo, qb_hi, true, a, threadIdx.x & 63)) {
        FaArgs c = a;
        c.mask_kind = kMaskCausal;
        fa_bwd_dkdv_body<T, D, false, false, false, NGK>(c);
        return;
      }
    }
  }
  fa_bwd_dkdv_body<T, D, BIAS, DROP, MASKT, NGK>(a);
}

// ---- launchers ----------------------------------------------------------------
template <typename T, int D, bool BIAS, bool DROP>
static hipError_t launch_bwd_t(FaArgs a, int stages, hipStream_t st) {
  hipError_t e = hipSuccess;
  bool dq_done = false;
  if constexpr (D == 128 && !BIAS && !DROP) {
    // head dim 128 without side inputs on aligned lengths: the kernel with 64 query rows per wave
    if ((stages & kStageDq) && dq64_applicable(a)) {
      e = launch_bwd_dq64(a, std::is_same<T, bf16>::value ? 1 : 0, st);
      if (e != hipSuccess) return e;
      dq_done = true;
    }
  }
  if ((stages & kStageDq) && !dq_done) {
    constexpr int QG = 1, NW = D > 128 ? 4 : 8;          // (wide head dims: one wave per SIMD has the registers)
    constexpr int BM = 32 * QG * NW;
    using CS = SwzCfg<D>;
    constexpr size_t tiles = 4 * 64 * (size_t)CS::PITCH + (BIAS ? (size_t)NW * QG * 4096 : 0) + (size_t)NW * 2 * DropRowStage<DROP, QG, 2>::BYTES, stage = (size_t)NW * 32 * (CS::DB * 64 + 16);
    const size_t smem = tiles > stage ? tiles : stage;
    a.n_tiles = (a.Sq + BM - 1) / BM;
    const bool mask_q = BIAS || DROP || a.mask_kind == kMaskDense || a.mask_kind == kMaskTile;
    auto kern = mask_q ? fa_bwd_dq_kernel<T, D, QG, NW, BIAS, DROP, true> : fa_bwd_dq_kernel<T, D, QG, NW, BIAS, DROP, BIAS || DROP>;
    e = allow_dynamic_lds((const void*)kern, smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)((long long)a.n_tiles * a.B * a.N)), dim3(64 * NW), smem, st, a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (stages & kStageDkDv) {
    using CS = SwzCfg<D>;
    constexpr int NGK = dkdv_groups<D>();
    constexpr size_t stageb = 2 * 64 * (size_t)CS::PITCH + 512 + (DROP ? 2048 : 0);
    constexpr size_t loopb = 2 * stageb + 8 * 2048 * NGK + 8 * (size_t)dkdv_park<D, BIAS, true>() * 1024 + (BIAS ? 4 * 4096 : 0),
                     epib = (size_t)8 * 32 * (CS::DB * 64 + 16);
    static_assert(loopb <= 160 * 1024 && epib <= 160 * 1024, "the workgroup's LDS must fit the CU's 160 KB");
    const size_t smem2 = loopb > epib ? loopb : epib;
    a.n_tiles = (a.Sk + 128 * NGK - 1) / (128 * NGK);
    const bool mask_t = BIAS || DROP || a.mask_kind == kMaskDense || a.mask_kind == kMaskTile;
    auto kern = mask_t ? fa_bwd_dkdv_kernel<T, D, BIAS, DROP, true, NGK> : fa_bwd_dkdv_kernel<T, D, BIAS, DROP, BIAS || DROP, NGK>;
    e = allow_dynamic_lds((const void*)kern, smem2);
    if (e != hipSuccess) return e;
    const long long n_wg = (long long)a.n_tiles * a.B * a.N;
    hipLaunchKernelGGL(kern, dim3((unsigned)(n_wg * (a.q_split > 1 ? a.q_split : 1))), dim3(512), smem2, st, a);
    e = hipGetLastError();
    if (e == hipSuccess && a.q_split > 1) {
      auto red = fa_bwd_dkdv_reduce_kernel<T, D, NGK>;
      e = allow_dynamic_lds((const void*)red, epib);
      if (e != hipSuccess) return e;
      hipLaunchKernelGGL(red, dim3((unsigned)n_wg), dim3(512), epib, st, a, DROP ? a.inv_keep : 1.0f);
      e = hipGetLastError();
    }
  }
  return e;
}

// SIDE: 2 = bias and dropout variants, 1 = the dropout variant only (head dims 40, 160, 256)
template <typename T, int D, int SIDE = 2>
static hipError_t launch_bwd_d(const FaArgs& a, int stages, hipStream_t st) {
  const bool bias = a.alibi != nullptr, drop = a.droprow != nullptr || a.dropcol != nullptr;
#ifndef ACCT_DEV_BUILD
  if constexpr (SIDE == 2) {
    if (bias) return drop ? launch_bwd_t<T, D, true, true>(a, stages, st) : launch_bwd_t<T, D, true, false>(a, stages, st);
  }
  if constexpr (SIDE >= 1) {
    if (drop && !bias) return launch_bwd_t<T, D, false, true>(a, stages, st);
  }
#endif
  if (bias || drop) return hipErrorNotSupported;       // (development build, head dims 40 / 160: plain variants only)
  return launch_bwd_t<T, D, false, false>(a, stages, st);
}

bool fwd_variants_complete();
#ifdef ACCT_DEV_BUILD
bool launch_variants_complete() { return false; }
#else
bool launch_variants_complete() { return fwd_variants_complete(); }
#endif

hipError_t launch_bwd(const FaArgs& a, int dtype, int Dr, int stages, hipStream_t st) {
  const int D = head_dim_class(Dr);
#ifdef ACCT_DEV_BUILD
  if (dtype != 0 || D != 128) return hipErrorNotSupported;
  return launch_bwd_d<f16, 128>(a, stages, st);
#else
  if (dtype == 0) {
    if (D == 128) return launch_bwd_d<f16, 128>(a, stages, st);
    if (D == 64) return launch_bwd_d<f16, 64>(a, stages, st);
    if (D == 80) return launch_bwd_d<f16, 80>(a, stages, st);
    if (D == 40) return launch_bwd_d<f16, 40, 1>(a, stages, st);
    if (D == 160) return launch_bwd_d<f16, 160, 1>(a, stages, st);
    if (D == 256) return launch_bwd_d<f16, 256, 1>(a, stages, st);
  } else {
    if (D == 128) return launch_bwd_d<bf16, 128>(a, stages, st);
    if (D == 64) return launch_bwd_d<bf16, 64>(a, stages, st);
    if (D == 80) return launch_bwd_d<bf16, 80>(a, stages, st);
    if (D == 40) return launch_bwd_d<bf16, 40, 1>(a, stages, st);
    if (D == 160) return launch_bwd_d<bf16, 160, 1>(a, stages, st);
    if (D == 256) return launch_bwd_d<bf16, 256, 1>(a, stages, st);
  }
  return hipErrorInvalidValue;
#endif
}

}  // namespace acct
