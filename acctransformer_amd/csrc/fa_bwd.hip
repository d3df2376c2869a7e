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

namespace acct {

ACCT_DEV void load_f32x4(const float* base, int idx, int limit, bool vec_ok, float fill, float out[4]) {
  if (vec_ok && idx + 4 <= limit) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(base + idx);
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = t[e];
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = (idx + e < limit) ? base[idx + e] : fill;
  }
}

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
template <typename T, int D, int QG, int NW, bool BIAS, bool DROP>
__global__ void __launch_bounds__(64 * NW) fa_bwd_dq_kernel(const FaArgs a) {
  using E = Elem<T>;
  using V8 = typename E::V8;
  using C = SwzCfg<D>;
  constexpr int BM = 32 * QG * NW;
  constexpr int TILEB = 64 * C::PITCH;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;   // [2 buffers][K tile | V tile]; reused by the epilogue

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, g = lane >> 5;
  const int BH = a.B * a.N;
  const int bh = blockIdx.x % BH;
  const int qt = a.n_tiles - 1 - (int)(blockIdx.x / BH);
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
      qf[gq][t] = *reinterpret_cast<const V8*>(qp + (int64_t)row_c * a.q_ss + 16 * t + 8 * g);
      dof[gq][t] = *reinterpret_cast<const V8*>(dop + (int64_t)row_c * a.o_ss + 16 * t + 8 * g);
      const V8 ov = *reinterpret_cast<const V8*>(op + (int64_t)row_c * a.o_ss + 16 * t + 8 * g);
#pragma unroll
      for (int e = 0; e < 8; e++) part += (float)dof[gq][t][e] * (float)ov[e];
    }
    dl[gq] = pair_sum(part);
    lq[gq] = INFINITY;                                   // rows past Sq: P = exp2(x - inf) = 0
    if (row < a.Sq) {
      lq[gq] = a.lse[(int64_t)bh * a.Sq + row] * kLog2e;
      if (g == 0) a.delta[(int64_t)bh * a.Sq + row] = dl[gq];
    }
  }

  // per-lane LDS offsets (tile-invariant)
  int koff[C::KS];
#pragma unroll
  for (int t = 0; t < C::KS; t++) koff[t] = l32 * C::PITCH + swz_off(2 * t + g, l32 & 7);
  const int trow = 4 * g + ((lane & 15) >> 2);
  const int tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
  int toff[C::DB];
#pragma unroll
  for (int db = 0; db < C::DB; db++) toff[db] = trow * C::PITCH + swz_off(4 * db + tchunk, trow) + 8 * (lane & 1);

  f32x16 acc[QG][C::DB];
#pragma unroll
  for (int gq = 0; gq < QG; gq++)
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[gq][db][r] = 0.f;

  const int mb = a.mask_sb ? b : 0;
  const uint8_t* maskp = a.mask ? a.mask + (a.mask_kind == kMaskDense ? (int64_t)mb * a.mask_sb : 0) : nullptr;
  const uint8_t* dropp = DROP ? a.drop + ((int64_t)bh * a.Sq) * a.Sk : nullptr;
  const T* alibip = BIAS ? (const T*)a.alibi + b * a.al_sb + h * a.al_sh : nullptr;
  const bool mask_vec = a.mask_kind == kMaskDense ? (((uintptr_t)a.mask | (uintptr_t)a.Sk | (uintptr_t)a.mask_sb) & 3) == 0
                                                  : ((uintptr_t)a.mask & 3) == 0;
  const bool drop_vec = DROP && (((uintptr_t)a.drop | (uintptr_t)a.Sk) & 3) == 0;
  const bool alibi_vec = BIAS && (((uintptr_t)a.alibi & 7) | ((a.al_sb | a.al_sh | a.al_sq) & 3)) == 0;

  if (j_lo <= j_hi) {
    tile_dma<T, D, 64, NW>(kp, a.k_ss, j_lo * 64, a.Sk, smem);
    tile_dma<T, D, 64, NW>(vp, a.v_ss, j_lo * 64, a.Sk, smem + TILEB);
    dma_wait();
    __syncthreads();

    for (int j = j_lo; j <= j_hi; j++) {
      const int buf = (j - j_lo) & 1;
      ACCT_LDS char* kbuf = smem + buf * 2 * TILEB;
      ACCT_LDS char* vbuf = kbuf + TILEB;
      if (j < j_hi) {
        tile_dma<T, D, 64, NW>(kp, a.k_ss, (j + 1) * 64, a.Sk, smem + (buf ^ 1) * 2 * TILEB);
        tile_dma<T, D, 64, NW>(vp, a.v_ss, (j + 1) * 64, a.Sk, smem + (buf ^ 1) * 2 * TILEB + TILEB);
      }
      const int kv0 = j * 64;
      const int kvb = j >> 1;
      bool act = (kvb - a.next_blk <= wqb) && (wqb <= kvb + a.prev_blk) && (wq0 < a.Sq);
      if (causal) act = act && (kv0 <= wq_end - 1);
      act = act && (kv0 < wkv_limit);
      bool apply_mask = false;
      if (a.mask_kind == kMaskDense && act) {
        const uint8_t f = a.blkflags[((int64_t)mb * a.Tr + wqb) * a.Tc + kvb];
        act = f != kBlkSkip;
        apply_mask = f == kBlkApply;
      } else if (a.mask_kind == kMaskTile) {
        apply_mask = wqb == kvb;
      }
      const bool edge = apply_mask || (causal && (kv0 + 63 > wq0)) || (kv0 + 64 > a.Sk);
      if (act) {
        V8 dsf[QG][2][2];
#pragma unroll
        for (int c = 0; c < 2; c++) {
          f32x16 s[QG], dp[QG];
#pragma unroll
          for (int gq = 0; gq < QG; gq++)
#pragma unroll
            for (int r = 0; r < 16; r++) { s[gq][r] = 0.f; dp[gq][r] = 0.f; }
          {
            V8 kf[C::KS], vf[C::KS];
#pragma unroll
            for (int t = 0; t < C::KS; t++) kf[t] = lds_read_frag<T>(kbuf + koff[t] + c * 32 * C::PITCH);
#pragma unroll
            for (int t = 0; t < C::KS; t++) vf[t] = lds_read_frag<T>(vbuf + koff[t] + c * 32 * C::PITCH);
#pragma unroll
            for (int t = 0; t < C::KS; t++)
#pragma unroll
              for (int gq = 0; gq < QG; gq++) s[gq] = E::mfma(kf[t], qf[gq][t], s[gq]);
#pragma unroll
            for (int t = 0; t < C::KS; t++)
#pragma unroll
              for (int gq = 0; gq < QG; gq++) dp[gq] = E::mfma(vf[t], dof[gq][t], dp[gq]);
          }
          // element (gq, r): q = wq0 + 32 gq + l32 ; kv = kv0 + 32 c + 8 (r/4) + 4 g + r%4
#pragma unroll
          for (int gq = 0; gq < QG; gq++) {
            const int qrow = wq0 + 32 * gq + l32;
            const int qrow_c = min(qrow, a.Sq - 1);
            float ds[16];
            if (!edge && !BIAS && !DROP) {                   // interior tile: no side inputs at all
#pragma unroll
              for (int r = 0; r < 16; r++) {
                const float p = fast_exp2(__builtin_fmaf(s[gq][r], a.scale_log2e, -lq[gq]));
                ds[r] = p * (dp[gq][r] - dl[gq]);
              }
            } else {
#pragma unroll
              for (int r4 = 0; r4 < 4; r4++) {
                const int kv = kv0 + 32 * c + 8 * r4 + 4 * g;
                float bias[4] = {0.f, 0.f, 0.f, 0.f};
                uint32_t mbits = 0, dbits = 0x01010101u;
                if (BIAS) load_bias4<T>(alibip + (int64_t)qrow_c * a.al_sq, kv, a.Sk, alibi_vec, bias);
                if (apply_mask) {
                  if (a.mask_kind == kMaskDense) mbits = load_u8x4(maskp + (int64_t)qrow_c * a.Sk, kv, a.Sk, mask_vec);
                  else mbits = load_u8x4(maskp + (qrow_c & 127) * 128, kv & 127, 128, mask_vec);
                }
                if (DROP) dbits = load_u8x4(dropp + (int64_t)qrow_c * a.Sk, kv, a.Sk, drop_vec);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                  const int r = 4 * r4 + e;
                  float x = __builtin_fmaf(s[gq][r], a.scale_log2e, -lq[gq]);
                  if (BIAS) x = __builtin_fmaf(bias[e], kLog2e, x);
                  if (((mbits >> (8 * e)) & 0xffu) || (causal && kv + e > qrow)) x += kMaskFill * kLog2e;
                  float p = fast_exp2(x);
                  if (kv + e >= a.Sk) p = 0.f;
                  float dpv = dp[gq][r];
                  if (DROP) dpv = ((dbits >> (8 * e)) & 0xffu) ? dpv * a.inv_keep : 0.f;
                  ds[r] = p * (dpv - dl[gq]);
                }
              }
            }
            dsf[gq][c][0] = pack8<T>(ds);
            dsf[gq][c][1] = pack8<T>(ds + 8);
          }
        }
        // ---- dQ^T += K^T dS^T ----
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
          for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int db = 0; db < C::DB; db++) {
              const ACCT_LDS char* kaddr = kbuf + toff[db] + (32 * c + 16 * hh) * C::PITCH;
              const V8 ktf = join_tr<T>(lds_read_tr(kaddr), lds_read_tr(kaddr + 8 * C::PITCH));
#pragma unroll
              for (int gq = 0; gq < QG; gq++) acc[gq][db] = E::mfma(ktf, dsf[gq][c][hh], acc[gq][db]);
            }
      }
      dma_wait();
      __syncthreads();
    }
  }

  // ---- epilogue: dQ = scale * dQ^T, transposed through the wave's own LDS region ----
  T* dqp = (T*)a.dq + b * a.q_sb + h * a.q_sh;
  constexpr int OPITCH = C::DB * 64 + 16;
  ACCT_LDS char* obuf = smem + wave * (32 * OPITCH);
#pragma unroll
  for (int gq = 0; gq < QG; gq++) {
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        typename E::V2 t0 = E::cvt2(acc[gq][db][4 * r4 + 0] * a.scale, acc[gq][db][4 * r4 + 1] * a.scale);
        typename E::V2 t1 = E::cvt2(acc[gq][db][4 * r4 + 2] * a.scale, acc[gq][db][4 * r4 + 3] * a.scale);
        typename E::V4 ov = {t0[0], t0[1], t1[0], t1[1]};
        *reinterpret_cast<ACCT_LDS typename E::V4*>(obuf + l32 * OPITCH + (32 * db + 8 * r4 + 4 * g) * 2) = ov;
      }
    constexpr int NCH = C::CPR;
#pragma unroll
    for (int i = 0; i < (32 * NCH + 63) / 64; i++) {
      const int idx = lane + 64 * i;
      const int r = idx / NCH, ch = idx % NCH;
      const int grow = wq0 + 32 * gq + r;
      if (idx < 32 * NCH && grow < a.Sq) {
        const u32x4 v = *reinterpret_cast<const ACCT_LDS u32x4*>(obuf + r * OPITCH + ch * 16);
        *reinterpret_cast<u32x4*>(dqp + (int64_t)grow * a.q_ss + ch * 8) = v;
      }
    }
  }
}

// ============================================================================
// dK/dV kernel: kv-tile owner.  Each wave owns 32*KG key rows; Q and dO tiles of
// 64 query rows are staged through LDS.
// ============================================================================
template <typename T, int D, int KG, bool BIAS, bool DROP>
__global__ void __launch_bounds__(256) fa_bwd_dkdv_kernel(const FaArgs a) {
  using E = Elem<T>;
  using V8 = typename E::V8;
  using C = TileCfg<D>;
  constexpr int BNK = 128 * KG;                     // key rows per workgroup
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;   // [2 buffers][Q tile | dO tile]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, g = lane >> 5;
  const int BH = a.B * a.N;
  const int bh = blockIdx.x % BH;
  const int kt = (int)(blockIdx.x / BH);            // causal: the first key tiles are the heaviest
  const int b = bh / a.N, h = bh % a.N;
  const int k0 = kt * BNK;
  const int wk0 = k0 + wave * 32 * KG;              // first key row of this wave
  const int k_end = min(k0 + BNK, a.Sk);

  const T* qp = (const T*)a.q + b * a.q_sb + h * a.q_sh;
  const T* kp = (const T*)a.k + b * a.k_sb + h * a.k_sh;
  const T* vp = (const T*)a.v + b * a.v_sb + h * a.v_sh;
  const T* dop = (const T*)a.dout + b * a.o_sb + h * a.o_sh;
  const float* lsep = a.lse + (int64_t)bh * a.Sq;
  const float* delp = a.delta + (int64_t)bh * a.Sq;

  // visible query tiles (64 rows) of this workgroup
  const int kb_lo = k0 / 128, kb_hi = (k_end - 1) / 128;
  const int qb_lo = max(0, kb_lo - a.next_blk), qb_hi = min(a.Tr - 1, kb_hi + a.prev_blk);
  int i_lo = qb_lo * 2, i_hi = min(qb_hi * 2 + 1, (a.Sq - 1) / 64);
  const bool causal = a.mask_kind == kMaskCausal;
  if (causal) i_lo = max(i_lo, k0 / 64);            // query tiles wholly above the diagonal contribute 0
  const int wkb = wk0 / 128;

  // K and V fragments of the wave's key rows (B operands): lane holds key row l32, d = 16t + 8g ..
  V8 kf[KG][C::KS], vf[KG][C::KS];
#pragma unroll
  for (int gk = 0; gk < KG; gk++) {
    const int row = wk0 + 32 * gk + l32;
#pragma unroll
    for (int t = 0; t < C::KS; t++) {
      V8 z = {};
      kf[gk][t] = z;
      vf[gk][t] = z;
      if (row < a.Sk) {
        kf[gk][t] = *reinterpret_cast<const V8*>(kp + (int64_t)row * a.k_ss + 16 * t + 8 * g);
        vf[gk][t] = *reinterpret_cast<const V8*>(vp + (int64_t)row * a.v_ss + 16 * t + 8 * g);
      }
    }
  }
  f32x16 dk[KG][C::DB], dv[KG][C::DB];
#pragma unroll
  for (int gk = 0; gk < KG; gk++)
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) { dk[gk][db][r] = 0.f; dv[gk][db][r] = 0.f; }

  const int mb = a.mask_sb ? b : 0;
  const uint8_t* maskp = a.mask ? a.mask + (a.mask_kind == kMaskDense ? (int64_t)mb * a.mask_sb : 0) : nullptr;
  const uint8_t* dropp = DROP ? a.drop + ((int64_t)bh * a.Sq) * a.Sk : nullptr;
  const T* alibip = BIAS ? (const T*)a.alibi + b * a.al_sb + h * a.al_sh : nullptr;
  const bool stat_vec = ((((uintptr_t)lsep | (uintptr_t)delp) & 15) == 0);

  if (i_lo <= i_hi) {
    u32x4 qreg[C::NLD], doreg[C::NLD];
    tile_load<T, D>(qp, a.q_ss, i_lo * 64, a.Sq, qreg);
    tile_load<T, D>(dop, a.o_ss, i_lo * 64, a.Sq, doreg);
    tile_store<D>(smem, qreg);
    tile_store<D>(smem + C::TILEB, doreg);
    __syncthreads();

    for (int i = i_lo; i <= i_hi; i++) {
      const int buf = (i - i_lo) & 1;
      ACCT_LDS char* qbuf = smem + buf * 2 * C::TILEB;
      ACCT_LDS char* dobuf = qbuf + C::TILEB;
      const bool more = i < i_hi;
      if (more) {
        tile_load<T, D>(qp, a.q_ss, (i + 1) * 64, a.Sq, qreg);
        tile_load<T, D>(dop, a.o_ss, (i + 1) * 64, a.Sq, doreg);
      }
      const int qt0 = i * 64;
      const int qb = i >> 1;
      bool act = (wkb - a.next_blk <= qb) && (qb <= wkb + a.prev_blk) && (wk0 < a.Sk);
      if (causal) act = act && (qt0 + 63 >= wk0);
      if (a.row_prefix) act = act && (wk0 < (qt0 / a.row_prefix + 1) * a.row_prefix);
      bool apply_mask = false;
      if (a.mask_kind == kMaskDense && act) {
        const uint8_t f = a.blkflags[((int64_t)mb * a.Tr + qb) * a.Tc + wkb];
        act = f != kBlkSkip;
        apply_mask = f == kBlkApply;
      } else if (a.mask_kind == kMaskTile) {
        apply_mask = wkb == qb;
      }
      const bool diag = causal && (wk0 + 32 * KG - 1 > qt0);
      if (act) {
#pragma unroll
        for (int c = 0; c < 2; c++) {                 // 32-row query chunk of the tile
          // rows of this lane's C registers: q = qt0 + 32 c + 8 (r/4) + 4 g + r%4
          float lrow[16], drow[16];
#pragma unroll
          for (int r4 = 0; r4 < 4; r4++) {
            const int q = qt0 + 32 * c + 8 * r4 + 4 * g;
            load_f32x4(lsep, q, a.Sq, stat_vec, INFINITY, lrow + 4 * r4);
            load_f32x4(delp, q, a.Sq, stat_vec, 0.f, drow + 4 * r4);
          }
          f32x16 s[KG], dp[KG];
#pragma unroll
          for (int gk = 0; gk < KG; gk++)
#pragma unroll
            for (int r = 0; r < 16; r++) { s[gk][r] = 0.f; dp[gk][r] = 0.f; }
#pragma unroll
          for (int t = 0; t < C::KS; t++) {
            const V8 qa = lds_read_frag<T>(qbuf + (32 * c + l32) * C::ROWB + (16 * t + 8 * g) * 2);
            const V8 doa = lds_read_frag<T>(dobuf + (32 * c + l32) * C::ROWB + (16 * t + 8 * g) * 2);
#pragma unroll
            for (int gk = 0; gk < KG; gk++) {
              s[gk] = E::mfma(qa, kf[gk][t], s[gk]);       // S[q, kv]
              dp[gk] = E::mfma(doa, vf[gk][t], dp[gk]);    // dP[q, kv]
            }
          }
          V8 pf[KG][2], dsf[KG][2];
#pragma unroll
          for (int gk = 0; gk < KG; gk++) {
            const int kv = wk0 + 32 * gk + l32;
            const int kv_c = min(kv, a.Sk - 1);
            float pv[16], ds[16];
#pragma unroll
            for (int r = 0; r < 16; r++) {
              const int q = qt0 + 32 * c + 8 * (r >> 2) + 4 * g + (r & 3);
              const int q_c = min(q, a.Sq - 1);
              float x = __builtin_fmaf(s[gk][r], a.scale_log2e, -lrow[r] * kLog2e);
              bool keep = true;
              if (BIAS) x = __builtin_fmaf((float)alibip[(int64_t)q_c * a.al_sq + kv_c], kLog2e, x);
              if (apply_mask) {
                const uint8_t mbyte = a.mask_kind == kMaskDense ? maskp[(int64_t)q_c * a.Sk + kv_c]
                                                                : maskp[(q_c & 127) * 128 + (kv_c & 127)];
                if (mbyte) x += kMaskFill * kLog2e;
              }
              if (DROP) keep = dropp[(int64_t)q_c * a.Sk + kv_c] != 0;
              if (diag && kv > q) x += kMaskFill * kLog2e;
              float p = fast_exp2(x);
              if (kv >= a.Sk) p = 0.f;
              float dpv = dp[gk][r];
              float pd = p;
              if (DROP) {
                dpv = keep ? dpv * a.inv_keep : 0.f;
                pd = keep ? p * a.inv_keep : 0.f;
              }
              pv[r] = pd;
              ds[r] = p * (dpv - drow[r]);
            }
            pf[gk][0] = pack8<T>(pv);
            pf[gk][1] = pack8<T>(pv + 8);
            dsf[gk][0] = pack8<T>(ds);
            dsf[gk][1] = pack8<T>(ds + 8);
          }
          // ---- dV^T += dO^T P ; dK^T += Q^T dS  (contract over the 32 query rows of chunk c) ----
#pragma unroll
          for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int db = 0; db < C::DB; db++) {
              const int off = (32 * c + 16 * hh + 4 * g + ((lane & 15) >> 2)) * C::ROWB +
                              (32 * db + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
              const V8 dot = join_tr<T>(lds_read_tr(dobuf + off), lds_read_tr(dobuf + off + 8 * C::ROWB));
              const V8 qtf = join_tr<T>(lds_read_tr(qbuf + off), lds_read_tr(qbuf + off + 8 * C::ROWB));
#pragma unroll
              for (int gk = 0; gk < KG; gk++) {
                dv[gk][db] = E::mfma(dot, pf[gk][hh], dv[gk][db]);
                dk[gk][db] = E::mfma(qtf, dsf[gk][hh], dk[gk][db]);
              }
            }
        }
      }
      if (more) {
        ACCT_LDS char* nq = smem + (buf ^ 1) * 2 * C::TILEB;
        tile_store<D>(nq, qreg);
        tile_store<D>(nq + C::TILEB, doreg);
      }
      __syncthreads();
    }
  }

  // ---- epilogue ----
  T* dkp = (T*)a.dk + b * a.k_sb + h * a.k_sh;
  T* dvp = (T*)a.dv + b * a.v_sb + h * a.v_sh;
#pragma unroll
  for (int gk = 0; gk < KG; gk++) {
    const int row = wk0 + 32 * gk + l32;
    if (row < a.Sk) {
#pragma unroll
      for (int db = 0; db < C::DB; db++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
          const int d = 32 * db + 8 * r4 + 4 * g;
          if (d < D) {
            typename E::V2 t0 = E::cvt2(dk[gk][db][4 * r4 + 0] * a.scale, dk[gk][db][4 * r4 + 1] * a.scale);
            typename E::V2 t1 = E::cvt2(dk[gk][db][4 * r4 + 2] * a.scale, dk[gk][db][4 * r4 + 3] * a.scale);
            typename E::V4 kvv = {t0[0], t0[1], t1[0], t1[1]};
            *reinterpret_cast<typename E::V4*>(dkp + (int64_t)row * a.k_ss + d) = kvv;
            typename E::V2 u0 = E::cvt2(dv[gk][db][4 * r4 + 0], dv[gk][db][4 * r4 + 1]);
            typename E::V2 u1 = E::cvt2(dv[gk][db][4 * r4 + 2], dv[gk][db][4 * r4 + 3]);
            typename E::V4 vvv = {u0[0], u0[1], u1[0], u1[1]};
            *reinterpret_cast<typename E::V4*>(dvp + (int64_t)row * a.v_ss + d) = vvv;
          }
        }
    }
  }
}

// ---- launchers ----------------------------------------------------------------
template <typename T, int D, bool BIAS, bool DROP>
static hipError_t launch_bwd_t(FaArgs a, int stages, hipStream_t st) {
  using C = TileCfg<D>;
  const size_t smem = 4 * (size_t)C::TILEB;
  hipError_t e = hipSuccess;
  if (stages & kStageDq) {
    constexpr int QG = 1, NW = 8;
    constexpr int BM = 32 * QG * NW;
    using CS = SwzCfg<D>;
    constexpr size_t tiles = 4 * 64 * (size_t)CS::PITCH, stage = (size_t)NW * 32 * (CS::DB * 64 + 16);
    const size_t smem = tiles > stage ? tiles : stage;
    a.n_tiles = (a.Sq + BM - 1) / BM;
    auto kern = fa_bwd_dq_kernel<T, D, QG, NW, BIAS, DROP>;
    e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)((long long)a.n_tiles * a.B * a.N)), dim3(64 * NW), smem, st, a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (stages & kStageDkDv) {
    constexpr int KG = 1;
    a.n_tiles = (a.Sk + 128 * KG - 1) / (128 * KG);
    auto kern = fa_bwd_dkdv_kernel<T, D, KG, BIAS, DROP>;
    e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)((long long)a.n_tiles * a.B * a.N)), dim3(256), smem, st, a);
    e = hipGetLastError();
  }
  return e;
}

template <typename T, int D>
static hipError_t launch_bwd_d(const FaArgs& a, int stages, hipStream_t st) {
  const bool bias = a.alibi != nullptr, drop = a.drop != nullptr;
#ifndef ACCT_DEV_BUILD
  if (bias) return drop ? launch_bwd_t<T, D, true, true>(a, stages, st) : launch_bwd_t<T, D, true, false>(a, stages, st);
  if (drop) return launch_bwd_t<T, D, false, true>(a, stages, st);
#endif
  return launch_bwd_t<T, D, false, false>(a, stages, st);
}

hipError_t launch_bwd(const FaArgs& a, int dtype, int D, int stages, hipStream_t st) {
#ifdef ACCT_DEV_BUILD
  return launch_bwd_d<f16, 128>(a, stages, st);
#else
  if (dtype == 0) {
    if (D == 128) return launch_bwd_d<f16, 128>(a, stages, st);
    if (D == 64) return launch_bwd_d<f16, 64>(a, stages, st);
    if (D == 80) return launch_bwd_d<f16, 80>(a, stages, st);
  } else {
    if (D == 128) return launch_bwd_d<bf16, 128>(a, stages, st);
    if (D == 64) return launch_bwd_d<bf16, 64>(a, stages, st);
    if (D == 80) return launch_bwd_d<bf16, 80>(a, stages, st);
  }
  return hipErrorInvalidValue;
#endif
}

}  // namespace acct
