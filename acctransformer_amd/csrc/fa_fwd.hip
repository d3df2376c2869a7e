// FlashAttention2 forward for gfx950 (CDNA4).
//
// Replaces the reference's forward kernel builder
// (train/acctransformer/flash_attention/ops/flash_attention/flash_attention_fwd.py:308-474:
// Q-outer / KV-inner loops, online softmax, O rescale, O/l and L = m + ln l).
//
// Work split: one workgroup (4 or 8 waves) owns 32*QG query rows per wave of one
// (batch, head).  K and V tiles of 64 rows (128 in the variants without side
// inputs) are staged through LDS (double buffered) and shared by the waves.  The wave computes
// the TRANSPOSED score tile S^T = K Q^T with 32x32x16 MFMAs, so every lane
// holds scores of a single query row (column l%32 of the MFMA C tile): the
// online-softmax state (running max, running sum) is per lane, row
// reductions are in-register plus one swap with lane l^32, and the C tile is
// directly the B operand of O^T += V^T P^T.  V^T fragments come from the
// row-major V tile through transposed LDS reads.
#include "fa_common.hpp"
#include "fa_launch.hpp"

namespace acct {

template <typename T, int D, int QG, int NW, bool BIAS, bool DROP, bool MASKT, int KT = 2>
ACCT_DEV void fa_fwd_body(const FaArgs& a) {
  static_assert(KT == 2 || KT == 4, "key tiles are 64 or 128 rows (with a bias, 128 rows take the key-only form of it only)");
  constexpr int BN = 32 * KT;                       // key rows per tile
  constexpr int FRING = 4, VRING = 3;   // fragment reads in flight ahead of their MFMA (K row-major / V transposed)
  constexpr int TPB = 128 / BN;                     // tiles per 128-column block
  using E = Elem<T>;
  using V8 = typename E::V8;
  using C = SwzCfg<D>;
  constexpr int BM = 32 * QG * NW;
  constexpr int TILEB = BN * C::PITCH;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;   // [2 buffers][K tile | V tile]; reused by the epilogue

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: everything derived from it stays in scalar registers
  const int BH = a.B * a.N;
  int bh, rank;
  wg_map(blockIdx.x, BH, a.n_tiles, bh, rank);
  const int qt = a.n_tiles - 1 - rank;                      // heaviest (latest) causal tiles first
  const int b = bh / a.N, h = bh % a.N;
  const int q0 = qt * BM;
  const int wq0 = q0 + wave * 32 * QG;                      // first query row of this wave
  const int q_end = min(q0 + BM, a.Sq);                     // one past the last valid row of the block
  const int wq_end = min(wq0 + 32 * QG, a.Sq);

  const T* qp = (const T*)a.q + b * a.q_sb + h * a.q_sh;
  const T* kp = (const T*)a.k + b * a.k_sb + h * a.k_sh;
  const T* vp = (const T*)a.v + b * a.v_sb + h * a.v_sh;

  // ---- visible kv tiles of this block (128-block band; causal and row-prefix clip the top) ----
  const int qb_lo = q0 / 128, qb_hi = (q_end - 1) / 128;
  const int kvb_lo = max(0, qb_lo - a.prev_blk), kvb_hi = min(a.Tc - 1, qb_hi + a.next_blk);
  int j_lo = kvb_lo * TPB, j_hi = min(kvb_hi * TPB + TPB - 1, (a.Sk - 1) / BN);
  const bool causal = a.mask_kind == kMaskCausal;
  if (causal) j_hi = min(j_hi, (q_end - 1) / BN);
  if (a.row_prefix) j_hi = min(j_hi, (((q_end - 1) / a.row_prefix + 1) * a.row_prefix - 1) / BN);
  const int wqb = wq0 / 128;                                // 128-block of this wave's rows
  BlkClassWindow flwin;                                     // block classes of a dense mask: 64 blocks at a time in scalar registers
  bool flwin_ready = false;
  if (MASKT && a.mask_kind == kMaskDense) {
    // tiles at either end whose 128x128 blocks are wholly masked for every row block of this workgroup are
    // not streamed at all (key padding: the padded tail of every sequence).  With at most 64 blocks in the
    // band, one round trip to memory yields both the trimmed range and the wave's class window.
    const uint8_t* fl = a.blkflags + ((int64_t)(a.mask_sb ? b : 0) * a.Tr) * a.Tc;
    int b_lo = j_lo / TPB, b_hi = j_hi / TPB;
    const uint8_t* tails = a.blktail ? a.blktail + ((int64_t)(a.mask_sb ? b : 0) * a.Tr) * a.Tc : nullptr;
    if (j_lo <= j_hi && flwin.init_trimmed(fl, 1, a.Tc, qb_lo, qb_hi - qb_lo + 1, min(wqb, qb_hi), b_lo, b_hi, lane, tails)) {
      j_lo = max(j_lo, b_lo * TPB);
      j_hi = min(j_hi, b_hi * TPB + TPB - 1);
      flwin_ready = true;
    } else {
      auto dead = [&](int j) {
        for (int qb = qb_lo; qb <= qb_hi; qb++)
          if (fl[(int64_t)qb * a.Tc + j / TPB] != kBlkSkip) return false;
        return true;
      };
      trim_dead_tiles(j_lo, j_hi, lane, dead);
    }
  }
  const int wkv_limit = a.row_prefix ? (wq0 / a.row_prefix + 1) * a.row_prefix : 0x7fffffff;   // keys past it are absent

  // ---- Q fragments (B operand of K Q^T): lane holds row l32, d = 16t + 8g .. +7 ----
  V8 qf[QG][C::KS];
#pragma unroll
  for (int gq = 0; gq < QG; gq++) {
    const int row = min(wq0 + 32 * gq + l32, a.Sq - 1);     // rows past Sq repeat the last row; never stored
#pragma unroll
    for (int t = 0; t < C::KS; t++) {
      // k-steps (or the upper half of one) past the head dim: zeros there make the products ignore whatever
      // the K tile holds in those slots
      const bool inside = 16 * t + 8 * g < a.hd;
      V8 z;
#pragma unroll
      for (int e = 0; e < 8; e++) z[e] = 0;
      qf[gq][t] = inside ? *reinterpret_cast<const V8*>(qp + (int64_t)row * a.q_ss + 16 * t + 8 * g) : z;
    }
  }

  // ---- per-lane LDS offsets (tile-invariant) ----
  // K fragment of k-step t: row l32, chunk 2t + g.  Chunk c + 8 of a row sits in slot (c ^ swz) ^ 8, so the
  // offsets of the upper half of the head dim are one XOR away from the lower four (wide rows only).
  constexpr int NKOFF = (C::CH >= 16 && C::KS > 4) ? 4 : C::KS;
  int koff_[NKOFF];
#pragma unroll
  for (int t = 0; t < NKOFF; t++) koff_[t] = l32 * C::PITCH + swz_off(2 * t + g, C::swz(l32));
  auto koff = [&](int t) { return t < NKOFF ? koff_[t] : (koff_[t & 3] ^ ((t >> 2) * 128)); };
  const int trow = 4 * g + ((lane & 15) >> 2);              // transposed reads: row within an 8-row group
  const int tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
  int voff[C::DB];                                          // V^T fragment of d block db
#pragma unroll
  for (int db = 0; db < C::DB; db++) voff[db] = trow * C::PITCH + swz_off(4 * db + tchunk, C::swz(trow)) + 8 * (lane & 1);

  f32x16 o[QG][C::DB];
  float m[QG], lsum[QG];
#pragma unroll
  for (int gq = 0; gq < QG; gq++) {
    m[gq] = -INFINITY;
    lsum[gq] = 0.f;
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[gq][db][r] = 0.f;
  }

  // Scores stay in raw q.k units (exp2 argument = s * scale*log2e - m * scale*log2e, one FMA) unless a
  // bias is added, in which case they become scale*s + bias first (one mixed-precision FMA per score:
  // the fp16 / bf16 bias is an operand as it is).
  // A key-only bias (row stride 0) that the DMA can stage goes in as the INITIAL value of the score accumulators
  // instead (bias / scale, the MFMAs add q.k): the scores stay in raw units and nothing is spent per score.
  const bool bias_staged = BIAS && (a.Sk & 7) == 0 && (((uintptr_t)a.alibi & 15) | ((a.al_sb | a.al_sh | a.al_sq) & 7)) == 0;
  // (the launcher picks 128-key tiles for a bias only when both hold: known at compile time there)
  const bool row_bias = BIAS && (KT == 4 || a.al_sq == 0);   // the bias depends on the key only: one row per tile
  const bool acc_bias = BIAS && (KT == 4 || (row_bias && bias_staged));
  const bool scaled = BIAS && !acc_bias;                   // scores are turned into scale*s + bias before the softmax
  const float cmul = scaled ? kLog2e : a.scale_log2e;
  const float madd = scaled ? kMaskFill : a.mask_add_raw;          // the additive -10000 in the units of s
  const float lazy_thr = 8.0f / cmul;                              // 8 octaves, in the units of s
  const int mb = a.mask_sb ? b : 0;
  const uint8_t* maskp = a.mask ? a.mask + (a.mask_kind == kMaskDense ? (int64_t)mb * a.mask_sb * a.mask_es : 0) : nullptr;
  const T* alibip = BIAS ? (const T*)a.alibi + b * a.al_sb + h * a.al_sh : nullptr;
  const bool mask_vec = a.mask_kind == kMaskDense ? ((((uintptr_t)a.mask / a.mask_es) | (uintptr_t)a.Sk | (uintptr_t)a.mask_sb) & 3) == 0
                                                  : ((uintptr_t)a.mask & (4 * a.mask_es - 1)) == 0;
  const bool alibi_vec = BIAS && (((uintptr_t)a.alibi & 7) | ((a.al_sb | a.al_sh | a.al_sq) & 3)) == 0;

  TileDma<T, D, BN, NW> kdma, vdma;
  const int cpr = a.hd >> 3;                                // valid 16-byte chunks per row
  kdma.plan(a.k_ss, cpr);
  vdma.plan(a.v_ss, cpr);
  // bias tiles of this wave's rows are staged through a wave-private LDS region one tile ahead
  // (with 128-key tiles only the key-only form is served: two 256-byte rows per wave)
  constexpr int BIASB = BIAS ? (KT == 4 ? 512 : QG * 4096) : 0;
  static_assert(KT == 2 || !BIAS || QG == 1, "128-key tiles with a bias: 32 rows per wave");
  ACCT_LDS char* bias_lds = smem + 4 * TILEB + wave * BIASB;
  // (a key-only bias: rows of consecutive tiles alternate between two 256-byte slots of the region, so the next
  // one is requested together with the next K/V tile; a tile bias has one slot and is requested once read)
  auto stage_bias = [&](int jn) {
#pragma unroll
    for (int gq = 0; gq < QG; gq++) {
      if (row_bias) bias_row_dma<T>(alibip, jn * BN, a.Sk, bias_lds + gq * 4096 + (acc_bias ? (jn & 1) * 256 : 0));
      else bias_tile_dma<T>(alibip, a.al_sq, wq0 + 32 * gq, a.Sq, jn * 64, a.Sk, bias_lds + gq * 4096);
    }
  };
  // keep bits of this wave's rows and one tile, staged with the tile's DMA (double buffered)
  using DropStage = DropRowStage<DROP, QG, KT>;
  ACCT_LDS char* drop_lds = smem + 4 * TILEB + NW * BIASB + wave * (2 * DropStage::BYTES);
  // ---- the phases of a tile step: classification, S^T = K Q^T, online softmax, O^T += V^T P^T ----
  const uint8_t* flrow = (MASKT && a.mask_kind == kMaskDense) ? a.blkflags + ((int64_t)mb * a.Tr + wqb) * a.Tc : nullptr;
  if (!flwin_ready && j_lo <= j_hi)
    flwin.init(flrow, 1, j_lo / TPB, j_hi / TPB, lane, (flrow && a.blktail) ? a.blktail + (flrow - a.blkflags) : nullptr);
  enum : uint32_t { kAct = 1u, kApply = 2u, kDiag = 4u, kTailShift = 8u };   // bits 8..15: key tail of the tile's block (0: none)
  // what this wave does with tile j (tiles must be asked for in ascending order)
  auto classify = [&](int j) -> uint32_t {
    const uint32_t fl_cur = flwin.get(j / TPB, lane);
    const int kv0 = j * BN, kvb = j / TPB;
    bool act = (kvb - a.next_blk <= wqb) && (wqb <= kvb + a.prev_blk) && (wq0 < a.Sq);
    if (causal) act = act && (kv0 <= wq_end - 1);
    act = act && (kv0 < wkv_limit);
    bool apply_mask = false;
    bool diag = causal;                                     // keys after the query are hidden, by index compare
    uint32_t tail = 0;
    if (MASKT && a.mask_kind == kMaskDense && act) {
      act = fl_cur != kBlkSkip;
      apply_mask = fl_cur == kBlkApply;
      if (fl_cur == kBlkTriu) { diag = true; act = kv0 <= wq_end - 1; }
      if (apply_mask && (tail = flwin.tail(kvb)) != 0) {
        // every row of the block hides exactly the keys from its tail-th on: an index compare, no mask loads
        apply_mask = false;
        act = kv0 < kvb * 128 + (int)tail;
      }
    } else if (MASKT && a.mask_kind == kMaskTile) {
      apply_mask = wqb == kvb;
    }
    return (act ? kAct : 0u) | (apply_mask ? kApply : 0u) | (diag ? kDiag : 0u) | (tail << kTailShift);
  };
  // stage key rows [j BN, (j+1) BN) of K or V into an LDS tile
  auto stage_tile = [&](const TileDma<T, D, BN, NW>& dma, const T* base, int64_t ss, int j, ACCT_LDS char* dst) {
    if ((j + 1) * BN <= a.Sk) dma.issue(base, ss, j * BN, dst);
    else tile_dma<T, D, BN, NW>(base, ss, j * BN, a.Sk, dst, cpr);   // ragged last tile: clamped rows
  };
  // S^T = K Q^T : s[gq][c] is the 32(kv) x 32(q) tile of kv chunk c
  auto gemm_s = [&](const ACCT_LDS char* kbuf, int j, f32x16 (&s)[QG][KT]) {
    if (BIAS && acc_bias) {
      // element (c, r) belongs to key 32 c + 8 (r/4) + 4 g + r%4 of the tile, whatever the lane's row
#pragma unroll
      for (int gq = 0; gq < QG; gq++)
#pragma unroll
        for (int c = 0; c < KT; c++)
#pragma unroll
          for (int r4 = 0; r4 < 4; r4++) {
            const typename E::V4 bv = bias_tile_read<T>(bias_lds + gq * 4096 + (j & 1) * 256, 0, 4 * c + r4, g);
#pragma unroll
            for (int e = 0; e < 4; e++) s[gq][c][4 * r4 + e] = (float)bv[e] * a.inv_scale;
          }
    } else {
#pragma unroll
      for (int gq = 0; gq < QG; gq++)
#pragma unroll
        for (int c = 0; c < KT; c++)
#pragma unroll
          for (int r = 0; r < 16; r++) s[gq][c][r] = 0.f;
    }
    // K fragments travel through a ring of FRING register sets: FRING reads are in flight ahead of the
    // MFMA that consumes the oldest one, so that a wave covers the LDS latency (well over one MFMA) by
    // itself.  The scheduling barriers keep the compiler from folding the ring back into read-wait-MFMA.
    constexpr int NF = KT * C::KS;
    constexpr int RING = FRING < NF ? FRING : NF;
    V8 ring[RING];
    auto kread = [&](int i) { return lds_read_frag<T>(kbuf + koff(i % C::KS) + (i / C::KS) * 32 * C::PITCH); };
#pragma unroll
    for (int i = 0; i < RING; i++) ring[i] = kread(i);
#pragma unroll
    for (int i = 0; i < NF; i++) {
      const int c = i / C::KS, t = i % C::KS;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int gq = 0; gq < QG; gq++) s[gq][c] = E::mfma(ring[i % RING], qf[gq][t], s[gq][c]);
      if (i + RING < NF)
        ring[i % RING] = kread(i + RING);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // O^T += V^T P^T, the transposed V fragments through a ring as well
  auto gemm_pv = [&](const ACCT_LDS char* vbuf, const V8 (&pf)[QG][KT][2]) {
    constexpr int NT = 2 * KT * C::DB;
    constexpr int RING = VRING < NT ? VRING : NT;
    auto tread = [&](int i) {
      const int db = i % C::DB, ch = i / C::DB;               // ch = 2 c + hh: rows 16 ch .. of the tile
      const ACCT_LDS char* vaddr = vbuf + voff[db] + 16 * ch * C::PITCH;
      return join_tr<T>(lds_read_tr(vaddr), lds_read_tr(vaddr + C::tr_hi(db)));
    };
    V8 ring[RING];
#pragma unroll
    for (int i = 0; i < RING; i++) ring[i] = tread(i);
#pragma unroll
    for (int i = 0; i < NT; i++) {
      const int db = i % C::DB, ch = i / C::DB;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int gq = 0; gq < QG; gq++) o[gq][db] = E::mfma(ring[i % RING], pf[gq][ch >> 1][ch & 1], o[gq][db]);
      if (i + RING < NT) ring[i % RING] = tread(i + RING);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // online softmax of the scores of tile j -> P^T fragments; `buf` = parity of the tile's staging buffers
  auto softmax = [&](int j, int buf, uint32_t info, f32x16 (&s)[QG][KT], V8 (&pf)[QG][KT][2]) {
    const int kv0 = j * BN;
    const bool apply_mask = MASKT && (info & kApply), diag = info & kDiag;
    const int tail = MASKT ? (int)((info >> kTailShift) & 0xffu) : 0;
    const int last_key = tail ? min(a.Sk, (j / TPB) * 128 + tail) - 1 : a.Sk - 1;     // last key that exists and is not behind a key tail
    // element (gq, c, r): q = wq0 + 32 gq + l32 ; kv = kv0 + 32 c + 8 (r/4) + 4 g + r%4
    const bool edge = apply_mask || (diag && (kv0 + BN - 1 > wq0)) || (kv0 + BN - 1 > last_key);
#pragma unroll
    for (int gq = 0; gq < QG; gq++) {
      const int qrow = wq0 + 32 * gq + l32;
      const int qrow_c = min(qrow, a.Sq - 1);            // clamped for side-input addressing
      if (BIAS && !acc_bias) {
        if (bias_staged) {
          typename E::V4 bv[2][4];
#pragma unroll
          for (int c = 0; c < 2; c++)
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) bv[c][r4] = bias_tile_read<T>(bias_lds + gq * 4096, row_bias ? 0 : l32, 4 * c + r4, g);
          if (gq == QG - 1) {
            // the tile is in registers: its LDS region can take the next tile, which has the rest of
            // this step to land (the end-of-step wait covers it)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (j < j_hi) stage_bias(j + 1);
          }
#pragma unroll
          for (int c = 0; c < 2; c++)
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++)
#pragma unroll
              for (int e = 0; e < 4; e++)
                s[gq][c][4 * r4 + e] = __builtin_fmaf(s[gq][c][4 * r4 + e], a.scale, (float)bv[c][r4][e]);
        } else {
#pragma unroll
          for (int c = 0; c < 2; c++)
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
              const int kv = kv0 + 32 * c + 8 * r4 + 4 * g;
              float bias[4];
              load_bias4<T>(alibip + (int64_t)qrow_c * a.al_sq, kv, a.Sk, alibi_vec, bias);
#pragma unroll
              for (int e = 0; e < 4; e++)
                s[gq][c][4 * r4 + e] = __builtin_fmaf(s[gq][c][4 * r4 + e], a.scale, bias[e]);
            }
        }
      }
      if (edge) {
        if (apply_mask) {
#pragma unroll
          for (int c = 0; c < KT; c++)
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
              const int kv = kv0 + 32 * c + 8 * r4 + 4 * g;
              uint32_t mbits;
              if (a.mask_kind == kMaskDense) mbits = load_mask4(maskp + (int64_t)qrow_c * a.Sk * a.mask_es, kv, a.Sk, mask_vec, a.mask_es);
              else mbits = load_mask4(maskp + (qrow_c & 127) * 128 * a.mask_es, kv & 127, 128, mask_vec, a.mask_es);
#pragma unroll
              for (int e = 0; e < 4; e++)
                if ((mbits >> (8 * e)) & 0xffu) s[gq][c][4 * r4 + e] += madd;
            }
        }
        {
          // Keys after the query (causal diagonal) and keys past Sk are removed outright: with the additive
          // mask their probability underflows to exactly 0 as well (the diagonal key is always visible), so
          // the result is the same bit for bit at a third of the vector instructions.
          int vis = last_key - kv0 - 4 * g;                  // last visible key, relative to this lane's first
          if (diag) vis = min(vis, qrow - kv0 - 4 * g);
          // (compare and select through VCC: see select_if_gt)
          const float ninf = -INFINITY;
#pragma unroll
          for (int c = 0; c < KT; c++) {
            const int visc = vis - 32 * c;
#pragma unroll
            for (int r = 0; r < 16; r++) s[gq][c][r] = select_if_gt(s[gq][c][r], 8 * (r >> 2) + (r & 3), visc, ninf);
          }
        }
      }
      // ---- online softmax for query row qrow ----
      float mx = s[gq][0][0];
#pragma unroll
      for (int c = 0; c < KT; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[gq][c][r]);
      mx = pair_max(mx);
      // Lazy running max: it only moves when a score beats it by more than 2^8 in probability
      // terms.  Until then P = exp2(s - m) may reach 256 instead of 1 (harmless in fp16/bf16 and in
      // the fp32 sums; O = acc / l and LSE = m + ln l are unchanged), and the O rescale below is
      // skipped for almost every tile after the first.
      const bool grow = mx > m[gq] + lazy_thr;
      const float m_new = grow ? mx : m[gq];
      const float alpha = grow ? fast_exp2((m[gq] - m_new) * cmul) : 1.0f;
      const float mc = m_new * cmul;
      m[gq] = m_new;
      float rs = 0.f;
      float p[KT][16];
#pragma unroll
      for (int c = 0; c < KT; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          p[c][r] = fast_exp2(__builtin_fmaf(s[gq][c][r], cmul, -mc));
          rs += p[c][r];
        }
      lsum[gq] = lsum[gq] * alpha + rs;                  // row sum BEFORE dropout
      if (DROP) {
        // keep bits of this row and tile: word c covers keys kv0 + 32c .. +31
#pragma unroll
        for (int c = 0; c < KT; c++) {
          const uint32_t w = DropStage::word(drop_lds + buf * DropStage::BYTES, 32 * gq + l32, c) >> (4 * g);
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int32_t sel = __builtin_amdgcn_sbfe((int)w, 8 * (r >> 2) + (r & 3), 1);   // keep ? ~0 : 0
            p[c][r] = __uint_as_float(__float_as_uint(p[c][r]) & (uint32_t)sel);        // (1 / keep_prob: once, on O)
          }
        }
      }
#pragma unroll
      for (int c = 0; c < KT; c++)
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
          typename E::V2 t0 = E::cvt2(p[c][8 * hh + 0], p[c][8 * hh + 1]);
          typename E::V2 t1 = E::cvt2(p[c][8 * hh + 2], p[c][8 * hh + 3]);
          typename E::V2 t2 = E::cvt2(p[c][8 * hh + 4], p[c][8 * hh + 5]);
          typename E::V2 t3 = E::cvt2(p[c][8 * hh + 6], p[c][8 * hh + 7]);
          V8 pv = {t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
          pf[gq][c][hh] = pv;
        }
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int db = 0; db < C::DB; db++)
#pragma unroll
          for (int r = 0; r < 16; r++) o[gq][db][r] *= alpha;
      }
    }
  };

  if (j_lo <= j_hi) {
    tile_dma<T, D, BN, NW>(kp, a.k_ss, j_lo * BN, a.Sk, smem, cpr);
    tile_dma<T, D, BN, NW>(vp, a.v_ss, j_lo * BN, a.Sk, smem + TILEB, cpr);
    if (BIAS && bias_staged && wq0 < a.Sq) stage_bias(j_lo);
    DropStage::issue(a, bh, wq0, j_lo, lane, drop_lds);
    // A full wait the compiler can see: every load issued so far (Q fragments included) is complete, so
    // it places no vmcnt wait inside the loop -- such a wait would also stall on the next tile's DMA.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (int j = j_lo; j <= j_hi; j++) {
      const int buf = (j - j_lo) & 1;
      ACCT_LDS char* kbuf = smem + buf * 2 * TILEB;
      ACCT_LDS char* vbuf = kbuf + TILEB;
      if (j < j_hi) {                                       // next tile streams into the other buffer meanwhile
        ACCT_LDS char* nb = smem + (buf ^ 1) * 2 * TILEB;
        stage_tile(kdma, kp, a.k_ss, j + 1, nb);
        stage_tile(vdma, vp, a.v_ss, j + 1, nb + TILEB);
        DropStage::issue(a, bh, wq0, j + 1, lane, drop_lds + (buf ^ 1) * DropStage::BYTES);
        if (BIAS && acc_bias && wq0 < a.Sq) stage_bias(j + 1);
      }
      const uint32_t info = classify(j);
      if (info & kAct) {
        f32x16 s[QG][KT];
        V8 pf[QG][KT][2];
        gemm_s(kbuf, j, s);
        softmax(j, buf, info, s, pf);
        gemm_pv(vbuf, pf);
      } else if (BIAS && bias_staged && !acc_bias && j < j_hi && wq0 < a.Sq) {
        stage_bias(j + 1);                                  // nothing to read in this step: the region is free
      }
      dma_wait();
      __syncthreads();
    }
  }

  // ---- epilogue: O = O^T / l, LSE = m + ln l.  Each wave transposes its rows through its own
  // LDS region (pitch 2D+16 keeps the 8-byte writes of 16 rows on distinct banks) so that the
  // global stores are whole rows. ----
  T* op = (T*)a.o + b * a.o_sb + h * a.o_sh;
  const float mnat = scaled ? 1.0f : a.scale;
  constexpr int OPITCH = C::DB * 64 + 16;
  ACCT_LDS char* obuf = smem + wave * (32 * OPITCH);
#pragma unroll
  for (int gq = 0; gq < QG; gq++) {
    const int row = wq0 + 32 * gq + l32;
    const float l = pair_sum(lsum[gq]);
    const float inv = l > 0.f ? (DROP ? a.inv_keep : 1.0f) / l : 0.f;
    if (row < a.Sq && g == 0) a.lse[(int64_t)bh * a.Sq + row] = l > 0.f ? m[gq] * mnat + __logf(l) : -INFINITY;
#pragma unroll
    for (int db = 0; db < C::DB; db++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        typename E::V2 t0 = E::cvt2(o[gq][db][4 * r4 + 0] * inv, o[gq][db][4 * r4 + 1] * inv);
        typename E::V2 t1 = E::cvt2(o[gq][db][4 * r4 + 2] * inv, o[gq][db][4 * r4 + 3] * inv);
        typename E::V4 ov = {t0[0], t0[1], t1[0], t1[1]};
        *reinterpret_cast<ACCT_LDS typename E::V4*>(obuf + l32 * OPITCH + (32 * db + 8 * r4 + 4 * g) * 2) = ov;
      }
    // read back row-contiguous: 16-byte chunk ch of row r
    const int nch = a.hd >> 3;                       // valid 16-byte chunks per row
    const uint32_t nch_inv = recip16(nch);
#pragma unroll
    for (int i = 0; i < (32 * C::CPR + 63) / 64; i++) {
      const int idx = lane + 64 * i;
      const int r = div_small(idx, nch_inv), ch = idx - r * nch;
      const int grow = wq0 + 32 * gq + r;
      if (idx < 32 * nch && grow < a.Sq) {
        const u32x4 v = *reinterpret_cast<const ACCT_LDS u32x4*>(obuf + r * OPITCH + ch * 16);
        *reinterpret_cast<u32x4*>(op + (int64_t)grow * a.o_ss + ch * 8) = v;
      }
    }
  }
}


// The variant that knows mask tensors but neither a bias nor dropout carries a second body: a workgroup whose
// rows see nothing but the causal pattern in a dense mask (block classes: clean before the diagonal, the
// causal diagonal, skipped after it) runs the code of the variant without side inputs, by index compare.
// A causal mask given as a tensor then costs one look at the class table per workgroup.
template <typename T, int D, int QG, int NW, bool BIAS, bool DROP, bool MASKT, int KT = 2>
__global__ void __launch_bounds__(64 * NW) fa_fwd_kernel(const FaArgs a) {
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
        fa_fwd_body<T, D, QG, NW, false, false, false, KT>(c);
        return;
      }
    }
  }
  fa_fwd_body<T, D, QG, NW, BIAS, DROP, MASKT, KT>(a);
}

template <typename T, int D, int QG, int NW, bool BIAS, bool DROP, int KT>
static hipError_t launch_fwd_kt(FaArgs a, hipStream_t st) {
  using C = SwzCfg<D>;
  constexpr int BM = 32 * QG * NW;
  a.n_tiles = (a.Sq + BM - 1) / BM;
  const bool mask_t = BIAS || DROP || a.mask_kind == kMaskDense || a.mask_kind == kMaskTile;
  constexpr size_t biasb = BIAS ? (KT == 4 ? 512 : QG * 4096) : 0;     // per wave, as in the kernel
  const size_t tiles = 4 * 32 * KT * (size_t)C::PITCH + NW * biasb + (size_t)NW * 2 * DropRowStage<DROP, QG, KT>::BYTES, stage = (size_t)NW * 32 * (C::DB * 64 + 16);
  static_assert(4 * 32 * KT * (size_t)C::PITCH + NW * biasb + (size_t)NW * 2 * DropRowStage<DROP, QG, KT>::BYTES <= 160 * 1024, "the workgroup's LDS must fit the CU's 160 KB");
  const size_t smem = tiles > stage ? tiles : stage;
  auto kern = mask_t ? fa_fwd_kernel<T, D, QG, NW, BIAS, DROP, true, KT> : fa_fwd_kernel<T, D, QG, NW, BIAS, DROP, BIAS || DROP, KT>;
  hipError_t e = allow_dynamic_lds((const void*)kern, smem);
  if (e != hipSuccess) return e;
  const long long nblk = (long long)a.n_tiles * a.B * a.N;
  hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(64 * NW), smem, st, a);
  return hipGetLastError();
}

template <typename T, int D, int QG, int NW, bool BIAS, bool DROP>
static hipError_t launch_fwd_t(const FaArgs& a, hipStream_t st) {
  // K/V stream in tiles of 128 keys where registers and LDS allow (8 waves x 32 rows, D <= 128): twice the
  // matrix work between two barriers, -2 % (causal) to -6 % (full).  A bias tile per wave does not fit beside
  // them; a key-only bias that the DMA can stage (the kernel's own test, repeated here) is a 256-byte row and does.
  constexpr bool BIG = QG == 1 && NW == 8 && D <= 128;
  if constexpr (BIG && BIAS) {
    const bool row_staged = a.al_sq == 0 && (a.Sk & 7) == 0 && (((uintptr_t)a.alibi & 15) | ((a.al_sb | a.al_sh) & 7)) == 0;
    return row_staged ? launch_fwd_kt<T, D, QG, NW, BIAS, DROP, 4>(a, st) : launch_fwd_kt<T, D, QG, NW, BIAS, DROP, 2>(a, st);
  } else {
    return launch_fwd_kt<T, D, QG, NW, BIAS, DROP, BIG ? 4 : 2>(a, st);
  }
}

// SIDE: 2 = bias and dropout variants, 1 = the dropout variant only (head dims 40, 160, 256)
template <typename T, int D, int QG, int NW, int SIDE = 2>
static hipError_t launch_fwd_q(const FaArgs& a, hipStream_t st) {
  const bool bias = a.alibi != nullptr, drop = a.droprow != nullptr || a.dropcol != nullptr;
#ifndef ACCT_DEV_BUILD
  if constexpr (SIDE == 2) {
    if (bias) return drop ? launch_fwd_t<T, D, QG, NW, true, true>(a, st) : launch_fwd_t<T, D, QG, NW, true, false>(a, st);
  }
  if constexpr (SIDE >= 1) {
    if (drop && !bias) return launch_fwd_t<T, D, QG, NW, false, true>(a, st);
  }
#endif
  if (bias || drop) return hipErrorNotSupported;       // (development build: plain variants only)
  return launch_fwd_t<T, D, QG, NW, false, false>(a, st);
}

// variant: 1 = 4 waves x 32 rows, 3 = 8 waves x 32 rows
template <typename T, int D>
static hipError_t launch_fwd_d(const FaArgs& a, int variant, hipStream_t st) {
  return variant == 3 ? launch_fwd_q<T, D, 1, 8>(a, st) : launch_fwd_q<T, D, 1, 4>(a, st);
}
// head dims 40 and 160: no bias variants
template <typename T, int D>
static hipError_t launch_fwd_plain(const FaArgs& a, int variant, hipStream_t st) {
  return variant == 3 ? launch_fwd_q<T, D, 1, 8, 1>(a, st) : launch_fwd_q<T, D, 1, 4, 1>(a, st);
}

#ifdef ACCT_DEV_BUILD
bool fwd_variants_complete() { return false; }
#else
bool fwd_variants_complete() { return true; }
#endif

hipError_t launch_fwd(const FaArgs& a, int dtype, int Dr, int qg, hipStream_t st) {
  const int D = head_dim_class(Dr);
#ifdef ACCT_DEV_BUILD
  if (dtype != 0 || D != 128) return hipErrorNotSupported;
  return launch_fwd_d<f16, 128>(a, qg, st);
#else
  if (dtype == 0) {
    if (D == 128) return launch_fwd_d<f16, 128>(a, qg, st);
    if (D == 64) return launch_fwd_d<f16, 64>(a, qg, st);
    if (D == 80) return launch_fwd_d<f16, 80>(a, qg, st);
    if (D == 40) return launch_fwd_plain<f16, 40>(a, qg, st);
    if (D == 160) return launch_fwd_plain<f16, 160>(a, qg, st);
    if (D == 256) return launch_fwd_q<f16, 256, 1, 4, 1>(a, st);     // one wave per SIMD: 128 accumulator registers
  } else {
    if (D == 128) return launch_fwd_d<bf16, 128>(a, qg, st);
    if (D == 64) return launch_fwd_d<bf16, 64>(a, qg, st);
    if (D == 80) return launch_fwd_d<bf16, 80>(a, qg, st);
    if (D == 40) return launch_fwd_plain<bf16, 40>(a, qg, st);
    if (D == 160) return launch_fwd_plain<bf16, 160>(a, qg, st);
    if (D == 256) return launch_fwd_q<bf16, 256, 1, 4, 1>(a, st);
  }
  return hipErrorInvalidValue;
#endif
}

}  // namespace acct
