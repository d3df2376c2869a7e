// Device-side building blocks shared by the gfx950 attention kernels:
// vector types, the 32x32x16 MFMA wrappers, LDS fragment reads and the
// kernel argument block.  CDNA4 only (wave64, MFMA, ds_read_*_tr_b16).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fa_index_math.hpp"

namespace acct {

typedef _Float16 f16;
typedef __bf16 bf16;
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define ACCT_LDS __attribute__((address_space(3)))
#define ACCT_DEV __device__ __forceinline__

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMaskFill = -10000.0f;   // additive mask value of the reference (constants.py:24)

// ---- element-type traits ---------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<f16> {
  using V8 = f16x8; using V4 = f16x4; using V2 = f16x2;
  static ACCT_DEV f32x16 mfma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static ACCT_DEV V2 cvt2(float x, float y) { f32x2 t = {x, y}; return __builtin_convertvector(t, V2); }
};
template <> struct Elem<bf16> {
  using V8 = bf16x8; using V4 = bf16x4; using V2 = bf16x2;
  static ACCT_DEV f32x16 mfma(V8 a, V8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static ACCT_DEV V2 cvt2(float x, float y) { f32x2 t = {x, y}; return __builtin_convertvector(t, V2); }
};

// The MFMA 32x32x16 register layouts used throughout (lane l, g = l / 32):
//   A (32 x 16): lane holds row  l % 32, k = 8g .. 8g+7
//   B (16 x 32): lane holds col  l % 32, k = 8g .. 8g+7
//   C (32 x 32): lane holds col  l % 32, rows 8*(r/4) + 4g + r%4 for r = 0..15
// A C tile can therefore be fed back as a B operand of a product that
// contracts over C's rows: registers 8h..8h+7 are the k = 8g..8g+7 slots of
// k-step h, i.e. rows 16h + 8*(e/4) + 4g + e%4 (e = 0..7) of the C tile.

// 16-byte LDS read of an A/B fragment stored row-major.
template <typename T>
ACCT_DEV typename Elem<T>::V8 lds_read_frag(const ACCT_LDS char* p) {
  return *reinterpret_cast<const ACCT_LDS typename Elem<T>::V8*>(p);
}

// Transposed LDS read (ds_read_b64_tr_b16).  Within each block of 16 lanes,
// lane i supplies the address of 4 consecutive 16-bit elements
// M[k0 + i/4][n0 + 4*(i%4) ..]; lane j receives M[k0 + 0..3][n0 + j].
ACCT_DEV i16x4 lds_read_tr(const ACCT_LDS char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((ACCT_LDS i16x4*)(p));
}

template <typename T>
ACCT_DEV typename Elem<T>::V8 join_tr(i16x4 lo, i16x4 hi) {
  typedef short i16x8 __attribute__((ext_vector_type(8)));
  i16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(typename Elem<T>::V8, v);
}

// reductions over the lane pair (l, l ^ 32): v_permlane32_swap leaves the low
// halves of both operands in one register and the high halves in the other.
ACCT_DEV float pair_max(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
ACCT_DEV float pair_sum(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

ACCT_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11): ten rounds of
// two 32x32->64 multiplies; the key is bumped by the Weyl constants after every round.
ACCT_DEV void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t (&out)[4]) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// ---- kernel arguments --------------------------------------------------------
struct FaArgs {
  const void* q; const void* k; const void* v;
  void* o; float* lse;                 // fwd outputs / bwd inputs
  const void* dout; void* dq; void* dk; void* dv;                // bwd only
  float* delta; float* nlse;           // bwd workspace: D = rowsum(dO*O) and -LSE*log2(e), [B,N,Sq] each
  float* dkdv_part;                    // q_split > 1: per-slice dK / dV sums of the dK/dV kernel, [q_split][workgroup][wave][regs x 64 lanes]
  const uint8_t* mask; const uint8_t* drop; const void* alibi;   // mask / drop: elements of mask_es / drop_es bytes
  const uint8_t* blkflags;             // [MB, Tr, Tc] block classes of a dense mask
  const uint8_t* blktail;              // [MB, Tr, Tc] or null: t > 0 for a mixed block whose every row masks exactly the keys from
                                       // the block's t-th on (key padding: no mask loads there, an index compare); else 0
  const uint32_t* droprow;             // [B*N*Sq, droprow_w] keep bits of the dropout mask by query row: bit k of word w = drop[row][32w+k] != 0
  const uint32_t* dropcol;             // [B*N, Tr, Sk, 4] the same by key column: bit r of the 128-bit entry = drop[128*qb + r][key] != 0
  const uint32_t* colbits;             // [MB, Tr, Sk, 4] dense mask of the 'apply' blocks packed by key column: bit r of the
                                       // 128-bit entry = mask[128*qb + r][key] (dK/dV kernel); may be null
  int B, N, Sq, Sk;
  int hd;                              // head dim (<= the kernel's template head dim, a multiple of 8): columns past it do not exist
  int Tr, Tc;                          // number of 128-row / 128-column blocks
  int64_t q_sb, q_sh, q_ss;
  int64_t k_sb, k_sh, k_ss;
  int64_t v_sb, v_sh, v_ss;
  int64_t o_sb, o_sh, o_ss;
  int64_t mask_sb;
  int64_t al_sb, al_sh, al_sq;
  float scale, scale_log2e, inv_keep, inv_scale;
  float mask_add_raw;                  // -10000 / scale: the mask in raw q.k units
  // The backward recomputes P = exp(S - LSE), normalised: with many keys its entries, and dS = P (dP - D), fall
  // into the subnormal range of fp16 before they feed the MFMAs.  The kernels therefore work with 2^p_shift P
  // (a shift of the exp2 argument: no instruction) and multiply dQ, dK, dV by p_unshift = 2^-p_shift at the end.
  float p_shift, p_unshift;
  int prev_blk, next_blk;
  int mask_kind;
  int mask_es, drop_es;                // bytes per element of mask and drop: 1 (uint8) or 2 (the I/O dtype); nonzero = masked / kept
  int row_prefix;                      // >0: row i sees keys j < (i/row_prefix + 1)*row_prefix only (multiple of 128)
  int n_tiles;                         // tiles along the owner dimension
  int q_split;                         // dK/dV kernel: slices of the query range, each on workgroups of its own (1 = no split)
  int droprow_w;                       // 32-bit words per row of droprow: 2 * ceil(Sk / 64)
  uint32_t philox_k0, philox_k1;       // counter-based dropout: key, call offset and keep threshold (byte < thr keeps)
  uint32_t philox_offset, philox_thr;
};

enum : int { kMaskNone = 0, kMaskDense = 1, kMaskTile = 3, kMaskCausal = 4 };
enum : uint8_t { kBlkClean = 0, kBlkApply = 1, kBlkSkip = 2, kBlkTriu = 3 };

// Shrinks the tile range [lo, hi] from both ends while dead(tile) holds.  The 64 lanes of the wave test 64
// tiles at a time (one round trip to memory per 64 tiles instead of one per tile); every wave of the
// workgroup arrives at the same range.
template <typename F>
ACCT_DEV void trim_dead_tiles(int& lo, int& hi, int lane, F dead) {
  while (lo <= hi) {
    const int j = lo + lane;
    const uint64_t live = __ballot(j > hi || !dead(j));
    if (live) { lo += __builtin_ctzll(live); break; }
    lo += 64;
  }
  while (lo <= hi) {
    const int j = hi - lane;
    const uint64_t live = __ballot(j < lo || !dead(j));
    if (live) { hi -= __builtin_ctzll(live); break; }
    hi -= 64;
  }
}

// Classes of 64 consecutive blocks of one row or column of the block-class table, as two 64-bit lane
// masks in scalar registers: one byte load per lane and two ballots fill the window, and a step of the
// tile loop then looks its block up with scalar shifts.  (A byte load per step would stall the step for
// a round trip to memory, since the class decides a wave-uniform branch.)  Blocks are asked for in
// ascending order (init) or in descending order (init_descending); the window moves on when the block asked
// for lies outside it.
struct BlkClassWindow {
  const uint8_t* p;
  const uint8_t* pt = nullptr;        // the same line of the key-tail table (FaArgs::blktail), or null
  int64_t stride;
  int first, last, base;
  uint64_t b0, b1;
  int tail_blk = -1;                  // the first block of the window with a key tail, and that tail (scalar registers; further
  uint32_t tail_t = 0;                // such blocks of the window are read as mixed blocks: same results)
  ACCT_DEV void init(const uint8_t* p_, int64_t stride_, int first_, int last_, int lane, const uint8_t* tails_line = nullptr) {
    p = p_; pt = tails_line; stride = stride_; first = first_; last = last_;
    load(first, lane);
  }
  ACCT_DEV void init_descending(const uint8_t* p_, int64_t stride_, int first_, int last_, int lane, const uint8_t* tails_line = nullptr) {
    p = p_; pt = tails_line; stride = stride_; first = first_; last = last_;
    load(max(first_, last_ - 63), lane);
  }
  // The window of the blocks [lo, hi] of line `own` and, in the same round trip to memory, the part of [lo, hi]
  // that is not 'skip' in every one of the `n` lines line0 .. line0 + n - 1 (the row or column blocks a
  // workgroup covers; line l, block x sits at tbl[l * line_step + x * stride]): lo and hi shrink to it (lo > hi
  // when nothing is left).  For at most 64 blocks; returns false, with nothing done, when there are more.
  // `tails`: the key-tail table, indexed like tbl, or null.
  ACCT_DEV bool init_trimmed(const uint8_t* tbl, int64_t stride_, int64_t line_step, int line0, int n, int own, int& lo, int& hi, int lane,
                             const uint8_t* tails = nullptr) {
    if (hi - lo >= 64 || n > 2) return false;
    p = tbl + (int64_t)own * line_step; stride = stride_; first = lo; last = hi; base = lo;
    pt = tails ? tails + (int64_t)own * line_step : nullptr;
    const int blk = lo + lane;
    const bool in = blk <= hi;
    // (all loads are issued before the first ballot waits for one)
    const uint32_t f0 = in ? tbl[(int64_t)line0 * line_step + blk * stride_] : (uint32_t)kBlkSkip;
    const uint32_t f1 = (in && n > 1) ? tbl[(int64_t)(line0 + 1) * line_step + blk * stride_] : (uint32_t)kBlkSkip;
    const uint32_t fo = own == line0 ? f0 : (own == line0 + 1 && n > 1 ? f1 : (in ? p[blk * stride_] : 0u));
    note_tail((pt && in) ? pt[blk * stride_] : 0u);
    const uint64_t live = __ballot(in && !(f0 == kBlkSkip && f1 == kBlkSkip));
    b0 = __ballot(in && (fo & 1u));
    b1 = __ballot(in && (fo & 2u));
    if (live) {
      hi = lo + 63 - __builtin_clzll(live);
      lo += __builtin_ctzll(live);
    } else {
      hi = lo - 1;
    }
    return true;
  }
  ACCT_DEV void load(int first, int lane) {
    base = first;
    const int blk = first + lane;
    const uint32_t f = (p && blk <= last) ? p[blk * stride] : 0u;
    note_tail((pt && blk <= last) ? pt[blk * stride] : 0u);
    b0 = __ballot(f & 1u);
    b1 = __ballot(f & 2u);
  }
  ACCT_DEV uint32_t get(int blk, int lane) {
    if (blk - base >= 64) load(blk, lane);
    else if (blk < base) load(max(first, blk - 63), lane);
    const int sh = blk - base;
    return (uint32_t)((b0 >> sh) & 1u) | ((uint32_t)((b1 >> sh) & 1u) << 1);
  }
  // tl: lane l holds the key tail of block base + l
  ACCT_DEV void note_tail(uint32_t tl) {
    const uint64_t any = __ballot(tl != 0);
    tail_blk = -1; tail_t = 0;
    if (any) {
      const int l = __builtin_ctzll(any);
      tail_blk = base + l;
      tail_t = (uint32_t)__builtin_amdgcn_readlane((int)tl, l);
    }
  }
  // key tail of a block inside the window (0: none, or not the window's first)
  ACCT_DEV uint32_t tail(int blk) const { return blk == tail_blk ? tail_t : 0u; }
};

// The same window with the key tail of EVERY block of the window, in one vector register.  A window along the key
// axis of a padded batch (forward, dQ) holds one key-tail block, which the two scalar registers above cover; a
// window along the query axis (the dK/dV kernel's) holds one per query block.
struct BlkClassWindowLaneTails {
  const uint8_t* p;
  const uint8_t* pt = nullptr;        // the same line of the key-tail table (FaArgs::blktail), or null
  int64_t stride;
  int first, last, base;
  uint64_t b0, b1;
  uint32_t tail_l = 0;                // lane l: key tail of block base + l
  ACCT_DEV void init(const uint8_t* p_, int64_t stride_, int first_, int last_, int lane, const uint8_t* tails_line = nullptr) {
    p = p_; pt = tails_line; stride = stride_; first = first_; last = last_;
    load(first, lane);
  }
  ACCT_DEV void init_descending(const uint8_t* p_, int64_t stride_, int first_, int last_, int lane, const uint8_t* tails_line = nullptr) {
    p = p_; pt = tails_line; stride = stride_; first = first_; last = last_;
    load(max(first_, last_ - 63), lane);
  }
  // The window of the blocks [lo, hi] of line `own` and, in the same round trip to memory, the part of [lo, hi]
  // that is not 'skip' in every one of the `n` lines line0 .. line0 + n - 1 (the row or column blocks a
  // workgroup covers; line l, block x sits at tbl[l * line_step + x * stride]): lo and hi shrink to it (lo > hi
  // when nothing is left).  For at most 64 blocks; returns false, with nothing done, when there are more.
  // `tails`: the key-tail table, indexed like tbl, or null.
  ACCT_DEV bool init_trimmed(const uint8_t* tbl, int64_t stride_, int64_t line_step, int line0, int n, int own, int& lo, int& hi, int lane,
                             const uint8_t* tails = nullptr) {
    if (hi - lo >= 64 || n > 2) return false;
    p = tbl + (int64_t)own * line_step; stride = stride_; first = lo; last = hi; base = lo;
    pt = tails ? tails + (int64_t)own * line_step : nullptr;
    const int blk = lo + lane;
    const bool in = blk <= hi;
    // (all loads are issued before the first ballot waits for one)
    const uint32_t f0 = in ? tbl[(int64_t)line0 * line_step + blk * stride_] : (uint32_t)kBlkSkip;
    const uint32_t f1 = (in && n > 1) ? tbl[(int64_t)(line0 + 1) * line_step + blk * stride_] : (uint32_t)kBlkSkip;
    const uint32_t fo = own == line0 ? f0 : (own == line0 + 1 && n > 1 ? f1 : (in ? p[blk * stride_] : 0u));
    note_tail((pt && in) ? pt[blk * stride_] : 0u);
    const uint64_t live = __ballot(in && !(f0 == kBlkSkip && f1 == kBlkSkip));
    b0 = __ballot(in && (fo & 1u));
    b1 = __ballot(in && (fo & 2u));
    if (live) {
      hi = lo + 63 - __builtin_clzll(live);
      lo += __builtin_ctzll(live);
    } else {
      hi = lo - 1;
    }
    return true;
  }
  ACCT_DEV void load(int first, int lane) {
    base = first;
    const int blk = first + lane;
    const uint32_t f = (p && blk <= last) ? p[blk * stride] : 0u;
    note_tail((pt && blk <= last) ? pt[blk * stride] : 0u);
    b0 = __ballot(f & 1u);
    b1 = __ballot(f & 2u);
  }
  ACCT_DEV uint32_t get(int blk, int lane) {
    if (blk - base >= 64) load(blk, lane);
    else if (blk < base) load(max(first, blk - 63), lane);
    const int sh = blk - base;
    return (uint32_t)((b0 >> sh) & 1u) | ((uint32_t)((b1 >> sh) & 1u) << 1);
  }
  ACCT_DEV void note_tail(uint32_t tl) { tail_l = tl; }
  ACCT_DEV uint32_t tail(int blk) const { return (uint32_t)__builtin_amdgcn_readlane((int)tail_l, blk - base); }
};

// True when the block classes of a dense mask say that, inside the band, the `n` (<= 2) lines line0 .. of the class
// table that a workgroup covers hold exactly the causal pattern: clean before the diagonal, the causal diagonal
// class on it, skipped after it.  Such a workgroup gives the same results by index compare alone, with the code
// that knows no mask tensor.  `lines_are_keys`: the lines are key blocks and the walk [lo, hi] runs over query
// blocks (the dK/dV kernel); else the lines are query blocks and the walk runs over key blocks.  Element
// (line l, block x) sits at tbl[l * line_step + x * stride].  At most 64 blocks are looked at (one load per
// lane and line); more give false.  Every wave of the workgroup arrives at the same answer.
ACCT_DEV bool dense_lines_are_causal(const uint8_t* tbl, int64_t stride, int64_t line_step, int line0, int n, int lo, int hi,
                                     bool lines_are_keys, const FaArgs& a, int lane) {
  if (hi - lo >= 64 || n > 2 || lo > hi) return false;
  const int blk = lo + lane;
  bool ok = true;
  uint32_t f[2];
#pragma unroll
  for (int l = 0; l < 2; l++) f[l] = (l < n && blk <= hi) ? tbl[(int64_t)(line0 + l) * line_step + blk * stride] : 0u;
#pragma unroll
  for (int l = 0; l < 2; l++)
    if (l < n && blk <= hi) {
      const int qb = lines_are_keys ? blk : line0 + l, kb = lines_are_keys ? line0 + l : blk;
      bool in_band = (kb - a.next_blk <= qb) && (qb <= kb + a.prev_blk);
      if (a.row_prefix) in_band = in_band && kb <= ((qb * 128 / a.row_prefix + 1) * a.row_prefix - 1) / 128;
      const uint32_t want = kb < qb ? (uint32_t)kBlkClean : (kb == qb ? (uint32_t)kBlkTriu : (uint32_t)kBlkSkip);
      ok = ok && (!in_band || f[l] == want);
    }
  return __all(ok);
}

// four consecutive mask / dropout bytes starting at column kv of a row
ACCT_DEV uint32_t load_u8x4(const uint8_t* row, int kv, int limit, bool vec_ok) {
  if (vec_ok && kv + 4 <= limit) return *reinterpret_cast<const uint32_t*>(row + kv);
  uint32_t r = 0;
#pragma unroll
  for (int e = 0; e < 4; e++)
    if (kv + e < limit) r |= (uint32_t)row[kv + e] << (8 * e);
  return r;
}

// mask / dropout element -> "is nonzero": a 2-byte element is a floating-point number, whose zero may carry a sign
template <int ES> ACCT_DEV bool elem_nonzero(const uint8_t* p, int64_t idx) {
  if (ES == 1) return p[idx] != 0;
  return (reinterpret_cast<const uint16_t*>(p)[idx] & 0x7fffu) != 0;
}
// the same four consecutive elements for a mask of `es`-byte elements, as four "nonzero" bytes (row = first byte of the row)
ACCT_DEV uint32_t load_mask4(const uint8_t* row, int kv, int limit, bool vec_ok, int es) {
  if (es == 1) return load_u8x4(row, kv, limit, vec_ok);
  const uint16_t* r16 = reinterpret_cast<const uint16_t*>(row);
  uint32_t r = 0;
  if (vec_ok && kv + 4 <= limit) {
    const u32x2 t = *reinterpret_cast<const u32x2*>(r16 + kv);
#pragma unroll
    for (int e = 0; e < 4; e++)
      if ((t[e >> 1] >> (16 * (e & 1))) & 0x7fffu) r |= 1u << (8 * e);
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (kv + e < limit && (r16[kv + e] & 0x7fffu)) r |= 1u << (8 * e);
  }
  return r;
}

template <typename T>
ACCT_DEV void load_bias4(const T* row, int kv, int limit, bool vec_ok, float out[4]) {
  if (vec_ok && kv + 4 <= limit) {
    typename Elem<T>::V4 t = *reinterpret_cast<const typename Elem<T>::V4*>(row + kv);
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = (float)t[e];
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = (kv + e < limit) ? (float)row[kv + e] : 0.f;
  }
}

// ---- swizzled LDS tiles filled by direct-to-LDS loads --------------------------
// (the swizzle itself: SwzCfg in fa_index_math.hpp)
#define ACCT_GLB __attribute__((address_space(1)))

// Stage rows [row0, row0 + ROWS) of a row-major global matrix into a swizzled LDS
// tile with NW waves.  Rows past nrows repeat the last valid row (finite data whose
// contribution is zeroed by the caller's masking), slots past the `cpr` valid 16-byte
// chunks of a row (head dim / 8) repeat the last valid chunk.
// `wv` < 0: the NW waves are the workgroup's first NW; else the calling wave's index among the NW.
template <typename T, int D, int ROWS, int NW>
ACCT_DEV void tile_dma(const T* base, int64_t row_stride, int row0, int nrows, ACCT_LDS char* buf, int cpr, int wv = -1) {
  using C = SwzCfg<D>;
  constexpr int NI = ROWS / C::RPI;
  static_assert(NI % NW == 0, "tile rows must split evenly over the waves");
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));                   // addresses are re-derived per call instead of living in registers
  const int lane = tid & 63, wave = wv < 0 ? tid >> 6 : wv;
#pragma unroll
  for (int i = 0; i < NI / NW; i++) {
    const int inst = wave * (NI / NW) + i;
    const int r = inst * C::RPI + lane / C::CH;
    const int lc = min((lane % C::CH) ^ C::swz(r), cpr - 1);
    const int grow = min(row0 + r, nrows - 1);
    const T* src = base + (int64_t)grow * row_stride + lc * 8;
    // Issued as inline assembly on purpose: the compiler then does not order every later LDS read
    // behind these loads (it cannot tell the two tile buffers apart), which would serialise the
    // prefetch of the next tile with the work on the current one.  dma_wait() + the workgroup
    // barrier publish the tile.
    const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(buf + inst * 1024));
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(dst) : "memory");
  }
}

// The same staging with everything tile-invariant hoisted: per-lane 32-bit byte offsets are
// computed once (plan), a tile then costs a 64-bit scalar base, and per wave instruction one m0
// write and one global_load_lds with scalar base + vector offset -- no vector ALU work in the loop.
// Only tiles that lie entirely inside the matrix may use it (no row clamping).
template <typename T, int D, int ROWS, int NW>
struct TileDma {
  using C = SwzCfg<D>;
  static constexpr int NI = ROWS / C::RPI;
  static constexpr int NIW = NI / NW;              // instructions per wave and tile
  // The swizzle repeats every 16 rows, i.e. every PER instructions: instruction i of a wave differs from
  // instruction i % PER by a whole number of 16-row groups, which goes into the scalar base address.
  static constexpr int PER = 16 / C::RPI;
  static constexpr int NV = NIW < PER ? NIW : PER;
  static_assert(NIW <= PER || NIW % PER == 0, "a wave's share of a tile must be whole 16-row groups");
  uint32_t voff[NV];
  uint32_t lds0;                                   // LDS byte offset of this wave's first 1 KB slab within a tile
  // `wv` < 0: the NW waves are the workgroup's first NW; else the calling wave's index among the NW
  ACCT_DEV void plan(int64_t row_stride, int cpr, int wv = -1) {
    static_assert(NI % NW == 0, "tile rows must split evenly over the waves");
    const int lane = threadIdx.x & 63, wave = wv < 0 ? (int)(threadIdx.x >> 6) : wv;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int inst = wave * NIW + i;
      const int r = inst * C::RPI + lane / C::CH;
      const int lc = min((lane % C::CH) ^ C::swz(r), cpr - 1);
      voff[i] = (uint32_t)((r * row_stride + lc * 8) * (int64_t)sizeof(T));
    }
    lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(wave * NIW * 1024));
  }
  // plan-free variant for kernels without registers to spare: the 32-bit offsets are re-derived
  // (a few 32-bit vector ops per instruction); rows [row0, row0 + ROWS) must exist
  static ACCT_DEV void issue_direct(const T* base, int64_t row_stride, int row0, ACCT_LDS char* buf, int cpr) {
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = tid >> 6;
    const T* tile = base + (int64_t)row0 * row_stride;
    {
      const uint64_t t = (uint64_t)(uintptr_t)tile;               // uniform: pinned in scalar registers
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)t);
      const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(t >> 32));
      tile = (const T*)(uintptr_t)(((uint64_t)hi << 32) | lo);
    }
    const uint32_t dst0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)buf + (uint32_t)(wave * NIW * 1024));
    const uint32_t rs = (uint32_t)row_stride * (uint32_t)sizeof(T);
#pragma unroll
    for (int i = 0; i < NIW; i++) {
      const int r = (wave * NIW + i) * C::RPI + lane / C::CH;
      const int lc = min((lane % C::CH) ^ C::swz(r), cpr - 1);
      const uint32_t voff = (uint32_t)r * rs + (uint32_t)lc * 16u;
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(tile), "s"(dst0 + i * 1024)
                   : "memory");
    }
  }
  // rows [row0, row0 + ROWS) must exist
  ACCT_DEV void issue(const T* base, int64_t row_stride, int row0, ACCT_LDS char* buf) const {
    const uint32_t dst0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)buf) + lds0;
#pragma unroll
    for (int grp = 0; grp < (NIW + PER - 1) / PER; grp++) {
      const T* tile = base + (int64_t)(row0 + 16 * grp) * row_stride;   // uniform: must live in scalar registers
      {
        const uint64_t t = (uint64_t)(uintptr_t)tile;               // (pinned there: under register pressure the
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)t);          // compiler may hold it in VGPRs)
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(t >> 32));
        tile = (const T*)(uintptr_t)(((uint64_t)hi << 32) | lo);
      }
#pragma unroll
      for (int i = 0; i < NV; i++)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff[i]), "s"(tile), "s"(dst0 + (grp * PER + i) * 1024)
                     : "memory");
    }
  }
};

// Wave-private staging of an additive-bias tile (32 query rows x 64 keys, 128 bytes per row) through LDS:
// the lanes of the attention kernels own query rows, so direct loads would touch 32 different cache lines
// per instruction; four 16-byte DMA instructions fetch whole rows instead.  The 16-byte chunk c of row r is
// stored in slot c ^ (r & 7), which spreads the 8-byte reads of 8 consecutive rows over all banks.
// Requires Sk % 8 == 0 and 16-byte aligned rows; rows past nrows repeat the last row, chunks past Sk repeat
// the last chunk (their scores are masked anyway).
// SWZ = false stores the rows plainly (for readers that walk down a column).
template <typename T, bool SWZ = true>
ACCT_DEV void bias_tile_dma(const T* base, int64_t row_stride, int row0, int nrows, int kv0, int Sk, ACCT_LDS char* dst) {
  int ln = threadIdx.x & 63;
  asm volatile("" : "+v"(ln));
  const int lcm = (Sk - kv0) / 8 - 1;              // last chunk of this tile that lies inside the row
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = 8 * i + (ln >> 3);
    const int lc = min(SWZ ? (ln & 7) ^ (r & 7) : (ln & 7), lcm);
    const T* src = base + (int64_t)min(row0 + r, nrows - 1) * row_stride + kv0 + 8 * lc;
    const uint32_t d = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(dst + i * 1024));
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(d) : "memory");
  }
}
// the 4 bias values of row `row` (0..31) for keys 8*cc + 4*half .. +3 of the staged tile
template <typename T>
ACCT_DEV typename Elem<T>::V4 bias_tile_read(const ACCT_LDS char* tile, int row, int cc, int half) {
  return *reinterpret_cast<const ACCT_LDS typename Elem<T>::V4*>(tile + row * 128 + ((cc ^ (row & 7)) << 4) + 8 * half);
}

// x = (k > v) ? y : x for a constant k, as one compare into VCC and one select.  Written in C++, a run of these
// is compiled into a batch of compares whose results sit in scalar register pairs; dozens of them push the
// kernel's other scalars into spill lanes.
ACCT_DEV float select_if_gt(float x, int k, int v, float y) {
  asm("v_cmp_gt_i32_e32 vcc, %2, %1\n\tv_cndmask_b32_e32 %0, %0, %3, vcc" : "+v"(x) : "v"(v), "i"(k), "v"(y) : "vcc");
  return x;
}
// all of this wave's direct-to-LDS loads have landed
ACCT_DEV void dma_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// one dword per lane from global memory to LDS at dst + 4 * lane (dst wave-uniform)
ACCT_DEV void dma4(const void* src, ACCT_LDS char* dst) {
  const uint32_t d = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(src), "s"(d) : "memory");
}

// A bias that depends on the key only (row stride 0, the reference's ALiBi form): the values of the keys
// kv0 .. kv0 + 127, one dword (two keys) per lane, land as row 0 of the region bias_tile_read reads (the
// chunks of row 0 are not swizzled), so a reader passes row 0 instead of its own.  Same requirements as
// bias_tile_dma; keys past Sk repeat the last pair.
template <typename T>
ACCT_DEV void bias_row_dma(const T* base, int kv0, int Sk, ACCT_LDS char* dst) {
  int ln = threadIdx.x & 63;
  asm volatile("" : "+v"(ln));
  dma4(base + min(kv0 + 2 * ln, Sk - 2), dst);
}

// Keep-bit words (dropout, packed by query row) of the 32*QG rows of a wave and the KT 32-key chunks of one
// K/V tile, brought into a wave-private LDS buffer [row][KT] by DMA together with the tile.  Read from LDS
// in the tile loop, they need no wait on the vector-memory counter, which would also wait for the K/V
// tile in flight.
template <bool DROP, int QG, int KT>
struct DropRowStage {
  static constexpr int BYTES = DROP ? QG * 32 * KT * 4 : 0;
  static ACCT_DEV void issue(const FaArgs& a, int bh, int wq0, int j, int lane, ACCT_LDS char* buf) {
    if constexpr (DROP) {
#pragma unroll
      for (int k = 0; k < QG * KT / 2; k++) {
        const int idx = lane + 64 * k;
        const int row = min(wq0 + idx / KT, a.Sq - 1), w = min(KT * j + idx % KT, a.droprow_w - 1);
        dma4(a.droprow + ((int64_t)bh * a.Sq + row) * a.droprow_w + w, buf + k * 256);
      }
    }
  }
  static ACCT_DEV uint32_t word(const ACCT_LDS char* buf, int row, int c) {
    return reinterpret_cast<const ACCT_LDS uint32_t*>(buf)[row * KT + c];
  }
};


}  // namespace acct
