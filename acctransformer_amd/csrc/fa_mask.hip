// Block classification of a dense attention mask (uint8, or the I/O dtype as the reference passes it;
// nonzero = masked either way).
//
// The reference adds -10000 to masked scores (attention.py:357-371 of the
// reference's flash_attention ops) instead of removing them.  A 128x128 block
// whose entries are all masked therefore contributes exp(-10000 + ...) = 0 in
// fp32 to every row that has at least one unmasked visible key elsewhere, and
// can be skipped without changing a bit of the result; a block with no masked
// entry needs no mask loads.  This pre-pass finds both kinds so the attention
// kernels touch the mask only on mixed blocks.  A diagonal block (same 128 rows and keys) whose entries
// are exactly "masked iff the key comes after the query" - every diagonal block of a causal mask given
// as a tensor, with or without padding elsewhere - gets a class of its own: the kernels then compare
// indices there, as they do for the causal mask kind, instead of loading mask bytes.
#include "fa_common.hpp"
#include "fa_launch.hpp"

namespace acct {

constexpr uint8_t kBlkAllMasked = 255;  // provisional: resolved to skip or apply below

// Fast path (Sk and the mask pointers 16-byte aligned): ONE launch that leaves the block classes and, for the
// dK/dV kernel, the column bitmaps of the mixed blocks (every launch costs a few microseconds of a step that
// takes a few hundred).  One workgroup of 256 threads per (mask batch, q block, key block) inside the band, so
// that the work spreads over the chip whatever the shape (a [1, 2048, 2048] mask has 16 row blocks but 256
// blocks).  Thread t owns 64 consecutive elements of row t % 128 (half t / 128 of the block's 128 columns),
// four or eight 16-byte loads, as a 64-bit "nonzero" mask.
//
// A wholly masked block may be skipped only if every row of its q block sees an unmasked key somewhere (see the
// top of the file).  A workgroup cannot see the other blocks of its row block's band, so it checks a sufficient
// condition on two of them that it reads itself: every row has an unmasked key in the first block of the band
// or in the diagonal block.  That holds for causal, banded, prefix and document masks (the diagonal entry is
// visible) and for key padding (the first keys are); where it fails although the rows do see keys elsewhere,
// the block is classed 'apply' instead of 'skip', which gives the same results bit for bit, only slower.
template <int ES>
__global__ void __launch_bounds__(256) fa_mask_prepass_kernel(const FaArgs a, uint8_t* flags, uint8_t* tails, uint32_t* colbits) {
  __shared__ unsigned long long s_bits[128][2];         // nonzero bits of the block: [row][column half]
  __shared__ unsigned long long s_seen[2];              // rows (bit = row % 64) with an unmasked key in the blocks probed
  __shared__ int s_lead[2];                             // unmasked leading columns of the block's first row, per column half
  const int kvb = blockIdx.x % a.Tc, qb = (blockIdx.x / a.Tc) % a.Tr, mb = blockIdx.x / (a.Tc * a.Tr);
  const int tid = threadIdx.x;
  int lo = max(0, qb - a.prev_blk), hi = min(a.Tc - 1, qb + a.next_blk);
  if (a.row_prefix) hi = min(hi, ((qb * 128 / a.row_prefix + 1) * a.row_prefix - 1) / 128);
  const int64_t blk = ((int64_t)mb * a.Tr + qb) * a.Tc + kvb;
  if (kvb < lo || kvb > hi) {                           // outside the band: never visited
    if (tid == 0) { flags[blk] = kBlkClean; tails[blk] = 0; }
    return;
  }
  const int rib = tid & 127, half = tid >> 7, row = qb * 128 + rib, c0 = half * 64;
  const uint8_t* mrow = a.mask + ((int64_t)mb * a.mask_sb + (int64_t)min(row, a.Sq - 1) * a.Sk) * ES;
  // this thread's 64 elements of key block kb: nz = nonzero bits, valid = bits of the elements that exist
  auto scan = [&](int kb, unsigned long long& nz, unsigned long long& valid) {
    nz = 0; valid = 0;
    if (row >= a.Sq) return;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int kv = kb * 128 + c0 + 16 * i;
      if (kv < a.Sk) {                                  // Sk % 16 == 0: a piece is entirely inside or outside
        uint32_t bits = 0;                              // bit e: element e of these 16 is nonzero
#pragma unroll
        for (int h = 0; h < ES; h++) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(mrow + (int64_t)kv * ES + 16 * h);
#pragma unroll
          for (int w = 0; w < 4; w++) {
            if (ES == 1) {
#pragma unroll
              for (int e = 0; e < 4; e++) bits |= (((v[w] >> (8 * e)) & 0xffu) != 0 ? 1u : 0u) << (4 * w + e);
            } else {
              // 2-byte floating-point elements: the sign of a zero does not count
              bits |= (((v[w] & 0x7fffu) != 0 ? 1u : 0u) | (((v[w] >> 16) & 0x7fffu) != 0 ? 2u : 0u)) << (8 * h + 2 * w);
            }
          }
        }
        nz |= (unsigned long long)bits << (16 * i);
        valid |= 0xffffull << (16 * i);
      }
    }
  };
  unsigned long long nz, valid;
  scan(kvb, nz, valid);
  // the causal pattern on the diagonal block: column c0 + e is masked iff it comes after row rib
  const int d = rib - c0;                               // columns above bit d are "after the row"
  const unsigned long long tri = d < 0 ? ~0ull : (d >= 63 ? 0ull : (~0ull << (d + 1)));
  const bool on_diag = kvb == qb;
  const int any_m = __syncthreads_or(nz != 0), any_u = __syncthreads_or((~nz & valid) != 0);
  const int bad = __syncthreads_or(on_diag && ((nz ^ tri) & valid) != 0);
  uint8_t cls = !any_m ? kBlkClean : (any_u ? ((on_diag && !bad) ? kBlkTriu : kBlkApply) : kBlkSkip);
  if (cls == kBlkSkip) {                                // (uniform: the whole workgroup takes the branch)
    if (tid < 2) s_seen[tid] = 0;
    __syncthreads();
    const int probe[2] = {lo, (qb >= lo && qb <= hi && qb != lo) ? qb : -1};
#pragma unroll
    for (int k = 0; k < 2; k++)
      if (probe[k] >= 0 && probe[k] != kvb) {
        unsigned long long pnz, pvalid;
        scan(probe[k], pnz, pvalid);
        const unsigned long long seen = __ballot((~pnz & pvalid) != 0);
        if ((tid & 63) == 0 && seen) atomicOr(&s_seen[(tid >> 6) & 1], seen);
      }
    __syncthreads();
    const int nrow = min(128, a.Sq - qb * 128);         // rows past Sq do not count
    bool ok = true;
#pragma unroll
    for (int w = 0; w < 2; w++) {
      const int n = min(64, max(0, nrow - 64 * w));
      const unsigned long long need = n >= 64 ? ~0ull : ((1ull << n) - 1ull);
      ok = ok && (s_seen[w] & need) == need;
    }
    if (!ok) cls = kBlkApply;
  }
  // A mixed block in which every row masks exactly the columns from the t-th on (1 <= t <= 127; key padding that
  // ends inside the block): the forward and dQ kernels compare key indices with t there instead of loading mask
  // bytes.  t is taken from the block's first row (which always exists) and checked against every row.
  int tail = 0;
  if (cls == kBlkApply) {                               // (uniform)
    if (rib == 0) s_lead[half] = nz ? __builtin_ctzll(nz) : 64;
    __syncthreads();
    const int t = s_lead[0] < 64 ? s_lead[0] : 64 + s_lead[1];
    const int rel = t - c0;                             // this thread's columns from bit `rel` on are masked
    const unsigned long long want = rel <= 0 ? ~0ull : (rel >= 64 ? 0ull : (~0ull << rel));
    const int differs = __syncthreads_or(row < a.Sq && ((nz ^ want) & valid) != 0);
    if (!differs && t >= 1 && t <= 127) tail = t;
  }
  if (tid == 0) { flags[blk] = cls; tails[blk] = (uint8_t)tail; }
  if (cls == kBlkApply && colbits) {
    // the block packed by key column: 128 bits per key, bit r = mask[128 qb + r][key]
    s_bits[rib][half] = nz;
    __syncthreads();
    const int col = tid & 127, kv = kvb * 128 + col;
    if (kv < a.Sk) {
      const ACCT_LDS uint32_t* sb = (const ACCT_LDS uint32_t*)&s_bits[0][0] + (col >> 5);   // the 32-bit piece that holds the column
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int i = 2 * half + j;
        uint32_t w = 0;
#pragma unroll 8
        for (int r = 0; r < 32; r++) w |= ((sb[(32 * i + r) * 4] >> (col & 31)) & 1u) << r;
        colbits[(((int64_t)mb * a.Tr + qb) * a.Sk + kv) * 4 + i] = w;
      }
    }
  }
}

// Generic path (any alignment): one workgroup per (mask batch, q block); thread t scans 64 columns of row t/2
template <int ES>
__global__ void __launch_bounds__(256) fa_mask_blocks_kernel(const FaArgs a, uint8_t* flags) {
  const int qb = blockIdx.x % a.Tr, mb = blockIdx.x / a.Tr;
  const int tid = threadIdx.x, row = qb * 128 + (tid >> 1), c0 = (tid & 1) * 64;
  const uint8_t* mrow = a.mask + ((int64_t)mb * a.mask_sb + (int64_t)min(row, a.Sq - 1) * a.Sk) * ES;
  const bool vec_ok = ((((uintptr_t)a.mask / ES) | (uintptr_t)a.Sk | (uintptr_t)a.mask_sb) & 3) == 0;
  uint8_t* frow = flags + ((int64_t)mb * a.Tr + qb) * a.Tc;
  int lo = max(0, qb - a.prev_blk), hi = min(a.Tc - 1, qb + a.next_blk);
  if (a.row_prefix) hi = min(hi, ((qb * 128 / a.row_prefix + 1) * a.row_prefix - 1) / 128);
  for (int kvb = tid; kvb < a.Tc; kvb += 256)
    if (kvb < lo || kvb > hi) frow[kvb] = kBlkClean;
  bool row_unmasked = false;
  bool tri_bad = false;
  for (int kvb = lo; kvb <= hi; kvb++) {
    bool any_m = false, any_u = false;
    if (row < a.Sq) {
#pragma unroll 4
      for (int c = 0; c < 64; c += 4) {
        const int kv = kvb * 128 + c0 + c;
        if (kv >= a.Sk) break;
        const int n = min(4, a.Sk - kv);
        const uint32_t bits = load_mask4(mrow, kv, a.Sk, vec_ok, ES);
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (e < n) {
            const bool masked = ((bits >> (8 * e)) & 0xffu) != 0;
            if (masked) any_m = true; else any_u = true;
            if (kvb == qb) tri_bad |= masked != (c0 + c + e > (tid >> 1));
          }
      }
    }
    row_unmasked |= any_u;
    const int blk_m = __syncthreads_or(any_m), blk_u = __syncthreads_or(any_u);
    if (tid == 0) frow[kvb] = !blk_m ? kBlkClean : (!blk_u ? kBlkAllMasked : kBlkApply);
  }
  row_unmasked |= (bool)__shfl_xor((int)row_unmasked, 1);
  const int rows_ok = __syncthreads_and(row >= a.Sq || row_unmasked);
  // (the barrier above also orders thread 0's provisional writes before the reads below)
  const int not_tri = __syncthreads_or(tri_bad);
  for (int kvb = lo + tid; kvb <= hi; kvb += 256) {
    if (frow[kvb] == kBlkAllMasked) frow[kvb] = rows_ok ? kBlkSkip : kBlkApply;
    else if (kvb == qb && frow[kvb] == kBlkApply && !not_tri) frow[kvb] = kBlkTriu;
  }
}

// Column bitmaps of the mixed ('apply') blocks for the dK/dV kernel, whose lanes own key columns: the 128
// rows of a block packed into 128 bits per key column, so that the kernel reads one 32-bit word per lane
// and 32-row chunk instead of 16 single bytes.  One thread per key column and word (32 rows): the loads
// of a thread are independent, and 512 threads keep enough of them in flight.
template <int ES>
__global__ void __launch_bounds__(512) fa_mask_colbits_kernel(const FaArgs a, const uint8_t* flags, uint32_t* out) {
  const int kvb = blockIdx.x % a.Tc, qb = (blockIdx.x / a.Tc) % a.Tr, mb = blockIdx.x / (a.Tc * a.Tr);
  if (flags[((int64_t)mb * a.Tr + qb) * a.Tc + kvb] != kBlkApply) return;
  const int kv = kvb * 128 + (threadIdx.x & 127), i = threadIdx.x >> 7;
  if (kv >= a.Sk) return;
  const uint8_t* col = a.mask + ((int64_t)mb * a.mask_sb + kv) * ES;
  uint32_t w = 0u;
#pragma unroll
  for (int r = 0; r < 32; r++) {
    const int row = qb * 128 + 32 * i + r;
    if (row < a.Sq && elem_nonzero<ES>(col, (int64_t)row * a.Sk)) w |= 1u << r;
  }
  out[(((int64_t)mb * a.Tr + qb) * a.Sk + kv) * 4 + i] = w;
}

// the same for the compact 128x128 tile that is applied on diagonal blocks: out[key][4]
template <int ES>
__global__ void __launch_bounds__(128) fa_mask_tilebits_kernel(const uint8_t* tile, uint32_t* out) {
  uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll 8
    for (int r = 0; r < 32; r++)
      if (elem_nonzero<ES>(tile, (32 * i + r) * 128 + threadIdx.x)) w[i] |= 1u << r;
  u32x4 v = {w[0], w[1], w[2], w[3]};
  *reinterpret_cast<u32x4*>(out + threadIdx.x * 4) = v;
}

hipError_t launch_mask_colbits(const FaArgs& a, const uint8_t* flags, uint32_t* out, int MB, hipStream_t st) {
  if (a.mask_kind == kMaskTile) {
    if (a.mask_es == 2) hipLaunchKernelGGL(fa_mask_tilebits_kernel<2>, dim3(1), dim3(128), 0, st, a.mask, out);
    else hipLaunchKernelGGL(fa_mask_tilebits_kernel<1>, dim3(1), dim3(128), 0, st, a.mask, out);
    return hipGetLastError();
  }
  const dim3 grid((unsigned)(MB * a.Tr * a.Tc));
  if (a.mask_es == 2) hipLaunchKernelGGL(fa_mask_colbits_kernel<2>, grid, dim3(512), 0, st, a, flags, out);
  else hipLaunchKernelGGL(fa_mask_colbits_kernel<1>, grid, dim3(512), 0, st, a, flags, out);
  return hipGetLastError();
}

// Column entries of the dropout bitmaps, written whole.  The four waves of a workgroup each hold, per lane and for
// sixteen keys, the 32-bit word of their 32 rows; a key's 16-byte entry is the four waves' words.  Written straight
// from the waves every entry would be four 4-byte stores from four places; instead the words cross LDS and every
// thread stores complete entries, consecutive threads consecutive entries.  cw[e]: bit r = row r of the wave's 32;
// key_of(lane, e): the key of a lane's e-th word.  (One spare entry after every sixteen keeps the word stores of a
// wave on different banks.)  `flags`: the class row of the attention mask for these query rows, or null: entries of
// key blocks classed 'skip' are never read and are not written.
template <typename KeyOf>
ACCT_DEV void store_col_entries(uint32_t* s_cw, const uint32_t (&cw)[16], int wave, int lane, int key0, int Sk, uint32_t* out,
                                const uint8_t* flags, KeyOf key_of) {
#pragma unroll
  for (int e = 0; e < 16; e++) {
    const int k = key_of(lane, e);                       // 0 .. 1023 within the span
    s_cw[(k + (k >> 4)) * 4 + wave] = cw[e];
  }
  __syncthreads();
#pragma unroll
  for (int m = 0; m < 4; m++) {
    const int k = threadIdx.x + 256 * m;
    if (key0 + k < Sk && !(flags && flags[(key0 + k) >> 7] == kBlkSkip))
      *reinterpret_cast<u32x4*>(out + (int64_t)(key0 + k) * 4) = *reinterpret_cast<const u32x4*>(s_cw + (k + (k >> 4)) * 4);
  }
}

// Dropout mask (uint8 {0,1}, or the reference's {0, 1/keep_prob} in the I/O dtype; nonzero = keep) packed into keep bits, by query row for the kernels whose lanes own
// query rows (forward, dQ) and by key column for the dK/dV kernel.  One workgroup of four waves per (batch*head,
// 128 query rows, 1024 keys), one wave per 32 rows -- enough waves to keep the memory system busy --: per row every lane loads the 16 bytes of keys 16*lane .. +15 (a kilobyte per wave
// instruction keeps enough bytes in flight) and turns them into 16 bits; lane pairs form the 32-bit row words.
//   rowbits [B*N*Sq, 2*ceil(Sk/64)] 32-bit: bit k of word w = keep[row][32w + k];
//   colbits [B*N, Tr, Sk, 4] 32-bit: bit r of the 128-bit entry = keep[128*qb + r][key].
template <int ES>
__global__ void __launch_bounds__(256) fa_drop_bits_kernel(const FaArgs a, uint32_t* rowbits, uint32_t* colbits) {
  __shared__ __attribute__((aligned(16))) uint32_t s_cw[(1024 + 64) * 4];
  // A lane's sixteen keys of the span come from ES 16-byte loads of 16 / ES keys each; load h of the wave reads one
  // contiguous kilobyte: keys 16*lane + e for bytes, keys 512 h + 8*lane + e for 2-byte elements.
  constexpr int NH = ES, KH = 16 / ES;
  const int nspan = (a.Sk + 1023) / 1024;
  const int i = threadIdx.x >> 6;                       // which 32 rows of the 128-row block: word i of the column entries
  const int blk = blockIdx.x;
  const int span = blk % nspan, qb = (blk / nspan) % a.Tr, bh = blk / (nspan * a.Tr);
  const int lane = threadIdx.x & 63;
  const bool aligned = (((uintptr_t)a.drop | (uintptr_t)a.Sk) & 15) == 0;     // (16 elements: aligned 16-byte loads)
  // Keys in a block that the attention mask's pre-pass classed 'skip' are never visited by the attention kernels:
  // their keep bits are not read, so their mask bytes are not loaded either (this pass is bound by the bytes it
  // reads; a padded batch skips a third to a half of them).
  const uint8_t* flags = a.blkflags ? a.blkflags + ((int64_t)(a.mask_sb ? bh / a.N : 0) * a.Tr + qb) * a.Tc : nullptr;
  int kv[NH];                                           // first key of each load
  bool vec[NH], dead[NH];
  const uint8_t* p[NH];
#pragma unroll
  for (int h = 0; h < NH; h++) {
    kv[h] = span * 1024 + (ES == 1 ? 16 * lane : 512 * h + 8 * lane);
    vec[h] = aligned && kv[h] + KH <= a.Sk;
    dead[h] = kv[h] >= a.Sk || (flags && flags[kv[h] / 128] == kBlkSkip);
    p[h] = a.drop + (((int64_t)bh * a.Sq + qb * 128 + 32 * i) * a.Sk + min(kv[h], max(a.Sk - KH, 0))) * ES;
  }
  // row words: 32 keys are two lanes' bits for bytes, four lanes' for 2-byte elements (whose second load fills
  // the words sixteen further on)
  constexpr int LPW = 32 / KH;                          // lanes per word
  const int widx = 32 * span + lane / LPW;
  const bool writer = rowbits && lane % LPW == 0;
  uint32_t* rowout = rowbits + ((int64_t)bh * a.Sq + qb * 128 + 32 * i) * a.droprow_w + widx;
  const int nrow = min(128, a.Sq - qb * 128);
  // cw[j]: the keep bits (bit e = this lane's key e) of rows j (low half) and j + 16 (high half) of the wave's 32
  uint32_t cw[16];
#pragma unroll
  for (int e = 0; e < 16; e++) cw[e] = 0u;
  for (int rh = 0; rh < 2; rh++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const int rr = 32 * i + 16 * rh + j;
      uint32_t nz = 0;                                  // bit KH*h + e: key e of this lane's load h is kept
#pragma unroll
      for (int h = 0; h < NH; h++) {
        if (rr < nrow && !dead[h]) {
          if (vec[h]) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(p[h]);
#pragma unroll
            for (int w = 0; w < 4; w++) {
              if (ES == 1) {
                // bit 8e: byte e is nonzero (no carry leaves a byte); then the four bits side by side
                const uint32_t y = ((((v[w] & 0x7f7f7f7fu) + 0x7f7f7f7fu) | v[w]) >> 7) & 0x01010101u;
                nz |= ((y | (y >> 7) | (y >> 14) | (y >> 21)) & 0xfu) << (4 * w);
              } else {
                // 2-byte floating-point elements: nonzero apart from the sign bit
                const uint32_t m = v[w] & 0x7fff7fffu;
                const uint32_t y = (((m + 0x7fff7fffu) | m) >> 15) & 0x00010001u;
                nz |= ((y | (y >> 15)) & 3u) << (KH * h + 2 * w);
              }
            }
          } else {
            const uint8_t* q = a.drop + ((int64_t)bh * a.Sq + qb * 128 + rr) * a.Sk * ES;
#pragma unroll
            for (int e = 0; e < KH; e++)
              if (kv[h] + e < a.Sk && elem_nonzero<ES>(q, kv[h] + e)) nz |= 1u << (KH * h + e);
          }
        }
        p[h] += (int64_t)a.Sk * ES;                     // per-lane pointers walk down the rows
      }
      cw[j] |= nz << (16 * rh);
#pragma unroll
      for (int h = 0; h < NH; h++) {
        uint32_t x = ((nz >> (KH * h)) & ((1u << KH) - 1u)) << (KH * (lane % LPW));
        x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xf, 0xf, true);                   // lane ^ 1
        if (LPW == 4) x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xf, 0xf, true);     // lane ^ 2
        if (writer && rr < nrow && !dead[h] && widx + 16 * h < a.droprow_w) rowout[16 * h] = x;   // (words of hidden key blocks are never read)
      }
      rowout += a.droprow_w;
    }
  }
  // The column words are the transpose of that 32 x 16 bit matrix: two 16 x 16 transposes side by side in the
  // sixteen registers (sub-blocks of 8, 4, 2, 1 swapped across the diagonal), after which bit r of cw[e] is the
  // keep bit of row r and key e.  (Shifting every key's bit into sixteen words row by row cost five times as many
  // instructions; this pass is bound by them, not by memory, once lanes of hidden key blocks load nothing.)
  {
    uint32_t mask = 0x00ff00ffu;
#pragma unroll
    for (int sft = 8; sft >= 1; sft >>= 1) {
#pragma unroll
      for (int k = 0; k < 16; k++) {
        if (k & sft) continue;
        const uint32_t t = ((cw[k] >> sft) ^ cw[k + sft]) & mask;
        cw[k + sft] ^= t;
        cw[k] ^= t << sft;
      }
      mask ^= mask << (sft >> 1);
    }
  }
  if (colbits)
    store_col_entries(s_cw, cw, i, lane, span * 1024, a.Sk, colbits + ((int64_t)bh * a.Tr + qb) * a.Sk * 4, flags,
                      [](int l, int e) { return ES == 1 ? 16 * l + e : 512 * (e >> 3) + 8 * l + (e & 7); });
}

// The same bitmaps for counter-based dropout: nothing is read, the keep decisions come from Philox4x32-10.
// One call yields the 16 bytes of one (query row, 32-key group M, half g): keys 32M + 8u + 4g + e for
// u = 0..3, e = 0..3 -- the keys one lane of the attention kernels owns in a 32-key group, so a kernel
// could also draw them in place.  One workgroup of four waves per (batch*head, 128 query rows, 1024 keys), one
// wave per 32 rows; lane 2L + g owns
// (M = 32*span + L, g), the lane pair forms the 32-bit row word of group M.
__global__ void __launch_bounds__(256) fa_drop_philox_kernel(const FaArgs a, uint32_t* rowbits, uint32_t* colbits) {
  __shared__ __attribute__((aligned(16))) uint32_t s_cw[(1024 + 64) * 4];
  const int nspan = (a.Sk + 1023) / 1024;
  const int i = threadIdx.x >> 6;                       // which 32 rows of the 128-row block: word i of the column entries
  const int blk = blockIdx.x;
  const int span = blk % nspan, qb = (blk / nspan) % a.Tr, bh = blk / (nspan * a.Tr);
  const int lane = threadIdx.x & 63, g = lane & 1;
  const int grp = 32 * span + (lane >> 1);              // 32-key group = word index within the row
  const bool writer = rowbits && g == 0 && grp < a.droprow_w;
  uint32_t* rowout = rowbits + ((int64_t)bh * a.Sq + qb * 128 + 32 * i) * a.droprow_w + grp;
  const int nrow = min(128, a.Sq - qb * 128);
  uint32_t cw[16];                                      // per key: the word of these 32 rows, most significant bit first
  {
#pragma unroll
    for (int t = 0; t < 16; t++) cw[t] = 0u;
#pragma unroll 2
    for (int r = 0; r < 32; r++) {
      const int rr = 32 * i + r;
      uint32_t v[4];
      philox4x32_10((uint32_t)(qb * 128 + rr), (uint32_t)(2 * grp + g), (uint32_t)bh, a.philox_offset, a.philox_k0, a.philox_k1, v);
      uint32_t bits = 0;
#pragma unroll
      for (int t = 0; t < 16; t++) {                    // t = 4u + e
        const uint32_t keep = ((v[t >> 2] >> (8 * (t & 3))) & 0xffu) < a.philox_thr ? 1u : 0u;
        bits |= keep << (8 * (t >> 2) + (t & 3));
        cw[t] = (cw[t] << 1) | (rr < nrow ? keep : 0u);
      }
      uint32_t x = bits << (4 * g);
      x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xf, 0xf, true);    // lane ^ 1
      if (writer && rr < nrow) *rowout = x;
      rowout += a.droprow_w;
    }
  }
  if (colbits) {
#pragma unroll
    for (int t = 0; t < 16; t++) cw[t] = __builtin_bitreverse32(cw[t]);
    store_col_entries(s_cw, cw, i, lane, span * 1024, a.Sk, colbits + ((int64_t)bh * a.Tr + qb) * a.Sk * 4, nullptr,
                      [](int l, int t) { return 32 * (l >> 1) + 8 * (t >> 2) + 4 * (l & 1) + (t & 3); });
  }
}

hipError_t launch_drop_philox(const FaArgs& a, uint32_t* rowbits, uint32_t* colbits, hipStream_t st) {
  const long long nblk = (long long)a.B * a.N * a.Tr * ((a.Sk + 1023) / 1024);
  hipLaunchKernelGGL(fa_drop_philox_kernel, dim3((unsigned)nblk), dim3(256), 0, st, a, rowbits, colbits);
  return hipGetLastError();
}

hipError_t launch_drop_bits(const FaArgs& a, uint32_t* rowbits, uint32_t* colbits, hipStream_t st) {
  const long long nblk = (long long)a.B * a.N * a.Tr * ((a.Sk + 1023) / 1024);
  if (a.drop_es == 2) hipLaunchKernelGGL(fa_drop_bits_kernel<2>, dim3((unsigned)nblk), dim3(256), 0, st, a, rowbits, colbits);
  else hipLaunchKernelGGL(fa_drop_bits_kernel<1>, dim3((unsigned)nblk), dim3(256), 0, st, a, rowbits, colbits);
  return hipGetLastError();
}

// true when launch_mask_blocks takes the fast path, which also writes the column bitmaps
bool mask_prepass_is_fused(const FaArgs& a) {
  // every 16-element piece of a row is 16-byte aligned and entirely inside or outside the row
  return (((uintptr_t)a.mask | (uintptr_t)a.Sk | (uintptr_t)a.mask_sb) & 15) == 0;
}

hipError_t launch_mask_blocks(const FaArgs& a, uint8_t* flags, uint32_t* colbits, int MB, hipStream_t st) {
  if (mask_prepass_is_fused(a)) {
    const dim3 grid((unsigned)((long long)MB * a.Tr * a.Tc));
    uint8_t* tails = flags + (size_t)MB * a.Tr * a.Tc;  // (the key-tail table follows the classes)
    if (a.mask_es == 2) hipLaunchKernelGGL(fa_mask_prepass_kernel<2>, grid, dim3(256), 0, st, a, flags, tails, colbits);
    else hipLaunchKernelGGL(fa_mask_prepass_kernel<1>, grid, dim3(256), 0, st, a, flags, tails, colbits);
    return hipGetLastError();
  }
  const dim3 grid((unsigned)(MB * a.Tr));
  if (a.mask_es == 2) hipLaunchKernelGGL(fa_mask_blocks_kernel<2>, grid, dim3(256), 0, st, a, flags);
  else hipLaunchKernelGGL(fa_mask_blocks_kernel<1>, grid, dim3(256), 0, st, a, flags);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !colbits) return e;
  return launch_mask_colbits(a, flags, colbits, MB, st);
}

}  // namespace acct
