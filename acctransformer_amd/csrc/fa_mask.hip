// Block classification of a dense uint8 attention mask.
//
// The reference adds -10000 to masked scores (attention.py:357-371 of the
// reference's flash_attention ops) instead of removing them.  A 128x128 block
// whose entries are all masked therefore contributes exp(-10000 + ...) = 0 in
// fp32 to every row that has at least one unmasked visible key elsewhere, and
// can be skipped without changing a bit of the result; a block with no masked
// entry needs no mask loads.  This pre-pass finds both kinds so the attention
// kernels touch the mask only on mixed blocks.
#include "fa_common.hpp"
#include "fa_launch.hpp"

namespace acct {

constexpr uint8_t kBlkAllMasked = 3;   // provisional: resolved to skip or apply below

// one workgroup per (mask batch, q block); thread t scans 64 columns of row t/2
__global__ void __launch_bounds__(256) fa_mask_blocks_kernel(const FaArgs a, uint8_t* flags) {
  const int qb = blockIdx.x % a.Tr, mb = blockIdx.x / a.Tr;
  const int tid = threadIdx.x, row = qb * 128 + (tid >> 1), c0 = (tid & 1) * 64;
  const uint8_t* mrow = a.mask + (int64_t)mb * a.mask_sb + (int64_t)min(row, a.Sq - 1) * a.Sk;
  const bool vec_ok = (((uintptr_t)a.mask | (uintptr_t)a.Sk | (uintptr_t)a.mask_sb) & 3) == 0;
  uint8_t* frow = flags + ((int64_t)mb * a.Tr + qb) * a.Tc;
  int lo = max(0, qb - a.prev_blk), hi = min(a.Tc - 1, qb + a.next_blk);
  if (a.row_prefix) hi = min(hi, ((qb * 128 / a.row_prefix + 1) * a.row_prefix - 1) / 128);
  for (int kvb = tid; kvb < a.Tc; kvb += 256)
    if (kvb < lo || kvb > hi) frow[kvb] = kBlkClean;
  bool row_unmasked = false;
  for (int kvb = lo; kvb <= hi; kvb++) {
    bool any_m = false, any_u = false;
    if (row < a.Sq) {
#pragma unroll 4
      for (int c = 0; c < 64; c += 4) {
        const int kv = kvb * 128 + c0 + c;
        if (kv >= a.Sk) break;
        const int n = min(4, a.Sk - kv);
        const uint32_t bits = load_u8x4(mrow, kv, a.Sk, vec_ok);
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (e < n) { if ((bits >> (8 * e)) & 0xffu) any_m = true; else any_u = true; }
      }
    }
    row_unmasked |= any_u;
    const int blk_m = __syncthreads_or(any_m), blk_u = __syncthreads_or(any_u);
    if (tid == 0) frow[kvb] = !blk_m ? kBlkClean : (!blk_u ? kBlkAllMasked : kBlkApply);
  }
  row_unmasked |= (bool)__shfl_xor((int)row_unmasked, 1);
  const int rows_ok = __syncthreads_and(row >= a.Sq || row_unmasked);
  // (the barrier above also orders thread 0's provisional writes before the reads below)
  for (int kvb = lo + tid; kvb <= hi; kvb += 256)
    if (frow[kvb] == kBlkAllMasked) frow[kvb] = rows_ok ? kBlkSkip : kBlkApply;
}

hipError_t launch_mask_blocks(const FaArgs& a, uint8_t* flags, int MB, hipStream_t st) {
  hipLaunchKernelGGL(fa_mask_blocks_kernel, dim3((unsigned)(MB * a.Tr)), dim3(256), 0, st, a, flags);
  return hipGetLastError();
}

}  // namespace acct
