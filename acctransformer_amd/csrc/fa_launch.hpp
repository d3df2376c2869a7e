// Host-side launchers of the gfx950 attention kernels (one per translation unit).
#pragma once
#include "fa_common.hpp"

#include <mutex>
#include <set>
#include <utility>

namespace acct {

// Raises a kernel's dynamic LDS limit once per (kernel, device) instead of on every launch.
inline hipError_t allow_dynamic_lds(const void* kern, size_t bytes) {
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> done;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(mu);
  if (done.count({kern, dev})) return hipSuccess;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess) done.insert({kern, dev});
  return e;
}

// forward: variant 3 = 8 waves x 32 query rows, 1 = 4 waves x 32 rows; the bias / dropout
// variants are picked from a.alibi / a.droprow
hipError_t launch_fwd(const FaArgs& a, int dtype, int D, int qg, hipStream_t st);

// backward: delta pre-pass, dK/dV kernel (kv-tile owner) and dQ kernel (q-tile owner)
enum : int { kStageDq = 1, kStageDkDv = 2 };
hipError_t launch_bwd(const FaArgs& a, int dtype, int D, int stages, hipStream_t st);

// the dQ kernel with 64 query rows per wave (fa_bwd_dq64.hip): head dim 128, no side inputs, aligned lengths
bool dq64_applicable(const FaArgs& a);
hipError_t launch_bwd_dq64(FaArgs a, int dtype, hipStream_t st);

// false when the kernel translation units were compiled with a reduced variant set (ACCT_DEV_BUILD)
bool launch_variants_complete();

// classify the 128x128 blocks of a dense mask into clean / apply / skip / causal diagonal and, with `colbits`
// non-null, pack its 'apply' blocks into per-key-column bitmaps [MB, Tr, Sk, 4 x u32] (one launch for aligned masks)
// true when launch_mask_blocks takes its one-launch path, which also fills the key-tail table behind the classes
bool mask_prepass_is_fused(const FaArgs& a);
hipError_t launch_mask_blocks(const FaArgs& a, uint8_t* flags, uint32_t* colbits, int MB, hipStream_t st);
// pack the dropout mask into keep bits by query row [B*N, Sq, droprow_w] and / or by key column [B*N, Tr, Sk, 4]
hipError_t launch_drop_bits(const FaArgs& a, uint32_t* rowbits, uint32_t* colbits, hipStream_t st);
// the same two bitmaps generated from (a.philox_k0, a.philox_k1, a.philox_offset, a.philox_thr) instead of read from a mask
hipError_t launch_drop_philox(const FaArgs& a, uint32_t* rowbits, uint32_t* colbits, hipStream_t st);
// the column bitmaps by themselves (and the compact tile's: out[key][4])
hipError_t launch_mask_colbits(const FaArgs& a, const uint8_t* flags, uint32_t* out, int MB, hipStream_t st);

}  // namespace acct
