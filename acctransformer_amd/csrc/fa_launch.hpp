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

// The kernels are built for the head dims 40, 64, 80, 128, 160 and 256.  Any other multiple of 8 runs on the next
// built size of its row layout (128-, 256- or 512-byte LDS rows): the columns past the head dim are never loaded
// as operands (zero fragments) and never stored.
inline int head_dim_class(int D) {
  if (D == 40 || D == 80 || D == 160) return D;
  return D <= 64 ? 64 : (D <= 128 ? 128 : 256);
}

// The dK/dV kernel gives every workgroup 256 keys (128 above head dim 128) of one head and all query rows.  With
// few heads and a short key sequence (cross attention on 77 keys) that is a handful of workgroups for 256 CUs:
// the query range is then cut into q_split slices that run side by side, and a second kernel adds their sums.
// Returns q_split (1 = no split) and the bytes of workspace the slices' sums take.
// `n_cu`: compute units of the device that runs the launch; the workspace-size query passes the 256 of a whole
// MI355X, which is also the upper bound of what a partition of it asks for.
struct DkdvSplit { int q_split; size_t part_bytes; };
inline DkdvSplit dkdv_split(int B, int N, int Sq, int Sk, int D, int n_cu = 256) {
  const int dc = head_dim_class(D), ngk = dc > 128 ? 1 : 2, db = (dc + 31) / 32;
  const long long n_wg = (long long)B * N * ((Sk + 128 * ngk - 1) / (128 * ngk));
  const long long tiles64 = (Sq + 63) / 64;
  long long s = (n_cu > 256 ? 256 : n_cu) / n_wg;
  if (tiles64 / 8 < s) s = tiles64 / 8;              // a slice keeps at least 512 query rows
  if (s > 16) s = 16;
  if (s < 2) return {1, 0};
  return {(int)s, (size_t)s * (size_t)n_wg * 8 * ngk * db * 1024 * sizeof(float)};
}

// forward: variant 3 = 8 waves x 32 query rows, 1 = 4 waves x 32 rows; the bias / dropout
// variants are picked from a.alibi / a.droprow
hipError_t launch_fwd(const FaArgs& a, int dtype, int D, int qg, hipStream_t st);

// backward: delta pre-pass, dK/dV kernel (kv-tile owner) and dQ kernel (q-tile owner)
enum : int { kStageDq = 1, kStageDkDv = 2 };
hipError_t launch_bwd(const FaArgs& a, int dtype, int D, int stages, hipStream_t st);

// false when the kernel translation units were compiled with a reduced variant set (ACCT_DEV_BUILD)
bool launch_variants_complete();

// classify the 128x128 blocks of a dense mask into clean / apply / skip / causal diagonal and, with `colbits`
// non-null, pack its 'apply' blocks into per-key-column bitmaps [MB, Tr, Sk, 4 x u32] (one launch for aligned masks)
hipError_t launch_mask_blocks(const FaArgs& a, uint8_t* flags, uint32_t* colbits, int MB, hipStream_t st);
// pack the dropout mask into keep bits by query row [B*N, Sq, droprow_w] and / or by key column [B*N, Tr, Sk, 4]
hipError_t launch_drop_bits(const FaArgs& a, uint32_t* rowbits, uint32_t* colbits, hipStream_t st);
// the same two bitmaps generated from (a.philox_k0, a.philox_k1, a.philox_offset, a.philox_thr) instead of read from a mask
hipError_t launch_drop_philox(const FaArgs& a, uint32_t* rowbits, uint32_t* colbits, hipStream_t st);
// the column bitmaps by themselves (and the compact tile's: out[key][4])
hipError_t launch_mask_colbits(const FaArgs& a, const uint8_t* flags, uint32_t* out, int MB, hipStream_t st);

}  // namespace acct
