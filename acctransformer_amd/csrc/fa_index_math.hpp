// Integer index arithmetic shared by the gfx950 attention kernels and their launchers: workgroup -> tile
// maps, LDS swizzles, head-dim classes, the query-range split of the dK/dV launch.  No HIP in here: the file
// also compiles with a host compiler, which is how the unit tests reach these functions.
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define ACCT_HD __host__ __device__ __forceinline__
#else
#define ACCT_HD inline
#endif

namespace acct {

// Workgroup id -> (batch*head, launch rank of the tile; rank 0 is launched first).  Workgroups are
// handed to the 8 XCDs round robin (id % 8), each XCD with its own L2.  With many heads the plain
// "head fastest" order gives every CU of an XCD a different head and nothing is shared; instead the
// heads of an XCD are taken 8 at a time and all tiles of those 8 heads are launched together, so
// that the workgroups streaming the same K/V (or Q/dO) rows run side by side on one L2.
ACCT_HD void wg_map(int id, int BH, int n_tiles, int& bh, int& rank) {
  if (BH > 64 && (BH & 63) == 0) {
    const int xcd = id & 7, slot = id >> 3;
    const int per_group = 8 * n_tiles;
    const int grp = slot / per_group, r = slot - grp * per_group;
    rank = r >> 3;
    bh = xcd + 8 * (grp * 8 + (r & 7));
  } else {
    bh = id % BH;
    rank = id / BH;
  }
}

// ---- swizzle of the LDS tiles that the direct-to-LDS loads fill ----
// Row pitch is a power of two (no padding, as the DMA writes 64 consecutive 16-byte
// slots per wave instruction); the 16-byte chunk c of row r lives in slot c ^ swz(r).
// The LDS serves a 16-byte read in groups of 16 lanes over 64 four-byte banks, so the
// fragment reads (lane = row) need the 16 rows of a group in 16 different slots of the
// 256 bytes the banks span: measured 4.3 clocks per wave instruction against 8.2 when
// only eight rows differ.  For 256-byte rows that is a four-bit swizzle,
// swz(r) = ((r & 3) << 1) | ((r >> 2) & 1) | (r & 8); its low three bits also put one
// 32-byte chunk PAIR of four consecutive rows into four different pairs of slots, which
// is what the transposed 8-byte reads (4 rows x 32 bytes per 16 lanes) need.  For
// 128-byte rows two consecutive rows span the banks and swz(r) = (r >> 1) & 7.
ACCT_HD int swz3(int row) { return ((row & 3) << 1) | ((row >> 2) & 1); }

template <int D> struct SwzCfg {
  static constexpr int KS = (D + 15) / 16;      // 16-wide k-steps across the head dim (the last one half empty when D % 16 == 8)
  static constexpr int DB = (D + 31) / 32;      // 32-wide blocks across the head dim
  static constexpr int CPR = D / 8;             // valid 16-byte chunks per row
  static constexpr int CH = D <= 64 ? 8 : (D <= 128 ? 16 : 32);   // chunk slots per LDS row
  static constexpr int PITCH = CH * 16;
  static constexpr int RPI = 64 / CH;           // rows covered by one wave-wide DMA instruction
  // (rows of 512 bytes wrap around the banks twice: the four-bit swizzle of the 256-byte rows serves them too)
  static ACCT_HD int swz(int row) { return CH >= 16 ? (swz3(row) | (row & 8)) : ((row >> 1) & 7); }
  // Transposed reads come in pairs, rows r..r+3 and r+8..r+11 with r % 16 < 8: the second row group has
  // the top swizzle bit set, so its slot differs in that bit.  Which way depends only on the 32-column
  // block db the read belongs to (chunk 4 db + 0..3), i.e. the distance is a compile-time constant.
  static constexpr int tr_hi(int db) {
    return 8 * PITCH + (CH >= 16 ? (((db >> 1) & 1) ? -128 : 128) : ((db & 1) ? -64 : 64));
  }
};

// idx / n for idx < 1024 and n <= 32 (the epilogues' chunk index -> row): exact with a 16-bit reciprocal
ACCT_HD int div_small(int idx, uint32_t inv16) { return (int)(((uint32_t)idx * inv16) >> 16); }
ACCT_HD uint32_t recip16(int n) { return (65536u + (uint32_t)n - 1u) / (uint32_t)n; }

// byte offset of logical chunk `lc` in a row whose swz3(row) is `swz`
ACCT_HD int swz_off(int lc, int swz) { return (lc ^ swz) << 4; }

// The kernels are built for the head dims 40, 64, 80, 128, 160 and 256.  Any other multiple of 8 runs on the next
// built size of its row layout (128-, 256- or 512-byte LDS rows): the columns past the head dim are never loaded
// as operands (zero fragments) and never stored.
ACCT_HD int head_dim_class(int D) {
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
ACCT_HD DkdvSplit dkdv_split(int B, int N, int Sq, int Sk, int D, int n_cu = 256) {
  const int dc = head_dim_class(D), ngk = dc > 128 ? 1 : 2, db = (dc + 31) / 32;
  const long long n_wg = (long long)B * N * ((Sk + 128 * ngk - 1) / (128 * ngk));
  const long long tiles64 = (Sq + 63) / 64;
  long long s = (n_cu > 256 ? 256 : n_cu) / n_wg;
  if (tiles64 / 8 < s) s = tiles64 / 8;              // a slice keeps at least 512 query rows
  if (s > 16) s = 16;
  if (s < 2) return {1, 0};
  return {(int)s, (size_t)s * (size_t)n_wg * 8 * ngk * db * 1024 * sizeof(float)};
}

}  // namespace acct
