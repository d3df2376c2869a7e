// Host-compiled unit tests of the integer index arithmetic the gfx950 kernels rest on
// (acctransformer_amd/csrc/fa_index_math.hpp).  Built and run by tests/test_index_math.py with g++;
// prints one line per failed check and exits with the number of failures.
// Test tier modelled on the reference's helper-level unit tests
// (tests/train/flash_attention/ut/test_split_core_strategy.py, test_tensor_transformat.py).
#include <cstdio>
#include <set>
#include <vector>

#include "../../acctransformer_amd/csrc/fa_index_math.hpp"

using namespace acct;

static int failures = 0;
#define CHECK(cond, ...)                                   \
  do {                                                     \
    if (!(cond)) {                                         \
      if (failures < 20) { printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } \
      failures++;                                          \
    }                                                      \
  } while (0)

// every (batch*head, tile rank) pair is produced by exactly one workgroup id, whichever branch of the map runs
static void test_wg_map() {
  const int tiles[] = {1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64};
  std::vector<char> seen;
  for (int BH = 1; BH <= 512; BH++)
    for (int nt : tiles) {
      seen.assign((size_t)BH * nt, 0);
      bool ok = true;
      for (int id = 0; id < BH * nt && ok; id++) {
        int bh = -1, rank = -1;
        wg_map(id, BH, nt, bh, rank);
        ok = bh >= 0 && bh < BH && rank >= 0 && rank < nt && !seen[(size_t)bh * nt + rank];
        if (ok) seen[(size_t)bh * nt + rank] = 1;
      }
      CHECK(ok, "wg_map is not a bijection for BH=%d n_tiles=%d", BH, nt);
    }
  // the grouped branch: the workgroups of one head all carry the same id % 8 (one XCD, one L2), ranks ascend with the id
  for (int BH : {128, 256, 512}) {
    const int nt = 16;
    std::vector<int> xcd(BH, -1), last_rank(BH, -1);
    for (int id = 0; id < BH * nt; id++) {
      int bh, rank;
      wg_map(id, BH, nt, bh, rank);
      CHECK(xcd[bh] < 0 || xcd[bh] == (id & 7), "head %d of BH=%d is spread over XCDs", bh, BH);
      xcd[bh] = id & 7;
      CHECK(rank > last_rank[bh], "ranks of head %d do not ascend with the workgroup id", bh);
      last_rank[bh] = rank;
    }
  }
  // the plain branch: head index fastest
  {
    int bh, rank;
    wg_map(64 * 3 + 5, 64, 8, bh, rank);
    CHECK(bh == 5 && rank == 3, "plain branch: got bh=%d rank=%d", bh, rank);
  }
}

// A 16-byte fragment read is served 16 lanes at a time; the 16 rows of such a group must land in 16 different
// 16-byte slots of the 256 bytes the banks span, for every logical chunk.
template <int D> static void test_swizzle_rows() {
  using C = SwzCfg<D>;
  for (int r0 = 0; r0 < 64; r0 += 16)
    for (int c = 0; c < C::CH; c++) {
      std::set<int> slots;
      for (int r = r0; r < r0 + 16; r++) {
        const int addr = r * C::PITCH + ((c ^ C::swz(r)) << 4);
        CHECK(((c ^ C::swz(r)) >= 0) && ((c ^ C::swz(r)) < C::CH), "D=%d: chunk %d of row %d leaves the row", D, c, r);
        slots.insert((addr % 256) / 16);
      }
      CHECK(slots.size() == 16, "D=%d rows %d..%d chunk %d: %zu distinct bank slots", D, r0, r0 + 15, c, slots.size());
    }
  // the swizzle is a permutation of a row's chunks and repeats every 16 rows
  for (int r = 0; r < 64; r++) {
    std::set<int> s;
    for (int c = 0; c < C::CH; c++) s.insert(c ^ C::swz(r));
    CHECK((int)s.size() == C::CH, "D=%d row %d: the swizzle is not a permutation", D, r);
    CHECK(C::swz(r) == C::swz(r + 16), "D=%d: the swizzle does not repeat after 16 rows at row %d", D, r);
  }
}

// Transposed reads: the lanes of a wave address rows trow = 4 g + (lane % 16) / 4 (g = lane / 32) of an 8-row group,
// chunk 4 db + tchunk; the partner read of rows + 8 must sit exactly tr_hi(db) bytes further, for every lane and db.
template <int D> static void test_tr_hi() {
  using C = SwzCfg<D>;
  for (int lane = 0; lane < 64; lane++) {
    const int g = lane >> 5;
    const int trow = 4 * g + ((lane & 15) >> 2);
    const int tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    for (int db = 0; db < C::DB; db++)
      for (int grp = 0; grp < 64; grp += 16) {
        const int lo = (grp + trow) * C::PITCH + swz_off(4 * db + tchunk, C::swz(grp + trow));
        const int hi = (grp + trow + 8) * C::PITCH + swz_off(4 * db + tchunk, C::swz(grp + trow + 8));
        CHECK(hi - lo == C::tr_hi(db), "D=%d lane %d db %d: rows +8 sit %d bytes away, tr_hi says %d", D, lane, db, hi - lo, C::tr_hi(db));
      }
  }
  // the four rows x two 16-byte chunks that a 16-lane group of a transposed read touches fall into 8 different slots
  // (256- and 512-byte rows; with 128-byte rows two consecutive rows share a swizzle value and the eight pieces
  // fall into 4 slots, a two-way conflict that the head dims up to 64 live with)
  for (int db = 0; db < C::DB; db++)
    for (int half = 0; half < 2; half++)
      for (int g = 0; g < 2; g++) {
        std::set<int> slots;
        for (int i = 0; i < 16; i++) {
          const int lane = 32 * g + 16 * half + i;
          const int trow = 4 * g + ((lane & 15) >> 2), tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
          const int addr = trow * C::PITCH + swz_off(4 * db + tchunk, C::swz(trow));
          slots.insert((addr % 256) / 16);
        }
        const size_t want = C::CH >= 16 ? 8 : 4;
        CHECK(slots.size() == want, "D=%d db %d: a transposed 16-lane group touches %zu slots, expected %zu", D, db, slots.size(), want);
      }
}

static void test_head_dim_class() {
  const int built[] = {40, 64, 80, 128, 160, 256};
  for (int D = 8; D <= 256; D += 8) {
    const int c = head_dim_class(D);
    bool is_built = false;
    for (int b : built) is_built |= b == c;
    CHECK(is_built && c >= D, "head dim %d runs on %d", D, c);
    // same LDS row layout: 128-, 256- or 512-byte rows
    auto layout = [](int d) { return d <= 64 ? 0 : (d <= 128 ? 1 : 2); };
    CHECK(layout(c) == layout(D), "head dim %d (layout %d) runs on %d (layout %d)", D, layout(D), c, layout(c));
    for (int b : built) CHECK(!(b >= D && b < c && layout(b) == layout(D) && (b == D)), "head dim %d skips its own built size", D);
  }
  CHECK(head_dim_class(40) == 40 && head_dim_class(48) == 64 && head_dim_class(72) == 128 && head_dim_class(136) == 256, "class table");
}

static void test_dkdv_split() {
  for (int B : {1, 2, 4, 16})
    for (int N : {1, 4, 16, 32})
      for (int Sq : {64, 511, 512, 1024, 4096, 131072})
        for (int Sk : {1, 77, 128, 256, 257, 2048})
          for (int D : {40, 64, 128, 160, 256})
            for (int n_cu : {32, 64, 256, 304}) {
              const DkdvSplit sp = dkdv_split(B, N, Sq, Sk, D, n_cu), full = dkdv_split(B, N, Sq, Sk, D);
              const int ngk = head_dim_class(D) > 128 ? 1 : 2, db = (head_dim_class(D) + 31) / 32;
              const long long n_wg = (long long)B * N * ((Sk + 128 * ngk - 1) / (128 * ngk));
              CHECK(sp.q_split >= 1 && sp.q_split <= 16, "q_split %d out of range", sp.q_split);
              CHECK(sp.q_split <= full.q_split && sp.part_bytes <= full.part_bytes,
                    "a device of %d CUs asks for more than the workspace query grants (B%d N%d Sq%d Sk%d D%d)", n_cu, B, N, Sq, Sk, D);
              if (sp.q_split > 1) {
                CHECK(sp.q_split * n_wg <= (n_cu > 256 ? 256 : n_cu), "split grid %lld exceeds the CUs", sp.q_split * n_wg);
                CHECK(((Sq + 63) / 64) / sp.q_split >= 8, "a slice has fewer than 512 query rows");
                CHECK(sp.part_bytes == (size_t)sp.q_split * n_wg * 8 * ngk * db * 4096, "part_bytes");
              } else {
                CHECK(sp.part_bytes == 0, "no split but %zu bytes", sp.part_bytes);
              }
            }
  // the cross-attention shape the split exists for, and the benchmark shape that must not split
  CHECK(dkdv_split(2, 16, 4096, 77, 40).q_split == 8, "B2 N16 Sq4096 Sk77 D40 -> %d", dkdv_split(2, 16, 4096, 77, 40).q_split);
  CHECK(dkdv_split(4, 16, 2048, 2048, 128).q_split == 1, "the benchmark shape splits");
}

static void test_div_small() {
  for (int n = 1; n <= 32; n++)
    for (int idx = 0; idx < 1024; idx++) CHECK(div_small(idx, recip16(n)) == idx / n, "div_small(%d, %d)", idx, n);
}

int main() {
  test_wg_map();
  test_swizzle_rows<64>();
  test_swizzle_rows<128>();
  test_swizzle_rows<256>();
  test_tr_hi<64>();
  test_tr_hi<128>();
  test_tr_hi<256>();
  test_head_dim_class();
  test_dkdv_split();
  test_div_small();
  if (failures) printf("%d checks failed\n", failures);
  else printf("index math: all checks passed\n");
  return failures > 255 ? 255 : failures;
}
