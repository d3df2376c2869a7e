// dQ kernel of the FlashAttention2 backward with 64 query rows per wave (head dim 128, no side inputs).
//
// Same algorithm and results layout as fa_bwd_dq_kernel (fa_bwd.hip; replaces the dQ part of the reference's
// backward builder, flash_attention_bwd.py:209-231, and its D = rowsum(dO*O), :138-159): a workgroup owns 256
// query rows of one (batch, head) and streams K/V tiles of 64 keys through LDS.  Here the workgroup is 4 waves
// of 64 rows -- one wave per SIMD, 512 registers each -- instead of 8 waves of 32 rows: every K, V and K^T
// fragment read from LDS feeds two MFMAs, which halves the LDS bytes per flop, the largest cost above the
// matrix work in that kernel.  A lone wave per SIMD has no partner to overlap with, so the tile loop is one
// block of hand-scheduled assembly (fa_bwd_dq64_asm.inc, written by gen_dq64_asm.py), software-pipelined three
// 32-key chunks deep: the vector work of one chunk rides behind the MFMAs of the score products of the next
// and of the dQ product of the one before; the accumulators and the Q / dO fragments live in AGPRs at fixed
// registers.  The code around the loop (prologue with the first two tiles' DMA, epilogue) is HIP.
//
// Served cases: head dim 128 exactly, no bias, no dropout, no mask tensor (mask none or the causal mask by
// index compare), no row-block prefix, the band open towards earlier keys, Sq a multiple of 256 and Sk of 64.
// Everything else stays with fa_bwd_dq_kernel.
#include "fa_common.hpp"
#include "fa_launch.hpp"
#ifndef ACCT_DQ64_ASM_INC
#define ACCT_DQ64_ASM_INC "fa_bwd_dq64_asm.inc"          // a timing build names another generated file here
#endif
#include ACCT_DQ64_ASM_INC

namespace acct {

typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef uint32_t u32x32 __attribute__((ext_vector_type(32)));
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

// The tile loop (fa_bwd_dq64_asm.inc): operands at the fixed registers the generated code names.
template <typename T> struct Dq64Asm;
#define DQ64_RUN(BODY)                                                                                                   \
  asm volatile(BODY                                                                                                      \
               : "+{a[0:31]}"(acc0), "+{a[32:63]}"(acc1), "+{a[64:95]}"(acc2), "+{a[96:127]}"(acc3)                     \
               : "{a[128:159]}"(qa), "{a[160:191]}"(qb), "{a[192:223]}"(doa), "{a[224:255]}"(dob), "{v[96:103]}"(koff), \
                 "{v[104:107]}"(toff), "{v108}"(nlq0), "{v109}"(nlq1), "{v110}"(dl0), "{v111}"(dl1),                      \
                 "{v[116:119]}"(kvoff), "{v[120:123]}"(vvoff), "{v124}"(rowrel0), "{v125}"(rowrel1),                      \
                 [kbuf0] "s"(s.kbuf0), [lds0] "s"(s.lds0), [kptr] "s"(s.kptr), [vptr] "s"(s.vptr), [kstep] "s"(s.kstep),       \
                 [vstep] "s"(s.vstep), [jhi] "s"(s.jhi), [jlast] "s"(s.jlast), [lastedge] "s"(s.lastedge), [scale] "s"(s.scale) \
               : DQ64_CLOBBERS)
struct Dq64Scalars {
  uint32_t kbuf0, lds0;              // LDS: first of the three K/V tile buffers, this wave's slab inside a tile
  uint64_t kptr, vptr;               // global address of the K / V rows of tile 2 (of the last tile when there are fewer)
  uint32_t kstep, vstep;             // bytes from one tile's rows to the next
  uint32_t jhi;                      // last tile of the workgroup
  uint32_t jlast, lastedge;          // last tile of this wave; whether the causal diagonal runs through it
  float scale;                       // scale * log2(e)
};
template <> struct Dq64Asm<f16> {
  static ACCT_DEV void run(const Dq64Scalars& s, f32x32& acc0, f32x32& acc1, f32x32& acc2, f32x32& acc3, const u32x32& qa, const u32x32& qb,
                           const u32x32& doa, const u32x32& dob, const u32x8& koff, const u32x4& toff, float nlq0, float nlq1, float dl0,
                           float dl1, const u32x4& kvoff, const u32x4& vvoff, int rowrel0, int rowrel1) {
    DQ64_RUN(DQ64_LOOP_F16);
  }
};
template <> struct Dq64Asm<bf16> {
  static ACCT_DEV void run(const Dq64Scalars& s, f32x32& acc0, f32x32& acc1, f32x32& acc2, f32x32& acc3, const u32x32& qa, const u32x32& qb,
                           const u32x32& doa, const u32x32& dob, const u32x8& koff, const u32x4& toff, float nlq0, float nlq1, float dl0,
                           float dl1, const u32x4& kvoff, const u32x4& vvoff, int rowrel0, int rowrel1) {
    DQ64_RUN(DQ64_LOOP_BF16);
  }
};
#undef DQ64_RUN

template <typename T>
__global__ void __launch_bounds__(256) fa_bwd_dq64_kernel(const FaArgs a) {
  using E = Elem<T>;
  using V8 = typename E::V8;
  constexpr int D = 128, NW = 4, BM = 256;
  using C = SwzCfg<D>;
  constexpr int TILEB = 64 * C::PITCH;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  ACCT_LDS char* smem = (ACCT_LDS char*)smem_raw;   // [3 buffers][K tile | V tile]; reused by the epilogue

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int bh, rank;
  wg_map(blockIdx.x, a.B * a.N, a.n_tiles, bh, rank);
  const int qt = a.n_tiles - 1 - rank;               // heaviest (latest) causal tiles first
  const int b = bh / a.N, h = bh % a.N;
  const int q0 = qt * BM, wq0 = q0 + wave * 64;      // every row exists: Sq is a multiple of 256
  const bool causal = a.mask_kind == kMaskCausal;

  const T* qp = (const T*)a.q + b * a.q_sb + h * a.q_sh;
  const T* kp = (const T*)a.k + b * a.k_sb + h * a.k_sh;
  const T* vp = (const T*)a.v + b * a.v_sb + h * a.v_sh;
  const T* op = (const T*)a.o + b * a.o_sb + h * a.o_sh;
  const T* dop = (const T*)a.dout + b * a.o_sb + h * a.o_sh;

  const int j_lo = 0;
  int j_hi = a.Sk / 64 - 1;
  if (causal) j_hi = min(j_hi, (q0 + BM - 1) / 64);

  // Q and dO fragments (B operands: lane holds row l32 of its group, d = 16 t + 8 g .. +7), D and LSE of the rows
  u32x32 qa, qb, doa, dob;
  float dl[2], nlq[2];
#pragma unroll
  for (int gq = 0; gq < 2; gq++) {
    const int row = wq0 + 32 * gq + l32;
    float part = 0.f;
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const V8 qv = *reinterpret_cast<const V8*>(qp + (int64_t)row * a.q_ss + 16 * t + 8 * g);
      const V8 dv = *reinterpret_cast<const V8*>(dop + (int64_t)row * a.o_ss + 16 * t + 8 * g);
      const V8 ov = *reinterpret_cast<const V8*>(op + (int64_t)row * a.o_ss + 16 * t + 8 * g);
#pragma unroll
      for (int e = 0; e < 8; e++) part += (float)dv[e] * (float)ov[e];
      const u32x4 qw = __builtin_bit_cast(u32x4, qv), dw = __builtin_bit_cast(u32x4, dv);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (gq == 0) { qa[4 * t + e] = qw[e]; doa[4 * t + e] = dw[e]; }
        else { qb[4 * t + e] = qw[e]; dob[4 * t + e] = dw[e]; }
      }
    }
    dl[gq] = pair_sum(part);
    // (minus p_shift: the recomputed probabilities carry a factor 2^p_shift, see FaArgs)
    const float lq = a.lse[(int64_t)bh * a.Sq + row] * kLog2e - a.p_shift;
    nlq[gq] = -lq;
    if (g == 0) {
      a.delta[(int64_t)bh * a.Sq + row] = dl[gq];
      a.nlse[(int64_t)bh * a.Sq + row] = -lq;          // p_shift - LSE*log2(e): the exp2 offset the dK/dV kernel adds
    }
  }

  // per-lane LDS offsets inside a tile: row-major fragment of k-step t (row l32, chunk 2t + g), transposed
  // fragment of 32-column block db
  u32x8 koff;
#pragma unroll
  for (int t = 0; t < 8; t++) koff[t] = (uint32_t)(l32 * C::PITCH + swz_off(2 * t + g, C::swz(l32)));
  u32x4 toff;
  {
    const int trow = 4 * g + ((lane & 15) >> 2);
    const int tchunk = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
#pragma unroll
    for (int db = 0; db < 4; db++) toff[db] = (uint32_t)(trow * C::PITCH + swz_off(4 * db + tchunk, C::swz(trow)) + 8 * (lane & 1));
  }

  f32x32 acc0, acc1, acc2, acc3;                      // dQ^T: group 0 blocks 0-1, 2-3; group 1 blocks 0-1, 2-3
#pragma unroll
  for (int i = 0; i < 32; i++) acc0[i] = acc1[i] = acc2[i] = acc3[i] = 0.f;

  TileDma<T, D, 64, NW> kdma, vdma;
  kdma.plan(a.k_ss, D / 8);
  vdma.plan(a.v_ss, D / 8);
  if (j_lo <= j_hi) {
    // tiles 0 and 1 have landed before the loop starts; inside it every tile is requested two steps ahead
    const int t1 = min(1, j_hi) * 64, t2 = min(2, j_hi) * 64;
    kdma.issue(kp, a.k_ss, 0, smem);
    vdma.issue(vp, a.v_ss, 0, smem + TILEB);
    kdma.issue(kp, a.k_ss, t1, smem + 2 * TILEB);
    vdma.issue(vp, a.v_ss, t1, smem + 3 * TILEB);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    auto uniform = [](uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };
    Dq64Scalars s;
    s.kbuf0 = uniform((uint32_t)(uintptr_t)smem);
    s.lds0 = uniform(kdma.lds0);
    const uint64_t kptr = (uint64_t)(uintptr_t)(kp + (int64_t)t2 * a.k_ss), vptr = (uint64_t)(uintptr_t)(vp + (int64_t)t2 * a.v_ss);
    s.kptr = ((uint64_t)uniform((uint32_t)(kptr >> 32)) << 32) | uniform((uint32_t)kptr);
    s.vptr = ((uint64_t)uniform((uint32_t)(vptr >> 32)) << 32) | uniform((uint32_t)vptr);
    s.kstep = uniform((uint32_t)(64 * a.k_ss * (int64_t)sizeof(T)));
    s.vstep = uniform((uint32_t)(64 * a.v_ss * (int64_t)sizeof(T)));
    s.jhi = uniform((uint32_t)j_hi);
    // under the causal mask the wave's 64 rows end with the 64 keys of tile wq0 / 64, if the keys reach that far
    const int jdiag = wq0 / 64;
    s.jlast = uniform((uint32_t)(causal ? min(jdiag, j_hi) : j_hi));
    s.lastedge = uniform(causal && jdiag <= j_hi ? 1u : 0u);
    s.scale = a.scale_log2e;
    const u32x4 kvoff = {kdma.voff[0], kdma.voff[1], kdma.voff[2], kdma.voff[3]};
    const u32x4 vvoff = {vdma.voff[0], vdma.voff[1], vdma.voff[2], vdma.voff[3]};
    Dq64Asm<T>::run(s, acc0, acc1, acc2, acc3, qa, qb, doa, dob, koff, toff, nlq[0], nlq[1], dl[0], dl[1], kvoff, vvoff,
                    wq0 + l32 - 4 * g, wq0 + 32 + l32 - 4 * g);
  }

  // ---- epilogue: dQ = scale * dQ^T, transposed through the wave's own LDS region so that the stores are whole rows ----
  const float dq_scale = a.scale * a.p_unshift;
  T* dqp = (T*)a.dq + b * a.q_sb + h * a.q_sh;
  constexpr int OPITCH = C::DB * 64 + 16;
  ACCT_LDS char* obuf = smem + wave * (32 * OPITCH);
#pragma unroll
  for (int gq = 0; gq < 2; gq++) {
#pragma unroll
    for (int db = 0; db < 4; db++) {
      const f32x32& src = gq == 0 ? (db < 2 ? acc0 : acc1) : (db < 2 ? acc2 : acc3);
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        const int i0 = 16 * (db & 1) + 4 * r4;
        typename E::V2 t0 = E::cvt2(src[i0 + 0] * dq_scale, src[i0 + 1] * dq_scale);
        typename E::V2 t1 = E::cvt2(src[i0 + 2] * dq_scale, src[i0 + 3] * dq_scale);
        typename E::V4 ov = {t0[0], t0[1], t1[0], t1[1]};
        *reinterpret_cast<ACCT_LDS typename E::V4*>(obuf + l32 * OPITCH + (32 * db + 8 * r4 + 4 * g) * 2) = ov;
      }
    }
#pragma unroll
    for (int i = 0; i < 32 * 16 / 64; i++) {
      const int idx = lane + 64 * i, r = idx >> 4, ch = idx & 15;
      const u32x4 v = *reinterpret_cast<const ACCT_LDS u32x4*>(obuf + r * OPITCH + ch * 16);
      *reinterpret_cast<u32x4*>(dqp + (int64_t)(wq0 + 32 * gq + r) * a.q_ss + ch * 8) = v;
    }
  }
}

bool dq64_applicable(const FaArgs& a) {
  const bool no_side = !a.alibi && !a.droprow && !a.dropcol && (a.mask_kind == kMaskNone || a.mask_kind == kMaskCausal);
  const bool band_open = a.prev_blk >= a.Tr && (a.mask_kind == kMaskCausal || a.next_blk >= a.Tc);
  // (the loop advances its tile addresses by 32-bit byte steps)
  const bool steps_fit = a.k_ss < (1 << 23) && a.v_ss < (1 << 23);
  return no_side && band_open && steps_fit && a.hd == 128 && a.row_prefix == 0 && a.Sq % 256 == 0 && a.Sk % 64 == 0;
}

hipError_t launch_bwd_dq64(FaArgs a, int dtype, hipStream_t st) {
  constexpr size_t smem = 6 * 64 * 256;               // three K/V tile pairs (the epilogue's transposition fits inside)
  a.n_tiles = a.Sq / 256;
  const dim3 grid((unsigned)((long long)a.n_tiles * a.B * a.N));
  hipError_t e;
  if (dtype == 0) {
    e = allow_dynamic_lds((const void*)fa_bwd_dq64_kernel<f16>, smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(fa_bwd_dq64_kernel<f16>, grid, dim3(256), smem, st, a);
  } else {
    e = allow_dynamic_lds((const void*)fa_bwd_dq64_kernel<bf16>, smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(fa_bwd_dq64_kernel<bf16>, grid, dim3(256), smem, st, a);
  }
  return hipGetLastError();
}

}  // namespace acct
