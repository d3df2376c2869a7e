// C ABI of the gfx950 attention kernels: argument validation, workspace
// carving, kernel selection.  Declared in include/acct_fa.h.
#include <hip/hip_runtime.h>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/acct_fa.h"
#include "fa_common.hpp"
#include "fa_launch.hpp"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Scratch memory of acct_fa_bwd_static: one copy per GPU the library runs on, held until the process ends.
// In host code the array's name is only a stand-in: its address on a device comes from
// hipGetSymbolAddress (static_scratch() below) and nothing else may be passed to a kernel.
static __device__ __align__(256) unsigned char g_static_scratch[ACCT_FA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<int> g_dev_state[kMaxDevices];   // 0 unknown, 1 gfx950, 2 other
std::atomic<int> g_dev_cus[kMaxDevices];

int check_device(int* n_cu) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(ACCT_E_ARCH, "no HIP device is current");
  if (dev < 0 || dev >= kMaxDevices) return fail(ACCT_E_ARCH, "device ordinal %d out of range", dev);
  int st = g_dev_state[dev].load(std::memory_order_acquire);
  if (st == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return fail(ACCT_E_ARCH, "hipGetDeviceProperties failed");
    g_dev_cus[dev].store(prop.multiProcessorCount, std::memory_order_relaxed);
    st = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
    g_dev_state[dev].store(st, std::memory_order_release);
  }
  if (st != 1) return fail(ACCT_E_ARCH, "device %d is not gfx950; this library carries gfx950 code only", dev);
  *n_cu = g_dev_cus[dev].load(std::memory_order_relaxed);
  return ACCT_OK;
}

std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of the current device's copy of g_static_scratch (looked up once per device, with that device current).
int static_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(ACCT_E_ARCH, "no HIP device is current");
  if (dev < 0 || dev >= kMaxDevices) return fail(ACCT_E_ARCH, "device ordinal %d out of range", dev);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess || !ptr) return fail(ACCT_E_LAUNCH, "hipGetSymbolAddress(static scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return ACCT_OK;
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// [B, N, S, D] rows of 2-byte floating-point elements -> float32, both sides with the same element strides
// (grad_f32: the gradients in the reference's registered output type)
template <typename T>
__global__ void __launch_bounds__(256) cast_rows_to_f32_kernel(const T* src, float* dst, int N, int S, int D8, int64_t sb, int64_t sh,
                                                              int64_t ss, long long chunks) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= chunks) return;
  const int c = (int)(idx % D8);
  const long long row = idx / D8;
  const int s_ = (int)(row % S), h = (int)((row / S) % N);
  const long long b = row / ((long long)S * N);
  const int64_t off = b * sb + h * sh + (int64_t)s_ * ss + 8 * c;
  typedef T t8 __attribute__((ext_vector_type(8)));
  const t8 v = *reinterpret_cast<const t8*>(src + off);
  acct::f32x4 lo = {(float)v[0], (float)v[1], (float)v[2], (float)v[3]}, hi = {(float)v[4], (float)v[5], (float)v[6], (float)v[7]};
  *reinterpret_cast<acct::f32x4*>(dst + off) = lo;
  *reinterpret_cast<acct::f32x4*>(dst + off + 4) = hi;
}

hipError_t cast_rows_to_f32(const void* src, float* dst, int dtype, int B, int N, int S, int D, int64_t sb, int64_t sh, int64_t ss, hipStream_t st) {
  const long long chunks = (long long)B * N * S * (D / 8);
  const unsigned grid = (unsigned)((chunks + 255) / 256);
  if (dtype == ACCT_F16)
    hipLaunchKernelGGL(cast_rows_to_f32_kernel<acct::f16>, dim3(grid), dim3(256), 0, st, (const acct::f16*)src, dst, N, S, D / 8, sb, sh, ss, chunks);
  else
    hipLaunchKernelGGL(cast_rows_to_f32_kernel<acct::bf16>, dim3(grid), dim3(256), 0, st, (const acct::bf16*)src, dst, N, S, D / 8, sb, sh, ss, chunks);
  return hipGetLastError();
}

// elements between the first and one past the last element of a [B, N, S, D] tensor with these strides
size_t span_elems(const int64_t st[3], int B, int N, int S, int D) {
  if (st[0] == 0 && st[1] == 0 && st[2] == 0) return (size_t)B * N * S * D;
  return (size_t)((B - 1) * st[0] + (N - 1) * st[1] + (S - 1) * st[2] + D);
}
// grad_f32: room for dQ, dK, dV in p->dtype, laid out like q, k, v
size_t grad_tmp_bytes(const acct_fa_params* p, int which) {
  if (!p->grad_f32) return 0;
  const int64_t* st = which == 0 ? p->q_stride : (which == 1 ? p->k_stride : p->v_stride);
  return align_up(span_elems(st, p->B, p->N, which == 0 ? p->Sq : p->Sk, p->D) * 2, 256);
}

bool strides_zero(const int64_t s[3]) { return s[0] == 0 && s[1] == 0 && s[2] == 0; }

bool mask_is_dense(const acct_fa_params* p) { return p->mask_kind == ACCT_MASK_DENSE_U8 || p->mask_kind == ACCT_MASK_DENSE_F16; }
bool mask_is_tile(const acct_fa_params* p) { return p->mask_kind == ACCT_MASK_TILE_U8 || p->mask_kind == ACCT_MASK_TILE_F16; }
int mask_elem_size(const acct_fa_params* p) { return (p->mask_kind == ACCT_MASK_DENSE_F16 || p->mask_kind == ACCT_MASK_TILE_F16) ? 2 : 1; }

// counter-based dropout is on: the keep mask comes from (drop_seed, drop_offset), not from a tensor
bool philox_on(const acct_fa_params* p) { return p->drop_philox != 0 && !p->drop_mask && p->keep_prob < 1.f; }
bool dropout_on(const acct_fa_params* p) { return p->drop_mask != nullptr || philox_on(p); }
uint32_t philox_threshold(float keep_prob) {
  long t = lroundf(256.f * keep_prob);
  return (uint32_t)(t < 1 ? 1 : t > 256 ? 256 : t);
}

// Checks that need no device: used by the entry points and by the workspace queries.
int validate(const acct_fa_params* p, bool backward) {
  if (!p) return fail(ACCT_E_NULLPTR, "params is NULL");
  if (p->dtype != ACCT_F16 && p->dtype != ACCT_BF16) return fail(ACCT_E_DTYPE, "dtype %d is neither ACCT_F16 nor ACCT_BF16", p->dtype);
  if (p->B <= 0 || p->N <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->D <= 0)
    return fail(ACCT_E_SHAPE, "extents must be positive: B=%d N=%d Sq=%d Sk=%d D=%d", p->B, p->N, p->Sq, p->Sk, p->D);
  {
    // grid sizes and (batch*head, tile) indices are 32-bit in the kernels
    const int64_t smax = p->Sq > p->Sk ? p->Sq : p->Sk;
    if ((int64_t)p->B * p->N > 0x7fffffff || (int64_t)p->B * p->N * ((smax + 31) / 32) > 0x7fffffff)
      return fail(ACCT_E_SHAPE, "B*N*ceil(S/32) must stay below 2^31: B=%d N=%d Sq=%d Sk=%d", p->B, p->N, p->Sq, p->Sk);
  }
  if (p->D > 256) return fail(ACCT_E_HEADDIM, "head_dim too large, reduce head_dim and try again. (D=%d > 256)", p->D);
  if (p->D % 8 != 0) return fail(ACCT_E_HEADDIM, "head_dim %d is not a multiple of 8", p->D);
  (void)backward;
  // bias variants are built for the head-dim classes 64, 80 and 128 (dropout: every head dim)
  if ((p->D == 40 || p->D > 128) && p->alibi)
    return fail(ACCT_E_HEADDIM, "head_dim %d is built without the bias variants", p->D);
  if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return fail(ACCT_E_PARAM, "scale must be positive and finite, got %g", (double)p->scale);
  if (!(p->keep_prob > 0.f && p->keep_prob <= 1.f)) return fail(ACCT_E_PARAM, "keep_prob must be in (0, 1], got %g", (double)p->keep_prob);
  if (p->prev_block_num < 0 || p->next_block_num < 0) return fail(ACCT_E_PARAM, "prev_block_num / next_block_num must be >= 0");
  if (p->row_block_prefix < 0 || p->row_block_prefix % 128 != 0) return fail(ACCT_E_PARAM, "row_block_prefix must be 0 or a positive multiple of 128, got %d", p->row_block_prefix);
  switch (p->mask_kind) {
    case ACCT_MASK_NONE: case ACCT_MASK_CAUSAL: break;
    case ACCT_MASK_DENSE_U8: case ACCT_MASK_TILE_U8: case ACCT_MASK_DENSE_F16: case ACCT_MASK_TILE_F16:
      if (!p->attn_mask) return fail(ACCT_E_NULLPTR, "attn_mask is NULL but mask_kind=%d needs a tensor", p->mask_kind);
      break;
    default: return fail(ACCT_E_PARAM, "unknown mask_kind %d", p->mask_kind);
  }
  if (p->mask_stride_b < 0 || (mask_is_dense(p) && p->mask_stride_b != 0 && p->mask_stride_b < (int64_t)p->Sq * p->Sk))
    return fail(ACCT_E_SHAPE, "mask_stride_b must be 0 (broadcast) or >= Sq*Sk");
  if (mask_elem_size(p) == 2 && ((uintptr_t)p->attn_mask & 1)) return fail(ACCT_E_SHAPE, "a 2-byte attn_mask must be 2-byte aligned");
  if (p->drop_mask_kind != ACCT_DROP_U8 && p->drop_mask_kind != ACCT_DROP_F16) return fail(ACCT_E_PARAM, "unknown drop_mask_kind %d", p->drop_mask_kind);
  if (p->drop_mask && p->drop_mask_kind == ACCT_DROP_F16 && ((uintptr_t)p->drop_mask & 1)) return fail(ACCT_E_SHAPE, "a 2-byte drop_mask must be 2-byte aligned");
  if (!p->q || !p->k || !p->v) return fail(ACCT_E_NULLPTR, "q, k and v must be non-NULL");
  const int64_t* st[4] = {p->q_stride, p->k_stride, p->v_stride, p->o_stride};
  const void* ptrs[3] = {p->q, p->k, p->v};
  for (int i = 0; i < 4; i++) {
    if (strides_zero(st[i])) continue;
    for (int j = 0; j < 3; j++)
      if (st[i][j] < 0 || st[i][j] % 8 != 0) return fail(ACCT_E_SHAPE, "strides must be non-negative multiples of 8 elements");
    if (st[i][2] < p->D) return fail(ACCT_E_SHAPE, "row stride smaller than D");
  }
  for (int i = 0; i < 3; i++)
    if ((uintptr_t)ptrs[i] & 15) return fail(ACCT_E_SHAPE, "q, k and v must be 16-byte aligned");
  if (p->alibi && (p->alibi_stride_b < 0 || p->alibi_stride_h < 0 || p->alibi_stride_q < 0))
    return fail(ACCT_E_SHAPE, "alibi strides must be >= 0");
  if ((uintptr_t)p->drop_bits & 255) return fail(ACCT_E_WORKSPACE, "drop_bits must be 256-byte aligned");
  if ((uintptr_t)p->mask_bits & 255) return fail(ACCT_E_WORKSPACE, "mask_bits must be 256-byte aligned");
  return ACCT_OK;
}

void fill_strides(const int64_t s[3], int N, int S, int D, int64_t* sb, int64_t* sh, int64_t* ss) {
  if (strides_zero(s)) { *ss = D; *sh = (int64_t)S * D; *sb = (int64_t)N * S * D; }
  else { *sb = s[0]; *sh = s[1]; *ss = s[2]; }
}

acct::FaArgs make_args(const acct_fa_params* p) {
  acct::FaArgs a;
  memset(&a, 0, sizeof(a));
  a.q = p->q; a.k = p->k; a.v = p->v;
  a.mask = (mask_is_dense(p) || mask_is_tile(p)) ? (const uint8_t*)p->attn_mask : nullptr;
  a.mask_es = mask_elem_size(p);
  a.drop = p->keep_prob < 1.f || p->drop_mask ? (const uint8_t*)p->drop_mask : nullptr;
  a.drop_es = p->drop_mask_kind == ACCT_DROP_F16 ? 2 : 1;
  a.alibi = p->alibi;
  a.B = p->B; a.N = p->N; a.Sq = p->Sq; a.Sk = p->Sk;
  a.hd = p->D;
  a.Tr = (p->Sq + 127) / 128; a.Tc = (p->Sk + 127) / 128;
  fill_strides(p->q_stride, p->N, p->Sq, p->D, &a.q_sb, &a.q_sh, &a.q_ss);
  fill_strides(p->k_stride, p->N, p->Sk, p->D, &a.k_sb, &a.k_sh, &a.k_ss);
  fill_strides(p->v_stride, p->N, p->Sk, p->D, &a.v_sb, &a.v_sh, &a.v_ss);
  fill_strides(p->o_stride, p->N, p->Sq, p->D, &a.o_sb, &a.o_sh, &a.o_ss);
  a.mask_sb = mask_is_dense(p) ? p->mask_stride_b : 0;
  a.al_sb = p->alibi_stride_b; a.al_sh = p->alibi_stride_h; a.al_sq = p->alibi_stride_q;
  a.scale = p->scale;
  a.scale_log2e = p->scale * acct::kLog2e;
  a.inv_keep = 1.0f / p->keep_prob;
  if (philox_on(p)) {
    a.philox_k0 = (uint32_t)p->drop_seed;
    a.philox_k1 = (uint32_t)(p->drop_seed >> 32);
    a.philox_offset = p->drop_offset;
    a.philox_thr = philox_threshold(p->keep_prob);
    a.inv_keep = 256.0f / (float)a.philox_thr;          // the reciprocal of the keep probability actually used
  }
  a.inv_scale = 1.0f / p->scale;
  {
    // 2^p_shift grows with the key count (average probability 1 / Sk): none up to 4096 keys, where P and
    // dS = P (dP - D) sit in fp16's normal range by themselves and the overflow bound of dS is the reference's
    // own (|dS| < 65504, its dS is fp16 too, flash_attention_bwd.py:161-181); one power of two per doubling of
    // Sk after that, up to 2^8.  With a shift the bound is 65504 / 2^p_shift.  bf16 runs keep the shift: the
    // P handed from the V-role to the K-role wave of the dK/dV kernel is fp16 in both cases.
    int lg = 0;
    while ((2 << lg) <= p->Sk) lg++;
    const int sh = lg - 12 < 0 ? 0 : (lg - 12 > 8 ? 8 : lg - 12);
    a.p_shift = (float)sh;
    a.p_unshift = 1.0f / (float)(1 << sh);
  }
  a.mask_add_raw = acct::kMaskFill / p->scale;
  a.prev_blk = p->prev_block_num > ACCT_BLOCK_UNBOUNDED ? ACCT_BLOCK_UNBOUNDED : p->prev_block_num;
  a.next_blk = p->next_block_num > ACCT_BLOCK_UNBOUNDED ? ACCT_BLOCK_UNBOUNDED : p->next_block_num;
  // the kernels know one dense and one tile kind; the element size travels beside it
  a.mask_kind = mask_is_dense(p) ? (int)acct::kMaskDense : (mask_is_tile(p) ? (int)acct::kMaskTile : p->mask_kind);
  a.row_prefix = p->row_block_prefix;
  return a;
}

// block classes of a dense mask, one byte per 128x128 block, followed by the key-tail table of the same size
size_t class_count(const acct_fa_params* p) {
  const size_t MB = p->mask_stride_b ? p->B : 1;
  return MB * (size_t)((p->Sq + 127) / 128) * (size_t)((p->Sk + 127) / 128);
}
size_t flag_bytes(const acct_fa_params* p) {
  if (!mask_is_dense(p)) return 0;
  return align_up(2 * class_count(p), 256);
}

// per-key-column bitmaps of the mixed blocks of a dense mask (backward only): 16 bytes per (q block, key)
size_t colbit_bytes(const acct_fa_params* p) {
  if (mask_is_tile(p)) return 128 * 16;
  if (!mask_is_dense(p)) return 0;
  const size_t MB = p->mask_stride_b ? p->B : 1;
  return align_up(MB * (size_t)((p->Sq + 127) / 128) * (size_t)p->Sk * 16, 256);
}

// keep bits of the dropout mask: by query row (forward, dQ) and by key column (dK/dV)
size_t droprow_words(const acct_fa_params* p) { return 2 * (size_t)((p->Sk + 63) / 64); }   // 32-bit words per row
size_t droprow_bytes(const acct_fa_params* p) {
  if (!dropout_on(p)) return 0;
  return align_up((size_t)p->B * p->N * p->Sq * droprow_words(p) * 4, 256);
}
size_t dropcol_bytes(const acct_fa_params* p) {
  if (!dropout_on(p)) return 0;
  return align_up((size_t)p->B * p->N * (size_t)((p->Sq + 127) / 128) * (size_t)p->Sk * 16, 256);
}

// Pre-passes over the attention mask: block classes of a dense mask (all three kernels) and the mask packed by
// key column (dK/dV kernel; also for the compact tile).  They run into `own` (a workspace region of
// flag_bytes + colbit_bytes) or, when the caller lends a mask_bits buffer, once into that buffer: the call that
// finds it unfilled runs BOTH pre-passes, whichever kernels it launches itself, so that the later calls of the
// step only read.
int mask_prepass(acct::FaArgs& a, const acct_fa_params* p, uint8_t* own, bool want_cols, hipStream_t st) {
  if (!mask_is_dense(p) && !mask_is_tile(p)) return ACCT_OK;
  uint8_t* base = p->mask_bits ? (uint8_t*)p->mask_bits : own;
  uint8_t* flags = base;                                            // (no classes for the tile kind: flag_bytes = 0)
  uint32_t* cbits = (uint32_t*)(base + flag_bytes(p));
  const bool filled = p->mask_bits && p->mask_bits_filled;
  const bool cols = p->mask_bits ? true : want_cols;
  if (mask_is_dense(p)) {
    a.blkflags = flags;
    // (only the one-launch pre-pass writes the key tails; which path runs follows from the arguments alone, so every
    // call of a step that shares a mask_bits buffer decides alike)
    a.blktail = acct::mask_prepass_is_fused(a) ? flags + class_count(p) : nullptr;
  }
  if (cols) a.colbits = cbits;
  if (filled) return ACCT_OK;
  hipError_t e = mask_is_dense(p) ? acct::launch_mask_blocks(a, flags, cols ? cbits : nullptr, p->mask_stride_b ? p->B : 1, st)
                                  : (cols ? acct::launch_mask_colbits(a, flags, cbits, 1, st) : hipSuccess);
  if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "mask pre-pass kernel: %s", hipGetErrorString(e));
  return ACCT_OK;
}

}  // namespace

extern "C" {

const char* acct_last_error(void) { return g_err; }
int acct_version(void) { return ACCT_FA_VERSION; }
int acct_build_is_complete(void) { return acct::launch_variants_complete() ? 1 : 0; }

size_t acct_fa_fwd_workspace_bytes(const acct_fa_params* p) {
  if (!p || p->B <= 0 || p->N <= 0 || p->Sq <= 0 || p->Sk <= 0) return 0;
  return (p->mask_bits ? 0 : flag_bytes(p)) + (p->drop_bits ? 0 : droprow_bytes(p));
}

size_t acct_fa_mask_bits_bytes(const acct_fa_params* p) {
  if (!p || p->B <= 0 || p->N <= 0 || p->Sq <= 0 || p->Sk <= 0) return 0;
  return flag_bytes(p) + colbit_bytes(p);
}

size_t acct_fa_drop_bits_bytes(const acct_fa_params* p) {
  if (!p || p->B <= 0 || p->N <= 0 || p->Sq <= 0 || p->Sk <= 0) return 0;
  return droprow_bytes(p) + dropcol_bytes(p);
}

// what the backward cannot do without: D and the exp2 offsets, the mask classes and bitmaps, the keep bits
static size_t bwd_min_workspace_bytes(const acct_fa_params* p) {
  return 2 * align_up((size_t)p->B * p->N * p->Sq * sizeof(float), 256) + (p->mask_bits ? 0 : flag_bytes(p) + colbit_bytes(p)) +
         (p->drop_bits ? 0 : droprow_bytes(p) + dropcol_bytes(p)) + grad_tmp_bytes(p, 0) + grad_tmp_bytes(p, 1) + grad_tmp_bytes(p, 2);
}

size_t acct_fa_bwd_workspace_bytes(const acct_fa_params* p) {
  if (!p || p->B <= 0 || p->N <= 0 || p->Sq <= 0) return 0;
  if (p->Sk <= 0 || p->D <= 0) return 0;
  // plus room for the per-slice sums of a dK/dV launch that splits the query range (few heads, short key
  // sequence); a caller that passes less gets the unsplit launch
  return align_up(bwd_min_workspace_bytes(p), 256) + acct::dkdv_split(p->B, p->N, p->Sq, p->Sk, p->D).part_bytes;
}

int acct_fa_fwd(const acct_fa_params* p, void* O, float* LSE, void* workspace, size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  int rc = validate(p, false);
  if (rc) return rc;
  if (!O || !LSE) return fail(ACCT_E_NULLPTR, "O and LSE must be non-NULL");
  if ((uintptr_t)O & 15) return fail(ACCT_E_SHAPE, "O must be 16-byte aligned");
  if (p->keep_prob < 1.f && !dropout_on(p)) return fail(ACCT_E_NULLPTR, "keep_prob < 1 needs a drop_mask or drop_philox");
  const size_t need = acct_fa_fwd_workspace_bytes(p);
  if (need && (!workspace || workspace_bytes < need))
    return fail(ACCT_E_WORKSPACE, "forward workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
  if (need && ((uintptr_t)workspace & 255)) return fail(ACCT_E_WORKSPACE, "workspace must be 256-byte aligned");
  int n_cu = 0;
  rc = check_device(&n_cu);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  acct::FaArgs a = make_args(p);
  a.o = O; a.lse = LSE;
  {
    rc = mask_prepass(a, p, (uint8_t*)workspace, /*want_cols=*/false, st);
    if (rc) return rc;
  }
  if (dropout_on(p)) {
    // own bits by query row in the workspace, or both layouts in the caller's buffer for the backward call
    uint32_t* rows = p->drop_bits ? (uint32_t*)p->drop_bits : (uint32_t*)((char*)workspace + (p->mask_bits ? 0 : flag_bytes(p)));
    uint32_t* cols = p->drop_bits ? (uint32_t*)((char*)p->drop_bits + droprow_bytes(p)) : nullptr;
    a.droprow = rows;
    a.droprow_w = (int)droprow_words(p);
    if (!(p->drop_bits && p->drop_bits_filled)) {
      hipError_t e = philox_on(p) ? acct::launch_drop_philox(a, rows, cols, st) : acct::launch_drop_bits(a, rows, cols, st);
      if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "dropout bitmap kernel: %s", hipGetErrorString(e));
    }
  }
  // 8 waves x 32 query rows (two waves per SIMD overlap MFMA and softmax work) once that still
  // fills the chip, else 4 waves x 32 rows for more workgroups
  int qg = ((long long)p->B * p->N * ((p->Sq + 255) / 256) >= n_cu) ? 3 : 1;
  hipError_t e = acct::launch_fwd(a, p->dtype, p->D, qg, st);
  if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "forward kernel: %s", hipGetErrorString(e));
  return ACCT_OK;
}

static int bwd_impl(const acct_fa_params* p, const void* O, const void* dO, const float* LSE, void* dQ, void* dK, void* dV,
                    void* workspace, size_t workspace_bytes, void* stream, int stages) {
  g_err[0] = 0;
  int rc = validate(p, true);
  if (rc) return rc;
  const bool want_dq = stages & acct::kStageDq, want_dkdv = stages & acct::kStageDkDv;
  if (!O || !dO || !LSE || (want_dq && !dQ) || (want_dkdv && (!dK || !dV)))
    return fail(ACCT_E_NULLPTR, "O, dO, LSE and the requested gradients must be non-NULL");
  if (((uintptr_t)O | (uintptr_t)dO | (uintptr_t)dQ | (uintptr_t)dK | (uintptr_t)dV) & 15)
    return fail(ACCT_E_SHAPE, "O, dO, dQ, dK and dV must be 16-byte aligned");
  if (p->keep_prob < 1.f && !dropout_on(p)) return fail(ACCT_E_NULLPTR, "keep_prob < 1 needs a drop_mask or drop_philox");
  const size_t need = bwd_min_workspace_bytes(p);
  if (!workspace || workspace_bytes < need)
    return fail(ACCT_E_WORKSPACE, "backward workspace too small: need %zu bytes (%zu to let the dK/dV kernel split the query range), got %zu",
                need, acct_fa_bwd_workspace_bytes(p), workspace_bytes);
  if ((uintptr_t)workspace & 255) return fail(ACCT_E_WORKSPACE, "workspace must be 256-byte aligned");
  int n_cu = 0;
  rc = check_device(&n_cu);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  acct::FaArgs a = make_args(p);
  a.o = const_cast<void*>(O); a.lse = const_cast<float*>(LSE);
  a.dout = dO; a.dq = dQ; a.dk = dK; a.dv = dV;
  const size_t stat_bytes = align_up((size_t)p->B * p->N * p->Sq * sizeof(float), 256);
  a.delta = (float*)workspace;
  a.nlse = (float*)((char*)workspace + stat_bytes);
  {
    // (without a caller-held mask_bits buffer the dkdv-only call re-derives the classes as well: the mask may
    // have been edited since)
    rc = mask_prepass(a, p, (uint8_t*)workspace + 2 * stat_bytes, want_dkdv, st);
    if (rc) return rc;
  }
  if (dropout_on(p)) {
    char* base = p->drop_bits ? (char*)p->drop_bits : (char*)workspace + 2 * stat_bytes + (p->mask_bits ? 0 : flag_bytes(p) + colbit_bytes(p));
    uint32_t* rows = (uint32_t*)base;
    uint32_t* cols = (uint32_t*)(base + droprow_bytes(p));
    a.droprow = rows;
    a.dropcol = cols;
    a.droprow_w = (int)droprow_words(p);
    if (p->drop_bits && p->drop_bits_filled) {
      // an earlier call of this step left both layouts in the caller's buffer
    } else if (p->drop_bits) {
      // the caller's buffer is filled completely, whichever half of the backward asked
      hipError_t e = philox_on(p) ? acct::launch_drop_philox(a, rows, cols, st) : acct::launch_drop_bits(a, rows, cols, st);
      if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "dropout bitmap kernel: %s", hipGetErrorString(e));
    } else {
      hipError_t e = philox_on(p) ? acct::launch_drop_philox(a, want_dq ? rows : nullptr, want_dkdv ? cols : nullptr, st)
                                  : acct::launch_drop_bits(a, want_dq ? rows : nullptr, want_dkdv ? cols : nullptr, st);
      if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "dropout bitmap kernel: %s", hipGetErrorString(e));
    }
  }
  void* out_f32[3] = {dQ, dK, dV};
  if (p->grad_f32) {
    if (stages != (acct::kStageDq | acct::kStageDkDv)) return fail(ACCT_E_PARAM, "grad_f32 needs the fused acct_fa_bwd call");
    if (((uintptr_t)dQ | (uintptr_t)dK | (uintptr_t)dV) & 15) return fail(ACCT_E_SHAPE, "dQ, dK and dV must be 16-byte aligned");
    // the kernels write p->dtype tensors into the tail of the workspace; a conversion pass fills the caller's
    char* tmp = (char*)workspace + need - grad_tmp_bytes(p, 0) - grad_tmp_bytes(p, 1) - grad_tmp_bytes(p, 2);
    a.dq = tmp;
    a.dk = tmp + grad_tmp_bytes(p, 0);
    a.dv = tmp + grad_tmp_bytes(p, 0) + grad_tmp_bytes(p, 1);
  }
  a.q_split = 1;
  if (want_dkdv) {
    const acct::DkdvSplit sp = acct::dkdv_split(p->B, p->N, p->Sq, p->Sk, p->D, n_cu);
    const size_t part_at = align_up(need, 256);
    if (sp.q_split > 1 && workspace_bytes >= part_at + sp.part_bytes) {
      a.q_split = sp.q_split;
      a.dkdv_part = (float*)((char*)workspace + part_at);
    }
  }
  hipError_t e = acct::launch_bwd(a, p->dtype, p->D, stages, st);
  if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "backward kernels: %s", hipGetErrorString(e));
  if (p->grad_f32) {
    e = cast_rows_to_f32(a.dq, (float*)out_f32[0], p->dtype, p->B, p->N, p->Sq, p->D, a.q_sb, a.q_sh, a.q_ss, st);
    if (e == hipSuccess) e = cast_rows_to_f32(a.dk, (float*)out_f32[1], p->dtype, p->B, p->N, p->Sk, p->D, a.k_sb, a.k_sh, a.k_ss, st);
    if (e == hipSuccess) e = cast_rows_to_f32(a.dv, (float*)out_f32[2], p->dtype, p->B, p->N, p->Sk, p->D, a.v_sb, a.v_sh, a.v_ss, st);
    if (e != hipSuccess) return fail(ACCT_E_LAUNCH, "gradient conversion kernel: %s", hipGetErrorString(e));
  }
  return ACCT_OK;
}

int acct_fa_bwd(const acct_fa_params* p, const void* O, const void* dO, const float* LSE, void* dQ, void* dK, void* dV,
                void* workspace, size_t workspace_bytes, void* stream) {
  return bwd_impl(p, O, dO, LSE, dQ, dK, dV, workspace, workspace_bytes, stream, acct::kStageDq | acct::kStageDkDv);
}

int acct_fa_bwd_static(const acct_fa_params* p, const void* O, const void* dO, const float* LSE, void* dQ, void* dK, void* dV,
                       void* stream) {
  g_err[0] = 0;
  int rc = validate(p, true);
  if (rc) return rc;
  if (p->grad_f32) return fail(ACCT_E_PARAM, "acct_fa_bwd_static does not take grad_f32");
  const size_t need = bwd_min_workspace_bytes(p);
  if (need > (size_t)ACCT_FA_STATIC_SCRATCH_BYTES)
    return fail(ACCT_E_WORKSPACE, "acct_fa_bwd_static: this problem needs %zu bytes of scratch, the built-in buffer holds %zu; "
                "use acct_fa_bwd with a caller-owned workspace", need, (size_t)ACCT_FA_STATIC_SCRATCH_BYTES);
  void* scratch = nullptr;
  rc = static_scratch(&scratch);
  if (rc) return rc;
  return bwd_impl(p, O, dO, LSE, dQ, dK, dV, scratch, (size_t)ACCT_FA_STATIC_SCRATCH_BYTES, stream, acct::kStageDq | acct::kStageDkDv);
}

int acct_fa_bwd_dq(const acct_fa_params* p, const void* O, const void* dO, const float* LSE, void* dQ,
                   void* workspace, size_t workspace_bytes, void* stream) {
  return bwd_impl(p, O, dO, LSE, dQ, nullptr, nullptr, workspace, workspace_bytes, stream, acct::kStageDq);
}

int acct_fa_bwd_dkdv(const acct_fa_params* p, const void* O, const void* dO, const float* LSE, void* dK, void* dV,
                     void* workspace, size_t workspace_bytes, void* stream) {
  return bwd_impl(p, O, dO, LSE, nullptr, dK, dV, workspace, workspace_bytes, stream, acct::kStageDkDv);
}

// Shape function of the inference operator.  Limits and accept / reject behaviour follow
// infer/flash_attention/tik/op_proto/flash_attention_tik.cpp:20-193 of the reference.
int acct_fa_infer_shape(const int64_t* q_dims, int q_rank, const int64_t* k_dims, int k_rank,
                        const int64_t* v_dims, int v_rank, int64_t* y_dims) {
  g_err[0] = 0;
  if (!q_dims || !k_dims || !v_dims) return fail(ACCT_E_NULLPTR, "q_dims, k_dims and v_dims must be non-NULL");
  if (q_rank != 3 && q_rank != 4) return fail(ACCT_E_SHAPE, "q must have 3 or 4 dimensions, got %d", q_rank);
  if (k_rank != q_rank || v_rank != q_rank) return fail(ACCT_E_SHAPE, "k and v must have q's number of dimensions");
  auto in_range = [](int64_t x, int64_t lo, int64_t hi) { return x >= lo && x <= hi; };
  auto same = [&](int i) { return k_dims[i] == q_dims[i] && v_dims[i] == q_dims[i]; };
  const int s = q_rank - 2;                                          // position of the sequence length
  if (q_rank == 3) {
    if (!in_range(q_dims[0], 1, 64) || !same(0)) return fail(ACCT_E_SHAPE, "batch*heads must be 1..64 and equal for q, k, v");
  } else {
    if (!in_range(q_dims[0], 1, 64) || !same(0)) return fail(ACCT_E_SHAPE, "batch must be 1..64 and equal for q, k, v");
    if (!in_range(q_dims[1], 1, 4096) || !same(1)) return fail(ACCT_E_SHAPE, "heads must be 1..4096 and equal for q, k, v");
  }
  if (!in_range(q_dims[s], 1, 8192) || !in_range(k_dims[s], 1, 8192) || v_dims[s] != k_dims[s])
    return fail(ACCT_E_SHAPE, "sequence lengths must be 1..8192 and equal for k and v");
  const int64_t d = q_dims[s + 1];
  if (q_rank == 3) {
    // the reference checks the last dimension of a 3-D input with its batch*heads rule (1..64 and equal),
    // op_proto/flash_attention_tik.cpp:104-112; the kernel builder then wants one of its head dims
    // (tbe/impl/flash_attention_fwd.py:38,104-106).  Both are applied here.
    if (!in_range(d, 1, 64) || !same(2)) return fail(ACCT_E_HEADDIM, "head dim of a 3-D input must be 1..64 and equal for q, k, v");
  }
  if ((d != 40 && d != 64 && d != 80 && d != 160) || !same(s + 1))
    return fail(ACCT_E_HEADDIM, "head dim must be one of 40, 64, 80, 160 and equal for q, k, v");
  if (y_dims)
    for (int i = 0; i < q_rank; i++) y_dims[i] = q_dims[i];
  return ACCT_OK;
}

}  // extern "C"
