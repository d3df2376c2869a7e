/*
 * acct_fa.h -- C ABI of the MI355X (gfx950) FlashAttention2 / TriangleAttention
 * hot path.  Plain pointers and sizes only; every pointer is a DEVICE pointer
 * unless a comment says otherwise; the caller owns every buffer; the library
 * never allocates, never throws, never synchronises: each call enqueues its
 * kernels on `stream` (a hipStream_t passed as void*; NULL = default stream).
 *
 * Citations are file:line in the reference tree (mindspore-ai/acctransformer):
 *   T = train/acctransformer/flash_attention/ops/flash_attention
 *   L = train/acctransformer/flash_attention/nn/layer
 *
 * Operator semantics (identical to the reference kernels, T/flash_attention_fwd.py
 * and T/flash_attention_bwd.py; blocks are 128 rows / 128 columns):
 *
 *   band(i,j) := j/128 - next_block_num <= i/128 <= j/128 + prev_block_num
 *   S[i,j] = scale * sum_d q[i,d] k[j,d] + alibi[b,h,(i|0),j] - 10000 * mask[(b|0),i,j]   for band(i,j)
 *   m = rowmax S;  Pt = exp(S - m);  l = rowsum Pt   (l is taken BEFORE dropout)
 *   LSE = m + ln l
 *   O = (Pt / l) * (drop / keep_prob) * v
 *   backward:  P = exp(S - LSE); Pd = P*drop/keep_prob; dV = Pd^T dO; dP = (dO v^T)*drop/keep_prob
 *              Dl = rowsum(dO*O); dS = P*(dP - Dl); dQ = scale dS k; dK = scale dS^T q
 */
#ifndef ACCT_FA_H_
#define ACCT_FA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ACCT_FA_VERSION 108

/* error codes (0 = success) */
#define ACCT_OK          0
#define ACCT_E_NULLPTR  (-1)   /* a required pointer is NULL */
#define ACCT_E_SHAPE    (-2)   /* non-positive or inconsistent extent / stride */
#define ACCT_E_DTYPE    (-3)   /* dtype is neither ACCT_F16 nor ACCT_BF16 */
#define ACCT_E_HEADDIM  (-4)   /* D unsupported: not a multiple of 8, above 256 (L/flash_attention.py:26,105-106), or 40 / above 128 together
                                  with a bias (kernels are built for 40, 64, 80, 128, 160, 256; other multiples of 8 run
                                  on the next built size; dropout is built for all of them) */
#define ACCT_E_ARCH     (-5)   /* current device is not gfx950 */
#define ACCT_E_LAUNCH   (-6)   /* HIP reported a launch error */
#define ACCT_E_WORKSPACE (-7)  /* workspace missing or too small */
#define ACCT_E_PARAM    (-8)   /* scale <= 0, keep_prob outside (0,1], bad mask_kind ... */

#define ACCT_F16  0
#define ACCT_BF16 1

/* attn_mask interpretation */
#define ACCT_MASK_NONE     0
#define ACCT_MASK_DENSE_U8 1   /* uint8 [1|B, Sq, Sk], nonzero = masked (adds -10000); T/attention.py:357-371 */
#define ACCT_MASK_DENSE_F16 2  /* the same mask in p->dtype (fp16 / bf16), the form the reference op takes
                                  (T/flash_attention_impl.py:43-45, T/attention.py:270-277,357-371): nonzero = masked.
                                  The reference multiplies the mask VALUE by -10000 and only ever feeds 0 / 1. */
#define ACCT_MASK_TILE_U8  3   /* uint8 [128,128] tile applied only where q_blk == kv_blk:
                                  the reference's compact causal mode, T/attention.py:279-285,363-365 */
#define ACCT_MASK_CAUSAL   4   /* no tensor: -10000 added where j > i, evaluated by index compare */
#define ACCT_MASK_TILE_F16 5   /* the compact [128,128] tile in p->dtype (the reference's own form of it) */

/* drop_mask interpretation (drop_mask_kind) */
#define ACCT_DROP_U8  0        /* uint8 [B,N,Sq,Sk] of {0,1}, nonzero = keep */
#define ACCT_DROP_F16 1        /* p->dtype [B,N,Sq,Sk] of {0, 1/keep_prob}, the form the reference op takes
                                  (T/flash_attention_impl.py:48-55, T/attention.py:373-395): nonzero = keep; the
                                  scaling comes from keep_prob, which the caller still passes */

#define ACCT_BLOCK_UNBOUNDED 65536   /* default prev/next_block_num, L/flash_attention.py:95-96 */

/*
 * One description of the problem for forward and backward.  Replaces the
 * tensor-descriptor dicts handed to the reference's kernel builders
 * (T/flash_attention_fwd.py:498-530, T/flash_attention_bwd.py:436-477) and
 * the primitive attrs prev_block_num / next_block_num
 * (T/flash_attention_impl.py:146-148).
 */
typedef struct acct_fa_params {
  int32_t dtype;                 /* ACCT_F16 | ACCT_BF16: type of q,k,v,O,dO,dQ,dK,dV and alibi */
  int32_t B, N, Sq, Sk, D;       /* q [B,N,Sq,D]; k,v [B,N,Sk,D] */
  float   scale;                 /* multiplies q k^T in fp32; 1.0 = the raw reference op, the
                                    layer passes fp16(D^-1/4)^2 (L/flash_attention.py:117,188-189) */
  float   keep_prob;             /* 1.0 = no dropout; P *= drop / keep_prob (T/attention.py:373-395) */
  int32_t prev_block_num;        /* band, in 128-row blocks (T/attention.py:162-167) */
  int32_t next_block_num;        /* 0 = causal block skip */
  int32_t mask_kind;             /* ACCT_MASK_* */
  int32_t row_block_prefix;      /* 0 = off; else a multiple of 128: query row i sees only keys
                                    j < (i / row_block_prefix + 1) * row_block_prefix -- the row-block prefixes of
                                    train/acctransformer/triangle_attention/triangle_attention.py:137-165 */
  int64_t mask_stride_b;         /* elements between batches of attn_mask; 0 = broadcast [1,Sq,Sk] */
  int64_t alibi_stride_b;        /* alibi element strides; stride_q = 0 is the reference's   */
  int64_t alibi_stride_h;        /* [B,N,1,Sk] row-bias form (L/flash_attention.py:185);      */
  int64_t alibi_stride_q;        /* stride_b = 0 / stride_h = 0 broadcast over batch / heads  */
  /* element strides (batch, head, row) of q/dQ, k/dK, v/dV and O/dO; the last
     dimension is contiguous.  All zeros = contiguous BNSD. */
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];
  const void*    q;
  const void*    k;
  const void*    v;
  const void*    attn_mask;      /* per mask_kind, contiguous; NULL when NONE / CAUSAL */
  const void*    drop_mask;      /* per drop_mask_kind, [B,N,Sq,Sk] contiguous; NULL = no dropout */
  const void*    alibi;          /* dtype, see strides; NULL = none (T/attention.py:347-355) */
  /* Counter-based dropout (fields added in version 101): with drop_philox != 0, drop_mask == NULL and
     keep_prob < 1 the keep mask is never materialised by the caller -- the library derives it from
     (drop_seed, drop_offset) with Philox4x32-10, the same way in forward and backward.  It stands in
     for the DropoutGenMask / DropoutDoMask chain of the reference layer (L/flash_attention.py:198-203),
     which draws a [B,N,Sq,Sk] mask per call.  Definition (so that a caller or a test can rebuild the mask):
       key     = (low 32 bits of drop_seed, high 32 bits of drop_seed)
       counter = (i, 2*(j/32) + (j/4)%2, b*N + h, drop_offset)           i = query row, j = key column
       byte    = byte 4*((j/8)%4) + j%4 of the 16 output bytes (word 0 first, little endian)
       keep[b,h,i,j] = byte < T,  T = round(256 * keep_prob) clamped to 1..256
     and kept probabilities are scaled by 256 / T (the reciprocal of the probability actually used).
     Callers advance drop_offset (or change drop_seed) for every call that must draw a fresh mask. */
  uint64_t drop_seed;
  uint32_t drop_offset;
  int32_t  drop_philox;
  /* Keep bits shared between the forward and the backward call of one training step (fields added in
     version 103; no counterpart in the reference, whose two operators each read the byte mask).  Both
     calls need the dropout mask as bit maps, packed from drop_mask or drawn from (drop_seed, drop_offset)
     by a pre-pass.  With drop_bits == NULL every call runs that pre-pass into its own workspace.  With
     drop_bits pointing at acct_fa_drop_bits_bytes(p) bytes of device memory (256-byte aligned) that the
     caller keeps from the forward to the backward call, a call with drop_bits_filled == 0 runs the pre-pass
     into that buffer and a call with drop_bits_filled != 0 reads what an earlier call left there.  The
     caller sets drop_bits_filled after the first call returns; the bits depend on drop_mask or on
     (drop_seed, drop_offset, keep_prob) and on B, N, Sq, Sk; with a dense attn_mask the bits of the 128x128
     blocks that the mask hides completely are left out (no kernel reads them), so the buffer belongs to the
     calls of one step on one attn_mask. */
  void*    drop_bits;
  int32_t  drop_bits_filled;
  int32_t  drop_mask_kind;       /* ACCT_DROP_* (field added in version 104; 0 = the uint8 form) */
  /* What the pre-passes derive from attn_mask, shared between the calls of one training step (fields added in
     version 108; no counterpart in the reference, whose kernels read the mask tile by tile,
     T/attention.py:357-371).  A dense mask is classified block by block (clean / apply / skip / causal
     diagonal; for a block in which every row hides exactly the keys from one position on -- key padding that
     ends inside the block -- that position) and, for the dK/dV kernel, packed by key column; the compact tile
     is packed by key column.
     With mask_bits == NULL every call runs the pre-passes into its own workspace.  With mask_bits pointing
     at acct_fa_mask_bits_bytes(p) bytes of device memory (256-byte aligned) that the caller keeps across the
     calls, a call with mask_bits_filled == 0 runs them into that buffer and a call with
     mask_bits_filled != 0 only reads it.  The caller sets mask_bits_filled after the first call returns, and
     clears it when the contents of attn_mask change; the bits depend on attn_mask, mask_kind, B, Sq, Sk,
     prev_block_num, next_block_num and row_block_prefix only, so a mask that stays the same from step to
     step needs them once. */
  void*    mask_bits;
  int32_t  mask_bits_filled;
  /* Backward only (field added in version 108): != 0 makes dQ, dK, dV float32 tensors (same element strides as
     q, k, v), the output types the reference registers for its grad op before its bprop casts them to fp16
     (T/flash_attention_impl.py:59-93,103-105,121-123) -- for graphs that keep that registration.  The values are
     the p->dtype results converted (the kernels round once, from their fp32 accumulators, either way); the
     workspace grows by room for the three p->dtype tensors (acct_fa_bwd_workspace_bytes accounts for it).
     Not available through acct_fa_bwd_static, acct_fa_bwd_dq or acct_fa_bwd_dkdv. */
  int32_t  grad_f32;
} acct_fa_params;

/* Forward: replaces the `flash_attention` TBE custom op, T/flash_attention_fwd.py:498-530
 * (outputs `output` and `rowsum`, T/flash_attention_impl.py:129-154).
 * O is [B,N,Sq,D] in p->dtype with p->o_stride; LSE is fp32 [B,N,Sq] contiguous
 * (L = m + ln l, T/flash_attention_fwd.py:302-306).  `workspace` must hold
 * acct_fa_fwd_workspace_bytes(p) bytes (0 unless mask_kind == DENSE_U8 or dropout is on). */
int acct_fa_fwd(const acct_fa_params* p, void* O, float* LSE,
                void* workspace, size_t workspace_bytes, void* stream);
size_t acct_fa_fwd_workspace_bytes(const acct_fa_params* p);
/* Size of the optional drop_bits buffer (0 without dropout): keep bits by query row for the forward and dQ
 * kernels, then by key column for the dK/dV kernel, a quarter of a byte per score in total. */
size_t acct_fa_drop_bits_bytes(const acct_fa_params* p);

/* Size of the optional mask_bits buffer (0 without an attn_mask tensor). */
size_t acct_fa_mask_bits_bytes(const acct_fa_params* p);

/* Backward: replaces the `flash_attention_grad` TBE custom op,
 * T/flash_attention_bwd.py:436-477 (the bprop of T/flash_attention_impl.py:117-124
 * casts its fp32 results to fp16; here dQ,dK,dV are written in p->dtype directly,
 * accumulated in fp32 registers).  O and dO use p->o_stride; dQ,dK,dV use the
 * strides of q,k,v.  Deterministic: no atomics. */
int acct_fa_bwd(const acct_fa_params* p, const void* O, const void* dO, const float* LSE,
                void* dQ, void* dK, void* dV,
                void* workspace, size_t workspace_bytes, void* stream);
/* Workspace of the backward, 256-byte aligned.  With few heads and a short key sequence (cross attention on 77
 * keys: a handful of key tiles for 256 CUs) the size includes room for a dK/dV launch that cuts the query range
 * into slices on workgroups of their own and adds the slices' sums in a second kernel (fixed order: still
 * deterministic).  A smaller workspace that still holds everything else is accepted and runs the unsplit launch;
 * the two launches differ in the last bits of dK and dV (another order of summation). */
size_t acct_fa_bwd_workspace_bytes(const acct_fa_params* p);

/* The two halves of acct_fa_bwd, for callers that need one side of the gradient
 * only or want to time the halves apart (same workspace size as acct_fa_bwd).
 * acct_fa_bwd_dq writes dQ (T/flash_attention_bwd.py:209-231) and leaves
 * D = rowsum(dO*O) (T/flash_attention_bwd.py:138-159) in the workspace;
 * acct_fa_bwd_dkdv writes dV and dK (T/flash_attention_bwd.py:183-207,233-257)
 * and reads that D: it must follow an acct_fa_bwd_dq or acct_fa_bwd call with
 * the same inputs and workspace, in stream order. */
int acct_fa_bwd_dq(const acct_fa_params* p, const void* O, const void* dO, const float* LSE,
                   void* dQ, void* workspace, size_t workspace_bytes, void* stream);
int acct_fa_bwd_dkdv(const acct_fa_params* p, const void* O, const void* dO, const float* LSE,
                     void* dK, void* dV, void* workspace, size_t workspace_bytes, void* stream);

/* acct_fa_bwd for callers that cannot allocate or pass a workspace (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments as acct_fa_bwd minus the
 * workspace, and the results of acct_fa_bwd with a workspace of ACCT_FA_STATIC_SCRATCH_BYTES, bit for bit: D = rowsum(dO*O), the exp2 offsets, the mask block classes and bitmaps and
 * the dropout keep bits go to a buffer of ACCT_FA_STATIC_SCRATCH_BYTES that is part of the library's device
 * image (each GPU the library runs on holds one copy until the process ends).  The call allocates nothing and
 * frees nothing.  A problem that needs more than the buffer even without the optional split of the dK/dV launch
 * is refused with ACCT_E_WORKSPACE (pass drop_bits to keep a large dropout mask's bits out of it).  All calls on one GPU share
 * the buffer: calls that may overlap on that GPU (different streams, different threads) race and must be
 * serialised by the caller; calls in one stream are ordered and safe.  Nothing in the buffer needs clearing
 * between calls: every region a call reads is written by that call first. */
#define ACCT_FA_STATIC_SCRATCH_BYTES (8u << 20)
int acct_fa_bwd_static(const acct_fa_params* p, const void* O, const void* dO, const float* LSE,
                       void* dQ, void* dK, void* dV, void* stream);

/* Shape function of the inference operator `FlashAttentionTik` (y = softmax(q k^T) v, no mask, no scale),
 * replacing FlashAttentionTikInferShape, infer/flash_attention/tik/op_proto/flash_attention_tik.cpp:160-193:
 * q, k, v are [batch*heads, seq, D] or [batch, heads, seq, D] (HOST arrays of extents); batch and
 * batch*heads 1..64, heads 1..4096, sequence lengths 1..8192 with k's equal to v's, D one of 40, 64, 80, 160
 * (a 3-D input is also held to the reference's 1..64 rule for its last dimension, :104-112).  Writes q's
 * extents to y_dims (may be NULL) and returns ACCT_OK, else an error code; no device is touched.
 * The operator itself is acct_fa_fwd with scale = 1, mask_kind = NONE (head dims 40 and 160 are built
 * without the bias variants). */
int acct_fa_infer_shape(const int64_t* q_dims, int q_rank, const int64_t* k_dims, int k_rank,
                        const int64_t* v_dims, int v_rank, int64_t* y_dims);

/* Thread-local text of the last error on the calling thread ("" if none).
 * Stands in for the Python exceptions the reference raises at build time
 * (L/flash_attention.py:105-108,193-196). */
const char* acct_last_error(void);

/* ACCT_FA_VERSION of the loaded library. */
int acct_version(void);

/* 1 when the library contains every element type, head dim and side-input variant; 0 for a development build
 * that was compiled with a reduced variant set (such a build refuses the calls it cannot serve with
 * ACCT_E_LAUNCH).  No counterpart in the reference: a guard for packaging and tests. */
int acct_build_is_complete(void);

/* Measurement aid, no counterpart in the reference: the rate (TFLOP/s, whole GPU) at which the current device
 * retires back-to-back independent v_mfma_f32_32x32x16_f16 from registers, two waves per SIMD on every CU and
 * nothing else running -- the ceiling of any fp16 kernel built on that instruction.  varying_operands != 0:
 * operands differ from lane to lane as real data does; 0: one value in every lane (the clock, and with it the
 * rate, depends on how much the operands toggle).  Runs about 0.1 s of kernels on `stream` and waits for them.
 * bench.py reports both figures beside the attention kernels' roofline fraction. */
int acct_probe_mfma_rate(int varying_operands, double* tflops, void* stream);

/* The same run, which also reports the shader clock (GHz) that one wave saw while it ran: shader-clock ticks
 * over wall-clock ticks across its MFMA loop.  An MFMA of this kind occupies the matrix pipe for 32 clocks whatever
 * the operands; what the power drawn changes is this clock.  Measurement aid, no counterpart in the reference. */
int acct_probe_mfma_clock(int varying_operands, double* tflops, double* shader_ghz, void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* ACCT_FA_H_ */
