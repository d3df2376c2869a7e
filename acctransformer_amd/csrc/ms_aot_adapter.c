/*
 * MindSpore `Custom(..., func_type="aot")` entry points over the C ABI of include/acct_fa.h: the binding a
 * maintainer of the reference adds in place of its two TBE registrations
 * (train/acctransformer/flash_attention/ops/flash_attention/flash_attention_impl.py:107-108,143-145).
 *
 * MindSpore calls an AOT custom op as
 *     int fn(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* stream, void* extra)
 * with the inputs first and the outputs after them, all device pointers.  The operand order is the reference's:
 *     forward   inputs  query, key, value, attn_mask, dropout_mask, alibi_mask        (flash_attention_impl.py:150)
 *               outputs output, rowsum [, workspace]                                  (:151-153)
 *     backward  inputs  query, key, value, output, dout, rowsum, attn_mask, dropout_mask, alibi_mask   (:113)
 *               outputs dq, dk, dv [, workspace]                                      (:114)
 * An optional input the graph does not feed arrives as a NULL pointer (the reference passes None,
 * attention.py:299-309).  Masks come in the reference's own forms: attn_mask fp16/bf16 [1|B,Sq,Sk] or the compact
 * (1,128,128) causal tile (attention.py:279-285), dropout_mask fp16/bf16 {0, 1/keep_prob}; uint8 masks are taken
 * too.  Output types are checked: `output` in the operands' dtype, `rowsum` float32, dq / dk / dv either in the
 * operands' dtype or float32 -- the reference registers float32 there and casts in its bprop
 * (flash_attention_impl.py:103-105,121-123); a graph that keeps that registration gets float32 tensors
 * (acct_fa_params.grad_f32).
 *
 * Attributes.  MindSpore hands `extra` to the main function: NULL when the op has no init function, else the
 * AotExtra object (a C++ class of MindSpore's; this file is plain C and does not know it).  The primitive
 * attributes (prev_block_num, next_block_num: flash_attention_impl.py:146-148) therefore come through an accessor
 * that the maintainer's init glue registers once with acct_ms_set_attrs_accessor(): given `extra`, it returns the
 * acct_ms_attrs block that the init function built from extra->Attr<T>(...) and parked as the op's kernel data.
 * Without a registered accessor, `extra` must be NULL (defaults: unbounded band, scale 1, keep_prob 1) or point
 * at an acct_ms_attrs block whose `magic` field holds ACCT_MS_ATTRS_MAGIC; anything else is refused with
 * ACCT_E_PARAM rather than read as attributes.
 *
 * Workspace.  A trailing workspace output (sized by the *WorkspaceBytes functions below, for the op's shape
 * function) is REQUIRED whenever the library needs scratch memory: the backward always, the forward with an
 * attn_mask tensor or dropout.  Without it those calls return ACCT_E_WORKSPACE.  Only when the attributes say
 * use_static_scratch != 0 does a backward without a workspace output go through acct_fa_bwd_static, whose one
 * buffer per GPU is shared by every call on that GPU: safe for a graph that runs on one stream, a race for
 * attention ops on several streams.  Plain C: builds with gcc, links libacct_fa.so.
 */
#include <stdint.h>
#include <string.h>

#include "../../include/acct_fa.h"

#define ACCT_MS_ATTRS_MAGIC 0x41434354u     /* "ACCT" */

typedef struct acct_ms_attrs {
  uint32_t magic;                           /* ACCT_MS_ATTRS_MAGIC */
  int32_t prev_block_num, next_block_num;   /* 65536 = unbounded */
  float scale;                              /* 1.0 = the raw op (the reference's layer pre-scales q and k) */
  float keep_prob;                          /* 1.0 = no dropout */
  int32_t use_static_scratch;               /* != 0: a backward without a workspace output may use acct_fa_bwd_static */
} acct_ms_attrs;

typedef const acct_ms_attrs* (*acct_ms_attrs_accessor)(void* extra);
static acct_ms_attrs_accessor g_accessor = 0;

/* registers the function that maps MindSpore's `extra` to the attribute block (NULL = back to the default rule) */
void acct_ms_set_attrs_accessor(acct_ms_attrs_accessor fn) { g_accessor = fn; }

/* returns 0 and *out (NULL = defaults) or an error code */
static int attrs_of(void* extra, const acct_ms_attrs** out) {
  *out = 0;
  if (g_accessor) {
    *out = g_accessor(extra);
    return (*out && (*out)->magic != ACCT_MS_ATTRS_MAGIC) ? ACCT_E_PARAM : ACCT_OK;
  }
  if (!extra) return ACCT_OK;
  if (((const acct_ms_attrs*)extra)->magic != ACCT_MS_ATTRS_MAGIC) return ACCT_E_PARAM;
  *out = (const acct_ms_attrs*)extra;
  return ACCT_OK;
}

static int dtype_code(const char* s) {
  if (!s) return -1;
  if (!strcmp(s, "float16")) return ACCT_F16;
  if (!strcmp(s, "bfloat16")) return ACCT_BF16;
  return -1;
}

/* fills the problem description from the q, k, v operands and the three optional side inputs */
static int describe(acct_fa_params* p, void** params, int* ndims, int64_t** shapes, const char** dtypes, int iq, int imask,
                    const acct_ms_attrs* at) {
  memset(p, 0, sizeof(*p));
  if (ndims[iq] != 4 || ndims[iq + 1] != 4 || ndims[iq + 2] != 4) return ACCT_E_SHAPE;
  p->dtype = dtype_code(dtypes[iq]);
  if (p->dtype < 0 || dtype_code(dtypes[iq + 1]) != p->dtype || dtype_code(dtypes[iq + 2]) != p->dtype) return ACCT_E_DTYPE;
  p->B = (int32_t)shapes[iq][0]; p->N = (int32_t)shapes[iq][1]; p->Sq = (int32_t)shapes[iq][2]; p->D = (int32_t)shapes[iq][3];
  p->Sk = (int32_t)shapes[iq + 1][2];
  p->scale = at ? at->scale : 1.0f;
  p->keep_prob = at ? at->keep_prob : 1.0f;
  p->prev_block_num = at ? at->prev_block_num : ACCT_BLOCK_UNBOUNDED;
  p->next_block_num = at ? at->next_block_num : ACCT_BLOCK_UNBOUNDED;
  p->q = params[iq]; p->k = params[iq + 1]; p->v = params[iq + 2];
  if (params[imask]) {                                      /* attn_mask */
    const int nd = ndims[imask];
    const int64_t* sh = shapes[imask];
    const int wide = dtype_code(dtypes[imask]) == p->dtype;
    if (!wide && strcmp(dtypes[imask], "uint8")) return ACCT_E_DTYPE;
    /* the compact causal tile: (128,128) or (1,128,128) (attention.py:279-285) */
    const int compact = (nd == 2 && sh[0] == 128 && sh[1] == 128) || (nd == 3 && sh[0] == 1 && sh[1] == 128 && sh[2] == 128);
    if (compact && !(p->Sq == 128 && p->Sk == 128 && nd == 3)) {
      p->mask_kind = wide ? ACCT_MASK_TILE_F16 : ACCT_MASK_TILE_U8;
    } else {
      if (nd != 3 || sh[1] != p->Sq || sh[2] != p->Sk || (sh[0] != 1 && sh[0] != p->B)) return ACCT_E_SHAPE;
      p->mask_kind = wide ? ACCT_MASK_DENSE_F16 : ACCT_MASK_DENSE_U8;
      p->mask_stride_b = sh[0] == 1 ? 0 : sh[1] * sh[2];
    }
    p->attn_mask = params[imask];
  }
  if (params[imask + 1]) {                                  /* dropout_mask */
    const int wide = dtype_code(dtypes[imask + 1]) == p->dtype;
    if (!wide && strcmp(dtypes[imask + 1], "uint8")) return ACCT_E_DTYPE;
    p->drop_mask = params[imask + 1];
    p->drop_mask_kind = wide ? ACCT_DROP_F16 : ACCT_DROP_U8;
    /* a dropout mask without a keep probability below 1 would leave the kept probabilities unscaled */
    if (!(p->keep_prob < 1.0f)) return ACCT_E_PARAM;
  }
  if (params[imask + 2]) {                                  /* alibi_mask [B|1, N|1, Sq|1, Sk] in the operands' dtype */
    const int64_t* sh = shapes[imask + 2];
    if (ndims[imask + 2] != 4 || sh[3] != p->Sk || dtype_code(dtypes[imask + 2]) != p->dtype) return ACCT_E_SHAPE;
    p->alibi = params[imask + 2];
    p->alibi_stride_q = sh[2] == 1 ? 0 : sh[3];
    p->alibi_stride_h = sh[1] == 1 ? 0 : sh[2] * sh[3];
    p->alibi_stride_b = sh[0] == 1 ? 0 : sh[1] * sh[2] * sh[3];
  }
  return ACCT_OK;
}

static int is_f32(const char* s) { return s && !strcmp(s, "float32"); }

int FlashAttentionFwd(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* stream, void* extra) {
  if (nparam < 8 || !params || !ndims || !shapes || !dtypes) return ACCT_E_NULLPTR;
  const acct_ms_attrs* at;
  int rc = attrs_of(extra, &at);
  if (rc) return rc;
  acct_fa_params p;
  rc = describe(&p, params, ndims, shapes, dtypes, 0, 3, at);
  if (rc) return rc;
  if (dtype_code(dtypes[6]) != p.dtype || !is_f32(dtypes[7])) return ACCT_E_DTYPE;   /* output, rowsum */
  void* ws = nparam > 8 ? params[8] : 0;
  return acct_fa_fwd(&p, params[6], (float*)params[7], ws, ws ? acct_fa_fwd_workspace_bytes(&p) : 0, stream);
}

int FlashAttentionGrad(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* stream, void* extra) {
  if (nparam < 12 || !params || !ndims || !shapes || !dtypes) return ACCT_E_NULLPTR;
  const acct_ms_attrs* at;
  int rc = attrs_of(extra, &at);
  if (rc) return rc;
  acct_fa_params p;
  rc = describe(&p, params, ndims, shapes, dtypes, 0, 6, at);
  if (rc) return rc;
  /* dq, dk, dv: all in the operands' dtype, or all float32 (the reference's registration) */
  const int f32 = is_f32(dtypes[9]);
  for (int i = 9; i < 12; i++)
    if (f32 ? !is_f32(dtypes[i]) : dtype_code(dtypes[i]) != p.dtype) return ACCT_E_DTYPE;
  if (dtype_code(dtypes[3]) != p.dtype || dtype_code(dtypes[4]) != p.dtype || !is_f32(dtypes[5])) return ACCT_E_DTYPE;
  p.grad_f32 = f32;
  if (nparam > 12 && params[12])
    return acct_fa_bwd(&p, params[3], params[4], (const float*)params[5], params[9], params[10], params[11], params[12],
                       acct_fa_bwd_workspace_bytes(&p), stream);
  if (!(at && at->use_static_scratch) || f32) return ACCT_E_WORKSPACE;
  return acct_fa_bwd_static(&p, params[3], params[4], (const float*)params[5], params[9], params[10], params[11], stream);
}

/* sizes of the workspace outputs, for the op's shape function (the backward's depends on the dq / dk / dv dtype) */
size_t FlashAttentionFwdWorkspaceBytes(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* extra) {
  acct_fa_params p;
  const acct_ms_attrs* at;
  if (nparam < 6 || attrs_of(extra, &at) || describe(&p, params, ndims, shapes, dtypes, 0, 3, at)) return 0;
  return acct_fa_fwd_workspace_bytes(&p);
}
size_t FlashAttentionGradWorkspaceBytes(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* extra) {
  acct_fa_params p;
  const acct_ms_attrs* at;
  if (nparam < 9 || attrs_of(extra, &at) || describe(&p, params, ndims, shapes, dtypes, 0, 6, at)) return 0;
  p.grad_f32 = nparam > 9 && is_f32(dtypes[9]);
  return acct_fa_bwd_workspace_bytes(&p);
}
