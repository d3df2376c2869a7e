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
 * too.  `extra` points at an acct_ms_attrs block that the op's init function fills from the primitive attributes
 * (prev_block_num, next_block_num: flash_attention_impl.py:146-148).  A trailing workspace output is used when
 * the graph declares one (sized by acct_fa_*_workspace_bytes); without it the forward needs none for mask-free
 * calls and the backward goes through acct_fa_bwd_static.  Plain C: builds with gcc, links libacct_fa.so.
 */
#include <stdint.h>
#include <string.h>

#include "../../include/acct_fa.h"

typedef struct acct_ms_attrs {
  int32_t prev_block_num, next_block_num;   /* 65536 = unbounded */
  float scale;                              /* 1.0 = the raw op (the reference's layer pre-scales q and k) */
  float keep_prob;                          /* 1.0 = no dropout */
} acct_ms_attrs;

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

int FlashAttentionFwd(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* stream, void* extra) {
  if (nparam < 8 || !params || !ndims || !shapes || !dtypes) return ACCT_E_NULLPTR;
  acct_fa_params p;
  int rc = describe(&p, params, ndims, shapes, dtypes, 0, 3, (const acct_ms_attrs*)extra);
  if (rc) return rc;
  void* ws = nparam > 8 ? params[8] : 0;
  return acct_fa_fwd(&p, params[6], (float*)params[7], ws, ws ? acct_fa_fwd_workspace_bytes(&p) : 0, stream);
}

int FlashAttentionGrad(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* stream, void* extra) {
  if (nparam < 12 || !params || !ndims || !shapes || !dtypes) return ACCT_E_NULLPTR;
  acct_fa_params p;
  int rc = describe(&p, params, ndims, shapes, dtypes, 0, 6, (const acct_ms_attrs*)extra);
  if (rc) return rc;
  if (nparam > 12 && params[12])
    return acct_fa_bwd(&p, params[3], params[4], (const float*)params[5], params[9], params[10], params[11], params[12],
                       acct_fa_bwd_workspace_bytes(&p), stream);
  return acct_fa_bwd_static(&p, params[3], params[4], (const float*)params[5], params[9], params[10], params[11], stream);
}

/* sizes of the optional workspace outputs, for the op's shape function */
size_t FlashAttentionFwdWorkspaceBytes(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* extra) {
  acct_fa_params p;
  if (nparam < 6 || describe(&p, params, ndims, shapes, dtypes, 0, 3, (const acct_ms_attrs*)extra)) return 0;
  return acct_fa_fwd_workspace_bytes(&p);
}
size_t FlashAttentionGradWorkspaceBytes(int nparam, void** params, int* ndims, int64_t** shapes, const char** dtypes, void* extra) {
  acct_fa_params p;
  if (nparam < 9 || describe(&p, params, ndims, shapes, dtypes, 0, 6, (const acct_ms_attrs*)extra)) return 0;
  return acct_fa_bwd_workspace_bytes(&p);
}
