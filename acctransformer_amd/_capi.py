"""ctypes binding of libacct_fa.so (the C ABI declared in include/acct_fa.h).

torch is used for device memory and the current HIP stream only; the compute
is the hand-written gfx950 kernels behind the C ABI.  There is no fallback:
if the shared library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os

import torch

_LIB_NAME = "libacct_fa.so"
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)

ACCT_F16, ACCT_BF16 = 0, 1
MASK_NONE, MASK_DENSE_U8, MASK_DENSE_F16, MASK_TILE_U8, MASK_CAUSAL, MASK_TILE_F16 = 0, 1, 2, 3, 4, 5
DROP_U8, DROP_F16 = 0, 1
BLOCK_UNBOUNDED = 65536

ERROR_NAMES = {
    0: "ACCT_OK", -1: "ACCT_E_NULLPTR", -2: "ACCT_E_SHAPE", -3: "ACCT_E_DTYPE", -4: "ACCT_E_HEADDIM",
    -5: "ACCT_E_ARCH", -6: "ACCT_E_LAUNCH", -7: "ACCT_E_WORKSPACE", -8: "ACCT_E_PARAM",
}


class AcctFaParams(ctypes.Structure):
    """Mirror of `acct_fa_params` (include/acct_fa.h)."""
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32), ("N", ctypes.c_int32), ("Sq", ctypes.c_int32), ("Sk", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("scale", ctypes.c_float), ("keep_prob", ctypes.c_float),
        ("prev_block_num", ctypes.c_int32), ("next_block_num", ctypes.c_int32),
        ("mask_kind", ctypes.c_int32), ("row_block_prefix", ctypes.c_int32),
        ("mask_stride_b", ctypes.c_int64),
        ("alibi_stride_b", ctypes.c_int64), ("alibi_stride_h", ctypes.c_int64), ("alibi_stride_q", ctypes.c_int64),
        ("q_stride", ctypes.c_int64 * 3), ("k_stride", ctypes.c_int64 * 3),
        ("v_stride", ctypes.c_int64 * 3), ("o_stride", ctypes.c_int64 * 3),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("attn_mask", ctypes.c_void_p), ("drop_mask", ctypes.c_void_p), ("alibi", ctypes.c_void_p),
        ("drop_seed", ctypes.c_uint64), ("drop_offset", ctypes.c_uint32), ("drop_philox", ctypes.c_int32),
        ("drop_bits", ctypes.c_void_p), ("drop_bits_filled", ctypes.c_int32), ("drop_mask_kind", ctypes.c_int32),
        ("mask_bits", ctypes.c_void_p), ("mask_bits_filled", ctypes.c_int32), ("grad_f32", ctypes.c_int32),
    ]


class AcctError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")
        self.code = code


_lib = None


def lib_path():
    return _LIB_PATH


def load():
    """Load libacct_fa.so (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} not found: build it with `make -C acctransformer_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path")
    lib = ctypes.CDLL(_LIB_PATH)
    P = ctypes.POINTER(AcctFaParams)
    lib.acct_fa_fwd.argtypes = [P, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.acct_fa_fwd.restype = ctypes.c_int
    lib.acct_fa_bwd.argtypes = [P] + [ctypes.c_void_p] * 7 + [ctypes.c_size_t, ctypes.c_void_p]
    lib.acct_fa_bwd.restype = ctypes.c_int
    lib.acct_fa_bwd_static.argtypes = [P] + [ctypes.c_void_p] * 7
    lib.acct_fa_bwd_static.restype = ctypes.c_int
    lib.acct_fa_bwd_dq.argtypes = [P] + [ctypes.c_void_p] * 5 + [ctypes.c_size_t, ctypes.c_void_p]
    lib.acct_fa_bwd_dq.restype = ctypes.c_int
    lib.acct_fa_bwd_dkdv.argtypes = [P] + [ctypes.c_void_p] * 6 + [ctypes.c_size_t, ctypes.c_void_p]
    lib.acct_fa_bwd_dkdv.restype = ctypes.c_int
    lib.acct_fa_fwd_workspace_bytes.argtypes = [P]
    lib.acct_fa_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.acct_fa_drop_bits_bytes.argtypes = [P]
    lib.acct_fa_drop_bits_bytes.restype = ctypes.c_size_t
    lib.acct_fa_mask_bits_bytes.argtypes = [P]
    lib.acct_fa_mask_bits_bytes.restype = ctypes.c_size_t
    lib.acct_fa_bwd_workspace_bytes.argtypes = [P]
    lib.acct_fa_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.acct_last_error.argtypes = []
    lib.acct_last_error.restype = ctypes.c_char_p
    lib.acct_build_is_complete.argtypes = []
    lib.acct_build_is_complete.restype = ctypes.c_int
    I64P = ctypes.POINTER(ctypes.c_int64)
    lib.acct_fa_infer_shape.argtypes = [I64P, ctypes.c_int, I64P, ctypes.c_int, I64P, ctypes.c_int, I64P]
    lib.acct_fa_infer_shape.restype = ctypes.c_int
    lib.acct_probe_mfma_rate.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    lib.acct_probe_mfma_rate.restype = ctypes.c_int
    lib.acct_probe_mfma_clock.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    lib.acct_probe_mfma_clock.restype = ctypes.c_int
    lib.acct_version.argtypes = []
    lib.acct_version.restype = ctypes.c_int
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise AcctError(rc, load().acct_last_error().decode())


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _bhs_strides(t):
    """(batch, head, row) element strides of a [B,N,S,D] tensor whose last dim is contiguous."""
    if t.stride(3) != 1 and t.size(3) != 1:
        raise ValueError("last dimension must be contiguous")
    return (ctypes.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def make_params(q, k, v, *, scale, keep_prob=1.0, prev_block_num=BLOCK_UNBOUNDED, next_block_num=BLOCK_UNBOUNDED,
                mask_kind=MASK_NONE, attn_mask=None, drop_mask=None, alibi=None, o_like=None, row_block_prefix=0,
                drop_seed=None, drop_offset=0):
    """Describe one attention problem.  q [B,N,Sq,D]; k,v [B,N,Sk,D] (any
    batch/head/row strides, unit stride along D); attn_mask [1|B,Sq,Sk]
    (DENSE) or [128,128] (TILE), uint8 for the _U8 kinds and q's dtype for the
    _F16 kinds (nonzero = masked); drop_mask [B,N,Sq,Sk], uint8 {0,1} or q's
    dtype {0, 1/keep_prob} (nonzero = keep); alibi in q's dtype, broadcastable
    to [B,N,Sq,Sk].  With drop_seed (and no drop_mask) and
    keep_prob < 1 the library draws the keep mask itself from
    (drop_seed, drop_offset), identically in forward and backward."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be 4-D [B,N,S,D]")
    B, N, Sq, D = q.shape
    Sk = k.shape[2]
    if k.shape != (B, N, Sk, D) or v.shape != (B, N, Sk, D):
        raise ValueError(f"inconsistent shapes q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
    if q.dtype == torch.float16:
        dt = ACCT_F16
    elif q.dtype == torch.bfloat16:
        dt = ACCT_BF16
    else:
        raise TypeError(f"q/k/v must be float16 or bfloat16, got {q.dtype}")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share one dtype")
    p = AcctFaParams()
    p.dtype = dt
    p.B, p.N, p.Sq, p.Sk, p.D = B, N, Sq, Sk, D
    p.scale, p.keep_prob = float(scale), float(keep_prob)
    p.prev_block_num, p.next_block_num = int(min(prev_block_num, BLOCK_UNBOUNDED)), int(min(next_block_num, BLOCK_UNBOUNDED))
    p.mask_kind = mask_kind
    p.row_block_prefix = int(row_block_prefix)
    p.q_stride, p.k_stride, p.v_stride = _bhs_strides(q), _bhs_strides(k), _bhs_strides(v)
    if o_like is not None:
        p.o_stride = _bhs_strides(o_like)
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    keep = [q, k, v]
    if mask_kind in (MASK_DENSE_U8, MASK_TILE_U8, MASK_DENSE_F16, MASK_TILE_F16):
        want = torch.uint8 if mask_kind in (MASK_DENSE_U8, MASK_TILE_U8) else q.dtype
        if attn_mask is None or attn_mask.dtype != want or not attn_mask.is_contiguous():
            raise TypeError(f"attn_mask must be a contiguous {want} tensor for mask_kind {mask_kind}")
        if mask_kind in (MASK_DENSE_U8, MASK_DENSE_F16):
            if attn_mask.dim() != 3 or attn_mask.shape[1:] != (Sq, Sk) or attn_mask.shape[0] not in (1, B):
                raise ValueError(f"attn_mask must be [1|B,{Sq},{Sk}], got {tuple(attn_mask.shape)}")
            p.mask_stride_b = 0 if attn_mask.shape[0] == 1 else Sq * Sk
        elif attn_mask.numel() != 128 * 128:
            raise ValueError("compact attn_mask must hold 128*128 elements")
        p.attn_mask = attn_mask.data_ptr()
        keep.append(attn_mask)
    if drop_mask is not None:
        if drop_mask.dtype not in (torch.uint8, q.dtype) or not drop_mask.is_contiguous() or drop_mask.shape != (B, N, Sq, Sk):
            raise TypeError(f"drop_mask must be contiguous [{B},{N},{Sq},{Sk}], uint8 or {q.dtype}")
        p.drop_mask = drop_mask.data_ptr()
        p.drop_mask_kind = DROP_U8 if drop_mask.dtype == torch.uint8 else DROP_F16
        keep.append(drop_mask)
    if drop_seed is not None:
        if drop_mask is not None:
            raise ValueError("give either drop_mask or drop_seed, not both")
        p.drop_seed = int(drop_seed) & 0xFFFFFFFFFFFFFFFF
        p.drop_offset = int(drop_offset) & 0xFFFFFFFF
        p.drop_philox = 1
    if alibi is not None:
        if alibi.dtype != q.dtype or alibi.dim() != 4 or alibi.shape[3] != Sk or alibi.stride(3) != 1:
            raise TypeError("alibi must be 4-D in q's dtype with a contiguous last dim of Sk")
        ab, ah, aq = alibi.shape[:3]
        if ab not in (1, B) or ah not in (1, N) or aq not in (1, Sq):
            raise ValueError(f"alibi {tuple(alibi.shape)} does not broadcast to [{B},{N},{Sq},{Sk}]")
        p.alibi = alibi.data_ptr()
        p.alibi_stride_b = 0 if ab == 1 else alibi.stride(0)
        p.alibi_stride_h = 0 if ah == 1 else alibi.stride(1)
        p.alibi_stride_q = 0 if aq == 1 else alibi.stride(2)
        keep.append(alibi)
    p._keepalive = keep
    return p


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _workspace(nbytes, device):
    if nbytes == 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def attach_drop_bits(p, device):
    """Give `p` a buffer for the keep bits of its dropout mask, so that the forward call packs (or draws)
    them once and the backward call of the same step reads them: set `p.drop_bits_filled = 1` after the
    first call.  Returns the buffer (the caller keeps it alive), or None when `p` has no dropout."""
    lib = load()
    n = lib.acct_fa_drop_bits_bytes(ctypes.byref(p))
    if n == 0:
        return None
    buf = torch.empty(n, dtype=torch.uint8, device=device)
    p.drop_bits = buf.data_ptr()
    p.drop_bits_filled = 0
    return buf


def attach_mask_bits(p, device):
    """Give `p` a buffer for what the pre-passes derive from its attn_mask (block classes, column bitmaps), so
    that the first call of a step runs them once and the later calls read them: set `p.mask_bits_filled = 1`
    after the first call.  Returns the buffer (the caller keeps it alive), or None when `p` has no mask tensor."""
    lib = load()
    n = lib.acct_fa_mask_bits_bytes(ctypes.byref(p))
    if n == 0:
        return None
    buf = torch.empty(n, dtype=torch.uint8, device=device)
    p.mask_bits = buf.data_ptr()
    p.mask_bits_filled = 0
    return buf


def fa_fwd(p, q):
    """Run acct_fa_fwd for params `p` built from q; returns (O, LSE)."""
    lib = load()
    if not q.is_cuda:
        raise RuntimeError("acct_fa_fwd needs device tensors (there is no CPU path)")
    o = torch.empty_like(q)
    if not any(p.o_stride):
        p.o_stride = _bhs_strides(o)
    lse = torch.empty((p.B, p.N, p.Sq), dtype=torch.float32, device=q.device)
    nws = lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p))
    ws = _workspace(nws, q.device)
    with torch.cuda.device(q.device):
        _check(lib.acct_fa_fwd(ctypes.byref(p), _ptr(o), _ptr(lse), _ptr(ws), nws, _stream(q)))
    return o, lse


def fa_bwd(p, q, k, v, o, do, lse, workspace_bytes=None):
    """Run acct_fa_bwd; returns (dQ, dK, dV) laid out like q, k, v.  `workspace_bytes`: the size of the
    workspace to pass instead of acct_fa_bwd_workspace_bytes (a smaller one that still holds the required
    parts makes the library run the dK/dV kernel without splitting the query range)."""
    lib = load()
    if not q.is_cuda:
        raise RuntimeError("acct_fa_bwd needs device tensors (there is no CPU path)")
    if do.stride() != o.stride():
        # the kernels read dO with O's strides: copy the values into a buffer laid out like O
        tmp = torch.empty_strided(o.size(), o.stride(), dtype=o.dtype, device=o.device)
        tmp.copy_(do)
        do = tmp
    p.o_stride = _bhs_strides(o)
    gdt = torch.float32 if p.grad_f32 else q.dtype       # (grad_f32: the reference's registered output type)
    dq = torch.empty_strided(q.size(), q.stride(), dtype=gdt, device=q.device)
    dk = torch.empty_strided(k.size(), k.stride(), dtype=gdt, device=k.device)
    dv = torch.empty_strided(v.size(), v.stride(), dtype=gdt, device=v.device)
    nws = lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p)) if workspace_bytes is None else int(workspace_bytes)
    ws = _workspace(nws, q.device)
    with torch.cuda.device(q.device):
        _check(lib.acct_fa_bwd(ctypes.byref(p), _ptr(o), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv),
                               _ptr(ws), nws, _stream(q)))
    return dq, dk, dv


def infer_shape(q_shape, k_shape, v_shape):
    """acct_fa_infer_shape: the output shape of the inference operator for these input shapes,
    or AcctError when the reference's shape function would reject them."""
    lib = load()
    arr = lambda s: (ctypes.c_int64 * max(len(s), 1))(*s)
    y = (ctypes.c_int64 * 4)()
    _check(lib.acct_fa_infer_shape(arr(q_shape), len(q_shape), arr(k_shape), len(k_shape), arr(v_shape), len(v_shape), y))
    return tuple(y[i] for i in range(len(q_shape)))
