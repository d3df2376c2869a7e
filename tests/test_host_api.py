"""CPU-side tests: the C-ABI library loads and exports what include/acct_fa.h
declares, argument validation returns the documented error codes without
touching a device, and the Python mirror of the reference interface keeps the
reference's names, argument checks and error texts."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from acctransformer_amd import _capi
from acctransformer_amd.flash_attention.nn.layer.flash_attention import FlashAttention
from acctransformer_amd.flash_attention.ops.flash_attention import flash_attention_impl as impl
from acctransformer_amd.triangle_attention.triangle_attention import TriangleAttention
from golden_cases import load_cases
from oracle import unfused_attention as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header():
    return open(os.path.join(ROOT, "include", "acct_fa.h")).read()


def test_library_exports_every_declared_symbol():
    lib = _capi.load()
    decl = re.findall(r"^\s*(?:int|size_t|const char\*)\s+(acct_\w+)\s*\(", _header(), flags=re.M)
    assert set(decl) >= {"acct_fa_fwd", "acct_fa_bwd", "acct_fa_bwd_dq", "acct_fa_bwd_dkdv",
                         "acct_fa_fwd_workspace_bytes", "acct_fa_bwd_workspace_bytes", "acct_last_error", "acct_version",
                         "acct_fa_infer_shape", "acct_build_is_complete", "acct_fa_drop_bits_bytes", "acct_fa_mask_bits_bytes"}
    for name in decl:
        assert hasattr(lib, name), name
    m = re.search(r"#define ACCT_FA_VERSION (\d+)", _header())
    assert lib.acct_version() == int(m.group(1))
    # the in-tree library must be the complete build, not a reduced development build
    assert lib.acct_build_is_complete() == 1


def test_struct_mirror_matches_header_field_order():
    body = re.search(r"typedef struct acct_fa_params \{(.*?)\} acct_fa_params;", _header(), flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.sub(r"\[\d+\]", "", part.strip().split()[-1]).lstrip("*"))
    assert names == [f[0] for f in _capi.AcctFaParams._fields_]
    assert ctypes.sizeof(_capi.AcctFaParams) == 272


def _params(**over):
    q = torch.zeros(1, 2, 128, 128, dtype=torch.float16)
    p = _capi.make_params(q, q.clone(), q.clone(), scale=1.0)
    for k, v in over.items():
        setattr(p, k, v)
    return p


@pytest.mark.parametrize("over, code", [
    (dict(dtype=7), -3), (dict(B=0), -2), (dict(D=512), -4), (dict(D=100), -4), (dict(scale=0.0), -8),
    (dict(keep_prob=1.5), -8), (dict(prev_block_num=-1), -8), (dict(mask_kind=6), -8), (dict(mask_kind=_capi.MASK_DENSE_F16), -1),
    (dict(drop_mask_kind=2), -8), (dict(B=1 << 20, N=1 << 12), -2), (dict(B=1 << 15, N=1 << 10, Sq=1 << 16), -2),
    (dict(mask_kind=_capi.MASK_DENSE_U8), -1), (dict(row_block_prefix=100), -8), (dict(q=None), -1),
])
def test_validation_error_codes(over, code):
    lib = _capi.load()
    p = _params(**over)
    buf = (ctypes.c_char * 64)()
    rc = lib.acct_fa_fwd(ctypes.byref(p), ctypes.addressof(buf), ctypes.addressof(buf), None, 0, None)
    assert rc == code
    assert lib.acct_last_error().decode() != ""
    rc = lib.acct_fa_bwd(ctypes.byref(p), *([ctypes.addressof(buf)] * 6), None, 0, None)
    assert rc == code


def test_null_outputs_and_workspace_sizes():
    lib = _capi.load()
    p = _params()
    assert lib.acct_fa_fwd(ctypes.byref(p), None, None, None, 0, None) == -1
    assert lib.acct_fa_fwd(None, None, None, None, 0, None) == -1
    assert lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p)) == 0
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p)) == 2 * (1 * 2 * 128 * 4)
    m = torch.zeros(1, 128, 128, dtype=torch.uint8)
    q = torch.zeros(2, 2, 128, 128, dtype=torch.float16)
    p2 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, mask_kind=_capi.MASK_DENSE_U8, attn_mask=m)
    # block classes (padded to 256)
    assert lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p2)) == 256
    raw = (ctypes.c_char * 128)()
    addr = (ctypes.addressof(raw) + 63) // 64 * 64
    # backward without its workspace is refused before any launch
    assert lib.acct_fa_bwd(ctypes.byref(p2), *([addr] * 6), None, 0, None) == -7
    # D and -LSE*log2e rows, block classes (padded to 256), key-column bitmaps: 16 bytes per (q block, key)
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p2)) == 2 * (2 * 2 * 128 * 4) + 256 + 1 * 1 * 128 * 16
    # a caller-held mask_bits buffer takes the classes and the bitmaps out of both workspaces
    assert lib.acct_fa_mask_bits_bytes(ctypes.byref(p2)) == 256 + 128 * 16
    assert lib.acct_fa_mask_bits_bytes(ctypes.byref(p)) == 0
    p2.mask_bits = 4096
    assert lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p2)) == 0
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p2)) == 2 * (2 * 2 * 128 * 4)
    p2.mask_bits = 4096 + 64
    assert lib.acct_fa_fwd(ctypes.byref(p2), addr, addr, None, 0, None) == -7     # misaligned buffer
    p2.mask_bits = None


def test_forward_rejects_misaligned_output_and_workspace():
    # O is stored in 16-byte rows and the workspace regions are 256-byte aligned: a misaligned pointer is an error
    # code, not a misaligned vector access (checked before any device is touched)
    lib = _capi.load()
    raw = (ctypes.c_char * 1024)()
    base = (ctypes.addressof(raw) + 255) // 256 * 256
    p = _params()
    assert lib.acct_fa_fwd(ctypes.byref(p), base + 8, base, None, 0, None) == -2
    m = torch.zeros(1, 128, 128, dtype=torch.uint8)
    q = torch.zeros(1, 2, 128, 128, dtype=torch.float16)
    p2 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, mask_kind=_capi.MASK_DENSE_U8, attn_mask=m)
    need = lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p2))
    assert need > 0
    assert lib.acct_fa_fwd(ctypes.byref(p2), base, base, base + 64, need, None) == -7
    assert "aligned" in lib.acct_last_error().decode()


def test_infer_shape_function():
    # accept / reject cases of the inference operator's shape function
    # (infer/flash_attention/tik/op_proto/flash_attention_tik.cpp:20-193 of the reference)
    ok = _capi.infer_shape
    assert ok((2, 8, 100, 160), (2, 8, 300, 160), (2, 8, 300, 160)) == (2, 8, 100, 160)
    assert ok((64, 4096, 1, 40), (64, 4096, 8192, 40), (64, 4096, 8192, 40)) == (64, 4096, 1, 40)
    assert ok((64, 77, 64), (64, 5, 64), (64, 5, 64)) == (64, 77, 64)
    assert ok((8, 100, 40), (8, 100, 40), (8, 100, 40)) == (8, 100, 40)
    bad = [
        (((65, 8, 100, 64),) * 3, -2),                                   # batch > 64
        (((2, 4097, 100, 64),) * 3, -2),                                 # heads > 4096
        (((2, 8, 8193, 64),) * 3, -2),                                   # sequence > 8192
        (((2, 8, 100, 64), (2, 8, 50, 64), (2, 8, 51, 64)), -2),         # k and v lengths differ
        (((2, 8, 100, 64), (2, 9, 100, 64), (2, 8, 100, 64)), -2),       # heads differ
        (((2, 8, 100, 128),) * 3, -4),                                   # head dim not in {40, 64, 80, 160}
        (((2, 8, 100, 64), (2, 8, 100, 80), (2, 8, 100, 64)), -4),       # head dims differ
        (((8, 100, 80),) * 3, -4),                                       # 3-D: last dimension held to 1..64
        (((65, 100, 64),) * 3, -2),                                      # 3-D: batch*heads > 64
        (((100, 64),) * 3, -2), (((1, 2, 8, 100, 64),) * 3, -2),         # rank
        (((2, 8, 100, 64), (8, 100, 64), (8, 100, 64)), -2),             # ranks differ
        (((2, 8, 0, 64),) * 3, -2),
    ]
    for shapes, code in bad:
        with pytest.raises(_capi.AcctError) as e:
            ok(*shapes)
        assert e.value.code == code, shapes
    lib = _capi.load()
    assert lib.acct_fa_infer_shape(None, 4, None, 4, None, 4, None) == -1


def test_extra_head_dims_take_forward_and_backward_and_dropout_but_no_bias():
    lib = _capi.load()
    buf = (ctypes.c_char * 64)()
    a = ctypes.addressof(buf)
    for D in (40, 160, 256):
        q = torch.zeros(1, 2, 128, D, dtype=torch.float16)
        p = _capi.make_params(q, q.clone(), q.clone(), scale=1.0)
        # the forward accepts the head dim (the call gets past validation to the NULL output check: nothing is launched)
        assert lib.acct_fa_fwd(ctypes.byref(p), None, None, None, 0, None) == -1
        # so does the backward (it gets past validation to the workspace check)
        assert lib.acct_fa_bwd(ctypes.byref(p), *([a] * 6), None, 0, None) == -7
        # dropout is built for every head dim (the reference's layer takes dropout_rate with any head dim up to 256,
        # nn/layer/flash_attention.py:92-130,198-203) ...
        p2 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, keep_prob=0.9, drop_seed=1)
        assert lib.acct_fa_fwd(ctypes.byref(p2), None, None, None, 0, None) == -1
        # ... a bias is not, and says so before anything is launched
        p3 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, alibi=torch.zeros(1, 1, 1, 128, dtype=torch.float16))
        assert lib.acct_fa_fwd(ctypes.byref(p3), None, None, None, 0, None) == -4
        assert "bias" in lib.acct_last_error().decode()


def test_no_cpu_fallback():
    q = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    p = _capi.make_params(q, q.clone(), q.clone(), scale=1.0)
    with pytest.raises(RuntimeError):
        _capi.fa_fwd(p, q)


# ---- the Python mirror of the reference interface -------------------------------
def test_layer_constructor_checks_match_reference():
    with pytest.raises(ValueError, match="head_dim too large"):
        FlashAttention(head_dim=512)
    with pytest.raises(ValueError, match="alibi not supported"):
        FlashAttention(head_dim=128, alibi=True)
    with pytest.raises(Exception, match="Strategy:foo not supported"):
        FlashAttention(head_dim=128, tiling_stgy_name="foo")
    with pytest.raises(ValueError, match="multiple of 8"):
        FlashAttention(head_dim=100)
    FlashAttention(head_dim=160, dropout_rate=0.1)          # dropout at every head dim the layer admits
    layer = FlashAttention(head_dim=128, dropout_rate=0.1, prev_block_num=7, next_block_num=0)
    assert np.isclose(layer.scale, orc.flash_attention_layer_scale(128))
    assert layer.shard(((2, 4, 1, 1),) * 3) is layer and (layer.dp, layer.mp) == (2, 4)
    q = torch.zeros(1, 2, 128, 128, dtype=torch.float16)
    k = torch.zeros(1, 3, 128, 128, dtype=torch.float16)
    with pytest.raises(ValueError, match="head_num of query, key and value must be the same"):
        layer(q, k, k)


def test_triangle_constructor_checks_match_reference():
    with pytest.raises(ValueError, match="block size must be positive"):
        TriangleAttention(block_size=0)
    with pytest.raises(ValueError, match="dropout rate must be between 0 and 1"):
        TriangleAttention(dropout_rate=1.0)
    with pytest.raises(ValueError, match="data parallel must be positive"):
        TriangleAttention(dp=0)
    with pytest.raises(ValueError, match="model parallel must be positive"):
        TriangleAttention(mp=-1)
    assert TriangleAttention().block_size == 512


def test_op_factories_keep_reference_signature():
    fwd = impl.get_flash_attention(prev_block_num=3, next_block_num=0, tiling_stgy_name="wukong")
    assert (fwd.prev_block_num, fwd.next_block_num, fwd.tiling_stgy_name) == (3, 0, "wukong")
    assert callable(impl.get_flash_attention_grad())
    with pytest.raises(Exception, match="not supported"):
        impl.get_flash_attention(tiling_stgy_name="nope")


def test_mask_classification():
    S = 256
    f16 = torch.float16
    tri = torch.triu(torch.ones(1, S, S, dtype=f16), 1)
    # by default a mask tensor goes to the library as it is (its pre-pass finds the causal diagonal on the device)
    assert not impl.DETECT_CAUSAL_MASKS
    kind, m = impl._classify_mask(tri, S, S, f16)
    assert kind == _capi.MASK_DENSE_F16 and m.data_ptr() == tri.data_ptr()
    tile0 = torch.triu(torch.ones(1, 128, 128, dtype=f16), 1)
    assert impl._classify_mask(tile0, S, S, f16)[0] == _capi.MASK_TILE_F16
    impl.DETECT_CAUSAL_MASKS = True                      # opt-in: one device compare and host sync per mask tensor
    try:
        _test_mask_classification_with_detection(S, f16, tri)
    finally:
        impl.DETECT_CAUSAL_MASKS = False


def _test_mask_classification_with_detection(S, f16, tri):
    assert impl._classify_mask(tri, S, S, f16)[0] == _capi.MASK_CAUSAL
    pad = torch.zeros(2, S, S, dtype=torch.uint8); pad[:, :, 200:] = 1
    kind, m8 = impl._classify_mask(pad, S, S, f16)
    assert kind == _capi.MASK_DENSE_U8 and m8.dtype == torch.uint8 and m8.shape == (2, S, S)
    tile = torch.triu(torch.ones(1, 128, 128, dtype=f16), 1)
    assert impl._classify_mask(tile, S, S, f16)[0] == _capi.MASK_CAUSAL
    odd = tile.clone(); odd[0, 5, 3] = 1
    kind, m = impl._classify_mask(odd, S, S, f16)
    assert kind == _capi.MASK_TILE_F16 and m.shape == (128, 128) and m.dtype == f16     # the reference's form, as it is
    kind, m = impl._classify_mask(odd.float(), S, S, f16)
    assert kind == _capi.MASK_TILE_U8 and m.dtype == torch.uint8                        # other dtypes are converted
    # remembered per tensor and version: an in-place edit is seen; a mask in the operands' dtype is not converted
    tri[0, 0, 1] = 0
    kind, m = impl._classify_mask(tri, S, S, f16)
    assert kind == _capi.MASK_DENSE_F16 and m.data_ptr() == tri.data_ptr()
    kind, m = impl._classify_mask(tri, S, S, torch.bfloat16)
    assert kind == _capi.MASK_DENSE_U8 and m.dtype == torch.uint8
    with pytest.raises(ValueError):
        impl._classify_mask(torch.zeros(1, 100, S), S, S, f16)


def test_dropout_mask_forms():
    f16 = torch.float16
    d = torch.tensor([[0.0, 1.25], [1.25, 0.0]], dtype=f16)
    m, keep, seed = impl._prepare_dropout(d, None, f16)
    assert m.data_ptr() == d.data_ptr() and np.isclose(keep, 0.8) and seed is None       # the reference's form, as it is
    m8, keep, seed = impl._prepare_dropout(d, None, torch.bfloat16)
    assert m8.tolist() == [[0, 1], [1, 0]] and m8.dtype == torch.uint8 and np.isclose(keep, 0.8)
    m8, keep, seed = impl._prepare_dropout(torch.tensor([[1, 0]], dtype=torch.uint8), 0.9, f16)
    assert keep == 0.9 and seed is None
    with pytest.raises(ValueError):
        impl._prepare_dropout(torch.tensor([[1, 0]], dtype=torch.uint8), None, f16)
    # a (seed, offset) pair asks the library to draw the mask itself
    m8, keep, seed = impl._prepare_dropout((1234, 5), 0.75, f16)
    assert m8 is None and keep == 0.75 and seed == (1234, 5)
    with pytest.raises(ValueError):
        impl._prepare_dropout((1234, 5), None, f16)


def test_counter_based_dropout_fields_and_workspace():
    lib = _capi.load()
    assert lib.acct_version() >= 101
    q = torch.zeros(2, 2, 128, 128, dtype=torch.float16)
    p = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, keep_prob=0.9, drop_seed=(7 << 40) + 3, drop_offset=11)
    assert (p.drop_seed, p.drop_offset, p.drop_philox) == ((7 << 40) + 3, 11, 1)
    # keep bits by query row: 2 * ceil(Sk / 64) words per row; by key column 16 bytes per (q block, key)
    rows = 2 * 2 * 128 * 4 * 4
    assert lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p)) == rows
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p)) == 2 * (2 * 2 * 128 * 4) + rows + 2 * 2 * 1 * 128 * 16
    # keep_prob = 1 switches dropout off whatever the seed
    p1 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, keep_prob=1.0, drop_seed=5)
    assert lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p1)) == 0
    # keep_prob < 1 with neither a mask nor a seed is refused
    p2 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, keep_prob=0.9)
    buf = (ctypes.c_char * 64)()
    assert lib.acct_fa_fwd(ctypes.byref(p2), ctypes.addressof(buf), ctypes.addressof(buf), None, 0, None) == -1
    with pytest.raises(ValueError):
        _capi.make_params(q, q.clone(), q.clone(), scale=1.0, keep_prob=0.9, drop_seed=1,
                          drop_mask=torch.ones(2, 2, 128, 128, dtype=torch.uint8))


def test_shared_keep_bits_buffer_sizes_and_alignment():
    lib = _capi.load()
    assert lib.acct_version() >= 103
    q = torch.zeros(2, 2, 128, 128, dtype=torch.float16)
    p = _capi.make_params(q, q.clone(), q.clone(), scale=1.0, keep_prob=0.9, drop_seed=3)
    rows, cols = 2 * 2 * 128 * 4 * 4, 2 * 2 * 1 * 128 * 16
    assert lib.acct_fa_drop_bits_bytes(ctypes.byref(p)) == rows + cols
    stats = 2 * (2 * 2 * 128 * 4)
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p)) == stats + rows + cols
    # with the caller's buffer attached, the calls no longer ask for room of their own for the bits
    p.drop_bits = 256 * 1000
    assert lib.acct_fa_fwd_workspace_bytes(ctypes.byref(p)) == 0
    assert lib.acct_fa_bwd_workspace_bytes(ctypes.byref(p)) == stats
    # the buffer must be 256-byte aligned (checked before anything is launched)
    p.drop_bits = 256 * 1000 + 16
    buf = (ctypes.c_char * 64)()
    assert lib.acct_fa_fwd(ctypes.byref(p), ctypes.addressof(buf), ctypes.addressof(buf), None, 0, None) == -7
    # no dropout: nothing to share
    p0 = _capi.make_params(q, q.clone(), q.clone(), scale=1.0)
    assert lib.acct_fa_drop_bits_bytes(ctypes.byref(p0)) == 0


# ---- the oracle still reproduces the committed fixtures -------------------------
@pytest.mark.parametrize("name", sorted(load_cases().keys()))
def test_oracle_reproduces_golden(name):
    c = load_cases()[name]
    kw = dict(scale=float(c["scale"]), attn_mask=c.get("attn_mask"), drop_mask=c.get("drop_mask"),
              alibi=None if "alibi" not in c else c["alibi"].astype(np.float32), keep_prob=float(c["keep_prob"]),
              prev_block_num=int(c["prev_block_num"]), next_block_num=int(c["next_block_num"]))
    O, L = orc.unfused_fwd(c["q"], c["k"], c["v"], **kw)
    dQ, dK, dV = orc.unfused_bwd(c["q"], c["k"], c["v"], c["dO"], **kw)
    for got, want in ((O, c["O"]), (L, c["L"]), (dQ, c["dQ"]), (dK, c["dK"]), (dV, c["dV"])):
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6)


# ---- the MindSpore AOT custom-op adapter (libacct_fa_ms.so) ---------------------------------------------
def _ms_lib():
    lib = ctypes.CDLL(os.path.join(ROOT, "acctransformer_amd", "libacct_fa_ms.so"))
    for name in ("FlashAttentionFwd", "FlashAttentionGrad"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_int),
                       ctypes.POINTER(ctypes.POINTER(ctypes.c_int64)), ctypes.POINTER(ctypes.c_char_p), ctypes.c_void_p, ctypes.c_void_p]
    return lib


class MsAttrs(ctypes.Structure):
    """acct_ms_attrs of csrc/ms_aot_adapter.c"""
    MAGIC = 0x41434354
    _fields_ = [("magic", ctypes.c_uint32), ("prev_block_num", ctypes.c_int32), ("next_block_num", ctypes.c_int32),
                ("scale", ctypes.c_float), ("keep_prob", ctypes.c_float), ("use_static_scratch", ctypes.c_int32)]


def ms_call_args(operands):
    """(nparam, params, ndims, shapes, dtypes) of MindSpore's AOT convention from a list of (pointer or None, shape, dtype name)."""
    n = len(operands)
    params = (ctypes.c_void_p * n)(*[op[0] for op in operands])
    ndims = (ctypes.c_int * n)(*[len(op[1]) for op in operands])
    rows = [(ctypes.c_int64 * max(len(op[1]), 1))(*op[1]) for op in operands]
    shapes = (ctypes.POINTER(ctypes.c_int64) * n)(*[ctypes.cast(r, ctypes.POINTER(ctypes.c_int64)) for r in rows])
    dtypes = (ctypes.c_char_p * n)(*[op[2].encode() for op in operands])
    return n, params, ndims, shapes, dtypes, rows


def test_mindspore_adapter_loads_and_validates_without_a_device():
    lib = _ms_lib()
    buf = (ctypes.c_char * 64)()
    a = ctypes.addressof(buf)
    sh = (1, 2, 128, 128)
    good = [(a, sh, "float16")] * 3 + [(None, (), "float16")] * 3 + [(a, sh, "float16"), (a, sh[:3], "float32")]
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(good)
    assert lib.FlashAttentionFwd(3, params, ndims, shapes, dtypes, None, None) == -1          # too few operands
    bad = list(good); bad[1] = (a, sh, "float32")
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(bad)
    assert lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, None) == -3          # q, k, v dtypes differ
    bad = list(good); bad[3] = (a, (1, 100, 128), "float16")
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(bad)
    assert lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, None) == -2          # mask shape
    bad = list(good); bad[3] = (a, (1, 128, 128), "int32")
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(bad)
    assert lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, None) == -3          # mask dtype
    # output types: `output` in the operands' dtype, `rowsum` float32
    bad = list(good); bad[7] = (a, sh[:3], "float16")
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(bad)
    assert lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, None) == -3
    # `extra` that is not an attribute block (MindSpore's own object, say) is refused, not read as attributes
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(good)
    junk = (ctypes.c_char * 64)()
    assert lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, ctypes.addressof(junk)) == -8
    # a dropout mask without a keep probability below 1 (no attributes: keep_prob defaults to 1) is refused
    bad = list(good); bad[4] = (a, (1, 2, 128, 128), "float16")
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(bad)
    assert lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, None) == -8
    # backward: dq, dk, dv all in the operands' dtype or all float32; a workspace output is required unless the
    # attributes allow the shared built-in scratch
    g = [(a, sh, "float16")] * 5 + [(a, sh[:3], "float32")] + [(None, (), "float16")] * 3 + [(a, sh, "float16")] * 3
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(g)
    assert lib.FlashAttentionGrad(n, params, ndims, shapes, dtypes, None, None) == -7
    mixed = list(g); mixed[10] = (a, sh, "float32")
    n, params, ndims, shapes, dtypes, _keep = ms_call_args(mixed)
    assert lib.FlashAttentionGrad(n, params, ndims, shapes, dtypes, None, None) == -3
    # the accessor hook: the maintainer's init glue maps MindSpore's `extra` to the attribute block
    at = MsAttrs(MsAttrs.MAGIC, 65536, 65536, 1.0, 1.0, 0)
    ACC = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_void_p)
    acc = ACC(lambda extra: ctypes.addressof(at))
    lib.acct_ms_set_attrs_accessor.argtypes = [ACC]
    lib.acct_ms_set_attrs_accessor.restype = None
    lib.acct_ms_set_attrs_accessor(acc)
    try:
        n, params, ndims, shapes, dtypes, _keep = ms_call_args(good)
        rc = lib.FlashAttentionFwd(n, params, ndims, shapes, dtypes, None, ctypes.addressof(junk))
        assert rc != -8                                    # the attributes were accepted (the call then needs a device)
    finally:
        lib.acct_ms_set_attrs_accessor(ctypes.cast(None, ACC))
