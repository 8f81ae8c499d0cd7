"""CPU-side checks of the C ABI: the library loads, exports every declared symbol, validates
arguments with the documented status codes (no kernel is launched), and its host tables equal
the oracle's and Hugging Face's golden tables bit for bit."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from turbodeberta_amd import _lib
from oracle import hf_eager as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "tdb_attn.h")).read()
    declared = set(re.findall(r"^\s*(?:const\s+char\*|int)\s+(tdb_\w+)\s*\(", header, re.M))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.tdb_version() == _lib.ABI_VERSION
    m = re.search(r"#define TDB_ABI_VERSION (\d+)", header)
    assert int(m.group(1)) == _lib.ABI_VERSION


def test_workgroup_limit_rounding():
    try:
        assert [_lib.set_workgroup_limit(n) for n in (1, 8, 15, 24, 250, 4096)] == [8, 8, 8, 24, 248, 4096]
        assert _lib.set_workgroup_limit(-3) == 0
    finally:
        assert _lib.set_workgroup_limit(0) == 0


def test_struct_layout_matches_header_field_order():
    header = open(os.path.join(ROOT, "include", "tdb_attn.h")).read()
    for cname, cls in (("tdb_pos_args", _lib.PosArgs), ("tdb_fixed_args", _lib.FixedArgs), ("tdb_varlen_args", _lib.VarlenArgs)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), header, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            # drop the type: everything up to the first declarator
            decl = re.sub(r"^(const\s+)?(int32_t|int64_t|float|void|tdb_pos_args)\s*\**", "", decl)
            names += [n.strip().lstrip("*").strip() for n in decl.split(",")]
        assert names == [f[0] for f in cls._fields_], cname


def test_host_tables_bit_exact(golden_dir):
    g = np.load(os.path.join(golden_dir, "hf_bucket_table.npz"))
    for key in g.files:
        if key.startswith("b"):
            b, p, l = (int(x[1:]) for x in key.split("_"))
            assert np.array_equal(_lib.bucket_table(l, b, p), g[key].astype(np.int32)), key
    for (b, p, l) in [(256, 512, 128), (256, 512, 512), (256, 512, 4096), (-1, 32, 100), (0, 64, 70), (16, 32, 40)]:
        assert np.array_equal(_lib.delta_table(l, b, p), O.delta_table(l, b, p)), (b, p, l)


def test_bucket_margin_refusal():
    # buckets 6 (mid 3), max_position 49: for |r| = 12 the ceil() argument is
    # log(12/3)/log(48/3)*2 = 1 exactly, so float32 rounding decides the bucket -> refused.
    with pytest.raises(ValueError, match="TDB_ERR_BUCKET_MARGIN"):
        _lib.bucket_table(60, 6, 49)
    _lib.bucket_table(12, 6, 49)        # |r| <= 11 never reaches the doubtful value


def test_check_cu_seqlens():
    ok = np.array([0, 3, 3, 10], dtype=np.int32)
    _lib.check_cu_seqlens(ok, 10, 7)
    for bad, total, mx in ((np.array([1, 3, 10]), 10, 9), (np.array([0, 5, 4, 10]), 10, 9),
                           (np.array([0, 3, 10]), 11, 9), (np.array([0, 3, 10]), 10, 6)):
        with pytest.raises(ValueError, match="TDB_ERR_CU_SEQLENS"):
            _lib.check_cu_seqlens(bad.astype(np.int32), total, mx)


def _fixed(**kw):
    a = _lib.FixedArgs()
    a.dtype, a.batch, a.heads, a.head_dim, a.seqlen = _lib.TDB_BF16, 2, 3, 64, 128
    a.sm_scale = 0.1
    a.q = a.k = a.v = a.o = 0x1000          # never dereferenced: validation fails first
    for nm in "qkvo":
        setattr(a, nm + "_stride_b", 3 * 128 * 64)
        setattr(a, nm + "_stride_h", 128 * 64)
        setattr(a, nm + "_stride_l", 64)
    for k, v in kw.items():
        obj = a
        *path, leaf = k.split(".")
        for p in path:
            obj = getattr(obj, p)
        setattr(obj, leaf, v)
    return a


@pytest.mark.parametrize("kw,err", [
    (dict(dtype=7), "TDB_ERR_DTYPE"),
    (dict(head_dim=12), "TDB_ERR_SHAPE"),
    (dict(head_dim=512), "TDB_ERR_SHAPE"),
    (dict(seqlen=0), "TDB_ERR_SHAPE"),
    (dict(heads=0), "TDB_ERR_SHAPE"),
    (dict(causal=1), "TDB_ERR_CAUSAL"),
    (dict(q=0), "TDB_ERR_NULL"),
    (dict(k=0x1004), "TDB_ERR_ALIGN"),
    (dict(q_stride_l=63), "TDB_ERR_STRIDE"),
    (dict(v_stride_l=32), "TDB_ERR_STRIDE"),
    (dict(o_stride_b=-64), "TDB_ERR_STRIDE"),
    ({"pos.pos_key": 0x2000, "pos.span": 0}, "TDB_ERR_POSITION"),
    ({"pos.pos_key": 0x2000, "pos.span": 256}, "TDB_ERR_POSITION"),                       # no LUT
    ({"pos.pos_key": 0x2000, "pos.span": 256, "pos.delta_lut": 0x3000, "pos.lut_half": 100}, "TDB_ERR_POSITION"),
    ({"pos.pos_key": 0x2000, "pos.c2p_strip": 0x4000, "pos.span": 256, "pos.delta_lut": 0x3000, "pos.lut_half": 511},
     "TDB_ERR_POSITION"),
    ({"pos.pos_query": 0x2002, "pos.span": 256, "pos.delta_lut": 0x3000, "pos.lut_half": 511}, "TDB_ERR_ALIGN"),
    ({"pos.pos_query": 0x2000, "pos.pos_query_stride_r": 60, "pos.span": 256, "pos.delta_lut": 0x3000,
      "pos.lut_half": 511}, "TDB_ERR_STRIDE"),
])
def test_fixed_argument_validation(kw, err):
    lib = _lib.load()
    a = _fixed(**kw)
    rc = lib.tdb_attn_fwd_fixed(C.byref(a), None)
    assert rc < 0 and _lib.ERROR_NAMES[rc] == err, (rc, lib.tdb_last_error())
    with pytest.raises(ValueError, match=err):
        _lib.check(rc)


def test_null_args_and_empty_batch():
    lib = _lib.load()
    assert _lib.ERROR_NAMES[lib.tdb_attn_fwd_fixed(None, None)] == "TDB_ERR_NULL"
    assert _lib.ERROR_NAMES[lib.tdb_attn_fwd_varlen(None, None)] == "TDB_ERR_NULL"
    assert lib.tdb_attn_fwd_fixed(C.byref(_fixed(batch=0)), None) == 0      # nothing to do, no launch


def test_varlen_argument_validation():
    lib = _lib.load()
    a = _lib.VarlenArgs()
    a.dtype, a.batch, a.heads, a.head_dim, a.total_tokens, a.max_seqlen = _lib.TDB_F32, 2, 2, 64, 100, 64
    a.q = a.k = a.v = a.o = 0x1000
    for nm in "qkvo":
        setattr(a, nm + "_stride_t", 128)
        setattr(a, nm + "_stride_h", 64)
    assert _lib.ERROR_NAMES[lib.tdb_attn_fwd_varlen(C.byref(a), None)] == "TDB_ERR_NULL"      # cu_seqlens
    a.cu_seqlens = 0x5000
    a.q_stride_t = 32
    assert _lib.ERROR_NAMES[lib.tdb_attn_fwd_varlen(C.byref(a), None)] == "TDB_ERR_STRIDE"
    a.q_stride_t = 128
    a.total_tokens = -1
    assert _lib.ERROR_NAMES[lib.tdb_attn_fwd_varlen(C.byref(a), None)] == "TDB_ERR_SHAPE"
    a.total_tokens = 0
    assert lib.tdb_attn_fwd_varlen(C.byref(a), None) == 0


def test_operators_refuse_cpu_tensors():
    import torch
    from turbodeberta_amd.ops.flash_attention import flash_attention_with_disentangled
    q = torch.zeros(1, 1, 8, 64)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        flash_attention_with_disentangled(q, q, q, None, None)
