"""CPU-side checks of the C-ABI library and the Python boundary: the library loads without a
GPU, exports every symbol include/tf24.h declares, its host-only validators reproduce the
reference's argument errors, and the Python API fails loudly instead of falling back."""
import ctypes
import importlib.util
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tf24.h")


@pytest.fixture(scope="module")
def native():
    from sparse import _native
    if not os.path.exists(_native.library_path()):      # build only when nothing is built
        spec = importlib.util.spec_from_file_location("tf24_build", os.path.join(ROOT, "2by4-pretrain_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_library()
    return _native


def _declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(tf24_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(native):
    names = _declared_symbols()
    assert len(names) >= 13 and "tf24_spmm" in names and "tf24_prune_compress" in names
    handle = ctypes.CDLL(native.library_path())
    for name in names:
        assert hasattr(handle, name), f"{name} declared in tf24.h but not exported"
    # and the binding knows every declared entry point
    assert set(names) == set(native._SIGNATURES)


def test_version_and_error_string(native):
    assert native.version().startswith("tf24 ") and "gfx950" in native.version()
    lib = native.lib()
    rc = lib.tf24_prune_compress_validate(native.F16, native.ROW_MAJOR, 64, 33, 64, native.PRUNE_MAGNITUDE, 0, 0, 0, 0, 0, native.F16)
    assert rc == -1 and b"multiple of (32, 64)" in lib.tf24_last_error()


@pytest.mark.parametrize("m,k,out,ok", [(32, 64, 1, True), (32, 128, 3, True), (32, 64, 3, False), (48, 64, 1, False),
                                        (32, 96, 1, False), (16, 64, 1, False), (3072, 768, 1, True), (11008, 4096, 2, True)])
def test_compress_shape_rules(native, m, k, out, ok):
    # sparse/semi_structured.py:24-30,188-200: rows % 32, cols % 64 (16-bit) / 128 (8-bit), and at least that
    rc = native.lib().tf24_prune_compress_validate(native.F32, native.ROW_MAJOR, k, m, k, native.PRUNE_MAGNITUDE, 0, 0, 0, 0, 0, out)
    assert (rc == 0) == ok


def test_compress_argument_rules(native):
    lib, N = native.lib(), native
    ok = dict(in_dtype=N.BF16, layout=N.ROW_MAJOR, ld=64, m=32, k=64, mode=N.PRUNE_MAGNITUDE, has_mask=0, mask_dtype=N.U8, mask_ld=0,
              has_rand=0, rand_ld=0, out=N.F16)

    def call(**kw):
        a = dict(ok, **kw)
        return lib.tf24_prune_compress_validate(a["in_dtype"], a["layout"], a["ld"], a["m"], a["k"], a["mode"], a["has_mask"],
                                                a["mask_dtype"], a["mask_ld"], a["has_rand"], a["rand_ld"], a["out"])
    assert call() == 0
    assert call(in_dtype=N.E4M3) == -2 and call(out=N.F32) == -2 and call(out=N.U8) == -2
    assert call(layout=7) == -5 and call(mode=9) == -5
    assert call(ld=32) == -3 and call(ld=68) == -3                      # too small / not a multiple of 8
    assert call(layout=N.COL_MAJOR, ld=32) == 0 and call(layout=N.COL_MAJOR, ld=24) == -3
    assert call(mode=N.PRUNE_MASK) == -5                                 # mask missing
    assert call(mode=N.PRUNE_MASK, has_mask=1, mask_ld=64) == 0
    assert call(mode=N.PRUNE_MASK, has_mask=1, mask_ld=64, mask_dtype=N.E4M3) == -2
    assert call(mode=N.PRUNE_MVUE) == -5                                 # uniforms missing
    assert call(mode=N.PRUNE_MVUE, has_rand=1, rand_ld=64) == 0
    assert call(mode=N.PRUNE_MVUE, has_rand=1, rand_ld=64, has_mask=1, mask_ld=64) == -5   # MVUE with mask
    assert b"MVUE24 with mask" in lib.tf24_last_error()


def test_transposable_and_spmm_validators(native):
    lib, N = native.lib(), native
    assert lib.tf24_transposable_mask_validate(N.BF16, N.ROW_MAJOR, 64, 32, 64) == 0
    assert lib.tf24_transposable_mask_validate(N.BF16, N.ROW_MAJOR, 64, 33, 64) == -1       # transposable_semi_structured.py:60-63
    assert lib.tf24_transposable_mask_validate(N.BF16, N.ROW_MAJOR, 32, 32, 32) == -1       # :64-67
    assert lib.tf24_transposable_mask_validate(N.E4M3, N.ROW_MAJOR, 64, 32, 64) == -2       # :58-59
    assert lib.tf24_transposable_mask_validate(N.F32, N.COL_MAJOR, 32, 32, 64) == 0
    # csrc .cu:101-109: sparse rows % 32, k % 64 | 128, dense extent % 8 | 16
    sp = lambda dt, n, k, nd, **kw: lib.tf24_spmm_validate(dt, n, k, kw.get("bl", N.ROW_MAJOR), kw.get("ldb", k), nd,
                                                             kw.get("out", N.F16), kw.get("cl", N.COL_MAJOR), kw.get("ldc", n), kw.get("act", 0))
    assert sp(N.F16, 32, 64, 8) == 0 and sp(N.BF16, 11008, 4096, 8192) == 0 and sp(N.E4M3, 8192, 8192, 16384, out=N.BF16) == 0
    assert sp(N.F16, 48, 64, 8) == -1 and sp(N.F16, 32, 96, 8) == -1 and sp(N.F16, 32, 64, 12) == -1
    assert sp(N.E4M3, 32, 64, 16) == -1 and sp(N.E4M3, 32, 128, 8) == -1
    assert sp(N.F32, 32, 64, 8) == -2 and sp(N.F16, 32, 64, 8, out=N.E4M3) == -2
    assert sp(N.F16, 32, 64, 8, ldb=32) == -3 and sp(N.F16, 32, 64, 8, ldc=16) == -3
    # output rows leave as 16-byte segments: ldc % 8 for 16-bit results, % 4 for 32-bit ones
    assert sp(N.F16, 32, 64, 8, ldc=36) == -3 and sp(N.F16, 32, 64, 8, ldc=40) == 0 and sp(N.F16, 32, 64, 8, ldc=36, out=N.F32) == 0
    assert sp(N.F16, 32, 64, 8, ldb=1 << 23) == 0 and sp(N.F16, 32, 64, 8, ldb=(1 << 23) + 8) == -3     # rows of the dense operand: at most 16 MiB
    assert sp(N.E4M3, 32, 128, 16, ldb=1 << 24) == 0 and sp(N.E4M3, 32, 128, 16, ldb=(1 << 24) + 16) == -3
    assert sp(N.F16, 32, 64, 8, act=5) == -5 and sp(N.F16, 32, 64, 8, bl=3) == -5


def test_misaligned_pointers_are_refused_before_any_launch(native):
    """The kernels use 128-bit accesses: entry points return TF24_ERR_STRIDE for a misaligned
    pointer instead of launching (no GPU is touched on this path, the addresses are made up)."""
    lib, N = native.lib(), native
    ok, off = 0x7f0000001000, 0x7f0000001008
    spmm = lambda a=ok, b=ok, c=ok, meta=ok: lib.tf24_spmm(a, meta, N.COMPRESSED_PANEL, N.F16, 64, 64, b, N.ROW_MAJOR, 64, 64,
                                                           c, N.F16, N.COL_MAJOR, 64, None, 1.0, 0, None, 0, None)
    assert spmm(b=off) == -3 and spmm(a=off) == -3 and spmm(c=off) == -3 and spmm(meta=ok + 4) == -3
    assert b"aligned" in lib.tf24_last_error()
    pc = lambda dense=ok, values=ok: lib.tf24_prune_compress(dense, N.F16, N.ROW_MAJOR, 64, 32, 64, N.PRUNE_MAGNITUDE, None, N.U8, 0,
                                                             None, 0, values, N.F16, ok, N.COMPRESSED_PANEL, None)
    assert pc(dense=off) == -3 and pc(values=off) == -3
    assert lib.tf24_transposable_mask(off, N.F16, N.ROW_MAJOR, 64, 32, 64, 1, None, ok, None) == -3
    assert lib.tf24_soft_threshold24(ok, N.F16, N.ROW_MAJOR, 64, 32, 64, off, ok, None) == -3
    assert lib.tf24_transpose(ok, N.F16, 64, 64, 64, off, 64, None) == -3
    assert lib.tf24_decompress(off, N.F16, ok, N.COMPRESSED_CANONICAL, 32, 64, ok, None) == -3


def test_int8_validators(native):
    """int8 values come from int8 matrices, take byte masks and no MVUE; the integer product gives
    int32 with no activation or ReLU (.cu:594-637)."""
    lib, N = native.lib(), native
    pc = lambda **a: lib.tf24_prune_compress_validate(a.get("dt", N.I8), a.get("layout", N.ROW_MAJOR), a.get("ld", 128), 32, 128,
                                                      a.get("mode", N.PRUNE_MAGNITUDE), a.get("has_mask", 0), a.get("mdt", N.U8),
                                                      a.get("mld", 0), a.get("has_rand", 0), a.get("rld", 0), a.get("out", N.I8))
    assert pc() == 0 and pc(mode=N.PRUNE_MASK, has_mask=1, mld=128) == 0
    assert pc(out=N.F16) == -2 and pc(dt=N.F16) == -2                    # int8 <-> int8 only
    assert pc(mode=N.PRUNE_MASK, has_mask=1, mld=128, mdt=N.F32) == -2   # byte masks only
    assert pc(mode=N.PRUNE_MVUE, has_rand=1, rld=128) == -5
    assert pc(layout=N.COL_MAJOR, ld=40) == -3 and pc(layout=N.COL_MAJOR, ld=48) == 0
    sp = lambda **a: lib.tf24_spmm_validate(N.I8, 32, 128, N.ROW_MAJOR, 128, 16, a.get("out", N.I32), N.COL_MAJOR, 32, a.get("act", 0))
    assert sp() == 0 and sp(act=N.ACT_RELU) == 0
    assert sp(out=N.F32) == -2 and sp(act=N.ACT_SILU) == -5 and sp(act=N.ACT_GELU) == -5
    assert lib.tf24_spmm_validate(N.F16, 32, 64, N.ROW_MAJOR, 64, 8, N.I32, N.COL_MAJOR, 32, 0) == -2
    assert lib.tf24_prune_compress_dual_validate(N.I8, 128, 128, 128, N.U8, 128, N.I8, N.COMPRESSED_PANEL) == 0
    assert lib.tf24_prune_compress_dual_validate(N.I8, 128, 128, 128, N.U8, 128, N.E4M3, N.COMPRESSED_PANEL) == -2
    assert lib.tf24_prune_compress_dual_validate(N.I8, 64, 64, 64, N.U8, 64, N.I8, N.COMPRESSED_PANEL) == -1


def test_dual_compress_validator(native):
    """Both W [m,k] and W^T [k,m] must be compressible: m and k multiples of 64 (128 for 8-bit values)."""
    lib, N = native.lib(), native
    dual = lambda m, k, **kw: lib.tf24_prune_compress_dual_validate(
        kw.get("dt", N.F32), kw.get("ld", k), m, k, kw.get("mdt", N.U8), kw.get("mld", k), kw.get("out", N.F16),
        kw.get("lay", N.COMPRESSED_PANEL))
    assert dual(64, 64) == 0 and dual(3072, 768) == 0 and dual(768, 3072, out=N.BF16, lay=N.COMPRESSED_CANONICAL) == 0
    assert dual(128, 256, out=N.E4M3) == 0 and dual(128, 256, out=N.E5M2, mdt=N.F32) == 0
    assert dual(96, 128) == -1 and dual(128, 96) == -1 and dual(32, 64) == -1
    assert dual(64, 128, out=N.E4M3) == -1 and dual(128, 192, out=N.E4M3) == -1
    assert dual(64, 64, dt=N.U8) == -2 and dual(64, 64, out=N.F32) == -2 and dual(64, 64, mdt=N.E4M3) == -2
    assert dual(64, 64, ld=56) == -3 and dual(64, 64, mld=68) == -3
    assert dual(64, 64, lay=2) == -5
    assert b"tf24_prune_compress_dual" in lib.tf24_last_error()


def test_python_api_rejects_cpu_tensors(native):
    import sparse
    with pytest.raises(RuntimeError, match="Only CUDA tensors"):
        sparse.to_sparse_semi_structured(torch.zeros(32, 64, dtype=torch.float16))
    with pytest.raises(RuntimeError):
        sparse.TransposableSparse()(torch.zeros(32, 64))
    with pytest.raises(RuntimeError):
        sparse.soft_threshold24_triton(torch.zeros(32, 64))
    with pytest.raises(AssertionError):
        sparse.masked_add_(torch.zeros(4), torch.zeros(4), torch.zeros(4), alpha=0.1)
    with pytest.raises(ValueError):
        sparse.SparseSemiStructuredTensor(None)


def test_missing_library_fails_loudly(native, monkeypatch):
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "library_path", lambda: "/nonexistent/lib2by4_gfx950.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        native.lib()


def test_product_path_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "2by4-pretrain_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f


def test_reference_api_names_present():
    import sparse
    for name in ["to_sparse_semi_structured", "SparseSemiStructuredTensor", "TransposableSparse", "masked_add_",
                 "soft_threshold24_triton", "sparse24_triton", "MVUE24_approx_triton", "SparseLinearTranspose",
                 "sparse_linear_transpose"]:
        assert hasattr(sparse, name), name
    import inspect
    sig = inspect.signature(sparse.to_sparse_semi_structured)
    assert list(sig.parameters)[:5] == ["original_tensor", "transposed", "MVUE24", "mask", "dtype"]
    assert sig.parameters["dtype"].default is torch.float16
    cls = sparse.SparseSemiStructuredTensor
    assert cls._FORCE_CUTLASS is True and cls._FUSE_TRANSPOSE is False
