"""SparseSemiStructuredTensor / to_sparse_semi_structured on the gfx950 2:4 library.

Mirrors the public surface of sparse/semi_structured.py of huyz2023/2by4-pretrain (class
:33-572, factory :575-631): same constructor arguments, attributes, dispatch rules and error
behaviour.  Differences, all deliberate:
  * one backend (hand-written HIP on SMFMAC); `_FORCE_CUTLASS` / `_FUSE_TRANSPOSE` are kept as
    inert attributes, `compressed_tensor_cusparselt` is always None;
  * the compressed operand is STORED in the panel layout the SMFMAC matmul streams (tf24.h:
    TF24_COMPRESSED_PANEL; class flag `_PANEL_LAYOUT`); `values()` / `indices()` /
    `sparse_tensor_cutlass` / `meta_tensor_cutlass` materialise the canonical row-major form
    (values [m, k/2], nibble metadata [m, k/16 | k/32]) on first use, also for column-major
    inputs (`W.T`); the metadata is the canonical nibble stream by default, and CUTLASS's reordered
    layout -- what the reference stores, returns from `indices()` and takes as `meta_tensor_cutlass=`
    (semi_structured.py:536-546, :133-144) -- when the class flag `_CUTLASS_METADATA` is set;
    `indices_cutlass()` / `indices_canonical()` give either form regardless of the flag;
  * MVUE24 takes its uniforms from an optional `rand` tensor, or generates them inside the kernel from
    (seed, offset) -- `rand=(seed, offset)`, or torch's generator state when `rand` is omitted;
  * `addmm` / `linear` with a bias work (the reference passes a wrong keyword there).
"""
import ctypes
import warnings
from collections import namedtuple
from typing import Any, Optional

import torch

from . import _native as N

__all__ = ["SparseSemiStructuredTensor", "to_sparse_semi_structured", "to_sparse_semi_structured_pair",
           "to_sparse_semi_structured_with_row_sums", "mvue_device_state"]

_Config = namedtuple("_SEMI_STRUCTURED_SPARSE_CONFIG",
                     "compression_factor sparse_min_rows sparse_min_cols dense_min_rows dense_min_cols")
# semi_structured.py:24-30 of the reference, restricted to what SMFMAC kernels exist for
_DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG = {
    torch.float8_e4m3fn: _Config(10, 32, 128, 16, 16),
    torch.float8_e5m2: _Config(10, 32, 128, 16, 16),
    torch.int8: _Config(10, 32, 128, 16, 16),
    torch.float16: _Config(9, 32, 64, 8, 8),
    torch.bfloat16: _Config(9, 32, 64, 8, 8),
}


_FLOAT8 = (torch.float8_e4m3fn, torch.float8_e5m2)
_EIGHT_BIT = _FLOAT8 + (torch.int8,)          # 128 dense columns per panel, int32 metadata words


def _indices_dtype(values_dtype):
    if values_dtype in _EIGHT_BIT:
        return torch.int32
    if values_dtype in (torch.float16, torch.bfloat16):
        return torch.int16
    raise RuntimeError(f"Datatype {values_dtype}  is not supported!")


def _panel_width(dtype):
    """Dense columns per panel: 128 bytes of the value dtype."""
    return 128 // torch.empty((), dtype=dtype).element_size()


def _to_canonical(values, meta, m, n, want_values=True, want_meta=True):
    """Panel-layout storage -> canonical (values [m, n/2], meta [m, n/16 | n/32]); None for a part not wanted."""
    v = torch.empty_like(values) if want_values else None
    mt = torch.empty_like(meta) if want_meta else None
    N.check(N.lib().tf24_repack_to(values.data_ptr(), meta.data_ptr(), N.operand_code(values.dtype), m, n, N.COMPRESSED_PANEL,
                                   N.COMPRESSED_CANONICAL, N.ptr(v), N.ptr(mt), N.stream_ptr()))
    return (v.view(m, n // 2) if want_values else None), (mt.view(m, -1) if want_meta else None)


class _HostWords:
    """A ctypes array passed where the binding expects a tensor's data_ptr()."""
    def __init__(self, array):
        self.array = array

    def data_ptr(self):
        return ctypes.addressof(self.array)


_DEVICE_PHILOX = {}        # device index -> int64[2] device tensor {seed, offset}


def mvue_device_state(device=None, seed=None, offset=None):
    """The {seed, offset} pair of MVUE24's in-kernel generator as a 2-element int64 tensor ON the device.

    A sampling call that is given this tensor as `rand` reads the pair when its kernel runs and leaves
    offset += 4 behind, in stream order -- so a HIP graph that holds MVUE24 conversions draws fresh,
    reproducible uniforms on every replay (a (seed, offset) pair of host integers would be frozen into
    the graph).  While a stream is being captured, MVUE24 conversions without an explicit `rand` use this
    state; it has to exist before the capture starts: call this function first (it allocates and
    copies).  `seed` / `offset` (re)initialise the state; by default it is created once from torch's
    generator for the device (torch.manual_seed applies) and returned unchanged afterwards."""
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    state = _DEVICE_PHILOX.get(index)
    if state is None or seed is not None or offset is not None:
        gen = torch.cuda.default_generators[index]
        s = gen.initial_seed() if seed is None else int(seed)
        o = (gen.get_offset() if state is None else 0) if offset is None else int(offset)
        signed = [v - (1 << 64) if v >= (1 << 63) else v for v in (s & (2 ** 64 - 1), o & (2 ** 64 - 1))]
        words = torch.tensor(signed, dtype=torch.int64)
        if state is None:
            state = _DEVICE_PHILOX[index] = words.to(torch.device("cuda", index))
        else:
            state.copy_(words)
    return state


def _next_philox_state(device):
    """(seed, offset) of torch's generator for `device`, advancing its offset the way a random op does,
    so that torch.manual_seed() makes the default MVUE24 sampling reproducible.  Under stream capture:
    the device-resident state of mvue_device_state()."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if torch.cuda.is_current_stream_capturing():
        state = _DEVICE_PHILOX.get(index)
        if state is None:
            raise RuntimeError("MVUE24 under HIP graph capture takes its generator state from device memory: "
                               "call sparse.mvue_device_state() once before the capture starts")
        return state
    gen = torch.cuda.default_generators[index]
    offset = gen.get_offset()
    gen.set_offset(offset + 4)
    return gen.initial_seed(), offset


def _compress(original, dtype, MVUE24, mask, rand, panel, row_sums=False):
    """One allocation of numel*cf/16 elements: values first, metadata in the tail
    (reference :215-243); then the HIP prune+compress kernel.  Returns flat storage views; with
    `row_sums` (column-major input only) also original.sum(1), taken from the same read."""
    m, n = original.shape
    cfg = _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG[dtype]
    buf = torch.empty((original.nelement() * cfg.compression_factor // 16,), dtype=dtype, device=original.device)
    values = buf[: m * n // 2]
    meta = buf[m * n // 2:].view(_indices_dtype(dtype))

    if (dtype == torch.int8) != (original.dtype == torch.int8):
        raise RuntimeError(f"int8 values are taken from an int8 dense tensor only (tensor {original.dtype}, dtype {dtype})")
    if dtype == torch.int8 and MVUE24:
        raise RuntimeError("MVUE24 rescales the kept values and is not defined for int8")
    dense = N.as_matrix(original)
    layout, ld = N.layout_of(dense)
    if dtype == torch.int8 and layout == N.COL_MAJOR and ld % 16:
        dense = dense.contiguous()                   # column-major int8 is read 16 rows at a time
        layout, ld = N.layout_of(dense)
    if dtype == torch.int8 and mask is not None and mask.dtype not in (torch.bool, torch.uint8):
        mask = mask != 0                             # int8 matrices take byte masks
    mode, mask_t, rand_t = N.PRUNE_MAGNITUDE, None, None
    mask_ld = rand_ld = 0
    mask_code = N.U8
    if mask is not None:
        if mask.shape != original.shape:
            raise RuntimeError(f"mask shape {tuple(mask.shape)} does not match tensor shape {tuple(original.shape)}")
        mode = N.PRUNE_MASK
        mask_t = N.as_matrix(mask, like=dense)
        mask_ld = N.layout_of(mask_t)[1]
        mask_code = N.dtype_code(mask_t.dtype)
    elif MVUE24:
        mode = N.PRUNE_MVUE
        if rand is None:
            rand = _next_philox_state(dense.device)  # uniforms generated inside the kernel
        if isinstance(rand, torch.Tensor) and rand.dtype in (torch.int64, torch.uint64) and rand.numel() == 2:
            if not rand.is_cuda or not rand.is_contiguous():
                raise RuntimeError("the {seed, offset} state tensor of MVUE24 must be a contiguous device tensor")
            mode = N.PRUNE_MVUE_SEEDED_DEVICE        # read by the kernel; the call leaves offset += 4 behind
            rand_t = rand
        elif isinstance(rand, tuple):
            mode = N.PRUNE_MVUE_SEEDED
            seed_offset = (ctypes.c_uint64 * 2)(int(rand[0]) & (2 ** 64 - 1), int(rand[1]) & (2 ** 64 - 1))
            rand_t = _HostWords(seed_offset)         # read by the library during the call
        else:
            if tuple(rand.shape) == (m, n // 2):
                mode = N.PRUNE_MVUE_PACKED           # group g of a row uses rand[r, 2g], rand[r, 2g+1]
            elif rand.shape != original.shape:
                raise RuntimeError(f"rand shape {tuple(rand.shape)} does not match tensor shape {tuple(original.shape)} "
                                   f"(or its packed form {(m, n // 2)})")
            rand_t = N.as_matrix(rand.float(), like=dense)
            rand_ld = N.layout_of(rand_t)[1]
    if row_sums:
        sums = torch.empty((m,), dtype=dense.dtype, device=dense.device)
        ws_bytes = N.lib().tf24_prune_compress_rowsum_workspace_bytes(m, n)
        workspace = torch.empty((ws_bytes // 4,), dtype=torch.float32, device=dense.device)
        N.check(N.lib().tf24_prune_compress_rowsum(
            dense.data_ptr(), N.operand_code(dense.dtype), layout, ld, m, n, mode,
            N.ptr(mask_t), mask_code, mask_ld, N.ptr(rand_t), rand_ld,
            values.data_ptr(), N.operand_code(dtype), meta.data_ptr(),
            N.COMPRESSED_PANEL if panel else N.COMPRESSED_CANONICAL,
            sums.data_ptr(), N.dtype_code(sums.dtype), workspace.data_ptr(), ws_bytes, N.stream_ptr()))
        return values, meta, sums
    N.check(N.lib().tf24_prune_compress(
        dense.data_ptr(), N.operand_code(dense.dtype), layout, ld, m, n, mode,
        N.ptr(mask_t), mask_code, mask_ld, N.ptr(rand_t), rand_ld,
        values.data_ptr(), N.operand_code(dtype), meta.data_ptr(),
        N.COMPRESSED_PANEL if panel else N.COMPRESSED_CANONICAL, N.stream_ptr()))
    return values, meta


_WORKSPACE_BYTES = {}      # (dtype, n, k, j) -> tf24_spmm_workspace_bytes, a pure function of the shape


def _spmm(sparse, dense, sparse_first, bias=None, out_dtype=None, scale=1.0, activation=N.ACT_NONE, keep_panel=True):
    """sparse_first: out = S @ dense  (S [n,k], dense [k,j])  -> [n, j]
       otherwise   : out = dense @ S^T (dense [j,k])          -> [j, n]
    keep_panel: an operand that arrives in canonical or CUTLASS form is repacked to the panel form; keep
    that copy in the wrapper (the wrapper owns its tensors) or drop it after the product (the wrapper
    only borrows tensors its caller may rewrite)."""
    values, meta, store_layout = sparse._store_values, sparse._store_meta, sparse._store_layout
    n, k = sparse._store_shape
    # An operand built from canonical values/metadata (the functional entry point) is brought to the
    # panel form once: the tiled kernel only streams that one.
    if store_layout != N.COMPRESSED_PANEL and n >= 64 and k % _panel_width(values.dtype) == 0:
        pv, pm = torch.empty_like(values), torch.empty_like(meta)
        N.check(N.lib().tf24_repack_to(values.data_ptr(), meta.data_ptr(), N.operand_code(values.dtype), n, k, store_layout,
                                       N.COMPRESSED_PANEL, pv.data_ptr(), pm.data_ptr(), N.stream_ptr()))
        if keep_panel:
            sparse._set_storage(pv, pm, (n, k), N.COMPRESSED_PANEL)
        values, meta, store_layout = pv, pm, N.COMPRESSED_PANEL
    vdtype = values.dtype
    if dense.dtype != vdtype:
        raise RuntimeError(f"dense operand dtype {dense.dtype} does not match the sparse operand's {vdtype}")
    # (layout, leading dimension) of the dense operand as it lies, or of a contiguous copy when the kernels cannot
    # address it (N.as_matrix + N.layout_of, written out: this function is on the training step's host path)
    d0, d1 = dense.shape
    s0, s1 = dense.stride()
    if s1 == 1 and s0 >= d1 and s0 % 8 == 0 and dense.data_ptr() % 16 == 0:
        lay, ld = N.ROW_MAJOR, s0
    elif s0 == 1 and s1 >= d0 and s1 % 8 == 0 and dense.data_ptr() % 16 == 0:
        lay, ld = N.COL_MAJOR, s1
    else:
        dense = dense.contiguous()
        lay, ld = N.ROW_MAJOR, dense.stride(0)
    # When k is the strided dimension of the dense operand (`S @ dense` with a row-major dense, e.g.
    # dW = MVUE(dY^T) @ x) the tiled kernel reads 16-bit operands as they are, transposing while it
    # loads fragments.  For 8-bit operands it wants k contiguous: one transposing copy of the dense
    # operand is far cheaper than running the general kernel.
    k_strided = (lay == N.ROW_MAJOR) if sparse_first else (lay == N.COL_MAJOR)
    if k_strided and store_layout == N.COMPRESSED_PANEL and dense.numel() // k <= 64:
        # a few dense columns: the kernels for them want k contiguous, and the operand is tiny
        flipped = (dense if sparse_first else dense.t()).t().contiguous()       # [j, k]
        dense = flipped.t() if sparse_first else flipped
        lay, ld = N.layout_of(dense)
    elif k_strided and dense.element_size() == 1 and store_layout == N.COMPRESSED_PANEL and dense.numel() >= (1 << 16):
        v = 16 // dense.element_size()
        row_major = dense if sparse_first else dense.t()          # the view that is row-major: [k, j]
        if row_major.shape[0] % v == 0 and row_major.shape[1] % v == 0:
            flipped = N.transposed_copy(row_major)                # [j, k], k contiguous
        else:
            flipped = row_major.t().contiguous()
        dense = flipped.t() if sparse_first else flipped
        lay, ld = N.layout_of(dense)
    if sparse_first:
        kk, j = dense.shape
        b_layout = N.COL_MAJOR if lay == N.ROW_MAJOR else N.ROW_MAJOR   # k strided when the [k,j] tensor is row-major
        c_layout, out_shape = N.ROW_MAJOR, (n, j)
    else:
        j, kk = dense.shape
        b_layout = N.ROW_MAJOR if lay == N.ROW_MAJOR else N.COL_MAJOR
        c_layout, out_shape = N.COL_MAJOR, (j, n)
    if kk != k:
        raise RuntimeError(f"inner dimensions do not match: sparse operand has k={k}, dense operand {tuple(dense.shape)}")
    if out_dtype is None:
        out_dtype = torch.int32 if vdtype == torch.int8 else torch.float32 if vdtype in _FLOAT8 else vdtype
    device = dense.device
    out = torch.empty(out_shape, dtype=out_dtype, device=device)
    if bias is not None:
        if bias.dtype != out_dtype or not bias.is_contiguous():
            bias = bias.to(out_dtype).contiguous()
        if bias.numel() != n:
            raise RuntimeError(f"bias must have {n} elements, got {bias.numel()}")
    code = N.operand_code(vdtype)
    lib = N.lib()
    ws_key = (vdtype, n, k, j)
    ws_bytes = _WORKSPACE_BYTES.get(ws_key)
    if ws_bytes is None:
        ws_bytes = _WORKSPACE_BYTES[ws_key] = lib.tf24_spmm_workspace_bytes(code, n, k, j)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=device) if ws_bytes else None
    N.check(lib.tf24_spmm(
        values.data_ptr(), meta.data_ptr(), store_layout, code, n, k,
        dense.data_ptr(), b_layout, ld, j, out.data_ptr(), N.operand_code(out_dtype), c_layout, out_shape[1],
        None if bias is None else bias.data_ptr(), float(scale), activation,
        None if workspace is None else workspace.data_ptr(), ws_bytes, N.stream_ptr()))
    return out


def _dense_times_sparse_t(dense2d, sparse, bias=None):
    """dense2d @ S.t() (+ bias): what `torch.mm(x, S.t())` / `torch.addmm(bias, x, S.t())` dispatch to, without
    building the transposed wrapper and without the dispatcher round trip (some 40 us of host time per
    product, which a training step that is bound by its launch rate pays three times)."""
    rows, cols = dense2d.shape
    cfg = _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG[dense2d.dtype]
    padded = dense2d if rows % cfg.dense_min_rows == 0 and cols % cfg.dense_min_cols == 0 else sparse._pad_tensor_for_matmul(dense2d)
    out_dtype = sparse._FP8_OUT_DTYPE if sparse._store_values.dtype in _FLOAT8 else None
    out = _spmm(sparse, padded, False, bias=bias, out_dtype=out_dtype)
    return out if padded is dense2d else out[:rows, :]


class SparseSemiStructuredTensor(torch.Tensor):
    """2:4 semi-structured sparse matrix as a wrapper tensor subclass: logically the dense
    [m, k] matrix, physically `sparse_tensor_cutlass` (kept values [m, k/2]) and
    `meta_tensor_cutlass` (2-bit positions, int16 [m, k/16] or int32 [m, k/32]).

    Supported ops: detach, t, mm, addmm, linear, values, indices; the sparse operand must be the
    first and untransposed or the second and transposed argument."""

    _FUSE_TRANSPOSE = False
    _FORCE_CUTLASS = True
    _PROTOTYPE_WARNING_SHOWN = False
    # output dtype of fp8 products (the reference's CUTLASS path returns float32)
    _FP8_OUT_DTYPE = torch.float32
    # store freshly compressed tensors in the SMFMAC panel layout (False: canonical row-major)
    _PANEL_LAYOUT = True
    # True: `indices()` / `meta_tensor_cutlass` return, and the `meta_tensor_cutlass=` constructor argument
    # is read as, the CUTLASS-reordered metadata of the reference (semi_structured.py:536-546; csrc
    # .cu:826-851) instead of the canonical nibble stream.  Set it before building tensors whose
    # metadata is exchanged with code written against the reference or upstream torch.sparse.
    _CUTLASS_METADATA = False

    @staticmethod
    def __new__(cls, original_tensor: Optional[torch.Tensor], original_shape: Optional[torch.Size] = None,
                compressed_tensor_cusparselt: Optional[torch.Tensor] = None,
                sparse_tensor_cutlass: Optional[torch.Tensor] = None,
                meta_tensor_cutlass: Optional[torch.Tensor] = None, transposed: bool = False,
                MVUE24: bool = False, mask: Optional[torch.Tensor] = None,
                dtype: Optional[torch.dtype] = None, rand: Optional[torch.Tensor] = None):
        assert compressed_tensor_cusparselt is None or (sparse_tensor_cutlass is None and meta_tensor_cutlass is None)
        cls._warn_once()
        if original_tensor is not None:
            previous, original_shape = original_tensor, original_tensor.shape
        elif compressed_tensor_cusparselt is not None:
            previous = compressed_tensor_cusparselt
        elif sparse_tensor_cutlass is not None:
            previous = sparse_tensor_cutlass
        else:
            raise ValueError("All of the tensor arguments are None!")
        return torch.Tensor._make_wrapper_subclass(
            cls, original_shape, device=previous.device, dtype=previous.dtype if dtype is None else dtype,
            layout=previous.layout, requires_grad=False)

    def __init__(self, original_tensor: Optional[torch.Tensor], original_shape: Optional[torch.Size] = None,
                 compressed_tensor_cusparselt: Optional[torch.Tensor] = None,
                 sparse_tensor_cutlass: Optional[torch.Tensor] = None,
                 meta_tensor_cutlass: Optional[torch.Tensor] = None, transposed: bool = False,
                 MVUE24: bool = False, mask: Optional[torch.Tensor] = None,
                 dtype: Optional[torch.dtype] = torch.float16, rand: Optional[torch.Tensor] = None) -> None:
        if original_tensor is not None:
            if not original_tensor.is_cuda:
                raise RuntimeError(f"Error original_tensor.device= {original_tensor.device} is not supported! "
                                   "Only CUDA tensors are currently supported.")
            if original_tensor.dim() != 2:
                raise RuntimeError(f"Error original_tensor.dim = {original_tensor.dim()} is not supported! "
                                   "Only 2d tensors are currently supported.")
            if dtype not in _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG:
                raise RuntimeError(f"Error dtype {dtype} is not a supported dtype! "
                                   f"dtype must be one of: {list(_DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG)}")
            m, n = original_tensor.shape
            cfg = _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG[dtype]
            if m < cfg.sparse_min_rows or m % cfg.sparse_min_rows or n < cfg.sparse_min_cols or n % cfg.sparse_min_cols:
                raise RuntimeError(f"Error original_tensor.shape {original_tensor.shape} is not supported! "
                                   "Both dimensions must be larger or equal than and a multiple of "
                                   f"({cfg.sparse_min_rows}, {cfg.sparse_min_cols})")
            if mask is not None and MVUE24:
                raise RuntimeError("Error using MVUE24 with mask is not supported! ")
            panel = bool(self._PANEL_LAYOUT)
            values, meta = _compress(original_tensor, dtype, MVUE24, mask, rand, panel)
            self._set_storage(values, meta, (m, n), N.COMPRESSED_PANEL if panel else N.COMPRESSED_CANONICAL)
        elif sparse_tensor_cutlass is not None:
            # built from pieces: values [m, k/2] row-major and metadata, canonical nibble stream or (class
            # flag) the reference's reordered words
            mm, half = sparse_tensor_cutlass.shape
            self._set_storage(sparse_tensor_cutlass.contiguous().view(-1), meta_tensor_cutlass.contiguous().view(-1),
                              (mm, 2 * half), N.COMPRESSED_CUTLASS if self._CUTLASS_METADATA else N.COMPRESSED_CANONICAL)
        else:
            self._set_storage(None, None, None, N.COMPRESSED_CANONICAL)
        self.original_tensor = None
        self.compressed_tensor_cusparselt = None
        self.transposed = transposed
        self.original_shape = original_shape

    def _set_storage(self, values, meta, shape, layout):
        self._store_values, self._store_meta = values, meta       # flat device tensors
        self._store_shape, self._store_layout = shape, layout     # (m, k) of the untransposed matrix

    def _canonical_pair(self, want_values=True, want_meta=True):
        """(values [m, k/2], canonical metadata) of the stored operand.  Made from the storage on every call
        (views where the storage is canonical, copies otherwise): the storage may be rewritten behind the
        wrapper's back -- a graph replay recompresses into the same buffers -- so nothing derived is kept."""
        m, n = self._store_shape
        if self._store_layout == N.COMPRESSED_PANEL:
            return _to_canonical(self._store_values, self._store_meta, m, n, want_values, want_meta)
        if self._store_layout == N.COMPRESSED_CUTLASS:
            return self._store_values.view(m, n // 2), (self._converted_meta(N.COMPRESSED_CANONICAL) if want_meta else None)
        return self._store_values.view(m, n // 2), self._store_meta.view(m, -1)

    def _converted_meta(self, to_layout):
        """The metadata in another storage form, [m, k/16 | k/32] words (HIP kernel; values untouched)."""
        m, n = self._store_shape
        out = torch.empty_like(self._store_meta)
        N.check(N.lib().tf24_repack_to(None, self._store_meta.data_ptr(), N.operand_code(self._store_values.dtype), m, n,
                                       self._store_layout, to_layout, None, out.data_ptr(), N.stream_ptr()))
        return out.view(m, -1)

    @property
    def sparse_tensor_cutlass(self):
        """Kept values, canonical [m, k/2] (the reference's attribute name)."""
        return None if self._store_values is None else self._canonical_pair(want_meta=False)[0]

    @property
    def meta_tensor_cutlass(self):
        """Metadata [m, k/16] int16 or [m, k/32] int32: the canonical nibble stream, or with the class flag
        `_CUTLASS_METADATA` the reference's reordered words."""
        if self._store_values is None:
            return None
        return self.indices_cutlass() if self._CUTLASS_METADATA else self._canonical_pair(want_values=False)[1]

    def __tensor_flatten__(self):
        return ["_store_values", "_store_meta"], (self.original_shape, self.transposed, self._store_shape, self._store_layout)

    @staticmethod
    def __tensor_unflatten__(inner_tensors, meta, outer_size, outer_stride):
        original_shape, transposed, store_shape, store_layout = meta
        if len(inner_tensors) != 2:
            raise RuntimeError(f"Expected 2 inner tensors but got {len(inner_tensors)}")
        return SparseSemiStructuredTensor._from_storage(
            inner_tensors["_store_values"], inner_tensors["_store_meta"], store_shape, store_layout, original_shape, transposed)

    @classmethod
    def _warn_once(cls):
        if not cls._PROTOTYPE_WARNING_SHOWN:
            warnings.warn(
                "The PyTorch API of SparseSemiStructuredTensor is in prototype stage and will change in the "
                "near future. Please open a Github issue for features requests and see our documentation on "
                "the torch.sparse module for further information about the project.", UserWarning)
            cls._PROTOTYPE_WARNING_SHOWN = True

    @classmethod
    def _from_storage(cls, values, meta, store_shape, store_layout, shape, transposed):
        """A wrapper around storage that already exists (flat values and metadata in `store_layout`): what the
        constructor builds from pieces, without its copies and checks -- the training layer makes six of these per step."""
        cls._warn_once()
        out = torch.Tensor._make_wrapper_subclass(cls, shape, device=values.device, dtype=values.dtype, layout=values.layout,
                                                  requires_grad=False)
        out._store_values, out._store_meta = values, meta
        out._store_shape, out._store_layout = store_shape, store_layout
        out.original_tensor = None
        out.compressed_tensor_cusparselt = None
        out.transposed = transposed
        out.original_shape = shape
        return out

    def __repr__(self) -> str:  # type: ignore[override]
        return (f"SparseSemiStructuredTensor(shape={self.shape}, transposed={self.transposed}"
                f"values={self.values()}metadata={self.indices()})")

    __torch_function__ = torch._C._disabled_torch_function_impl

    def _clone_view(self, shape, transposed):
        return SparseSemiStructuredTensor._from_storage(
            self._store_values, self._store_meta, self._store_shape, self._store_layout, shape, transposed)

    def _pad_tensor_for_matmul(self, original_tensor: torch.Tensor) -> torch.Tensor:
        """Zero-pads a 2-d dense operand to the multiples the kernel wants (reference :351-368)."""
        assert original_tensor.dim() == 2
        m, n = original_tensor.shape
        cfg = _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG[original_tensor.dtype]
        to_pad_m = -m % cfg.dense_min_rows
        to_pad_n = -n % cfg.dense_min_cols
        if to_pad_m or to_pad_n:
            return torch.nn.functional.pad(original_tensor, (0, to_pad_n, 0, to_pad_m))
        return original_tensor

    def _out_dtype(self):
        return self._FP8_OUT_DTYPE if self.dtype in _FLOAT8 else None

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs) -> Any:
        if func is torch.ops.aten.detach.default:
            return args[0]._clone_view(args[0].shape, args[0].transposed)

        # the compressed form cannot be transposed; only the number of transposes is tracked
        if func is torch.ops.aten.t.default:
            s = args[0]
            return s._clone_view(torch.Size([s.shape[1], s.shape[0]]), not s.transposed)

        if func is torch.ops.aten.addmm.default:
            bias, input_A, input_B = args
            # F.linear(x) = addmm(bias, x, W.t()) = (W x' + b')'
            if isinstance(input_B, cls) and input_B.transposed:
                row, _ = input_A.shape
                padded = input_B._pad_tensor_for_matmul(input_A)
                return _spmm(input_B, padded, False, bias=bias, out_dtype=input_B._out_dtype())[:row, :]

        if func is torch.ops.aten.mm.default:
            input_A, input_B = args
            if isinstance(input_A, cls) and not input_A.transposed:          # first operand sparse
                _, col = input_B.shape
                padded = input_A._pad_tensor_for_matmul(input_B)
                return _spmm(input_A, padded, True, out_dtype=input_A._out_dtype())[:, :col]
            if isinstance(input_B, cls) and input_B.transposed:              # second operand sparse
                row, _ = input_A.shape
                padded = input_B._pad_tensor_for_matmul(input_A)
                return _spmm(input_B, padded, False, out_dtype=input_B._out_dtype())[:row, :]

        # inference mode does not decompose linear into t + addmm
        if func is torch.ops.aten.linear.default:
            input_tensor, weight, bias = args
            if isinstance(weight, cls):
                shape = input_tensor.shape
                x2d = input_tensor.reshape(-1, shape[-1])
                row, _ = x2d.shape
                padded = weight._pad_tensor_for_matmul(x2d)
                res = _spmm(weight, padded, False, bias=bias, out_dtype=weight._out_dtype())
                return res[:row, :].view(*shape[:-1], -1)

        if func is torch.ops.aten.values.default:
            return args[0].sparse_tensor_cutlass.detach()

        if func is torch.ops.aten.indices.default:
            return args[0].meta_tensor_cutlass

        error_string = "\n".join([f"func {func} with args: "] + [f"arg{i}: {arg}" for i, arg in enumerate(args)])
        raise NotImplementedError(error_string)

    def to_dense(self):
        """Decompress to a dense [m, k] tensor of the value dtype (reference :554-572)."""
        values, meta = self._store_values, self._store_meta
        m, k = self._store_shape
        out = torch.empty((m, k), dtype=values.dtype, device=values.device)
        N.check(N.lib().tf24_decompress(values.data_ptr(), N.operand_code(values.dtype), meta.data_ptr(), self._store_layout,
                                        m, k, out.data_ptr(), N.stream_ptr()))
        return out

    def indices_canonical(self):
        """Metadata as the canonical nibble stream, whatever `_CUTLASS_METADATA` says."""
        return self._canonical_pair(want_values=False)[1]

    def indices_cutlass(self):
        """Metadata in the CUTLASS-reordered layout the reference's `indices()` returns
        (reorder_meta + ColumnMajorInterleaved<2>; csrc .cu:826-851; semi_structured.py:536-546)."""
        if self._store_layout == N.COMPRESSED_CUTLASS:
            m, _ = self._store_shape
            return self._store_meta.view(m, -1)
        return self._converted_meta(N.COMPRESSED_CUTLASS)


def to_sparse_semi_structured(original_tensor: torch.Tensor, transposed: bool = False, MVUE24: bool = False,
                              mask: Optional[torch.Tensor] = None, dtype: torch.dtype = torch.float16,
                              rand: Optional[torch.Tensor] = None) -> SparseSemiStructuredTensor:
    """Dense [m, k] device tensor -> SparseSemiStructuredTensor, pruned 2:4 along k.

    Without `mask`/`MVUE24` the two largest |x| of every 4 are kept (ties: larger index);
    `mask` (same shape, nonzero = keep) selects explicitly; `MVUE24=True` samples the
    minimum-variance unbiased estimator, taking its uniforms from `rand`: a tensor of the same shape
    (or the packed [m, k/2] form) in [0,1), or a (seed, offset) pair for uniforms generated inside the
    kernel, or the device-resident pair of mvue_device_state() (then graph replays draw fresh uniforms);
    when omitted, the pair is taken from torch's generator (torch.manual_seed applies).  `dtype` is the value dtype of the result
    (float16, bfloat16, float8_e4m3fn, float8_e5m2, or int8 for an int8 tensor).  Rows must be a
    multiple of 32, columns of 64 (128 for 8-bit values).  Same signature as the reference's factory (semi_structured.py:575-631)
    plus `rand`.
    """
    return SparseSemiStructuredTensor(
        original_tensor, original_shape=original_tensor.shape, transposed=transposed,
        MVUE24=MVUE24, mask=mask, dtype=dtype, rand=rand)


def to_sparse_semi_structured_pair(original_tensor: torch.Tensor, mask: torch.Tensor,
                                   dtype: torch.dtype = torch.float16):
    """(to_sparse_semi_structured(w, mask=mask, dtype=dtype), to_sparse_semi_structured(w.T, mask=mask.T, dtype=dtype))
    from one pass over w and mask: the two compressed copies a transposable-mask training layer
    rebuilds every optimizer step (README.md:165-166).  Both results are bit-identical to the
    separate calls.  w [m, k] row-major, both dimensions a multiple of 64 (128 for float8); with
    any other input the two separate conversions run instead."""
    w = original_tensor
    if not w.is_cuda or w.dim() != 2 or dtype not in _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG or mask is None:
        return (to_sparse_semi_structured(w, mask=mask, dtype=dtype), to_sparse_semi_structured(w.T, mask=mask.T, dtype=dtype))
    m, k = w.shape
    unit = _panel_width(dtype)
    if mask.dtype == torch.bool:
        mask = mask.view(torch.uint8)
    lay_w, lay_m = N.layout_of(w), N.layout_of(mask) if mask.dim() == 2 and mask.shape == w.shape else None
    fits = (m >= unit and k >= unit and m % unit == 0 and k % unit == 0 and ((w.dtype == torch.int8) == (dtype == torch.int8))
            and w.dtype in (torch.float32, torch.float16, torch.bfloat16, torch.int8)
            and lay_w is not None and lay_m is not None and lay_w[0] == N.ROW_MAJOR and lay_m[0] == N.ROW_MAJOR
            and lay_w[1] % 8 == 0 and lay_m[1] % 8 == 0 and w.data_ptr() % 16 == 0 and mask.data_ptr() % 16 == 0
            and mask.dtype in N._DTYPES and SparseSemiStructuredTensor._PANEL_LAYOUT)
    if not fits:
        return (to_sparse_semi_structured(w, mask=mask, dtype=dtype), to_sparse_semi_structured(w.T, mask=mask.T, dtype=dtype))
    cfg = _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG[dtype]
    per = w.nelement() * cfg.compression_factor // 16
    buf = torch.empty((2 * per,), dtype=dtype, device=w.device)          # [values | meta | values_t | meta_t]
    half = m * k // 2
    values, meta = buf[:half], buf[half:per].view(_indices_dtype(dtype))
    values_t, meta_t = buf[per:per + half], buf[per + half:].view(_indices_dtype(dtype))
    N.check(N.lib().tf24_prune_compress_dual(
        w.data_ptr(), N.operand_code(w.dtype), lay_w[1], m, k, mask.data_ptr(), N.dtype_code(mask.dtype), lay_m[1],
        values.data_ptr(), meta.data_ptr(), values_t.data_ptr(), meta_t.data_ptr(),
        N.operand_code(dtype), N.COMPRESSED_PANEL, N.stream_ptr()))
    s = SparseSemiStructuredTensor._from_storage(values, meta, (m, k), N.COMPRESSED_PANEL, torch.Size((m, k)), False)
    s_t = SparseSemiStructuredTensor._from_storage(values_t, meta_t, (k, m), N.COMPRESSED_PANEL, torch.Size((k, m)), False)
    return s, s_t


def to_sparse_semi_structured_with_row_sums(original_tensor: torch.Tensor, MVUE24: bool = False,
                                            mask: Optional[torch.Tensor] = None, dtype: torch.dtype = torch.float16,
                                            rand: Optional[torch.Tensor] = None):
    """(to_sparse_semi_structured(t, MVUE24=..., mask=..., dtype=..., rand=...), t.sum(1)).

    For a column-major `t` (the `grad_output.t()` of the training layer's backward, README.md:190-197,
    where the row sums are the bias gradient `grad_output.sum(0)`) both results come from one pass over
    `t`; the sums are added in float32 and rounded once to t's dtype.  Any other input runs the
    conversion and torch's sum separately."""
    t = original_tensor
    cfg = _DTYPE_TO_SEMI_STRUCTURED_SPARSE_CONFIG.get(dtype)
    fusable = (t.is_cuda and t.dim() == 2 and cfg is not None and t.dtype in (torch.float32, torch.float16, torch.bfloat16)
               and dtype != torch.int8 and not (mask is not None and MVUE24) and SparseSemiStructuredTensor._PANEL_LAYOUT)
    if fusable:
        m, n = t.shape
        lay = N.layout_of(t)
        fusable = (m >= cfg.sparse_min_rows and m % cfg.sparse_min_rows == 0 and n >= cfg.sparse_min_cols
                   and n % cfg.sparse_min_cols == 0 and lay is not None and lay[0] == N.COL_MAJOR and lay[1] % 8 == 0
                   and t.data_ptr() % 16 == 0 and t.stride(0) == 1)
    if not fusable:
        return (to_sparse_semi_structured(t, MVUE24=MVUE24, mask=mask, dtype=dtype, rand=rand), t.sum(1))
    values, meta, sums = _compress(t, dtype, MVUE24, mask, rand, True, row_sums=True)
    return SparseSemiStructuredTensor._from_storage(values, meta, (m, n), N.COMPRESSED_PANEL, torch.Size((m, n)), False), sums
