"""tf24_prune_compress_rowsum_static -- the entry point that allocates nothing (partial row sums in a
fixed array inside the library) -- against tf24_prune_compress_rowsum with a caller workspace, through
the C ABI: compressed values, metadata and row sums bit-equal, on two calls in a row, the second on
a smaller matrix (the array keeps the first call's contents), and once more on the first shape."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(cuda, m, k, mode, seed):
    from sparse import _native as N
    lib = N.lib()
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(k, m, generator=g).half().to(cuda).t()          # [m, k] column-major: the dY.t() of the backward pass
    so = (ctypes.c_uint64 * 2)(seed, 4 * seed)                        # {seed, offset} of the in-kernel uniforms
    rand = ctypes.addressof(so) if mode == N.PRUNE_MVUE_SEEDED else None

    def outputs():
        return (torch.empty(m * k // 2, dtype=torch.float16, device=cuda), torch.empty(m * k // 16, dtype=torch.int16, device=cuda),
                torch.empty(m, dtype=torch.float16, device=cuda))

    v0, m0, s0 = outputs()
    ws_bytes = lib.tf24_prune_compress_rowsum_workspace_bytes(m, k)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=cuda)
    N.check(lib.tf24_prune_compress_rowsum(t.data_ptr(), N.F16, N.COL_MAJOR, t.stride(1), m, k, mode, None, N.U8, 0, rand, 0,
                                           v0.data_ptr(), N.F16, m0.data_ptr(), N.COMPRESSED_PANEL, s0.data_ptr(), N.F16,
                                           ws.data_ptr(), ws_bytes, N.stream_ptr()))
    v1, m1, s1 = outputs()
    before = torch.cuda.memory_allocated(cuda)
    N.check(lib.tf24_prune_compress_rowsum_static(t.data_ptr(), N.F16, N.COL_MAJOR, t.stride(1), m, k, mode, None, N.U8, 0, rand, 0,
                                                  v1.data_ptr(), N.F16, m1.data_ptr(), N.COMPRESSED_PANEL, s1.data_ptr(), N.F16,
                                                  N.stream_ptr()))
    assert torch.cuda.memory_allocated(cuda) == before
    torch.cuda.synchronize()
    assert v1.view(torch.int16).equal(v0.view(torch.int16)), (m, k, "values")
    assert m1.equal(m0), (m, k, "metadata")
    assert s1.view(torch.int16).equal(s0.view(torch.int16)), (m, k, "row sums")
    want = t.float().sum(1)
    assert ((s1.float() - want).abs() <= 2e-3 * want.abs() + 0.05).all()


def test_static_scratch_matches_workspace_entry_point(cuda):
    from sparse import _native as N
    _both(cuda, 3072, 12288, N.PRUNE_MVUE_SEEDED, 11)      # config 4's c_fc gradient: 1.2 MiB of partial sums
    _both(cuda, 64, 256, N.PRUNE_MAGNITUDE, 12)            # smaller: the array still holds the first call's sums
    _both(cuda, 768, 12288, N.PRUNE_MVUE_SEEDED, 13)
    _both(cuda, 3072, 12288, N.PRUNE_MAGNITUDE, 14)


def test_static_scratch_rejects_what_does_not_fit(cuda):
    from sparse import _native as N
    lib = N.lib()
    limit = lib.tf24_prune_compress_rowsum_static_max_bytes()
    assert limit == 4 << 20
    m, k = 8192, 32768                                     # 8192 * 256 partial sums = 8 MiB
    assert lib.tf24_prune_compress_rowsum_workspace_bytes(m, k) > limit
    one = torch.zeros(16, device=cuda)
    rc = lib.tf24_prune_compress_rowsum_static(one.data_ptr(), N.F16, N.COL_MAJOR, m, m, k, N.PRUNE_MAGNITUDE, None, N.U8, 0, None, 0,
                                               one.data_ptr(), N.F16, one.data_ptr(), N.COMPRESSED_PANEL, one.data_ptr(), N.F16,
                                               N.stream_ptr())
    assert rc == -1 and b"built-in scratch" in lib.tf24_last_error()
