"""HIP graph capture of the 2:4 training path: the MVUE24 generator state in device memory (fresh
uniforms on every replay) and one whole training step of the MLP of config 4 replayed against the same
steps run eagerly."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F16 = torch.float16


def _full_uniforms(seed, offset, m, k):
    packed = oracle.mvue_uniforms(seed, offset, m, k)
    full = torch.zeros(m, k)
    full[:, 0::4], full[:, 1::4] = packed[:, 0::2], packed[:, 1::2]
    return full


@pytest.mark.parametrize("col_major", [False, True])
def test_mvue_generator_state_on_the_device(cuda, col_major):
    """rand = the {seed, offset} tensor of mvue_device_state(): the kernel reads the pair from device memory and
    the call leaves offset += 4 behind; every call equals the oracle's MVUE24 on the oracle's Philox uniforms
    at the offset it found.  Also through the C ABI with the pair at an arbitrary device address."""
    import sparse
    from sparse import _native as N
    m, k = 96, 320
    seed, offset = 0x1234567890abcdef, 40
    g = torch.Generator().manual_seed(31)
    w = torch.randn(m, k, generator=g).half()
    wd = w.to(cuda)
    if col_major:
        wd = wd.t().contiguous().t()
    state = sparse.mvue_device_state(cuda, seed=seed, offset=offset)
    assert state.dtype == torch.int64 and state.is_cuda and state.numel() == 2
    assert sparse.mvue_device_state(cuda) is state
    for call in range(3):
        s = sparse.to_sparse_semi_structured(wd, MVUE24=True, dtype=F16, rand=state)
        want_v, want_m, _ = oracle.mvue24(w, _full_uniforms(seed, offset + 4 * call, m, k), out_dtype=F16)
        assert s.values().cpu().view(torch.int16).equal(want_v.view(torch.int16)), call
        assert s.indices().cpu().equal(want_m), call
        same = sparse.to_sparse_semi_structured(wd, MVUE24=True, dtype=F16, rand=(seed, offset + 4 * call))
        assert same.values().equal(s.values()) and same.indices().equal(s.indices())
    got = state.cpu().view(torch.uint64)
    assert int(got[0]) == seed and int(got[1]) == offset + 12
    if col_major:       # the fused conversion + row sums of the training layer's backward
        s2, sums = sparse.to_sparse_semi_structured_with_row_sums(wd, MVUE24=True, dtype=F16, rand=state)
        want_v, want_m, _ = oracle.mvue24(w, _full_uniforms(seed, offset + 12, m, k), out_dtype=F16)
        assert s2.values().cpu().view(torch.int16).equal(want_v.view(torch.int16)) and s2.indices().cpu().equal(want_m)
        assert int(state.cpu()[1]) == offset + 16
    # C ABI: the pair anywhere in device memory (8-byte aligned)
    raw = torch.zeros(5, dtype=torch.int64, device=cuda)
    raw[3], raw[4] = 77, 1000
    values = torch.empty(m * k // 2, dtype=F16, device=cuda)
    meta = torch.empty(m * k // 16, dtype=torch.int16, device=cuda)
    lay, ld = N.layout_of(wd)
    N.check(N.lib().tf24_prune_compress(wd.data_ptr(), N.F16, lay, ld, m, k, N.PRUNE_MVUE_SEEDED_DEVICE, None, N.U8, 0,
                                        raw.data_ptr() + 24, 0, values.data_ptr(), N.F16, meta.data_ptr(), N.COMPRESSED_CANONICAL,
                                        N.stream_ptr()))
    want_v, want_m, _ = oracle.mvue24(w, _full_uniforms(77, 1000, m, k), out_dtype=F16)
    assert values.cpu().view(m, k // 2).view(torch.int16).equal(want_v.view(torch.int16)) and meta.cpu().view(m, -1).equal(want_m)
    assert raw.cpu().tolist() == [0, 0, 0, 77, 1004]
    with pytest.raises(RuntimeError):
        N.check(N.lib().tf24_prune_compress(wd.data_ptr(), N.F16, lay, ld, m, k, N.PRUNE_MVUE_SEEDED_DEVICE, None, N.U8, 0,
                                            raw.data_ptr() + 4, 0, values.data_ptr(), N.F16, meta.data_ptr(), N.COMPRESSED_CANONICAL,
                                            N.stream_ptr()))


def test_mvue_in_a_graph_draws_fresh_uniforms_on_every_replay(cuda):
    """An MVUE24 conversion recorded into a HIP graph (no `rand`: under capture the device-resident state is
    used): every replay -- with eager work and synchronisations between the replays -- gives the oracle's
    result at the offset the state held, and replays differ from each other."""
    import sparse
    m, k = 128, 512
    seed, offset = 2024, 8
    g = torch.Generator().manual_seed(32)
    w = torch.randn(m, k, generator=g).half()
    wd = w.to(cuda).t().contiguous().t()            # column-major, as dY^T in the layer's backward
    state = sparse.mvue_device_state(cuda, seed=seed, offset=offset)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sparse.to_sparse_semi_structured_with_row_sums(wd, MVUE24=True, dtype=F16, rand=state)       # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    offset += 4
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s, sums = sparse.to_sparse_semi_structured_with_row_sums(wd, MVUE24=True, dtype=F16)
    assert int(state.cpu()[1]) == offset                        # capture itself ran nothing
    seen = []
    for replay in range(4):
        graph.replay()
        torch.cuda.synchronize()
        values, meta = s.values().cpu().clone(), s.indices().cpu().clone()
        want_v, want_m, _ = oracle.mvue24(w, _full_uniforms(seed, offset + 4 * replay, m, k), out_dtype=F16)
        assert values.view(torch.int16).equal(want_v.view(torch.int16)) and meta.equal(want_m), replay
        assert torch.allclose(sums.float().cpu(), w.float().sum(1), rtol=2e-3, atol=2e-2)
        assert all(not values.equal(v) for v in seen)
        seen.append(values)
        # eager work between the replays (its own host-side pair: the device state is untouched)
        eager = sparse.to_sparse_semi_structured(wd, MVUE24=True, dtype=F16, rand=(seed, 12345))
        torch.mm(torch.ones(8, k, dtype=F16, device=cuda), eager.t())
        torch.cuda.synchronize()
    assert int(state.cpu()[1]) == offset + 16


@pytest.mark.parametrize("kind", ["sparse", "sparse_one_pass"])
def test_whole_training_step_replayed_from_graphs_equals_eager_steps(cuda, kind):
    """The config-4 training step (here 1024 tokens, 256 -> 512 -> 256, mask refresh every 4 steps) recorded into two
    HIP graphs (a step that refreshes the transposable masks, a step that does not) and replayed for 9 steps,
    against the same model stepped eagerly: masks, weights, biases and optimizer moments bit-equal after every
    step.  Both models draw MVUE24 uniforms from the same (seed, offset) sequence -- the eager one from torch's
    generator on the host, the replayed one from the state in device memory -- so any node of the graph that
    misbehaved on a replay (a memset node, a frozen offset, a stale mask buffer) would show.  kind "sparse": masked_add_
    + torch's fused AdamW; "sparse_one_pass": MaskedDecayAdamW with its step count on the device."""
    import bench
    kw = dict(tokens=1024, d=256, h=512, freq=4, capturable=True)
    eager = bench.MlpTrainer(kind, **kw)
    for _ in range(3):
        eager.step()
    graphed = bench.MlpTrainer(kind, **kw).capture(eager_steps=3)
    assert graphed.opt_steps == 3 and set(graphed.graphs) == {"refresh", "regular"}
    losses = []
    for step in range(3, 12):
        want = eager.step()
        got = graphed.replay_step()
        torch.cuda.synchronize()
        losses.append(got.item())
        assert got.item() == want.item(), step
        for pe, pg in zip(eager.params, graphed.params):
            assert torch.equal(pe, pg), step
            if hasattr(pe, "mask"):
                assert torch.equal(pe.mask, pg.mask), step
            se, sg = eager.opt.state[pe], graphed.opt.state[pg]
            assert torch.equal(se["exp_avg"], sg["exp_avg"]) and torch.equal(se["exp_avg_sq"], sg["exp_avg_sq"]), step
            assert float(se["step"]) == float(sg["step"]) == step + 1
    assert losses[-1] < losses[0]
    # the state moved on by 4 per MVUE24 conversion: two layers per step
    import sparse
    gen = torch.cuda.default_generators[0]
    assert int(sparse.mvue_device_state(cuda).cpu()[1]) == gen.get_offset()
