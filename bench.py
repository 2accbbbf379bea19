"""Benchmark of the 2:4 sparse hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload spmm|train|fp8|int8|decode|traffic] [--no-cpu] [--no-convert] [--no-extra]

Default workload: BASELINE config 3 -- fp16 2:4 spMM forward  Y[8192,11008] = X[8192,4096] . W^T
(W[11008,4096] magnitude-pruned along K) plus the transposed product dX[8192,4096] = dY . W with
the transposable-masked W compressed along its other axis.  One "step" = those two matmuls.
Prints ONE JSON line: whole-step throughput, the dominant kernel's roofline (HIP-event timed in
the same region), the dense hipBLASLt GEMM on the same shapes, per-kernel GB/s of the conversion
kernels at BASELINE config 2 sizes, the fp8 product of configs[4] and the training step of configs[3]
with their dense comparators, and the CPU oracle timed on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "2by4-pretrain_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_DENSE_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA; SMFMAC executes MACs at this rate
MFMA_DENSE_PEAK_FP8_TFLOPS = 5000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "spmm_cfg3_hbm_traffic_counters.md")


def profiled_traffic():
    """Bytes that cross the L2 <-> memory-fabric boundary per spmm launch of config 3 (mean of forward and
    transposed), as the committed byte-counter summary records them: its `traffic_record:` line holds the
    FETCH_SIZE / WRITE_SIZE readings (KiB per dispatch) of two `rocprofv3 --pmc` runs of
    `bench.py --workload traffic`, the factors that a plain device copy of known size gives each counter
    in the same runs, and the commit whose kernels were profiled.  A profiled figure, not something this
    run measures: (bytes, source) or (None, reason)."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith("traffic_record:"):
                    r = json.loads(line[len("traffic_record:"):])
                    nbytes = int(r["fetch_kib"] * 1024 * r["fetch_factor"] + r["write_kib"] * 1024 * r["write_factor"])
                    return nbytes, (f"profiles/{os.path.basename(TRAFFIC_PROFILE)}: rocprofv3 --pmc FETCH_SIZE {r['fetch_kib']} KiB x {r['fetch_factor']} + "
                                    f"WRITE_SIZE {r['write_kib']} KiB x {r['write_factor']} per dispatch over `bench.py --workload traffic`, factors from the "
                                    f"128 MiB device copy of the same runs; kernels of commit {r['kernel_commit']}; L2 <-> fabric bytes (infinity cache behind it)")
    except (OSError, ValueError, KeyError) as ex:
        return None, f"no traffic record ({ex})"
    return None, "no traffic record in the profile summary"


def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


SETTLE_S = 0.4


def settle(fn, seconds=SETTLE_S):
    """Run fn back to back for `seconds` before a timed region.  The shader clock takes tens of
    milliseconds of continuous load to leave its idle state and settle at the sustained (power
    managed) frequency; timings taken in the first ~50 ms of load read 15-20% slow.  Every timed
    leg (ours, the hipBLASLt comparator, the conversion kernels) is settled the same way."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn(i); i += 1
        torch.cuda.synchronize()


def time_rotating(fn, nsets, iters, warmup, batch=10):
    """Device time per call of fn(i % nsets) in microseconds, HIP events on the current stream: `iters`
    timed launches in batches of `batch` back-to-back launches (an event pair around every single
    launch would put the launch latency of each kernel inside its own interval).  Returns the
    median, the mean, the fastest and the slowest of the batch means."""
    settle(lambda i: fn(i % nsets))
    for i in range(warmup):
        fn(i % nsets)
    nb = max(1, (iters + batch - 1) // batch)
    ev = _events(nb + 1)
    torch.cuda.synchronize()
    i = 0
    ev[0].record()
    for b in range(nb):
        for _ in range(batch):
            fn(i % nsets); i += 1
        ev[b + 1].record()
    torch.cuda.synchronize()
    per = sorted(ev[b].elapsed_time(ev[b + 1]) * 1e3 / batch for b in range(nb))
    return {"median": per[len(per) // 2] if len(per) % 2 else 0.5 * (per[len(per) // 2 - 1] + per[len(per) // 2]),
            "mean": sum(per) / len(per), "min": per[0], "max": per[-1], "launches": nb * batch}


# --------------------------------------------------------------------------------------------
def conversion_kernels(iters=100, warmup=16, nsets=8):
    """BASELINE config 2: W[8192,8192] bf16 ~ N(0,1) seed 1; direct C-ABI launches on preallocated
    buffers, inputs and outputs rotated over `nsets` buffer sets (8 x 128 MiB of the smallest input,
    8 x 256 MiB of the float32 ones) so that the 256 MB last-level cache cannot serve repeats."""
    from sparse import _native as N
    lib = N.lib()
    dev = torch.device("cuda:0")
    m = k = 8192
    n = m * k
    gen = torch.Generator(device=dev).manual_seed(1)
    W = [torch.randn(m, k, device=dev, generator=gen).bfloat16() for _ in range(nsets)]
    U = [torch.rand(m, k, device=dev, generator=gen) for _ in range(nsets)]
    G = [1e-3 * torch.randn(m, k, device=dev, generator=gen) for _ in range(nsets)]
    P = [w.float() for w in W]
    values = [torch.empty(m, k // 2, dtype=torch.float16, device=dev) for _ in range(nsets)]
    meta = [torch.empty(m, k // 16, dtype=torch.int16, device=dev) for _ in range(nsets)]
    sp = [torch.empty_like(w) for w in W]
    mk = [torch.empty_like(w) for w in W]
    bmask = [torch.empty(m, k, dtype=torch.bool, device=dev) for _ in range(nsets)]
    st = N.stream_ptr()

    def magnitude(i):
        N.check(lib.tf24_prune_compress(W[i].data_ptr(), N.BF16, N.ROW_MAJOR, k, m, k, N.PRUNE_MAGNITUDE, None, N.U8, 0,
                                        None, 0, values[i].data_ptr(), N.F16, meta[i].data_ptr(), N.COMPRESSED_PANEL, st))

    def magnitude_canonical(i):
        N.check(lib.tf24_prune_compress(W[i].data_ptr(), N.BF16, N.ROW_MAJOR, k, m, k, N.PRUNE_MAGNITUDE, None, N.U8, 0,
                                        None, 0, values[i].data_ptr(), N.F16, meta[i].data_ptr(), N.COMPRESSED_CANONICAL, st))

    def mvue(i):
        N.check(lib.tf24_prune_compress(W[i].data_ptr(), N.BF16, N.ROW_MAJOR, k, m, k, N.PRUNE_MVUE, None, N.U8, 0,
                                        U[i].data_ptr(), k, values[i].data_ptr(), N.F16, meta[i].data_ptr(), N.COMPRESSED_PANEL, st))

    def transposable(i):
        N.check(lib.tf24_transposable_mask(W[i].data_ptr(), N.BF16, N.ROW_MAJOR, k, m, k, 1, sp[i].data_ptr(),
                                           bmask[i].data_ptr(), st))

    def soft(i):
        N.check(lib.tf24_soft_threshold24(W[i].data_ptr(), N.BF16, N.ROW_MAJOR, k, m, k, sp[i].data_ptr(), mk[i].data_ptr(), st))

    def decay(i):
        N.check(lib.tf24_masked_add(G[i].data_ptr(), N.F32, P[i].data_ptr(), N.F32, bmask[i].data_ptr(), N.U8, n, 2e-4, st))

    def mask_compress(i):
        N.check(lib.tf24_prune_compress(P[i].data_ptr(), N.F32, N.ROW_MAJOR, k, m, k, N.PRUNE_MASK, bmask[i].data_ptr(), N.U8, k,
                                        None, 0, values[i].data_ptr(), N.F16, meta[i].data_ptr(), N.COMPRESSED_PANEL, st))

    values_t = [torch.empty(k, m // 2, dtype=torch.float16, device=dev) for _ in range(nsets)]
    meta_t = [torch.empty(k, m // 16, dtype=torch.int16, device=dev) for _ in range(nsets)]

    def mask_compress_pair(i):
        N.check(lib.tf24_prune_compress_dual(P[i].data_ptr(), N.F32, k, m, k, bmask[i].data_ptr(), N.U8, k,
                                             values[i].data_ptr(), meta[i].data_ptr(), values_t[i].data_ptr(),
                                             meta_t[i].data_ptr(), N.F16, N.COMPRESSED_PANEL, st))

    def copy(i):
        sp[i].copy_(W[i])

    # algorithmic bytes: every input read once, every output written once
    table = [
        ("magnitude_prune_compress_bf16_to_f16", magnitude, 2 * n + n + n // 8),
        ("magnitude_prune_compress_bf16_to_f16 (canonical row-major output instead of the matmul's panel layout)",
         magnitude_canonical, 2 * n + n + n // 8),
        ("mvue24_prune_compress_bf16_u32_to_f16", mvue, 2 * n + 4 * n + n + n // 8),
        ("transposable_mask_select_bf16", transposable, 2 * n + 2 * n + n),
        ("soft_threshold24_bf16", soft, 2 * n + 2 * n + 2 * n),
        ("masked_add_f32", decay, 4 * n + 4 * n + 4 * n + n),
        ("mask_prune_compress_f32_to_f16", mask_compress, 4 * n + n + n + n // 8),
        ("mask_prune_compress_W_and_WT_f32_to_f16 (both compressed copies from one read)", mask_compress_pair,
         4 * n + n + 2 * (n + n // 8)),
        ("device_copy_bf16 (practical HBM ceiling)", copy, 4 * n),
    ]
    out = []
    for i in range(nsets):
        transposable(i)     # masks for the decay / mask-compress legs
    for name, fn, nbytes in table:
        t = time_rotating(fn, nsets, iters, warmup)
        us = t["median"]
        gbps = nbytes / us / 1e3
        out.append({"kernel": name, "us": round(us, 2), "us_mean": round(t["mean"], 2), "us_min": round(t["min"], 2),
                    "us_max": round(t["max"], 2), "launches": t["launches"], "buffer_sets": nsets, "bytes": nbytes,
                    "GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)})
    return out


# --------------------------------------------------------------------------------------------
def spmm_workload(steps, warmup):
    """BASELINE config 3.  Returns (ms_per_step wall, per-kernel event times, extras)."""
    import sparse
    dev = torch.device("cuda:0")
    M, K, Nw = 8192, 4096, 11008
    gen = torch.Generator().manual_seed(3)
    X = torch.randn(M, K, generator=gen).half().to(dev)
    W = (0.02 * torch.randn(Nw, K, generator=gen)).half().to(dev)
    dY = torch.randn(M, Nw, generator=gen).half().to(dev)

    w_fwd = sparse.to_sparse_semi_structured(W)                        # magnitude 2:4 along K
    _, tmask = sparse.TransposableSparse()(W)                          # transposable mask
    w_bwd = sparse.to_sparse_semi_structured(W.T, mask=tmask.T)        # 2:4 copy along the other axis
    w_fwd_t, w_bwd_t = w_fwd.t(), w_bwd.t()

    def fwd():
        return torch.mm(X, w_fwd_t)

    def bwd():
        return torch.mm(dY, w_bwd_t)

    settle(lambda i: (fwd(), bwd()))
    for _ in range(warmup):
        fwd(); bwd()
    ev = [_events(3) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        ev[s][0].record(); fwd(); ev[s][1].record(); bwd(); ev[s][2].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / steps

    # dense comparator: hipBLASLt fp16 GEMM on the masked dense weights, same shapes
    Wd_f = w_fwd.to_dense()
    Wd_b = torch.where(tmask, W, torch.zeros_like(W))
    settle(lambda i: (torch.mm(X, Wd_f.t()), torch.mm(dY, Wd_b)))
    e = _events(3)
    torch.cuda.synchronize()
    reps = max(3, steps)
    e[0].record()
    for _ in range(reps):
        torch.mm(X, Wd_f.t())
    e[1].record()
    for _ in range(reps):
        torch.mm(dY, Wd_b)
    e[2].record()
    torch.cuda.synchronize()
    dense_fwd_ms, dense_bwd_ms = e[0].elapsed_time(e[1]) / reps, e[1].elapsed_time(e[2]) / reps

    # accuracy spot check against the dense fp32-accumulate product of the same masked weights
    y, yd = fwd().float(), torch.mm(X.float(), Wd_f.float().t())
    rel_fwd = ((y - yd).norm() / yd.norm()).item()
    dx, dxd = bwd().float(), torch.mm(dY.float(), Wd_b.float())
    rel_bwd = ((dx - dxd).norm() / dxd.norm()).item()
    flops = 2.0 * M * Nw * K
    return wall_ms, fwd_ms, bwd_ms, dense_fwd_ms, dense_bwd_ms, rel_fwd, rel_bwd, flops, (M, K, Nw)



def forward_width_sweep(widths=(10240, 12288), steps=50):
    """The forward product of config 3 with W of other row counts (X[8192,4096] . W^T, W[n,4096]): n = 10240
    and 12288 are whole numbers of 256-row tiles per compute unit (5 and 6) and multiples of 256, where the
    dense library is at its best; config 3's own 11008 is neither.  ms, dense-equivalent TFLOP/s and the
    ratio to the dense GEMM on the masked weights, per width."""
    import sparse
    dev = torch.device("cuda:0")
    M, K = 8192, 4096
    gen = torch.Generator().manual_seed(3)
    X = torch.randn(M, K, generator=gen).half().to(dev)
    rows = []
    for n in widths:
        W = (0.02 * torch.randn(n, K, generator=gen)).half().to(dev)
        ws = sparse.to_sparse_semi_structured(W)
        wt, Wd = ws.t(), ws.to_dense()

        def timed(fn):
            settle(lambda i: fn())
            e = _events(2)
            e[0].record()
            for _ in range(steps):
                fn()
            e[1].record()
            torch.cuda.synchronize()
            return e[0].elapsed_time(e[1]) / steps
        ours, dense = timed(lambda: torch.mm(X, wt)), timed(lambda: torch.mm(X, Wd.t()))
        rows.append({"n": n, "ms": round(ours, 4), "tflops_dense_equivalent": round(2.0 * M * n * K / (ours * 1e-3) / 1e12, 1),
                     "dense_gemm_ms": round(dense, 4), "speedup_vs_dense_gemm": round(dense / ours, 3)})
        del W, ws, wt, Wd
    return rows


# --------------------------------------------------------------------------------------------
class MlpTrainer:
    """The training step of BASELINE config 4 -- GPT-2-124M MLP (c_fc d->h, GELU, c_proj h->d), fp16 autocast, mean
    squared error against a fixed target, fixed loss scale, AdamW -- run eagerly (step) or as replays of HIP graphs
    that hold one whole step each (capture / replay_step).

    kind  "sparse": SparseLinearTranspose layers (transposable mask refreshed every `freq` optimizer steps, W and
                    W^T recompressed each step, MVUE24 dW), masked decay alpha = 2e-4 by masked_add_, torch's fused AdamW;
          "sparse_one_pass": the same with MaskedDecayAdamW (decay folded into the update);
          "dense":  nn.Linear layers under autocast, torch's fused AdamW.
    Graphs: the layer's bookkeeping (`cnt`, `counter`: when to refresh the mask, when to recompress) is host
    logic that a graph freezes, so two graphs are recorded, a step that refreshes the masks and a step that does
    not, and replay_step picks by the optimizer step count.  MVUE24 takes its generator state from device memory
    under capture (sparse.mvue_device_state), so every replay samples afresh; the optimizer keeps its step count
    on the device (capturable=True)."""

    def __init__(self, kind, tokens=12 * 1024, d=768, h=3072, seed=2, capturable=False, freq=40, loss_scale=4096.0):
        import sparse
        self.sparse, self.kind, self.freq, self.loss_scale = sparse, kind, freq, loss_scale
        dev = torch.device("cuda:0")
        torch.manual_seed(seed)
        self.x = torch.randn(tokens, d, device=dev)
        self.target = torch.randn(tokens, d, device=dev)
        torch.manual_seed(seed)
        if kind != "dense":
            self.fc, self.proj = sparse.SparseLinearTranspose(d, h).to(dev), sparse.SparseLinearTranspose(h, d).to(dev)
            for layer in (self.fc, self.proj):
                layer.weight.freq = freq
        else:
            self.fc, self.proj = torch.nn.Linear(d, h).to(dev), torch.nn.Linear(h, d).to(dev)
        for layer in (self.fc, self.proj):
            torch.nn.init.normal_(layer.weight, std=0.02)
        self.params = list(self.fc.parameters()) + list(self.proj.parameters())
        if kind == "sparse_one_pass":      # masked decay folded into the optimizer update
            self.opt = sparse.MaskedDecayAdamW(self.params, lr=1e-4, weight_decay=0.0, alpha=2e-4, capturable=capturable)
        else:
            self.opt = torch.optim.AdamW(self.params, lr=1e-4, weight_decay=0.0, fused=True, capturable=capturable)
        self.opt_steps = 0
        self.graphs = None
        self.flops = 6 * 2.0 * tokens * d * h          # 3 GEMMs per layer, 2 layers, dense-equivalent

    def _body(self):
        import torch.nn.functional as F
        if self.kind != "dense":
            out = self.proj(F.gelu(self.fc(self.x)))
        else:
            with torch.autocast(device_type="cuda", dtype=torch.float16):
                out = self.proj(F.gelu(self.fc(self.x)))
        # a mean over tokens x d outputs puts dY near 1e-7, below fp16's normal range: fixed loss scale
        # (a power of two), gradients unscaled in one multi-tensor launch, in every model
        loss = F.mse_loss(out.float(), self.target)
        self.opt.zero_grad(set_to_none=True)
        (loss * self.loss_scale).backward()
        torch._foreach_mul_([p.grad for p in self.params], 1.0 / self.loss_scale)
        if self.kind == "sparse":
            with torch.no_grad():
                for p in self.params:
                    if hasattr(p, "mask") and p.mode == "sparse":
                        p.grad = p.grad.float()
                        self.sparse.masked_add_(p.grad.data, p.data, p.mask, alpha=2e-4)
                        p.cnt = 0
        self.opt.step()
        return loss

    def step(self):
        loss = self._body()
        self.opt_steps += 1
        return loss

    def _set_layer_clock(self, counter):
        for layer in (self.fc, self.proj):
            if hasattr(layer.weight, "counter"):
                layer.weight.counter, layer.weight.cnt = counter, 0

    def capture(self, eager_steps=3):
        """`eager_steps` steps on a side stream (allocator and library warm-up, optimizer state), then the
        recordings.  Nothing runs during a recording."""
        assert self.graphs is None
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(eager_steps):
                self.step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graphs, self.losses = {}, {}
        if self.kind != "dense":
            gen = torch.cuda.default_generators[0]
            self.sparse.mvue_device_state(self.x.device, seed=gen.initial_seed(), offset=gen.get_offset())
        for name in (("refresh", "regular") if self.kind != "dense" else ("regular",)):
            self._set_layer_clock(0 if name == "refresh" else 1)        # the mask is searched when counter % freq == 0
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self.losses[name] = self._body()
            self.graphs[name] = g
        self._set_layer_clock(self.opt_steps)
        return self

    def replay_step(self):
        name = "refresh" if (self.kind != "dense" and self.opt_steps % self.freq == 0) else "regular"
        self.graphs[name].replay()
        self.opt_steps += 1
        return self.losses[name]


def train_workload(steps, warmup):
    """BASELINE config 4: GPT-2-124M MLP (c_fc 768->3072, GELU, c_proj 3072->768) on 12x1024 tokens,
    fp16 autocast, SparseLinearTranspose layers (transposable mask refreshed every 40 optimizer steps,
    W and W^T recompressed each step, MVUE24 dW), masked decay alpha=2e-4, fused AdamW; seed 2.
    ms/step of the sparse model and of the same MLP with dense nn.Linear layers, each issued eagerly and as
    replays of whole-step HIP graphs."""
    def timed(step_fn):
        # median of three timed blocks of `steps` steps: the eager steps are issued by a Python thread whose
        # pace moves by several per cent from one moment to the next on a shared host
        settle(lambda i: step_fn())
        for _ in range(warmup):
            step_fn()
        blocks = []
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                loss = step_fn()
            torch.cuda.synchronize()
            blocks.append((time.perf_counter() - t0) * 1e3 / steps)
        return sorted(blocks)[1], loss.item()

    out = {}
    for kind in ("sparse", "dense", "sparse_one_pass"):
        t = MlpTrainer(kind)
        out[kind + "_ms"], out[kind + "_loss"] = timed(t.step)
        out["flops"] = t.flops
        del t
        torch.cuda.empty_cache()
    for kind in ("sparse", "dense", "sparse_one_pass"):
        t = MlpTrainer(kind, capturable=True).capture()
        out[kind + "_graph_ms"], out[kind + "_graph_loss"] = timed(t.replay_step)
        del t
        torch.cuda.empty_cache()
    return out


def train_record(r):
    """The training-step figures as they go into the JSON line."""
    return {
        "timing": "every figure is the median of three consecutive timed blocks of `steps` steps",
        "ms_per_step": round(r["sparse_ms"], 4), "ms_per_step_with_MaskedDecayAdamW": round(r["sparse_one_pass_ms"], 4),
        "dense_autocast_ms_per_step": round(r["dense_ms"], 4),
        "speedup_vs_dense_step": round(r["dense_ms"] / r["sparse_ms"], 3),
        "speedup_vs_dense_step_with_MaskedDecayAdamW": round(r["dense_ms"] / r["sparse_one_pass_ms"], 3),
        "hip_graph_replay": {
            "what": "one whole step (forward, backward, masked decay, fused AdamW) per graph replay; the sparse model replays "
                    "a mask-refresh graph every 40th step and a regular one otherwise; MVUE24 state on the device",
            "ms_per_step": round(r["sparse_graph_ms"], 4), "dense_autocast_ms_per_step": round(r["dense_graph_ms"], 4),
            "ms_per_step_with_MaskedDecayAdamW": round(r["sparse_one_pass_graph_ms"], 4),
            "speedup_vs_dense_step": round(r["dense_graph_ms"] / r["sparse_graph_ms"], 3),
            "speedup_vs_dense_step_with_MaskedDecayAdamW": round(r["dense_graph_ms"] / r["sparse_one_pass_graph_ms"], 3),
            "speedup_vs_eager_dense_step": round(r["dense_ms"] / r["sparse_graph_ms"], 3)},
        "tflops_dense_equivalent": round(r["flops"] / (r["sparse_ms"] * 1e-3) / 1e12, 1),
        "final_loss": {"sparse (2:4 weights, MVUE24 weight gradients)": r["sparse_loss"],
                       "dense (unmasked dense model: all weights trained, exact gradients)": r["dense_loss"]}}


def int8_workload(steps):
    """Not a BASELINE config (the reference's int8 branch, csrc .cu:594-637): int8 A[16384,8192] x magnitude-pruned
    int8 B[8192,8192]^T, int32 accumulate and output; comparator torch._int_mm on the dense masked operand.
    Exact: checked against an int64 product on a slab of rows."""
    import sparse
    dev = torch.device("cuda:0")
    M, K, Nb = 16384, 8192, 8192
    gen = torch.Generator(device=dev).manual_seed(7)
    A = torch.randint(-127, 128, (M, K), device=dev, generator=gen, dtype=torch.int32).to(torch.int8)
    B = torch.randint(-127, 128, (Nb, K), device=dev, generator=gen, dtype=torch.int32).to(torch.int8)
    w = sparse.to_sparse_semi_structured(B, dtype=torch.int8)
    Bd = w.to_dense()
    del B

    def timed(fn):
        settle(lambda i: fn())
        e = _events(2)
        e[0].record()
        for _ in range(steps):
            fn()
        e[1].record()
        torch.cuda.synchronize()
        return e[0].elapsed_time(e[1]) / steps

    mm_ms = timed(lambda: torch.mm(A, w.t()))
    dense_ms = None
    try:
        dense_ms = timed(lambda: torch._int_mm(A, Bd.t()))
    except Exception as ex:
        print(f"bench.py: dense int8 comparator unavailable: {ex}", file=sys.stderr)
    rows = slice(0, 256)
    exact = bool(torch.mm(A[rows], w.t()).cpu().long().equal(A[rows].cpu().long() @ Bd.cpu().long().t()))
    return mm_ms, dense_ms, exact, 2.0 * M * K * Nb


def fp8_workload(steps, warmup):
    """BASELINE configs[4]: e4m3 2:4 spMM A[16384,8192] x B[8192,8192]^T with B MVUE24-pruned from seeded
    uniforms, bf16 output; one step = soft_threshold24 on the bf16 B + MVUE24 prune/compress to e4m3 +
    the product.  The dense comparator is torch._scaled_mm (hipBLASLt fp8) on the dense masked operand."""
    import sparse
    dev = torch.device("cuda:0")
    M, K, Nb = 16384, 8192, 8192
    gen = torch.Generator(device=dev).manual_seed(5)
    A = torch.randn(M, K, device=dev, generator=gen)
    B = torch.randn(Nb, K, device=dev, generator=gen)
    U = torch.rand(Nb, K, device=dev, generator=gen)
    sa, sb = 448.0 / A.abs().max().item(), 224.0 / B.abs().max().item()   # MVUE rescales kept values by up to 2x
    Aq = (A * sa).to(torch.float8_e4m3fn)
    Bs = (B * sb).bfloat16()
    del A, B
    scale = 1.0 / (sa * sb)

    def step():
        sparse.soft_threshold24_triton(Bs)
        w = sparse.to_sparse_semi_structured(Bs, MVUE24=True, rand=U, dtype=torch.float8_e4m3fn)
        return sparse.sparse_semi_structured_linear(Aq, w, out_dtype=torch.bfloat16, scale=scale), w

    w = sparse.to_sparse_semi_structured(Bs, MVUE24=True, rand=U, dtype=torch.float8_e4m3fn)

    def mm():
        return sparse.sparse_semi_structured_linear(Aq, w, out_dtype=torch.bfloat16, scale=scale)

    settle(lambda i: step())
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) * 1e3 / steps
    settle(lambda i: mm())
    e = _events(2)
    e[0].record()
    for _ in range(steps):
        mm()
    e[1].record()
    torch.cuda.synchronize()
    mm_ms = e[0].elapsed_time(e[1]) / steps
    # the same product with the output type the reference gives 8-bit operands (float32, .cu:729, 772)
    mm32 = lambda: sparse.sparse_semi_structured_linear(Aq, w, scale=scale)
    settle(lambda i: mm32())
    e = _events(2)
    e[0].record()
    for _ in range(steps):
        mm32()
    e[1].record()
    torch.cuda.synchronize()
    mm32_ms = e[0].elapsed_time(e[1]) / steps

    Bd = w.to_dense()                                   # e4m3, 2:4 zeros in place
    dense_ms = None
    try:
        one = torch.ones((), device=dev)
        f = lambda: torch._scaled_mm(Aq, Bd.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
        settle(lambda i: f())
        e = _events(2)
        e[0].record()
        for _ in range(steps):
            f()
        e[1].record()
        torch.cuda.synchronize()
        dense_ms = e[0].elapsed_time(e[1]) / steps
    except Exception as ex:                             # no fp8 GEMM in this torch build
        print(f"bench.py: dense fp8 comparator unavailable: {ex}", file=sys.stderr)
    # accuracy on a slab of rows against the dense fp32 product of the same quantised operands
    rows = slice(0, 1024)
    ref = (Aq[rows].float() @ Bd.float().t()) * scale
    rel = ((mm()[rows].float() - ref).norm() / ref.norm()).item()
    return step_ms, mm_ms, dense_ms, rel, 2.0 * M * K * Nb, mm32_ms


def decode_workload(iters=200):
    """Not a BASELINE config: 8 to 1024 tokens against the config-3 weight (W[11008,4096] fp16, 2:4 along K), the
    shapes of decoding and of small batches with a compressed weight.  Bound by one pass over the compressed operand (values +
    metadata = 1.125 bytes per dense weight element).  Direct C-ABI launches on preallocated buffers;
    returns one row per token count with the dense hipBLASLt time on the decompressed weight beside it."""
    import sparse
    from sparse import _native as N
    lib = N.lib()
    dev = torch.device("cuda:0")
    Nw, K = 11008, 4096
    gen = torch.Generator().manual_seed(3)
    W = (0.02 * torch.randn(Nw, K, generator=gen)).half().to(dev)
    S = sparse.to_sparse_semi_structured(W)
    Wd_t = S.to_dense().t()
    v, mt, st = S._store_values, S._store_meta, N.stream_ptr()
    rows = []
    for tokens in (8, 16, 32, 64, 128, 256, 512, 1024):
        x = torch.randn(tokens, K, generator=gen).half().to(dev)
        out = torch.empty(tokens, Nw, dtype=torch.float16, device=dev)
        wsb = lib.tf24_spmm_workspace_bytes(N.F16, Nw, K, tokens)
        ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=dev)

        def sparse_mm(_i):
            N.check(lib.tf24_spmm(v.data_ptr(), mt.data_ptr(), N.COMPRESSED_PANEL, N.F16, Nw, K, x.data_ptr(), N.ROW_MAJOR, K, tokens,
                                  out.data_ptr(), N.F16, N.COL_MAJOR, Nw, None, 1.0, 0, ws.data_ptr() if wsb else None, wsb, st))

        def dense_mm(_i):
            torch.mm(x, Wd_t, out=out)
        us = time_rotating(sparse_mm, 1, iters, 20)["median"]
        ref = x.float() @ Wd_t.float()
        rel = ((out.float() - ref).norm() / ref.norm()).item()
        dus = time_rotating(dense_mm, 1, iters, 20)["median"]
        nbytes = Nw * K * 9 // 8 + tokens * K * 2 + tokens * Nw * 2
        rows.append({"tokens": tokens, "us": round(us, 2), "dense_hipblaslt_us": round(dus, 2), "speedup_vs_dense": round(dus / us, 3),
                     "GBps": round(nbytes / us / 1e3, 1), "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                     "rel_err_vs_dense_fp32": rel})
    return rows


def cpu_baseline_spmm(threads):
    """The oracle (pure-PyTorch port of the reference semantics) on the host cores, on config 3 itself:
    prune+compress and transposable mask of W, then both dense masked fp32 products; one warm-up
    repetition and three timed ones, the median reported."""
    import oracle
    torch.set_num_threads(threads)
    gen = torch.Generator().manual_seed(3)
    M, K, Nw = 8192, 4096, 11008
    X = torch.randn(M, K, generator=gen).half()
    W = (0.02 * torch.randn(Nw, K, generator=gen)).half()
    dY = torch.randn(M, Nw, generator=gen).half()

    def timed(fn, reps=3):
        fn()                                             # warm-up
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    mask = oracle.prune24_mask(W)
    w_t, _ = oracle.transposable_mask(W)
    Wm = torch.where(mask, W, torch.zeros_like(W))
    Wt = w_t.t().contiguous()
    t_conv = timed(lambda: oracle.compress24(W, mask=oracle.prune24_mask(W)))
    t_tr = timed(lambda: oracle.transposable_mask(W))
    t_mm = timed(lambda: (oracle.spmm_ref(X, Wm), oracle.spmm_ref(dY, Wt)))
    tflops = 2 * 2.0 * M * Nw * K / t_mm / 1e12
    return {"value": round(tflops, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"the whole of config 3, 1 warm-up + 3 timed repetitions, median: oracle.spmm_ref fp32 forward + transposed ({t_mm:.2f} s); "
                      f"oracle prune+compress of W {t_conv:.2f} s ({3.125 * Nw * K / t_conv / 1e9:.2f} GB/s algorithmic), "
                      f"oracle transposable mask of W {t_tr:.2f} s ({5.0 * Nw * K / t_tr / 1e9:.2f} GB/s algorithmic)"}


def cpu_baseline_configs(threads):
    """The oracle on the host cores beside the other single-GPU configs (2a-e, one training step of config 4,
    config 5), each on a stated sample -- a slab of rows where the whole matrix would take long -- one warm-up
    and three timed repetitions, the median; rates are algorithmic bytes (or dense-equivalent flops) of the
    sample per second."""
    import oracle
    torch.set_num_threads(threads)

    def timed(fn, reps=3):
        fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    out = []
    gen = torch.Generator().manual_seed(1)
    rows, k = 8192, 8192                     # config 2 itself
    n = rows * k
    W = torch.randn(rows, k, generator=gen).bfloat16()
    U = torch.rand(rows, k, generator=gen)
    G = 1e-3 * torch.randn(rows, k, generator=gen)
    P = W.float()
    _, tmask = oracle.transposable_mask(W)
    sample = "the whole 8192 x 8192 matrix of config 2"
    for name, fn, nbytes in (
            ("2a magnitude prune+compress bf16 -> f16", lambda: oracle.compress24(W, out_dtype=torch.float16), 3.125 * n),
            ("2b MVUE24 prune+compress (U float32)", lambda: oracle.mvue24(W, U, out_dtype=torch.float16), 7.125 * n),
            ("2c transposable mask select", lambda: oracle.transposable_mask(W), 5.0 * n),
            ("2d soft_threshold24 bf16", lambda: oracle.soft_threshold24(W), 6.0 * n),
            ("2e masked_add_ f32", lambda: oracle.masked_add(G, P, tmask, alpha=2e-4), 13.0 * n)):
        t = timed(fn)
        out.append({"config": name, "seconds": round(t, 4), "value": round(nbytes / t / 1e9, 3), "unit": "GB/s", "sample": sample})
    del W, U, G, P, tmask

    # config 4: one training step of the MLP in float32 with the oracle's operators (mask search, both compressed
    # copies, MVUE24 of dY^T for each layer, the six products as dense masked products)
    tokens, d, h = 12 * 1024, 768, 3072
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(tokens, d, generator=gen)
    target = torch.randn(tokens, d, generator=gen)
    w1, w2 = 0.02 * torch.randn(h, d, generator=gen), 0.02 * torch.randn(d, h, generator=gen)
    u1, u2 = torch.rand(h, tokens, generator=gen), torch.rand(d, tokens, generator=gen)

    def train_step():
        grads = []
        m1, m2 = oracle.transposable_mask(w1)[1], oracle.transposable_mask(w2)[1]
        for w, m in ((w1, m1), (w2, m2)):
            oracle.compress24(w, mask=m)
            oracle.compress24(w.t().contiguous(), mask=m.t().contiguous())
        w1m, w2m = torch.where(m1, w1, torch.zeros(())), torch.where(m2, w2, torch.zeros(()))
        a = oracle.spmm_ref(x, w1m)
        hid = torch.nn.functional.gelu(a)
        y = oracle.spmm_ref(hid, w2m)
        dy = 2.0 * (y - target) / y.numel()
        dhid = dy @ w2m
        dgelu = 0.5 * (1 + torch.erf(a * 0.7071067811865476)) + a * torch.exp(-0.5 * a * a) * 0.3989422804014327
        for g, inp, u in ((dy, hid, u2), (dhid * dgelu, x, u1)):
            grads.append(oracle.mvue24_dense(g.t().contiguous(), u) @ inp)
        for w, g, m in ((w1, grads[1], m1), (w2, grads[0], m2)):
            oracle.masked_add(g, w, m, alpha=2e-4)
        return grads
    t = timed(train_step, reps=1)
    out.append({"config": "4 one training step (float32, oracle operators; 1 warm-up + 1 timed)", "seconds": round(t, 3),
                "value": round(6 * 2.0 * tokens * d * h / t / 1e12, 4), "unit": "TFLOP/s dense-equivalent", "sample": "the whole step at full size"})
    del x, target, w1, w2, u1, u2

    # config 5: MVUE24 of a slab of B, the fp8-quantised product of A against it in float32
    gen = torch.Generator().manual_seed(5)
    ra, rb, kk = 4096, 4096, 8192
    A = torch.randn(ra, kk, generator=gen)
    B = torch.randn(rb, kk, generator=gen)
    U = torch.rand(rb, kk, generator=gen)
    sa, sb = 448.0 / A.abs().max().item(), 224.0 / B.abs().max().item()
    Aq, Bs = (A * sa).to(torch.float8_e4m3fn), (B * sb).bfloat16()

    def fp8_step():
        oracle.soft_threshold24(Bs)
        v, meta, _ = oracle.mvue24(Bs, U, out_dtype=torch.float8_e4m3fn)
        dense = oracle.decompress24(v, meta).float()
        return oracle.spmm_ref(Aq.float(), dense)
    t = timed(fp8_step)
    out.append({"config": "5 soft threshold + MVUE24 to e4m3 + product (float32 arithmetic on the e4m3 values)", "seconds": round(t, 3),
                "value": round(2.0 * ra * rb * kk / t / 1e12, 4), "unit": "TFLOP/s dense-equivalent",
                "sample": f"A rows 0..{ra - 1} of 16384 against B rows 0..{rb - 1} of 8192 (1/8 of the product, half of the conversions)"})
    return out


def host_threads():
    """Threads for the CPU leg: what the host gives this process (its affinity mask, and the
    OMP_NUM_THREADS the box sets), not the machine's core count."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit() and int(env) > 0:
        n = min(n, int(env))
    return max(1, n)


def traffic_workload(reps=8):
    """Kernels of known footprint, then the config-3 products, each launched `reps` times on rotated
    buffers: the workload of the `rocprofv3 --pmc` runs that calibrate the L2 <-> fabric byte counters
    (counted / known bytes on the streaming kernels) and size the matmul's traffic with them."""
    import sparse
    from sparse import _native as N
    lib = N.lib()
    dev = torch.device("cuda:0")
    m = k = 8192
    n = m * k
    nsets = 8
    gen = torch.Generator(device=dev).manual_seed(1)
    W = [torch.randn(m, k, device=dev, generator=gen).bfloat16() for _ in range(nsets)]
    G = [1e-3 * torch.randn(m, k, device=dev, generator=gen) for _ in range(nsets)]
    P = [torch.randn(m, k, device=dev, generator=gen) for _ in range(nsets)]
    bmask = [torch.rand(m, k, device=dev, generator=gen) < 0.5 for _ in range(nsets)]
    values = [torch.empty(m, k // 2, dtype=torch.float16, device=dev) for _ in range(nsets)]
    meta = [torch.empty(m, k // 16, dtype=torch.int16, device=dev) for _ in range(nsets)]
    dense = [torch.empty(m, k, dtype=torch.float16, device=dev) for _ in range(nsets)]
    st = N.stream_ptr()
    known = {}
    for i in range(reps):
        j = i % nsets
        N.check(lib.tf24_masked_add(G[j].data_ptr(), N.F32, P[j].data_ptr(), N.F32, bmask[j].data_ptr(), N.U8, n, 2e-4, st))
    known["masked_add_vec"] = {"read": 9 * n, "written": 4 * n}
    for i in range(reps):
        j = i % nsets
        N.check(lib.tf24_prune_compress(W[j].data_ptr(), N.BF16, N.ROW_MAJOR, k, m, k, N.PRUNE_MAGNITUDE, None, N.U8, 0,
                                        None, 0, values[j].data_ptr(), N.F16, meta[j].data_ptr(), N.COMPRESSED_PANEL, st))
    known["prune_compress_row_mag16_panel"] = {"read": 2 * n, "written": n + n // 8}
    for i in range(reps):
        j = i % nsets
        N.check(lib.tf24_decompress(values[j].data_ptr(), N.F16, meta[j].data_ptr(), N.COMPRESSED_PANEL, m, k, dense[j].data_ptr(), st))
    known["decompress_kernel"] = {"read": n + n // 8, "written": 2 * n}
    for i in range(reps):
        j = i % nsets
        dense[j].view(torch.bfloat16).copy_(W[(j + 1) % nsets])
    known["torch copy (bf16, 8192 x 8192)"] = {"read": 2 * n, "written": 2 * n}
    torch.cuda.synchronize()
    del W, G, P, bmask, values, meta, dense
    M, K, Nw = 8192, 4096, 11008
    g = torch.Generator().manual_seed(3)
    X = torch.randn(M, K, generator=g).half().to(dev)
    Wt = (0.02 * torch.randn(Nw, K, generator=g)).half().to(dev)
    dY = torch.randn(M, Nw, generator=g).half().to(dev)
    w_fwd = sparse.to_sparse_semi_structured(Wt)
    _, tmask = sparse.TransposableSparse()(Wt)
    w_bwd = sparse.to_sparse_semi_structured(Wt.T, mask=tmask.T)
    for _ in range(reps):
        torch.mm(X, w_fwd.t())
        torch.mm(dY, w_bwd.t())
    torch.cuda.synchronize()
    known["spmm_pipe (config 3, per launch, algorithmic)"] = {"read": M * K * 2 + Nw * K * 9 // 8, "written": M * Nw * 2}
    return {"launches_per_kernel": reps, "buffer_sets": nsets, "known_bytes_per_launch": known}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["spmm", "train", "fp8", "int8", "decode", "traffic"], default="spmm",
                    help="spmm: BASELINE configs[2] (default, the judged line); train: configs[3] MLP training step; "
                         "fp8: configs[4] e4m3 MVUE + spMM; decode: 8-1024 tokens against the config-3 weight (not a BASELINE config); "
                         "traffic: kernels of known footprint + the config-3 products, for rocprofv3 --pmc byte-counter runs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-convert", action="store_true", help="skip the conversion-kernel table")
    ap.add_argument("--no-extra", action="store_true", help="skip the fp8 (configs[4]) and training-step (configs[3]) legs of the default line")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the 2:4 path has no multi-GPU component (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    if a.workload == "traffic":
        print(json.dumps(traffic_workload()))
        return

    if a.workload == "train":
        r = train_workload(a.steps, a.warmup)
        line = {
            "metric": "2:4 sparse MLP training step, dense-equivalent TFLOP/s of its 6 GEMMs", "value": round(r["flops"] / (r["sparse_ms"] * 1e-3) / 1e12, 2),
            "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "clock_settle_s": SETTLE_S, "ms_per_step": round(r["sparse_ms"], 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "BASELINE configs[3]: SparseLinearTranspose GPT-2-124M MLP step, 12288 tokens, 768->3072->768, "
                                   "masked decay 2e-4, fused AdamW, mask refresh every 40 steps", "seed": 2}}
        line.update(train_record(r))
        print(json.dumps(line))
        return

    if a.workload == "decode":
        rows = decode_workload()
        first = rows[0]
        print(json.dumps({
            "metric": "2:4 spMM with a narrow dense operand: GB/s over the compressed weight (8 tokens)", "value": first["GBps"],
            "unit": "GB/s", "n_gpus": 1, "steps": 200, "warmup": 20, "ms_per_step": round(first["us"] / 1e3, 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "not a BASELINE config: tokens x W[11008,4096]^T, fp16, W 2:4 along K (decoding shapes)", "seed": 3},
            "roofline": {"bound": "hbm", "kernel": "spmm_narrow_shared (8 tokens)", "achieved": first["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": first["frac_of_hbm_peak"], "traffic": None},
            "by_tokens": rows, "cpu_baseline": None}))
        return

    if a.workload == "int8":
        mm_ms, dense_ms, exact, ops = int8_workload(a.steps)
        executed = (ops / 2) / (mm_ms * 1e-3) / 1e12
        print(json.dumps({
            "metric": "int8 2:4 spMM TOP/s (dense-equivalent 2MNK)", "value": round(ops / (mm_ms * 1e-3) / 1e12, 2),
            "unit": "TOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "clock_settle_s": SETTLE_S, "ms_per_step": round(mm_ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
            "config": {"workload": "not a BASELINE config: int8 A[16384,8192] x magnitude-pruned int8 B[8192,8192]^T, int32 accumulate and output", "seed": 7},
            "roofline": {"bound": "mfma", "kernel": "spmm (SMFMAC int8)", "achieved": round(executed, 2), "peak": 5000.0, "unit": "TOP/s",
                         "frac": round(executed / 5000.0, 4), "traffic": None},
            "dense_int8_gemm_ms": None if dense_ms is None else round(dense_ms, 4),
            "speedup_vs_dense_gemm": None if dense_ms is None else round(dense_ms / mm_ms, 3),
            "exact_vs_int64_product": exact, "cpu_baseline": None}))
        return

    if a.workload == "fp8":
        step_ms, mm_ms, dense_ms, rel, flops, mm32_ms = fp8_workload(a.steps, a.warmup)
        executed = (flops / 2) / (mm_ms * 1e-3) / 1e12
        print(json.dumps({
            "metric": "fp8 2:4 spMM TFLOP/s (dense-equivalent 2MNK)", "value": round(flops / (mm_ms * 1e-3) / 1e12, 2),
            "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "clock_settle_s": SETTLE_S, "ms_per_step": round(mm_ms, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "e4m3", "data": "synthetic",
            "config": {"workload": "BASELINE configs[4]: e4m3 A[16384,8192] x MVUE24-pruned B[8192,8192]^T, fp32 accumulate, bf16 out", "seed": 5},
            "roofline": {"bound": "mfma", "kernel": "spmm (SMFMAC fp8)", "achieved": round(executed, 2), "peak": 5000.0, "unit": "TFLOP/s",
                         "frac": round(executed / 5000.0, 4), "traffic": None},
            "iteration_ms_with_soft_threshold_and_mvue_compress": round(step_ms, 4),
            "ms_per_step_with_float32_output": round(mm32_ms, 4),
            "dense_fp8_gemm_ms": None if dense_ms is None else round(dense_ms, 4),
            "speedup_vs_dense_gemm": None if dense_ms is None else round(dense_ms / mm_ms, 3),
            "rel_err_vs_dense_fp32": rel, "cpu_baseline": None}))
        return

    wall_ms, fwd_ms, bwd_ms, dfwd_ms, dbwd_ms, rel_f, rel_b, flops, (M, K, Nw) = spmm_workload(a.steps, a.warmup)
    value = 2 * flops / (wall_ms * 1e-3) / 1e12
    traffic_bytes, traffic_source = profiled_traffic()
    dom_ms = (fwd_ms + bwd_ms) / 2                       # two products per step (the forward one: chained tiles + a launch for the last tile rows)
    executed_tflops = (flops / 2) / (dom_ms * 1e-3) / 1e12
    line = {
        "metric": "2:4 spMM TFLOP/s (dense-equivalent 2MNK; fwd X.W^T + transposed dY.W per step)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "clock_settle_s": SETTLE_S,
        "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: fp16 2:4 spMM X[8192,4096].W^T (W[11008,4096]) + dY[8192,11008].W, fp32 accumulate",
                   "M": M, "K": K, "N": Nw, "seed": 3},
        "roofline": {"bound": "mfma", "kernel": "spmm (SMFMAC)", "achieved": round(executed_tflops, 2),
                     "peak": MFMA_DENSE_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(executed_tflops / MFMA_DENSE_PEAK_TFLOPS, 4),
                     "traffic": traffic_bytes,
                     "traffic_source": traffic_source,
                     "algorithmic_bytes": M * K * 2 + Nw * K * 9 // 8 + M * Nw * 2,
                     "note": "achieved = executed flops (M*N*K, half the dense-equivalent 2MNK) per product / HIP-event "
                             "time of the product (one tf24_spmm call: the transposed product is one launch of the "
                             "chained-tile kernel, the forward product that kernel on 1280 tiles + a launch on "
                             "256 x 128 tiles for the last 3 tile rows); SMFMAC executes MACs at the dense MFMA rate, "
                             "so frac also equals dense-equivalent rate / (2 x dense peak)",
                     "fwd_ms": round(fwd_ms, 4), "transposed_ms": round(bwd_ms, 4)},
        "dense_gemm": {"library": "torch.mm fp16 (hipBLASLt) on the masked dense weights",
                       "fwd_ms": round(dfwd_ms, 4), "transposed_ms": round(dbwd_ms, 4),
                       "tflops": round(2 * flops / ((dfwd_ms + dbwd_ms) * 1e-3) / 1e12, 2)},
        "speedup_vs_dense_gemm": round((dfwd_ms + dbwd_ms) / (fwd_ms + bwd_ms), 3),
        "rel_err_vs_dense_fp32": {"fwd": rel_f, "transposed": rel_b},
    }
    if not a.no_extra:
        line["forward_other_widths"] = forward_width_sweep()
        torch.cuda.empty_cache()
        # the other two single-GPU configs of the baseline, in the same line (each also runs alone
        # with --workload fp8 / train)
        torch.cuda.empty_cache()
        step_ms, mm_ms, dense_ms, rel, f8, mm32_ms = fp8_workload(a.steps, a.warmup)
        ex8 = (f8 / 2) / (mm_ms * 1e-3) / 1e12
        line["fp8_config5"] = {
            "workload": "BASELINE configs[4]: e4m3 A[16384,8192] x MVUE24-pruned B[8192,8192]^T, fp32 accumulate, bf16 out",
            "spmm_ms": round(mm_ms, 4), "spmm_ms_with_float32_output": round(mm32_ms, 4),
            "tflops_dense_equivalent": round(f8 / (mm_ms * 1e-3) / 1e12, 1),
            "roofline_frac": round(ex8 / MFMA_DENSE_PEAK_FP8_TFLOPS, 4),
            "dense_fp8_gemm_ms": None if dense_ms is None else round(dense_ms, 4),
            "speedup_vs_dense_gemm": None if dense_ms is None else round(dense_ms / mm_ms, 3),
            "iteration_ms_with_soft_threshold_and_mvue_compress": round(step_ms, 4), "rel_err_vs_dense_fp32": rel}
        torch.cuda.empty_cache()
        line["train_config4"] = {
            "workload": "BASELINE configs[3]: SparseLinearTranspose GPT-2-124M MLP step, 12288 tokens, 768->3072->768, fp16 autocast, "
                        "masked decay 2e-4, fused AdamW, mask refresh every 40 steps"}
        line["train_config4"].update(train_record(train_workload(a.steps, a.warmup)))
        torch.cuda.empty_cache()
    if not a.no_convert:
        line["conversion_kernels_GBps"] = conversion_kernels()
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline_spmm(host_threads())
        line["cpu_baseline"]["other_configs"] = cpu_baseline_configs(host_threads())
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
