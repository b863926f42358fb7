"""Headline benchmark: power_retention forward + backward at the reference's benchmark shape
(b=1, t=65536, h=8, d=64, bf16, deg=2, chunk_size=1024, gated; ref: perf/benchmark.py:58-61,335-343)
on one MI355X.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms T] [--no-cpu] [--no-breakdown] [--no-decode]
                    [--no-short-chunks]

A step = one forward + one backward over one synthetic batch already resident in HBM.  After the W warm-up steps the
step keeps running untimed for T ms (default 60) so that the chip's clock has settled; then K steps are timed back to
back, and K steps each after a cache flush (their median is the headline).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 matrix-core peak
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E peak
CFG = dict(b=1, t=65536, h=8, d=64, chunk=1024, deg=2)


def flops(b, t, h, d, c, D):
    """Canonical algorithmic count: compact D = C(d+1, 2), causal-halved attention, state contractions on
    n-1 chunks, multiply-add = 2."""
    n = t // c
    attn = n * d * c * (c + 1)
    state = (n - 1) * c * D * d
    fwd = b * h * (2 * attn + 4 * state)
    bwd = b * h * (5 * attn + 8 * state)
    return fwd, bwd


def make_inputs(b, t, h, d, device, seed=42):
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn(b, t, h, d, generator=g).to(torch.bfloat16).to(device) for _ in range(4))
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g)).to(device)
    return Q, K, V, lg, dO


def event_time_ms(fn, iters, settle_ms=30.0):
    """Average duration of fn() on the current stream, by HIP events on that stream, after fn has run untimed for about
    settle_ms (the clock governor's ramp; the lead-in calls sit in the same queue, directly ahead of the timed ones)."""
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    e0.record(st)
    fn()
    e1.record(st)
    e1.synchronize()
    lead = int(settle_ms / max(e0.elapsed_time(e1), 1e-3)) + 1
    for _ in range(lead):
        fn()
    e0.record(st)
    for _ in range(iters):
        fn()
    e1.record(st)
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def op_breakdown(pra, Q, K, V, lg, dO, cfg, iters=5):
    """Per-kernel-family timings of the pieces of one step, each launched alone (HIP events) through the operator
    wrappers.  Those make no promise about the state's symmetry, so their query_state / update_state backward take
    both folds through the diagonal feature blocks (the fused step promises it and is ~20 us per launch faster,
    which the "sympow_grad(dK)" entry, launched as the step launches it, shows)."""
    from retention_integration_amd import ops
    b, t, h, d, c = cfg["b"], cfg["t"], cfg["h"], cfg["d"], cfg["chunk"]
    n = t // c
    Kc, Vc, Qc = K.view(b, n, c, h, d), V.view(b, n, c, h, d), Q.view(b, n, c, h, d)
    A = lg.view(b, n, c, h).cumsum(2)
    lcs = A[:, :, -1].contiguous()
    res = {}
    S, s = ops.update_state_fwd(Kc, Vc)
    res["update_state_fwd"] = event_time_ms(lambda: ops.update_state_fwd(Kc, Vc), iters)
    Sc = ops.discumsum_fwd(S, lcs, n)
    sc = ops.discumsum_fwd(s, lcs, n)
    res["discumsum_fwd(S)"] = event_time_ms(lambda: ops.discumsum_fwd(S, lcs, n), iters)
    Af = A.view(b * n, c, h).contiguous()
    Qf, Kf, Vf = Q.view(b * n, c, h, d), K.view(b * n, c, h, d), V.view(b * n, c, h, d)
    scale = d ** -0.5
    Ya, la, rm = ops.attention_fwd(Qf, Kf, Vf, Af, 2, scale, False)
    res["attention_fwd"] = event_time_ms(lambda: ops.attention_fwd(Qf, Kf, Vf, Af, 2, scale, False), iters)
    Ya5, la5, rm5 = Ya.view(b, n, c, h, d), la.view(b, n, c, h), rm.view(b, n, c, h)
    qs = lambda: ops.query_state_fwd(Qc, Sc, sc, Ya5, la5, rm5, scale ** 2, True)  # noqa: E731
    O, den = qs()
    res["query_state_fwd"] = event_time_ms(qs, iters)
    dOc = dO.view(b, n, c, h, d)
    res["query_state_bwd"] = event_time_ms(lambda: ops.query_state_bwd(Qc, Sc, sc, rm5, O, den, dOc, scale ** 2, True), iters)
    dOf = dO.view(b * n, c, h, d)
    res["attention_bwd"] = event_time_ms(lambda: ops.attention_bwd(Qf, Kf, Vf, Af, rm, dOf, la, None, 2, scale), iters)
    res["discumsum_bwd(S)"] = event_time_ms(lambda: ops.discumsum_bwd(Sc, Sc, lcs), iters)
    res["update_state_bwd"] = event_time_ms(lambda: ops.update_state_bwd(Kc, Vc, S, s), iters)
    # the single kernel with the largest share of a step: the feature-gradient contraction (sympow_grad), here as
    # the dK half of update_state backward, launched alone through the C ABI (dV = NULL skips the other half)
    from retention_integration_amd import _lib
    lib = _lib.load()
    dK = torch.empty_like(Kc)
    grad_only = lambda: _lib.check(lib.pr_update_state_bwd(  # noqa: E731
        _lib.ptr(Kc), _lib.ptr(Vc), _lib.ptr(S), _lib.ptr(s), None, None, None, None, _lib.ptr(dK), None, b * n, c, h, d, 2, 1, 0,
        _lib.dtype_code(Kc.dtype), _lib.stream()), "update_state_bwd(dK)")
    res["sympow_grad(dK)"] = event_time_ms(grad_only, iters)
    return {k: round(v, 4) for k, v in res.items()}


def counter_run(pra, Q, K, V, lg, cfg, dev, kernel):
    """For the byte counters (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE): three launches of one kernel alone, each followed
    by a plain copy of 256 MiB (read 256 MiB + write 256 MiB) that calibrates the counter.  kernel: "sympow_grad" (the dK
    half of update_state's backward), "chunk_fwd" (the forward of all chunks in one kernel) or "chunk_bwd_dq" (the query
    side of the backward in one kernel)."""
    from retention_integration_amd import _lib, ops
    b, t, h, d, c = cfg["b"], cfg["t"], cfg["h"], cfg["d"], cfg["chunk"]
    n = t // c
    p, st = _lib.ptr, _lib.stream()
    with torch.no_grad():
        Kc, Vc = K.view(b, n, c, h, d), V.view(b, n, c, h, d)
        S, s = ops.update_state_fwd(Kc, Vc)
        lib = _lib.load()
        lib.pr_set_gate_skipping(0)   # (every tile visited: the traffic of the whole algorithmic work)
        code = _lib.dtype_code(Kc.dtype)
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        if kernel == "sympow_grad":
            dK = torch.empty_like(Kc)

            def launch():
                _lib.check(lib.pr_update_state_bwd(p(Kc), p(Vc), p(S), p(s), None, None, None, None, p(dK), None, b * n, c, h, d,
                                                   2, 1, 0, code, st),
                           "update_state_bwd(dK)")
        elif kernel == "chunk_fwd":
            A = lg.view(b * n, c, h).cumsum(1).contiguous()
            lcs = A[:, -1].contiguous().view(b, n, h)
            Sc, sc = ops.discumsum_fwd(S, lcs, n), ops.discumsum_fwd(s, lcs, n)
            O = torch.empty_like(Q)
            rm, den = (torch.empty(b * n, c, h, dtype=torch.float32, device=dev) for _ in range(2))

            def launch():
                _lib.check(lib.pr_chunk_fwd(p(Q), p(K), p(V), p(A), p(Sc), p(sc), None, None, None, p(O), p(rm), p(den), b * n, n,
                                            c, h, 1, d,
                                            d ** -0.5, 2, 1, code, st), "chunk_fwd")
        elif kernel == "chunk_bwd_dq":
            from retention_integration_amd import fused
            O, A, _, _, Sc, sc, rm, den = fused.chunked_fwd(Q, K, V, lg, 2, d ** -0.5, c)[:8]
            dO = torch.randn_like(Q)
            rows = b * t * h
            qws = torch.empty(lib.pr_query_state_bwd_workspace(b * n, c, h, 1, d, code), dtype=torch.uint8, device=dev)
            dla, dys = torch.empty_like(den), torch.empty_like(den)
            # the row-wise preparation alone (no dQ, no dS): fills the workspace and the two row vectors
            _lib.check(lib.pr_query_state_bwd(p(Q), p(Sc), p(sc), p(rm), p(A), p(O), p(den), p(dO), None, None, None, None,
                                              p(dla), p(dys), p(qws), None, b * n, n, c, h, 1, d, 1.0 / d, 2, 2, 1, 0, code,
                                              st),
                       "query_state_bwd(prep)")
            cvec = qws.data_ptr() + (rows * d * 2 + 255) // 256 * 256
            dQ, dGq = torch.empty_like(Q), torch.empty_like(den)

            def launch():
                _lib.check(lib.pr_chunk_bwd_dq(p(Q), p(K), p(V), p(A), p(rm), p(den), p(dO), p(dla), p(dys), cvec, p(Sc),
                                               p(sc), None, None, None, p(dQ), p(dGq), b * n, n, c, h, 1, d, d ** -0.5, 2, 1,
                                               code, st),
                           "chunk_bwd_dq")
        else:
            sys.exit(f"--counter-run: unknown kernel {kernel!r} (sympow_grad, chunk_fwd, chunk_bwd_dq)")
        torch.cuda.synchronize()
        for _ in range(3):
            launch()
            dst.copy_(src)
        torch.cuda.synchronize()
    print(f"counter run done: 3 x {kernel}, 3 x 256 MiB device copy")


def attention_scaling(pra, dev, chunk):
    """For a kernel trace: the three attention kernels alone (operator level, 64 forward + backward calls) on the
    headline's 65536 x 8 rows cut into chunks of `chunk` keys.  The tile work of a launch is proportional to the chunk
    length while everything per row and per workgroup (loading the block's own rows, storing its results, set-up) is
    not, so two chunk lengths separate the two."""
    from retention_integration_amd import ops
    t, h, d = CFG["t"], CFG["h"], CFG["d"]
    Q, K, V, lg, dO = make_inputs(1, t, h, d, dev)
    n = t // chunk
    Qf, Kf, Vf, dOf = (x.view(n, chunk, h, d) for x in (Q, K, V, dO))
    A = lg.view(n, chunk, h).cumsum(1).contiguous()
    calls = 64   # ~35 ms of lead-in for the clock governor; a summary takes the last few launches
    with torch.no_grad():
        for _ in range(calls):
            Ya, la, rm = ops.attention_fwd(Qf, Kf, Vf, A, 2, d ** -0.5, False)
            ops.attention_bwd(Qf, Kf, Vf, A, rm, dOf, la, None, 2, d ** -0.5)
        torch.cuda.synchronize()
    print(f"attention scaling run done: {calls} x (attention_fwd, attention_bwd) at chunk {chunk}, {n} chunks x {h} heads")


def decode_bench(pra, dev, steps=512):
    """The inference configuration of the benchmark contract (configs[3]): b=32, h=8, d=64 bf16; prefill of 2048 tokens
    with switch_over_seq_len=1024, then `steps` single-token steps.  Loops timed:
      recurrent           every token folded into the state (switch_over_seq_len=1), one library call per token,
                          through power_retention_inference;
      recurrent_graph     the same steps through RetentionCache.step, captured once in a HIP graph and replayed;
      growing_cache       the reference caller's loop: torch.cat of the cache + power_retention_inference with the whole
                          cache, the state only queried (ref: deploy/models/powercoder/modeling_powercoder.py:181-196);
      growing_cache_prealloc  the same arithmetic through RetentionCache.step (append in place, no torch.cat)."""
    b, h, d = 32, 8, 64
    g = torch.Generator().manual_seed(4)
    mk = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16).to(dev)  # noqa: E731
    K, V, Q = mk(b, 2048, h, d), mk(b, 2048, h, d), mk(b, 1, h, d)
    lg = torch.nn.functional.logsigmoid(torch.randn(b, 2048, h, generator=g)).to(dev)
    qs, ks, vs = mk(steps, b, 1, h, d), mk(steps, b, 1, h, d), mk(steps, b, 1, h, d)
    lgs = torch.nn.functional.logsigmoid(torch.randn(steps, b, 1, h, generator=g)).to(dev)
    out = {}

    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        return {"us_per_step": round(dt / steps * 1e6, 1), "tokens_per_s": round(b * steps / dt, 1)}

    with torch.no_grad():
        pra.power_retention_inference(Q, K, V, lg, switch_over_seq_len=1024)   # warm-up
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _, S, s = pra.power_retention_inference(Q, K, V, lg, switch_over_seq_len=1024)
        torch.cuda.synchronize()
        out["prefill_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
        St, st = S, s
        for i in range(8):
            _, St, st = pra.power_retention_inference(qs[i], ks[i], vs[i], lgs[i], St, st, switch_over_seq_len=1)

        def recurrent():
            St, st = S, s
            for i in range(steps):
                _, St, st = pra.power_retention_inference(qs[i], ks[i], vs[i], lgs[i], St, st, switch_over_seq_len=1)
        out["recurrent"] = timed(recurrent)

        # the same steps captured in a HIP graph (state updated in place in the cache's own buffers)
        cache = pra.RetentionCache(b, h, d, capacity=steps, device=dev)
        ys = torch.empty(steps, b, 1, h, d, dtype=torch.bfloat16, device=dev)

        def rec_steps():
            for i in range(steps):
                cache.step(qs[i], ks[i], vs[i], lgs[i], switch_over_seq_len=1, out=ys[i])
        cache.update_state(S, s)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            rec_steps()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            rec_steps()
        cache.update_state(S, s)
        graph.replay()
        cache.update_state(S, s)
        out["recurrent_graph"] = timed(graph.replay)

        def growing():
            Kc = torch.empty(b, 0, h, d, dtype=torch.bfloat16, device=dev)
            Vc, Gc = Kc.clone(), torch.empty(b, 0, h, device=dev)
            for i in range(steps):
                Kc, Vc, Gc = torch.cat([Kc, ks[i]], 1), torch.cat([Vc, vs[i]], 1), torch.cat([Gc, lgs[i]], 1)
                pra.power_retention_inference(qs[i], Kc, Vc, Gc, S, s, switch_over_seq_len=1024)
        out["growing_cache"] = timed(growing)

        def growing_prealloc():
            cache.clean_kv()
            for i in range(steps):
                cache.step(qs[i], ks[i], vs[i], lgs[i], switch_over_seq_len=1024)
        cache.update_state(S, s)
        growing_prealloc()
        out["growing_cache_prealloc"] = timed(growing_prealloc)
    state_bytes = b * h * (pra.expanded_dim(d) * d * 2 + pra.expanded_dim(d) * 4)
    out["state_bytes"] = state_bytes
    for key in ("recurrent", "recurrent_graph"):
        out[key]["state_GBps"] = round(2 * state_bytes / (out[key]["us_per_step"] * 1e-6) / 1e9, 1)
    out["workload"] = f"power_retention_inference bf16 b={b} h={h} d={d}: prefill 2048 (switch_over_seq_len=1024), {steps} decode steps"
    return out


class KernelTimers:
    """Times every kernel of the library where it runs: the library's launch hook (pr_set_launch_hook) calls back right
    before and right after each kernel launch, and a HIP event is recorded on the launch stream at both points.
    `per_step()` gives, in launch order, the label of every kernel of a step (name#k for the k-th launch of that name in
    the step) and its average duration in ms over the steps recorded (the first `skip` steps left out)."""

    def __init__(self, _lib):
        self._lib, self.lib = _lib, _lib.load()
        self.records, self.steps = [], []
        self._t0 = None

        self._streams = {}

        def hook(name, phase, stream, user):
            sp = stream or 0
            if sp not in self._streams:
                self._streams[sp] = torch.cuda.current_stream() if sp == torch.cuda.current_stream().cuda_stream \
                    else torch.cuda.ExternalStream(sp)
            ev = torch.cuda.Event(enable_timing=True)
            ev.record(self._streams[sp])
            if phase == 0:
                self._t0 = ev
            else:
                self.records.append((name.decode(), self._t0, ev))
        self._cb = _lib.LAUNCH_HOOK(hook)   # (kept alive for as long as it is registered)

    def __enter__(self):
        # One stream while the kernels are timed: a kernel timed while another one runs beside it says nothing about
        # either (so the sum of these times exceeds a step of the node as it normally runs).
        from retention_integration_amd import fused
        self._flags = (fused.FWD_TWO_STREAMS, fused.BWD_TWO_STREAMS, fused.ATTN_BWD_TWO_STREAMS)
        fused.FWD_TWO_STREAMS = fused.BWD_TWO_STREAMS = fused.ATTN_BWD_TWO_STREAMS = False
        self.lib.pr_set_launch_hook(self._cb, None)
        return self

    def __exit__(self, *exc):
        from retention_integration_amd import fused
        self.lib.pr_set_launch_hook(None, None)
        fused.FWD_TWO_STREAMS, fused.BWD_TWO_STREAMS, fused.ATTN_BWD_TWO_STREAMS = self._flags

    def end_step(self):
        self.steps.append(self.records)
        self.records = []

    def per_step(self, skip=2):
        torch.cuda.synchronize()
        steps = self.steps[skip:] or self.steps
        out = {}
        for rec in steps:
            seen = {}
            for name, e0, e1 in rec:
                k = seen.get(name, 0)
                seen[name] = k + 1
                out.setdefault(f"{name}#{k}", []).append(e0.elapsed_time(e1))
        return {k: sum(v) / len(v) for k, v in out.items()}


def kernel_work(cfg, D_stored):
    """Algorithmic work per launch of every kernel of the headline step, by kernel name: ("mfma", flops) for the
    contractions (canonical count: compact D, causal-halved attention products, the n-1 chunks whose state is read),
    ("hbm", bytes) for the streaming kernels (what the stored layouts make them move).  The five products of the
    attention backward are split over its two kernels as 3 (dK/dV: its own two results and half of the two
    recomputed products S and dP that both kernels need) and 2 (dQ)."""
    b, t, h, d, c = cfg["b"], cfg["t"], cfg["h"], cfg["d"], cfg["chunk"]
    n, bh = t // c, b * h
    Dc = d * (d + 1) // 2
    attn = bh * n * d * c * (c + 1)          # one causal-halved product over all chunks
    state = 2.0 * bh * (n - 1) * c * Dc * d  # one state contraction
    R = b * t * h * d * 2                    # one [b, t, h, d] 16-bit tensor
    St = bh * n * D_stored * (d * 2 + 4)     # one state tensor with its fp32 key sums, all chunks
    return {
        "sympow_tn": ("mfma", state), "sympow_nn": ("mfma", state), "sympow_grad": ("mfma", state),
        "attention_fwd": ("mfma", 2.0 * attn), "chunk_fwd": ("mfma", 2.0 * attn + state),
        "attention_bwd_dkv": ("mfma", 3.0 * attn), "chunk_bwd_dq": ("mfma", 2.0 * attn + state),
        "attention_bwd_dq": ("mfma", 2.0 * attn),
        "discumsum_pair_fwd": ("hbm", 2.0 * St * (n - 1) / n), "discumsum_pair_bwd": ("hbm", 3.0 * St * (n - 1) / n),
        "qs_bwd_prep": ("hbm", 3.0 * R), "gate_apply_fwd": ("hbm", 2.0 * R), "chunk_prep_fwd": ("hbm", 2.0 * R),
    }


def roofline_block(label, ms, work):
    kind, amount = work
    if kind == "mfma":
        ach, peak, unit = amount / ms / 1e9, PEAK_BF16_TFLOPS, "TFLOP/s"
    else:
        ach, peak, unit = amount / ms / 1e6, PEAK_HBM_GBS, "GB/s"
    return {"kernel": label, "bound": kind, "achieved": round(ach, 2), "peak": peak, "unit": unit,
            "frac": round(ach / peak, 4), "ms_per_launch": round(ms, 4)}


def measured_traffic(name):
    """HBM bytes per launch of the roofline kernel as measured with rocprofv3 byte counters: read from the line
    'total HBM traffic <x> MB' of the tracked summary profiles/<name> (which gives the commands and the calibration).
    None when the file is absent or has no such line -- never a number typed in here."""
    import re
    path = os.path.join(ROOT, "profiles", name)
    try:
        m = re.search(r"total HBM traffic ([0-9.]+) MB", open(path).read())
    except OSError:
        return None, "profiles/" + name + " not found"
    if not m:
        return None, "profiles/" + name + " has no 'total HBM traffic' line"
    return float(m.group(1)) * 1e6, "profiles/" + name + " (rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated with a plain copy)"


def cpu_baseline(cfg, seconds_hint=20):
    """The CPU oracle (a port of the reference's pure-torch backend), fwd+bwd in fp32 on the host cores,
    on a bounded sample: the same shape with t cut to 32 chunks (cost is linear in the number of chunks)."""
    import oracle
    t_s = 32 * cfg["chunk"]
    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(1)
    Q, K, V, dO = (torch.randn(cfg["b"], t_s, cfg["h"], cfg["d"], generator=g).to(torch.bfloat16).float() for _ in range(4))
    lg = torch.nn.functional.logsigmoid(torch.randn(cfg["b"], t_s, cfg["h"], generator=g))
    xs = [x.requires_grad_(True) for x in (Q, K, V, lg)]
    # one untimed pass over two chunks first: thread pool, allocator and the oracle's cached index tables are warm
    w = 2 * cfg["chunk"]
    oracle.power_retention(*(x[:, :w] for x in xs), deg=2, chunk_size=cfg["chunk"]).backward(dO[:, :w])
    for x in xs:
        x.grad = None
    t0 = time.perf_counter()
    Y = oracle.power_retention(*xs, deg=2, chunk_size=cfg["chunk"])
    Y.backward(dO)
    dt = time.perf_counter() - t0
    return {"value": round(cfg["b"] * t_s / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"fwd+bwd fp32, same shape with t={t_s} (32 chunks of {cfg['chunk']}), "
                                      f"{dt:.1f} s wall after one untimed warm-up pass"}


def short_chunks(pra, dev, steps, warmup):
    """BASELINE configs[4]: many short chunks of a wide head -- the state tensors (19.3 GB each) dominate, and the
    chained state kernels apply.  Returns the figures of that workload (also printed on its own by --short-chunks):
    ms per step, tokens/s, canonical TFLOP/s, and the chained state kernel's rate over the state tensor it writes."""
    from retention_integration_amd import _lib
    b, t, h, d, c = 4, 16384, 16, 128, 128
    g = torch.Generator().manual_seed(42)
    Q, K, V = ((0.5 * torch.randn(b, t, h, d, generator=g)).to(torch.float16).to(dev).requires_grad_(True)
               for _ in range(3))
    dO = torch.randn(b, t, h, d, generator=g).to(torch.float16).to(dev)

    def step():
        for x in (Q, K, V):
            x.grad = None
        pra.power_retention(Q, K, V, None, deg=2, chunk_size=c).backward(dO)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    with KernelTimers(_lib) as kt:
        for _ in range(3):
            step()
            kt.end_step()
        per = kt.per_step(skip=1)
    f_fwd, f_bwd = flops(b, t, h, d, c, d * (d + 1) // 2)
    state_bytes = b * (t // c) * h * pra.expanded_dim(d) * d * 2
    out = {
        "metric": "fwd+bwd tokens/s at b=4,t=16384,h=16,d=128,deg=2,chunk=128 (no gating, fp16)",
        "value": round(b * t / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "power_retention fwd+bwd b=4 t=16384 h=16 d=128 deg=2 chunk_size=128 gating=False "
                               "(BASELINE configs[4])"},
        "tflops": round((f_fwd + f_bwd) / dt / 1e12, 2),
        "state_bytes_per_tensor": state_bytes,
        "kernels_us": {k: round(v * 1e3, 1) for k, v in per.items()}}
    chain = [v for k, v in per.items() if k.startswith("sympow_tn_chain#")]
    if chain:
        out["sympow_tn_chain_hbm"] = [
            {"ms_per_launch": round(v, 3), "achieved": round(state_bytes / v / 1e6, 1), "peak": PEAK_HBM_GBS,
             "unit": "GB/s", "frac": round(state_bytes / v / 1e6 / PEAK_HBM_GBS, 4)} for v in chain]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="after the warm-up steps, keep stepping untimed for this long so that the chip's clock governor "
                         "reaches its sustained state before anything is timed (0: time straight after the warm-up)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle baseline leg")
    ap.add_argument("--no-breakdown", action="store_true", help="skip the per-operator timings")
    ap.add_argument("--no-decode", action="store_true", help="skip the inference (prefill + decode) leg")
    ap.add_argument("--no-short-chunks", action="store_true", help="skip the BASELINE configs[4] leg (short_chunks key)")
    ap.add_argument("--no-chained-calls", action="store_true", help="skip the state_across_calls leg")
    ap.add_argument("--gate-runs", default="on,off,dense",
                    help="which of the three measurements of the headline step to make: on (gate skipping on: the value), "
                         "off (every tile visited: the kernel-quality figures), dense (gates that forget nothing); a "
                         "profiler run picks one so that its trace holds one kind of step")
    ap.add_argument("--counter-run", nargs="?", const="sympow_grad", default=None, metavar="KERNEL",
                    help="for rocprofv3 --pmc: launch only one kernel a few times -- sympow_grad (dK of update_state "
                         "backward, the default), chunk_fwd or chunk_bwd_dq -- and a plain device copy of 256 MiB for calibrating "
                         "byte counters")
    ap.add_argument("--attention-chunk", type=int, default=0,
                    help="for rocprofv3 --kernel-trace: run only the attention kernels, 64 times, with the headline's "
                         "rows cut into chunks of this length")
    ap.add_argument("--short-chunks", action="store_true",
                    help="instead of the headline workload: BASELINE configs[4] (fp16, b=4, t=16384, h=16, d=128, "
                         "chunk 128, no gating, inputs N(0,1)*0.5), fwd+bwd; prints its own JSON line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported", file=sys.stderr)
        sys.exit(2)
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    import retention_integration_amd as pra
    from retention_integration_amd import expanded_dim

    dev = torch.device("cuda:0")
    if args.short_chunks:
        print(json.dumps(short_chunks(pra, dev, args.steps, args.warmup)))
        return
    if args.attention_chunk:
        attention_scaling(pra, dev, args.attention_chunk)
        return
    cfg = CFG
    Q, K, V, lg, dO = make_inputs(cfg["b"], cfg["t"], cfg["h"], cfg["d"], dev)
    if args.counter_run:
        counter_run(pra, Q.detach(), K.detach(), V.detach(), lg.detach(), cfg, dev, args.counter_run)
        return
    from retention_integration_amd import _lib, fused
    lib = _lib.load()
    # gates that forget nothing inside a chunk (the distribution of the reference's own inference inputs,
    # ref: retention/create_inputs.py:39): the same step with nothing for gate skipping to leave out
    g2 = torch.Generator().manual_seed(43)
    lg_dense = torch.nn.functional.logsigmoid(6.906768 + torch.randn(cfg["b"], cfg["t"], cfg["h"], generator=g2)).to(dev)

    def median(v):
        v = sorted(v)
        return v[len(v) // 2] if len(v) % 2 else 0.5 * (v[len(v) // 2 - 1] + v[len(v) // 2])

    flush = torch.empty(512 * 1024 * 1024, dtype=torch.int8, device=dev)   # (allocated before anything is timed)

    def measure(gates, skipping):
        """The whole protocol for one choice of gates and of the library's gate skipping switch: -> dict with the median
        of the flushed steps (ms), the back-to-back figures, the first steps, and every kernel's time inside a step."""
        lib.pr_set_gate_skipping(1 if skipping else 0)
        leaves = [x.detach().clone().requires_grad_(True) for x in (Q, K, V, gates)]

        def step():
            for x in leaves:
                x.grad = None
            Y = pra.power_retention(*leaves, deg=cfg["deg"], chunk_size=cfg["chunk"])
            Y.backward(dO)

        def timed_steps(k, before=None, lead=0):
            """k steps, each bracketed by HIP events of its own; `before` is enqueued ahead of every step, outside them.
            `lead` untimed iterations of the same sequence go first, in the same queue (the host work between two
            phases idles the GPU long enough for its clock to drop)."""
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(k)]
            torch.cuda.synchronize()
            for _ in range(lead):
                if before is not None:
                    before()
                step()
            for e0, e1 in ev:
                if before is not None:
                    before()
                e0.record()
                step()
                e1.record()
            torch.cuda.synchronize()
            return [a.elapsed_time(b_) for a, b_ in ev]

        for _ in range(args.warmup):
            step()
        # The chip's clock governor drops the clock within a fraction of a millisecond of idling (an allocation, a long
        # device-side pause) and needs ~25 ms of sustained load to bring it back: straight after a few warm-up steps the
        # first step takes 2.08 ms and the twelfth 1.80.  The figures of a training loop are the settled ones, so the
        # steps run untimed for `settle_ms` before anything is timed; the unsettled steps are reported as well.
        first = timed_steps(min(args.steps, 5)) if args.settle_ms > 0 else []
        settle_steps = int(args.settle_ms / median(first)) + 1 if args.settle_ms > 0 else 0
        for _ in range(settle_steps):
            step()
        # (a) K steps back to back between two synchronisations
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        dt_b2b = (time.perf_counter() - t0) / args.steps
        # (a') the same steps once more with EVERY kernel timed where it runs: HIP events on the launch stream around
        # each launch (the library's launch hook).  For these steps the kernels run one after the other: in the steps
        # above, independent kernels of a step share the GPU on two streams, and a kernel timed while another one runs
        # beside it says nothing about either.  (So the sum of these times exceeds a headline step.)
        overlap = (fused.FWD_TWO_STREAMS, fused.BWD_TWO_STREAMS, fused.ATTN_BWD_TWO_STREAMS)
        fused.FWD_TWO_STREAMS = fused.BWD_TWO_STREAMS = fused.ATTN_BWD_TWO_STREAMS = False
        try:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                step()
            torch.cuda.synchronize()
            dt_seq = (time.perf_counter() - t0) / args.steps
            with KernelTimers(_lib) as kt:
                for _ in range(args.steps + 2):
                    step()
                    kt.end_step()
                in_step = kt.per_step(skip=2)
        finally:
            fused.FWD_TWO_STREAMS, fused.BWD_TWO_STREAMS, fused.ATTN_BWD_TWO_STREAMS = overlap
        # (b) the headline, by the reference's protocol (ref: perf/_timing.py:77-110): before every step the caches are
        # flushed (a fill of 512 MB: L2 and the 256 MB memory-side cache), then a short device-side pause lets the host
        # run ahead (launch latency is not measured), the step is bracketed by HIP events of its own, and the MEDIAN over
        # the K steps is reported.  (The reference pauses for 25 ms; here that alone would cost 10 %, see above: 0.1 ms.)
        times = timed_steps(args.steps, lambda: (flush.zero_(), torch.cuda._sleep(200_000)), lead=settle_steps // 2)
        lib.pr_set_gate_skipping(1)
        return {"dt": median(times) * 1e-3, "times": times, "b2b": dt_b2b, "seq": dt_seq, "first": first,
                "settle_steps": settle_steps, "in_step_ms": in_step}

    # The headline: the gates the benchmark contract names, the library as it ships (gate skipping on).  Beside it the
    # same step with skipping switched off -- every tile visited whatever the gates: the figures that say how good the
    # kernels are (rooflines, matrix-core share) come from THAT run -- and with gates that forget nothing.
    runs = [r for r in args.gate_runs.split(",") if r]
    assert runs and all(r in ("on", "off", "dense") for r in runs), "--gate-runs takes on, off, dense"
    head = measure(lg, True) if "on" in runs else None
    every = measure(lg, False) if "off" in runs else None
    dense = measure(lg_dense, True) if "dense" in runs else None
    head = head or every or dense      # (a run that leaves measurements out reports what it has in their place)
    every = every or head
    del flush
    dt, times, dt_b2b, dt_seq, first, settle_steps = (head[k] for k in ("dt", "times", "b2b", "seq", "first", "settle_steps"))
    in_step_ms = every["in_step_ms"]

    D_compact = cfg["d"] * (cfg["d"] + 1) // 2
    f_fwd, f_bwd = flops(cfg["b"], cfg["t"], cfg["h"], cfg["d"], cfg["chunk"], D_compact)
    canon = f_fwd + f_bwd
    tflops = canon / every["dt"] / 1e12   # (every product of the canonical count executed: skipping off)

    def summary(m):
        return {"ms_per_step": round(m["dt"] * 1e3, 4), "tokens_per_s": round(cfg["b"] * cfg["t"] / m["dt"], 1),
                "flushed_ms": {"median": round(m["dt"] * 1e3, 4), "min": round(min(m["times"]), 4),
                               "max": round(max(m["times"]), 4)},
                "back_to_back_ms_per_step": round(m["b2b"] * 1e3, 4),
                "back_to_back_one_stream_ms_per_step": round(m["seq"] * 1e3, 4),
                "kernels_us": {k: round(v * 1e3, 1) for k, v in m["in_step_ms"].items()},
                "kernels_us_sum": round(sum(m["in_step_ms"].values()) * 1e3, 1)}
    out = {
        "metric": "fwd+bwd tokens/s at t=65536,h=8,d=64,deg=2,chunk=1024 (gated, bf16)",
        "value": round(cfg["b"] * cfg["t"] / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "power_retention fwd+bwd b=1 t=65536 h=8 d=64 deg=2 chunk_size=1024 gating=True, "
                               "log_G = logsigmoid(N(0,1)) (BASELINE configs[1]+[2])", "D_state": expanded_dim(cfg["d"])},
        # value: the library as it ships -- gate skipping on -- on the gates the benchmark contract names.  Those gates
        # fall by 0.8 per step, so inside a chunk of 1024 most weights are exact zeros in fp32 and the kernels leave them
        # out (outputs and gradients identical bit for bit: tests/test_gpu_gate_skipping.py).  What a step costs when
        # nothing can be left out is reported beside it, and every kernel-quality figure (tflops, pct_bf16_mfma_peak,
        # the roofline blocks, kernels_us) is from the run with skipping OFF, in which every product is executed.
        "gate_skipping": {
            "value_measured_with": "on (library default)",
            "identical_results": "bit for bit, skipping on vs off: tests/test_gpu_gate_skipping.py",
            "on": summary(head),
            "off_every_tile_visited": summary(every),
            "gates_that_forget_nothing": dict(summary(dense or every),
                                              gates="log_G = logsigmoid(6.906768 + N(0,1)), skipping on"),
            "measured": runs,
            "canonical_tflops_at_value": round(canon / dt / 1e12, 2),
            "note": "canonical_tflops_at_value counts products the kernels did not execute: a rate of useful work, not a "
                    "matrix-core utilisation"},
        "value_every_tile_visited": round(cfg["b"] * cfg["t"] / every["dt"], 1),
        "ms_per_step_every_tile_visited": round(every["dt"] * 1e3, 4),
        "tflops": round(tflops, 2), "pct_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
        "tflops_measured_with": "gate skipping off (every product of the canonical count executed)",
        "timing": {"protocol": "W warm-up steps, then untimed steps for settle_ms (the clock governor's ramp); value = "
                               "median over K steps, each after a 512 MB cache flush and a short device-side pause, HIP "
                               "events per step (ref: perf/_timing.py:77-110); back_to_back = wall clock of K "
                               "consecutive steps / K; first_steps = the steps right after the W warm-up steps, "
                               "before settling",
                   "flushed_ms": {"median": round(dt * 1e3, 4), "min": round(min(times), 4), "max": round(max(times), 4)},
                   "back_to_back_ms_per_step": round(dt_b2b * 1e3, 4),
                   "back_to_back_one_stream_ms_per_step": round(dt_seq * 1e3, 4),
                   "first_steps_ms": [round(x, 4) for x in first],
                   "settle_ms": args.settle_ms, "settle_steps": settle_steps},
    }
    n = cfg["t"] // cfg["chunk"]
    bh = cfg["b"] * cfg["h"]
    # Roofline blocks, from the run with gate skipping off (in_step_ms = its kernel times): every product of the
    # algorithmic count is executed there.  `roofline` is the LONGEST single kernel of that step; its work per launch is
    # the algorithmic count of kernel_work().  HBM traffic of a launch comes from the tracked rocprofv3 counter summary of
    # that kernel when profiles/ holds one (parsed at run time, never typed in here).
    work = kernel_work(cfg, expanded_dim(cfg["d"]))
    out["kernels_us"] = {k: round(v * 1e3, 1) for k, v in in_step_ms.items()}
    out["kernels_us_sum"] = round(sum(in_step_ms.values()) * 1e3, 1)
    out["kernels_us_measured_with"] = "gate skipping off; gate_skipping.on.kernels_us has the kernels of the headline step"
    longest = max(in_step_ms, key=in_step_ms.get)
    base = longest.split("#")[0]
    blk = roofline_block(longest, in_step_ms[longest], work.get(base, ("hbm", 0.0)))
    traffic, traffic_src = measured_traffic(base + "_t65536_hbm_traffic.txt")
    blk["traffic"], blk["traffic_source"] = traffic, traffic_src
    out["roofline"] = blk
    # The attention backward: its two kernels together (canonical 5 products) where both run; where the query side is
    # one kernel with the query gradient through the state (chunk_bwd_dq), that kernel and the key side on their own.
    ab = [k for k in in_step_ms if k.startswith("attention_bwd_")]
    if len(ab) == 2:
        ms = sum(in_step_ms[k] for k in ab)
        out["roofline_attention_bwd"] = roofline_block(" + ".join(ab), ms, ("mfma", 5.0 * bh * n * cfg["d"] * cfg["chunk"] * (cfg["chunk"] + 1)))
    for key, label in (("roofline_attention_bwd_dkv", "attention_bwd_dkv#0"), ("roofline_chunk_bwd_dq", "chunk_bwd_dq#0")):
        if label in in_step_ms and len(ab) != 2:
            out[key] = roofline_block(label, in_step_ms[label], work[label.split("#")[0]])
    # (forward: one kernel for the attention inside the chunks, the state query and their merge where the library has it,
    # else attention_fwd and sympow_nn#0; sympow_nn's other launch is update_state's dV)
    one_kernel = "chunk_fwd#0" in in_step_ms
    for key, label in (("roofline_chunk_fwd", "chunk_fwd#0"), ("roofline_attention_fwd", "attention_fwd#0"),
                       ("roofline_update_state_fwd", "sympow_tn#0"),
                       ("roofline_update_state_bwd_dV" if one_kernel else "roofline_query_state_fwd", "sympow_nn#0"),
                       ("roofline_update_state_bwd_dK", "sympow_grad#0" if "chunk_bwd_dq#0" in in_step_ms else "sympow_grad#1"),
                       ("roofline_state_scan_fwd", "discumsum_pair_fwd#0"), ("roofline_state_scan_bwd", "discumsum_pair_bwd#0")):
        if label in in_step_ms:
            out[key] = roofline_block(label, in_step_ms[label], work[label.split("#")[0]])
    mf = sum(v for k, v in in_step_ms.items() if work.get(k.split("#")[0], ("hbm",))[0] == "mfma")
    out["kernel_time_split_us"] = {"mfma_bound": round(mf * 1e3, 1), "hbm_bound": round((sum(in_step_ms.values()) - mf) * 1e3, 1)}
    detach = [x.detach() for x in (Q, K, V, lg)]
    lib.pr_set_gate_skipping(0)   # the legs below time operators and chained calls as such: every tile visited
    if not args.no_breakdown:
        with torch.no_grad():
            bd = op_breakdown(pra, *detach, dO, cfg)
        out["breakdown_ms"] = bd
        scan_bytes = bh * expanded_dim(cfg["d"]) * cfg["d"] * (2 * n - 1) * 2
        out["discumsum_hbm"] = {"achieved": round(scan_bytes / bd["discumsum_fwd(S)"] / 1e6, 1), "peak": PEAK_HBM_GBS,
                                "unit": "GB/s", "frac": round(scan_bytes / bd["discumsum_fwd(S)"] / 1e6 / PEAK_HBM_GBS, 4)}
    if not args.no_decode:
        with torch.no_grad():
            out["decode"] = decode_bench(pra, dev)
    # chunked prefill: the forward of the same sequence in one call and in two calls that hand the state over
    # (initial_state / return_final_state), each timed like the breakdown entries (HIP events after a lead-in)
    if not args.no_chained_calls:
        with torch.no_grad():
            half = cfg["t"] // 2
            dq, dk, dv, dg = detach

            def one_call():
                return pra.power_retention(dq, dk, dv, dg, deg=cfg["deg"], chunk_size=cfg["chunk"])

            def two_calls():
                y1, st = pra.power_retention(dq[:, :half], dk[:, :half], dv[:, :half], dg[:, :half], deg=cfg["deg"],
                                             chunk_size=cfg["chunk"], return_final_state=True)
                y2 = pra.power_retention(dq[:, half:], dk[:, half:], dv[:, half:], dg[:, half:], deg=cfg["deg"],
                                         chunk_size=cfg["chunk"], initial_state=st)
                return y1, y2
            t1, t2 = event_time_ms(one_call, 10), event_time_ms(two_calls, 10)
            out["state_across_calls"] = {"forward_one_call_ms": round(t1, 4), "forward_two_calls_ms": round(t2, 4),
                                         "ratio": round(t2 / t1, 4),
                                         "workload": "forward only, the headline sequence whole vs as two halves chained "
                                                     "through (state, sum_of_keys); gate skipping off"}
    lib.pr_set_gate_skipping(1)
    if not args.no_short_chunks:
        torch.cuda.empty_cache()
        sc = short_chunks(pra, dev, 5, 2)
        out["short_chunks"] = {k: sc[k] for k in ("config", "dtype", "ms_per_step", "value", "unit", "tflops",
                                                  "state_bytes_per_tensor", "kernels_us", "sympow_tn_chain_hbm") if k in sc}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
