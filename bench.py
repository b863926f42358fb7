"""Headline benchmark: power_retention forward + backward at the reference's benchmark shape
(b=1, t=65536, h=8, d=64, bf16, deg=2, chunk_size=1024, gated; ref: perf/benchmark.py:58-61,335-343)
on one MI355X.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-breakdown]

A step = one forward + one backward over one synthetic batch already resident in HBM.
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


def event_time_ms(fn, iters, warmup=2):
    """Average duration of fn() on the current stream, by HIP events on that stream."""
    for _ in range(warmup):
        fn()
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(st)
    for _ in range(iters):
        fn()
    e1.record(st)
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def op_breakdown(pra, Q, K, V, lg, dO, cfg, iters=5):
    """Per-kernel-family timings of the pieces of one step, each launched alone (HIP events)."""
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
    return {k: round(v, 4) for k, v in res.items()}


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
    t0 = time.perf_counter()
    Y = oracle.power_retention(*xs, deg=2, chunk_size=cfg["chunk"])
    Y.backward(dO)
    dt = time.perf_counter() - t0
    return {"value": round(cfg["b"] * t_s / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"fwd+bwd fp32, same shape with t={t_s} (32 chunks of {cfg['chunk']}), "
                                      f"{dt:.1f} s wall"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle baseline leg")
    ap.add_argument("--no-breakdown", action="store_true", help="skip the per-operator timings")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported", file=sys.stderr)
        sys.exit(2)
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    import retention_integration_amd as pra
    from retention_integration_amd import expanded_dim

    cfg = CFG
    dev = torch.device("cuda:0")
    Q, K, V, lg, dO = make_inputs(cfg["b"], cfg["t"], cfg["h"], cfg["d"], dev)
    leaves = [x.requires_grad_(True) for x in (Q, K, V, lg)]

    def step():
        for x in leaves:
            x.grad = None
        Y = pra.power_retention(*leaves, deg=cfg["deg"], chunk_size=cfg["chunk"])
        Y.backward(dO)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps

    D_compact = cfg["d"] * (cfg["d"] + 1) // 2
    f_fwd, f_bwd = flops(cfg["b"], cfg["t"], cfg["h"], cfg["d"], cfg["chunk"], D_compact)
    tflops = (f_fwd + f_bwd) / dt / 1e12
    out = {
        "metric": "fwd+bwd tokens/s at t=65536,h=8,d=64,deg=2,chunk=1024 (gated, bf16)",
        "value": round(cfg["b"] * cfg["t"] / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "power_retention fwd+bwd b=1 t=65536 h=8 d=64 deg=2 chunk_size=1024 gating=True "
                               "(BASELINE configs[1]+[2])", "D_state": expanded_dim(cfg["d"])},
        "tflops": round(tflops, 2), "pct_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2),
    }
    detach = [x.detach() for x in (Q, K, V, lg)]
    if not args.no_breakdown:
        with torch.no_grad():
            bd = op_breakdown(pra, *detach, dO, cfg)
        out["breakdown_ms"] = bd
        n = cfg["t"] // cfg["chunk"]
        bh = cfg["b"] * cfg["h"]
        # dominant single kernel: the update_state forward contraction (sympow_tn), one launch = all chunks
        k_flops = 2.0 * bh * n * cfg["chunk"] * D_compact * cfg["d"]
        k_ms = bd["update_state_fwd"]
        out["roofline"] = {"kernel": "sympow_tn_kernel (update_state forward)", "bound": "mfma",
                           "achieved": round(k_flops / k_ms / 1e9, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                           "frac": round(k_flops / k_ms / 1e9 / PEAK_BF16_TFLOPS, 4), "traffic": None}
        scan_bytes = bh * expanded_dim(cfg["d"]) * cfg["d"] * (2 * n - 1) * 2
        out["discumsum_hbm"] = {"achieved": round(scan_bytes / bd["discumsum_fwd(S)"] / 1e6, 1), "peak": PEAK_HBM_GBS,
                                "unit": "GB/s", "frac": round(scan_bytes / bd["discumsum_fwd(S)"] / 1e6 / PEAK_HBM_GBS, 4)}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
