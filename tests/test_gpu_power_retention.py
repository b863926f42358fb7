"""GPU parity of the composed functions against the CPU oracle, the golden vectors written from the
reference, and size-independent invariants at larger shapes (ref test strategy:
perf/tests/chunk_consistency_tests.py:21-45, perf/tests/inference_tests.py:38-51, perf/tests/gqa_tests.py:72-129).
"""
import os

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

OUT_TOL, GRAD_TOL = 1e-2, 2e-2
# The fused node against the operator composition, rel-L2.  Both are checked against the oracle at the bars above; the
# one-kernel forward keeps the attention part of a row in fp32 until the merge where the composition rounds it (and its
# gradient) to 16 bits, which puts the two at 5.0e-3 to 6.1e-3 of each other on gradients, the fused node being the one
# closer to the oracle.
FUSED_VS_COMPOSED = 8e-3
DEV = "cuda"
G = os.path.join(os.path.dirname(__file__), "golden")


def rel_l2(got, want):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def check(name, got, want, tol):
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    err = rel_l2(got, want)
    print(f"  {name}: rel-L2 {err:.3e}", flush=True)
    assert err <= tol, f"{name}: rel-L2 {err:.3e} > {tol}"


def make_inputs(b, t, h, r, d, dtype, gated, seed=0, std=1.0):
    g = torch.Generator().manual_seed(seed)
    Q = (torch.randn(b, t, h * r, d, generator=g) * std).to(dtype)
    K = (torch.randn(b, t, h, d, generator=g) * std).to(dtype)
    V = (torch.randn(b, t, h, d, generator=g) * std).to(dtype)
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g)) if gated else None
    return Q, K, V, lg


@pytest.fixture(scope="module")
def pra():
    import retention_integration_amd as pra
    return pra


def run_both(pra, Q, K, V, lg, chunk, dO=None, **kw):
    gi = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    oi = [x.float().clone().requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    Y = pra.power_retention(*gi, deg=2, chunk_size=chunk, **kw)
    Yo = oracle.power_retention(*oi, deg=2, chunk_size=chunk, **kw)
    check("Y", Y, Yo, OUT_TOL)
    if dO is not None:
        Y.backward(dO.to(DEV))
        Yo.backward(dO.float())
        tol = {n: GRAD_TOL for n in ("dQ", "dK", "dV", "dlog_G")}
        if chunk is None:
            # Quadratic path on a short sequence: the first rows see one or two keys, their true gradient is a
            # cancellation to ~0 and any 16-bit run leaves a residual there.  Use the reference's own bar for such
            # cases (ref: perf/_checks.py:272-320): no worse than a small multiple of the 16-bit reference's error.
            ri = [x.clone().requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
            Yr = oracle.power_retention(*ri, deg=2, chunk_size=chunk, **kw)
            Yr.backward(dO)
            for nm, r_, g_ in zip(tol, ri, oi):
                if r_ is not None:
                    tol[nm] = max(GRAD_TOL, 2.0 * rel_l2(r_.grad, g_.grad))
        for nm, a, b_ in zip(["dQ", "dK", "dV", "dlog_G"], gi, oi):
            if a is not None:
                check(nm, a.grad, b_.grad, tol[nm])
    return Y


@pytest.mark.parametrize("dtype,b,t,h,r,d,chunk,gated", [
    (torch.bfloat16, 2, 1024, 8, 1, 64, 128, True),     # the benchmark contract's CPU-runnable shape (there in fp32)
    (torch.bfloat16, 1, 512, 2, 2, 64, 128, True),      # GQA
    (torch.bfloat16, 1, 300, 2, 1, 32, 64, True),       # padding (300 -> 320), d = 32
    (torch.float16, 1, 512, 2, 1, 128, 128, False),     # config 5 flavour: fp16, d = 128, ungated
    (torch.bfloat16, 1, 2048, 1, 1, 64, 1024, True),    # headline chunk size
    (torch.bfloat16, 1, 96, 2, 1, 64, None, True),      # quadratic path
    (torch.bfloat16, 1, 384, 2, 3, 64, 128, True),      # GQA ratio that is not a power of two (irregular tile copies)
    (torch.float16, 2, 320, 1, 3, 32, 64, True),        # the same with d = 32, fp16, padding
    (torch.bfloat16, 1, 512, 1, 8, 64, 128, True),      # GQA ratio 8 (ref: perf/tests/test_list.py:50-84)
    (torch.bfloat16, 1, 256, 1, 16, 32, 64, True),      # GQA ratio 16 (ref: perf/tests/test_list.py:189-218)
    (torch.bfloat16, 1, 128, 2, 8, 64, None, True),     # ratio 8 on the quadratic path
])
def test_power_retention_fwd_bwd(pra, dtype, b, t, h, r, d, chunk, gated):
    std = 0.5 if dtype == torch.float16 else 1.0
    Q, K, V, lg = make_inputs(b, t, h, r, d, dtype, gated, seed=t + d, std=std)
    g = torch.Generator().manual_seed(7)
    dO = torch.randn(b, t, h * r, d, generator=g).to(dtype)
    run_both(pra, Q, K, V, lg, chunk, dO)


@pytest.mark.parametrize("gated,r", [(True, 1), (True, 2), (False, 1), (True, 8), (True, 16)])
def test_fused_node_equals_operator_composition(pra, gated, r):
    """power_retention (one fused autograd node) vs the same function assembled from the four operators
    through make_power_retention: same kernels, so agreement is at rounding level."""
    Q, K, V, lg = make_inputs(2, 512, 2, r, 64, torch.bfloat16, gated, seed=21)
    dO = torch.randn(2, 512, 2 * r, 64, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(DEV)
    outs = []
    for fn in (pra.power_retention, pra.power_retention_composed):
        xs = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
        Y = fn(*xs, deg=2, chunk_size=128)
        Y.backward(dO)
        outs.append([Y] + [x.grad for x in xs if x is not None])
    for nm, a, b_ in zip(["Y", "dQ", "dK", "dV", "dlog_G"], *outs):
        # (two bf16 roundings apart: the composed path writes the attention part of the output and its gradient in 16
        # bits, the fused path keeps the first in its accumulators and scales dO on the fly)
        check(f"fused vs composed {nm}", a, b_, FUSED_VS_COMPOSED)


def test_shape_sweep_fused_vs_composed_vs_oracle(pra):
    """A seeded sweep over shapes the kernels treat differently (row counts that are not multiples of a tile, GQA
    ratios, head dims, chunk sizes from one tile to several, both dtypes, gated or not): the fused node against the
    operator composition (tight bar: same arithmetic, different kernels for the glue) and against the oracle."""
    rng = torch.Generator().manual_seed(1234)
    pick = lambda xs: xs[int(torch.randint(len(xs), (1,), generator=rng))]  # noqa: E731
    for case in range(10):
        dtype = pick([torch.bfloat16, torch.float16])
        d, r, h, b = pick([32, 64, 128]), pick([1, 2, 3, 4]), pick([1, 2]), pick([1, 2])
        chunk = pick([32, 64, 128, 256])
        n = pick([2, 3, 5])
        t = chunk * n - pick([0, 0, 1, 17])          # ragged lengths are padded up to a chunk multiple
        gated = pick([True, True, False])
        print(f"case {case}: {dtype} b={b} t={t} h={h} r={r} d={d} chunk={chunk} gated={gated}", flush=True)
        Q, K, V, lg = make_inputs(b, t, h, r, d, dtype, gated, seed=100 + case, std=0.5 if dtype == torch.float16 else 1.0)
        dO = torch.randn(b, t, h * r, d, generator=rng).to(dtype)
        outs = []
        for fn in (pra.power_retention, pra.power_retention_composed):
            xs = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
            Y = fn(*xs, deg=2, chunk_size=chunk)
            Y.backward(dO.to(DEV))
            outs.append([Y] + [x.grad for x in xs if x is not None])
        for nm, a, b_ in zip(["Y", "dQ", "dK", "dV", "dlog_G"], *outs):
            check(f"fused vs composed {nm}", a, b_, FUSED_VS_COMPOSED)
        xo = [x.float().clone().requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
        Yo = oracle.power_retention(*xo, deg=2, chunk_size=chunk)
        Yo.backward(dO.float())
        for nm, a, b_ in zip(["Y", "dQ", "dK", "dV", "dlog_G"], outs[0], [Yo] + [x.grad for x in xo if x is not None]):
            check(f"fused vs oracle {nm}", a, b_, OUT_TOL if nm == "Y" else GRAD_TOL)


@pytest.mark.parametrize("dtype,b,t,h,r,d,chunk,gated", [
    (torch.bfloat16, 2, 512, 2, 1, 64, 64, True),      # one stage per chunk
    (torch.bfloat16, 1, 640, 3, 2, 64, 128, True),     # GQA: 4 stages of folded rows per chunk, odd chunk count
    (torch.float16, 2, 512, 2, 1, 128, 128, False),    # BASELINE config 5's kind: d = 128, no gates
    (torch.bfloat16, 2, 384, 1, 4, 32, 64, True),
    (torch.float16, 1, 256, 2, 1, 32, 128, True),      # two chunks: only chunk 0 is ever accumulated
    (torch.bfloat16, 1, 512, 2, 2, 128, 128, True),    # d = 128 (32-row stages) with GQA and gates
])
def test_chained_state_kernels(pra, dtype, b, t, h, r, d, chunk, gated):
    _chained_case(pra, dtype, b, t, h, r, d, chunk, gated, 1.0)


@pytest.mark.parametrize("dtype,b,t,h,r,d,chunk", [
    (torch.bfloat16, 2, 512, 2, 1, 64, 64),
    (torch.float16, 1, 640, 2, 2, 128, 128),
    (torch.bfloat16, 1, 384, 2, 4, 32, 64),
])
def test_chained_state_kernels_weak_gates(pra, dtype, b, t, h, r, d, chunk):
    """Gates close to 1 (a chunk keeps 30-50 % of the state): every earlier chunk matters to every later one, so a
    decay applied with the wrong chunk's gate, or in the wrong order, shows (with logsigmoid(N(0,1)) gates a chunk of
    64 tokens forgets the state entirely and the scan degenerates to a shift)."""
    _chained_case(pra, dtype, b, t, h, r, d, chunk, True, 0.02)


def test_weak_gates(pra):
    """The same for the separate scan kernels (the default path at this shape)."""
    b, t, h, r, d, chunk = 2, 1024, 2, 2, 64, 128
    Q, K, V, lg = make_inputs(b, t, h, r, d, torch.bfloat16, True, seed=41)
    dO = torch.randn(b, t, h * r, d, generator=torch.Generator().manual_seed(42)).to(torch.bfloat16)
    run_both(pra, Q, K, V, lg * 0.01, chunk, dO)


def _chained_case(pra, dtype, b, t, h, r, d, chunk, gated, gate_scale):
    """Short chunks: update_state + scan, and the scan's backward + query_state's dS, as single passes that keep
    the running state in registers, against the separate kernels (tight bar: same products, but the running state
    is not rounded to 16 bits between the two steps) and against the oracle."""
    from retention_integration_amd import fused
    Q, K, V, lg = make_inputs(b, t, h, r, d, dtype, gated, seed=31, std=0.5 if dtype == torch.float16 else 1.0)
    if gated:
        lg = lg * gate_scale
    dO = torch.randn(b, t, h * r, d, generator=torch.Generator().manual_seed(32)).to(dtype)
    outs = []
    try:
        for chain in (True, False):
            fused.CHAIN = chain
            xs = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
            Y = pra.power_retention(*xs, deg=2, chunk_size=chunk)
            Y.backward(dO.to(DEV))
            outs.append([Y] + [x.grad for x in xs if x is not None])
    finally:
        fused.CHAIN = None
    names = ["Y", "dQ", "dK", "dV", "dlog_G"]
    for nm, a, b_ in zip(names, *outs):
        check(f"chained vs separate {nm}", a, b_, 6e-3)
    xo = [x.float().clone().requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    Yo = oracle.power_retention(*xo, deg=2, chunk_size=chunk)
    Yo.backward(dO.float())
    for nm, a, b_ in zip(names, outs[0], [Yo] + [x.grad for x in xo if x is not None]):
        check(f"chained vs oracle {nm}", a, b_, OUT_TOL if nm == "Y" else GRAD_TOL)


def test_chained_state_kernels_at_full_size(pra):
    """BASELINE configs[4] at its full size (fp16, b=4, t=16384, h=16, d=128, chunk 128, no gating; 19.3 GB per
    state tensor): the chained kernels, which the library picks there, against the separate ones."""
    from retention_integration_amd import fused
    b, t, h, d, c = 4, 16384, 16, 128, 128
    g = torch.Generator(device=DEV).manual_seed(7)
    Q, K, V = ((0.5 * torch.randn(b, t, h, d, generator=g, device=DEV)).half().requires_grad_(True) for _ in range(3))
    dO = torch.randn(b, t, h, d, generator=g, device=DEV).half()
    assert fused._chained(__import__("retention_integration_amd")._lib.load(), b, t // c, c, h, 1, d)
    outs = []
    try:
        for chain in (None, False):
            fused.CHAIN = chain
            for x in (Q, K, V):
                x.grad = None
            Y = pra.power_retention(Q, K, V, None, deg=2, chunk_size=c)
            Y.backward(dO)
            outs.append([Y.detach()] + [x.grad for x in (Q, K, V)])
            del Y
    finally:
        fused.CHAIN = None
    for nm, a, b_ in zip(["Y", "dQ", "dK", "dV"], *outs):
        assert torch.isfinite(a).all()
        err = ((a.float() - b_.float()).norm() / b_.float().norm()).item()
        print(f"  chained vs separate {nm}: rel-L2 {err:.3e}", flush=True)
        assert err <= 6e-3, (nm, err)
    del outs
    torch.cuda.empty_cache()


def test_chained_form_is_chosen_for_many_short_chunks(pra):
    """The library's own choice: chained where batch x heads x feature blocks fill the chip, separate kernels at the
    headline shape (8 heads, one batch element), nothing where a chunk is not a whole number of 64-row stages."""
    from retention_integration_amd import _lib
    lib = _lib.load()
    assert lib.pr_state_chain_supported(4, 128, 128, 16, 1, 128) == 2
    assert lib.pr_state_chain_supported(1, 64, 1024, 8, 1, 64) == 1
    assert lib.pr_state_chain_supported(2, 4, 96, 2, 1, 64) == 0
    assert lib.pr_state_chain_supported(2, 4, 64, 2, 3, 64) == 0
    assert lib.pr_state_chain_supported(2, 1, 64, 2, 1, 64) == 0


def test_strong_gates(pra):
    """log_G around -3 per step: weights across a chunk span e^-300, the reference gates of the kernels must keep
    every intermediate in range (same bar as the other cases)."""
    b, t, h, r, d, chunk = 1, 512, 2, 1, 64, 128
    Q, K, V, _ = make_inputs(b, t, h, r, d, torch.bfloat16, False, seed=5)
    g = torch.Generator().manual_seed(6)
    lg = -3.0 + 0.5 * torch.randn(b, t, h, generator=g)
    dO = torch.randn(b, t, h * r, d, generator=g).to(torch.bfloat16)
    run_both(pra, Q, K, V, lg.clamp(max=-0.01), chunk, dO)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("chunk", [None, 128])
def test_rows_whose_every_weight_is_tiny(pra, dtype, chunk):
    """Rows that see only keys with |q.k| ~ 1e-4 or exactly 0 (a first token orthogonal to its own key; leading
    all-zero keys).  The reference normalises the weights by the row maximum before it rounds them to 16 bits
    (retention/_attention/reference.py:50-52), so such a row is an exact average of the values it sees; in fp16 an
    unnormalised weight of 1e-8 would round to zero.  Checked row by row, not as a norm over the tensor."""
    b, t, h, r, d = 2, 256, 2, 2, 64
    Q, K, V, lg = make_inputs(b, t, h, r, d, dtype, True, seed=51, std=0.5 if dtype == torch.float16 else 1.0)
    Qf, Kf = Q.float(), K.float()
    K0 = Kf[:, 0].repeat_interleave(r, dim=1)                       # [b, hq, d]
    Qf[:, 0] -= (Qf[:, 0] * K0).sum(-1, keepdim=True) / (K0 * K0).sum(-1, keepdim=True) * K0   # q_0 orthogonal to k_0
    Kf[1, :3] = 0.0                                                 # batch 1: the first three keys are zero
    Qf[0, 5] = 0.0                                                  # a zero query: every weight is the eps term
    Qf[1, 200] = 0.0                                                # ... also deep inside a later chunk
    Q, K = Qf.to(dtype), Kf.to(dtype)
    dO = torch.randn(b, t, h * r, d, generator=torch.Generator().manual_seed(52)).to(dtype)
    xs = [x.to(DEV).requires_grad_(True) for x in (Q, K, V, lg)]
    xo = [x.float().clone().requires_grad_(True) for x in (Q, K, V, lg)]
    Y = pra.power_retention(*xs, deg=2, chunk_size=chunk)
    Yo = oracle.power_retention(*xo, deg=2, chunk_size=chunk)
    Y.backward(dO.to(DEV))
    Yo.backward(dO.float())
    row_err = (Y.float().cpu() - Yo).norm(dim=-1) / Yo.norm(dim=-1).clamp_min(1e-6)
    print(f"  worst row of Y: {row_err.max().item():.3e} (rows 0-3: {row_err[:, :4].max().item():.3e})", flush=True)
    assert row_err.max().item() <= 5e-2, "a row of Y is off"
    # Gradients.  The orthogonal first row's own dQ and dK are left out of the norm: its output does not depend on
    # its one weight, so they are a cancellation to ~0 (of dO.v against rowsum(O dO) with O rounded to 16 bits)
    # multiplied by 1/|q.k| ~ 1e4 -- any run that keeps O in 16 bits leaves a residual there.  They must be finite.
    for nm, x, o in zip(["dQ", "dK", "dV", "dlog_G"], xs, xo):
        got, want = x.grad, o.grad
        assert torch.isfinite(got.float()).all(), f"{nm}: non-finite values"
        if nm in ("dQ", "dK"):
            got, want = got[:, 1:], want[:, 1:]
        check(nm, got, want, GRAD_TOL)
    # the gate gradient of the rows that see only all-zero keys comes from the eps term of the weights alone
    got, want = xs[3].grad[1, 1:3].float().cpu(), xo[3].grad[1, 1:3]
    assert torch.allclose(got, want, rtol=5e-2, atol=1e-3), (got, want)


def test_fp32_inputs_are_rejected_loudly(pra):
    Q, K, V, lg = make_inputs(1, 256, 1, 1, 64, torch.float32, True)
    with pytest.raises((AssertionError, TypeError, RuntimeError)):
        pra.power_retention(*(x.to(DEV) for x in (Q, K, V, lg)), deg=2, chunk_size=128)


def test_chunked_equals_quadratic_on_gpu(pra):
    Q, K, V, lg = (x.to(DEV) for x in make_inputs(1, 1024, 4, 1, 64, torch.bfloat16, True, seed=3))
    a = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=128)
    b_ = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=None)
    c_ = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=256)
    check("chunk128 vs quadratic", a, b_, OUT_TOL)
    check("chunk256 vs quadratic", c_, b_, OUT_TOL)


def test_gqa_equals_repeated_heads_on_gpu(pra):
    Q, K, V, lg = (x.to(DEV) for x in make_inputs(1, 512, 2, 4, 64, torch.bfloat16, True, seed=4))
    a = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=128)
    b_ = pra.power_retention(Q, K.repeat_interleave(4, 2), V.repeat_interleave(4, 2), lg.repeat_interleave(4, 2),
                             deg=2, chunk_size=128)
    check("gqa vs mha", a, b_, 2e-3)


def load(name):
    z = np.load(os.path.join(G, name))
    return {k: torch.from_numpy(z[k]) if z[k].ndim else float(z[k]) for k in z.files}


def test_golden_power_retention(pra):
    v = load("power_retention_d32.npz")
    bf = lambda x: x.to(torch.bfloat16).to(DEV)  # noqa: E731
    Y = pra.power_retention(bf(v["Q"]), bf(v["K"]), bf(v["V"]), v["log_G"].to(DEV), deg=2, chunk_size=16)
    check("Y vs reference (chunked)", Y, v["Y_chunked"], 1.5e-2)  # golden ran on unrounded fp32 inputs
    Yq = pra.power_retention(bf(v["Q"]), bf(v["K"]), bf(v["V"]), v["log_G"].to(DEV), deg=2, chunk_size=None)
    check("Y vs reference (quadratic)", Yq, v["Y_quadratic"], 1.5e-2)


def test_golden_update_state_layout(pra):
    v = load("update_state_d32.npz")
    S, s = pra.update_state(v["K"].to(torch.bfloat16).to(DEV), v["V"].to(torch.bfloat16).to(DEV), 2)
    check("S vs reference", S, v["S"], 1.5e-2)
    check("s vs reference", s, v["N"], 1.5e-2)


def test_golden_inference(pra):
    v = load("inference_d32.npz")
    bf = lambda x: x.to(torch.bfloat16).to(DEV)  # noqa: E731
    Y0, st, sk = pra.power_retention_inference(bf(v["Q0"]), bf(v["K0"]), bf(v["V0"]), v["log_G0"].to(DEV), None, None,
                                               deg=2, switch_over_seq_len=16)
    check("Y0", Y0, v["Y0"], 1.5e-2)
    check("state0", st, v["state0"], 1.5e-2)
    check("sum_of_keys0", sk, v["sum_of_keys0"], 1.5e-2)
    Y1, st1, sk1 = pra.power_retention_inference(bf(v["Q1"]), bf(v["K1"]), bf(v["V1"]), v["log_G1"].to(DEV),
                                                 bf(v["state0"]), v["sum_of_keys0"].to(DEV), deg=2,
                                                 switch_over_seq_len=3)
    check("Y1", Y1, v["Y1"], 1.5e-2)
    check("state1", st1, v["state1"], 1.5e-2)
    check("sum_of_keys1", sk1, v["sum_of_keys1"], 1.5e-2)


@pytest.mark.parametrize("gated", [True, False])
def test_inference_prefill_then_decode_matches_oracle(pra, gated):
    b, h, r, d, t0, steps = 2, 2, 2, 64, 256, 4
    Q, K, V, lg = make_inputs(b, t0 + steps, h, r, d, torch.bfloat16, gated, seed=11)
    sl = lambda x, a, e: None if x is None else x[:, a:e]  # noqa: E731
    dv = lambda x: None if x is None else x.to(DEV)  # noqa: E731
    f32 = lambda x: None if x is None else x.float()  # noqa: E731
    Y, st, sk = pra.power_retention_inference(dv(Q[:, :t0]), dv(K[:, :t0]), dv(V[:, :t0]), dv(sl(lg, 0, t0)), None, None,
                                              deg=2, switch_over_seq_len=t0)
    Yo, sto, sko = oracle.power_retention_inference(f32(Q[:, :t0]), f32(K[:, :t0]), f32(V[:, :t0]), sl(lg, 0, t0), None,
                                                    None, deg=2, switch_over_seq_len=t0)
    check("prefill Y", Y, Yo, OUT_TOL)
    check("prefill state", st, sto, OUT_TOL)
    check("prefill sum_of_keys", sk, sko, OUT_TOL)
    for i in range(t0, t0 + steps):  # recurrent decode: query the state, then fold the new token in
        a = (dv(Q[:, i:i + 1]), dv(K[:, i:i + 1]), dv(V[:, i:i + 1]), dv(sl(lg, i, i + 1)))
        o = (f32(Q[:, i:i + 1]), f32(K[:, i:i + 1]), f32(V[:, i:i + 1]), sl(lg, i, i + 1))
        Y, st, sk = pra.power_retention_inference(*a, st, sk, deg=2, switch_over_seq_len=1)
        Yo, sto, sko = oracle.power_retention_inference(*o, sto, sko, deg=2, switch_over_seq_len=1)
        check(f"decode {i} Y", Y, Yo, OUT_TOL)
    check("final state", st, sto, OUT_TOL)
    check("final sum_of_keys", sk, sko, OUT_TOL)


def test_inference_state_parity_on_gpu(pra):
    Q, K, V, _ = make_inputs(1, 129, 2, 2, 64, torch.bfloat16, False, seed=12)
    q = Q[:, -1:].to(DEV)
    Y, st, sk = pra.power_retention_inference(q, K.to(DEV), V.to(DEV), None, None, None, deg=2, switch_over_seq_len=129)
    Y2, st2, sk2 = pra.power_retention_inference(q, None, None, None, st, sk, deg=2, switch_over_seq_len=129)
    check("Y from state vs Y from cache", Y2, Y, OUT_TOL)
    assert st2 is st and sk2 is sk


def test_large_shape_invariants(pra):
    """Headline shape: finite output, normalised rows (V = 1 -> Y = 1), linearity in V."""
    b, t, h, d, c = 1, 65536, 8, 64, 1024
    Q, K, V, lg = (x.to(DEV) for x in make_inputs(b, t, h, 1, d, torch.bfloat16, True, seed=5))
    Y = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=c)
    assert Y.shape == (b, t, h, d) and torch.isfinite(Y.float()).all()
    ones = pra.power_retention(Q, K, torch.ones_like(V), lg, deg=2, chunk_size=c)
    err = (ones.float() - 1).abs()
    print(f"  V=1 -> max |Y-1| = {err.max().item():.3e}, rms = {err.pow(2).mean().sqrt().item():.3e}", flush=True)
    assert err.pow(2).mean().sqrt().item() < 1e-2 and err.max().item() < 1e-1  # bf16 state: a few ulp at worst
    Y2 = pra.power_retention(Q, K, 2 * V, lg, deg=2, chunk_size=c)
    check("linearity in V", Y2, 2 * Y.float(), 1e-2)
    # the first chunk sees no state: it must equal quadratic attention on that chunk alone
    Yq = pra.power_retention(Q[:, :c], K[:, :c], V[:, :c], lg[:, :c], deg=2, chunk_size=None)
    check("chunk 0 vs quadratic", Y[:, :c], Yq, 1e-2)


@pytest.mark.parametrize("dtype,d,r,gated", [(torch.bfloat16, 64, 1, True), (torch.bfloat16, 32, 4, True),
                                             (torch.float16, 128, 2, False), (torch.bfloat16, 64, 8, True),
                                             # ratios 12 and 16 (ref: perf/tests/test_list.py:270-320, :189-218): one
                                             # pass over the state up to 16 query rows per kv head
                                             (torch.bfloat16, 64, 12, True), (torch.bfloat16, 32, 16, True),
                                             # beyond 16 rows the operator chain takes over (both names, same values)
                                             (torch.bfloat16, 32, 24, True)])
def test_fused_decode_step_equals_operator_chain(pra, dtype, d, r, gated):
    """The one-pass decode step (query + fold of one token) against the maker-assembled operator chain and the
    oracle: with a growing cache (no fold), with a one-token cache folded every step, and from the state alone."""
    b, h, t0, steps = 3, 2, 128, 3
    std = 0.5 if dtype == torch.float16 else 1.0
    Q, K, V, lg = make_inputs(b, t0 + steps, h, r, d, dtype, gated, seed=21 + d, std=std)
    dv = lambda x: None if x is None else x.to(DEV)  # noqa: E731
    sl = lambda x, a, e: None if x is None else x[:, a:e]  # noqa: E731
    f32 = lambda x: None if x is None else x.float()  # noqa: E731
    _, st, sk = pra.power_retention_inference(dv(Q[:, :t0]), dv(K[:, :t0]), dv(V[:, :t0]), dv(sl(lg, 0, t0)), None, None,
                                              deg=2, switch_over_seq_len=t0)
    sto, sko = st.float().cpu(), sk.float().cpu()
    # (i) cache grows, the state is only queried
    for n_cached in (1, 3):
        a = (dv(Q[:, t0 + n_cached - 1:t0 + n_cached]), dv(K[:, t0:t0 + n_cached]), dv(V[:, t0:t0 + n_cached]),
             dv(sl(lg, t0, t0 + n_cached)))
        Yf, sf, kf = pra.power_retention_inference(*a, st, sk, deg=2, switch_over_seq_len=64)
        Yc, _, _ = pra.power_retention_inference_composed(*a, st, sk, deg=2, switch_over_seq_len=64)
        Yo, _, _ = oracle.power_retention_inference(f32(Q[:, t0 + n_cached - 1:t0 + n_cached]), f32(K[:, t0:t0 + n_cached]),
                                                    f32(V[:, t0:t0 + n_cached]), sl(lg, t0, t0 + n_cached), sto, sko,
                                                    deg=2, switch_over_seq_len=64)
        assert sf is st and kf is sk
        check(f"cache of {n_cached}: fused vs chain", Yf, Yc, OUT_TOL)
        check(f"cache of {n_cached}: fused vs oracle", Yf, Yo, OUT_TOL)
    # (ii) one-token cache folded into the state at every step
    st_f, sk_f, st_c, sk_c = st, sk, st, sk
    for i in range(t0, t0 + steps):
        a = (dv(Q[:, i:i + 1]), dv(K[:, i:i + 1]), dv(V[:, i:i + 1]), dv(sl(lg, i, i + 1)))
        Yf, st_f, sk_f = pra.power_retention_inference(*a, st_f, sk_f, deg=2, switch_over_seq_len=1)
        Yc, st_c, sk_c = pra.power_retention_inference_composed(*a, st_c, sk_c, deg=2, switch_over_seq_len=1)
        Yo, sto, sko = oracle.power_retention_inference(f32(Q[:, i:i + 1]), f32(K[:, i:i + 1]), f32(V[:, i:i + 1]),
                                                        sl(lg, i, i + 1), sto, sko, deg=2, switch_over_seq_len=1)
        check(f"step {i}: fused vs chain", Yf, Yc, OUT_TOL)
        check(f"step {i}: fused vs oracle", Yf, Yo, OUT_TOL)
    check("state: fused vs chain", st_f, st_c, OUT_TOL)
    check("state: fused vs oracle", st_f, sto, OUT_TOL)
    check("sum_of_keys: fused vs oracle", sk_f, sko, OUT_TOL)
    # (iii) no cache at all
    q = dv(Q[:, -1:])
    Yf, _, _ = pra.power_retention_inference(q, None, None, None, st_f, sk_f, deg=2)
    Yc, _, _ = pra.power_retention_inference_composed(q, None, None, None, st_f, sk_f, deg=2)
    check("state only: fused vs chain", Yf, Yc, OUT_TOL)


def test_decode_step_in_place_through_the_c_abi(pra):
    """pr_decode_step with S_out = S, s_out = s (the serving loop's in-place state) gives the out-of-place results."""
    from retention_integration_amd import _lib, ops
    lib, st, p = _lib.load(), _lib.stream(), _lib.ptr
    b, h, r, d = 3, 2, 2, 64
    D = pra.expanded_dim(d)
    g = torch.Generator().manual_seed(21)
    dt = torch.bfloat16
    S = (torch.randn(b, h, D, d, generator=g) * 0.3).to(dt).to(DEV)
    s = torch.rand(b, h, D, generator=g).to(DEV) + 0.5
    Q = torch.randn(b, 1, h * r, d, generator=g).to(dt).to(DEV)
    K, V = (torch.randn(b, h, d, generator=g).to(dt).to(DEV) for _ in range(2))
    lg = torch.nn.functional.logsigmoid(torch.randn(b, h, generator=g)).to(DEV)
    out, S2, s2 = ops.decode_step(Q, lg, S, s, None, None, None, K, V, lg, 0.125 ** 2, True)
    Si, si, oi = S.clone(), s.clone(), torch.empty_like(Q)
    ws = torch.empty(lib.pr_decode_step_workspace(b, 1, h, r, d), dtype=torch.uint8, device=DEV)
    _lib.check(lib.pr_decode_step(p(Q), p(lg), p(Si), p(si), None, None, None, p(K), p(V), p(lg), p(Si), p(si), p(oi),
                                  p(ws), b, 1, h, r, d, 0.125 ** 2, 2, _lib.dtype_code(dt), 1, st), "decode_step")
    assert torch.equal(oi, out) and torch.equal(Si, S2) and torch.equal(si, s2)


@pytest.mark.parametrize("dtype,d,r,mode", [(torch.bfloat16, 64, 1, "new"), (torch.bfloat16, 64, 2, "cache"),
                                            (torch.float16, 128, 1, "new"), (torch.bfloat16, 32, 2, "state"),
                                            (torch.bfloat16, 64, 4, "new")])
def test_decode_step_large_batch_equals_small_batches(pra, dtype, d, r, mode):
    """With at least 256 (batch, kv head) pairs and at most two query rows the decode step runs as one kernel with a
    workgroup per pair; smaller batches (and more rows: the r = 4 case) slice the features and merge in a second
    kernel, the form the other tests pin to the oracle.  The same rows must come out of both, and the oracle's
    recurrent step (ref: retention/power_retention_maker.py:358-382) must agree on a slice."""
    from retention_integration_amd import ops
    b, h, t0 = 32, 8, 64
    std = 0.5 if dtype == torch.float16 else 1.0
    Q, K, V, lg = make_inputs(b, t0 + 1, h, r, d, dtype, True, seed=77 + d + r, std=std)
    Q, K, V, lg = (x.to(DEV) for x in (Q, K, V, lg))
    S, s = pra.update_state(K[:, :t0].contiguous(), V[:, :t0].contiguous(), 2)
    q = Q[:, t0:].contiguous()
    kn, vn, g1 = K[:, t0].contiguous(), V[:, t0].contiguous(), lg[:, t0].contiguous()
    gen = torch.Generator().manual_seed(5)
    hq = h * r
    scale_p = (1.0 / d ** 0.5) ** 2
    if mode == "new":
        args = lambda i: (q[i], g1[i], S[i], s[i], None, None, None, kn[i], vn[i], g1[i], scale_p, True)  # noqa: E731
    elif mode == "cache":
        Ya = torch.randn(b, 1, hq, d, generator=gen).to(dtype).to(DEV)
        la = (torch.rand(b, 1, hq, generator=gen) + 0.5).to(DEV)
        rm = torch.randn(b, 1, hq, generator=gen).to(DEV)
        args = lambda i: (q[i], g1[i], S[i], s[i], Ya[i], la[i], rm[i], None, None, None, scale_p, False)  # noqa: E731
    else:
        args = lambda i: (q[i], None, S[i], s[i], None, None, None, None, None, None, scale_p, False)  # noqa: E731
    out, S2, s2 = ops.decode_step(*args(slice(None)))
    assert torch.isfinite(out.float()).all()
    for sl in (slice(0, 3), slice(b - 3, b)):
        o_s, S_s, s_s = ops.decode_step(*[x.contiguous() if torch.is_tensor(x) else x for x in args(sl)])
        check(f"rows {sl.start}:{sl.stop} out", out[sl], o_s, 2e-3)
        if mode == "new":
            # same arithmetic element by element; in fp16 the compiler may fuse the final rounding into the multiply-add
            # in one kernel and not in the other (a last-bit difference in a few elements per million)
            check(f"rows {sl.start}:{sl.stop} state", S2[sl], S_s, 1e-4)
            assert torch.equal(s2[sl], s_s)
    if mode == "new":
        sl = slice(0, 2)
        f = lambda x: x[sl].float().cpu()  # noqa: E731
        Yo, So, so = oracle.power_retention_inference(f(q), f(K[:, t0:]), f(V[:, t0:]), lg[sl, t0:].cpu(), f(S), f(s),
                                                      deg=2, switch_over_seq_len=1)
        check("oracle out", out[sl], Yo, OUT_TOL)
        check("oracle state", S2[sl], So, OUT_TOL)
        check("oracle sum_of_keys", s2[sl], so, OUT_TOL)


def _short_d128_inputs(seed):
    dtype, b, t, h, r, d = torch.bfloat16, 1, 256, 2, 2, 128
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(b, t, h * r, d, generator=g).to(dtype)
    K, V = (torch.randn(b, t, h, d, generator=g).to(dtype) for _ in range(2))
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g))
    dO = torch.randn(b, t, h * r, d, generator=g).to(dtype)
    return Q, K, V, lg, dO


def _short_d128_case(pra, seed, chain, dO_mask=None):
    """bf16, b=1, t=256, h=2, r=2, d=128, chunk 64, gated: errors of the HIP path and of the oracle run in bf16, both
    against the fp32 oracle on the same inputs; also returns the three sets of tensors.  dO_mask [b, t, hq] zeroes the
    output gradient of some rows in all three runs."""
    from retention_integration_amd import fused
    chunk = 64
    Q, K, V, lg, dO = _short_d128_inputs(seed)
    if dO_mask is not None:
        dO = dO * dO_mask.unsqueeze(-1).to(dO.dtype)
    xo = [x.float().clone().requires_grad_(True) for x in (Q, K, V, lg)]
    Yo = oracle.power_retention(*xo, deg=2, chunk_size=chunk)
    Yo.backward(dO.float())
    xr = [x.clone().requires_grad_(True) for x in (Q, K, V, lg)]
    Yr = oracle.power_retention(*xr, deg=2, chunk_size=chunk)
    Yr.backward(dO)
    want = [Yo] + [x.grad for x in xo]
    ref16 = [Yr] + [x.grad for x in xr]
    e16 = [rel_l2(a, w) for a, w in zip(ref16, want)]
    fused.CHAIN = chain
    try:
        xs = [x.to(DEV).requires_grad_(True) for x in (Q, K, V, lg)]
        Y = pra.power_retention(*xs, deg=2, chunk_size=chunk)
        Y.backward(dO.to(DEV))
    finally:
        fused.CHAIN = None
    got = [Y] + [x.grad for x in xs]
    assert all(torch.isfinite(x.float()).all() for x in got)
    return [rel_l2(a, w) for a, w in zip(got, want)], e16, (got, ref16, want)


def _row_weight_totals(Q, K, lg, r):
    """L[b, hq, i] = sum_{j <= i} (q_i . k_j / sqrt(d))^2 exp(sum of the log gates after j up to i) in fp64: the
    normaliser of row i over its whole history (ref: retention/_attention/reference.py:42-55 without the chunking)."""
    d = Q.shape[-1]
    A = lg.double().cumsum(1).repeat_interleave(r, 2).permute(0, 2, 1)
    s = torch.einsum("bihd,bjhd->bhij", Q.double(), K.double().repeat_interleave(r, 2)) / d ** 0.5
    return torch.tril(s ** 2 * torch.exp(A[..., :, None] - A[..., None, :])).sum(-1)


def test_short_d128_chunks_against_the_16_bit_oracle(pra):
    """Four short chunks of a wide head, with the chained and the separate state kernels.  Averaged over seeds the HIP
    path must stay inside the fixed bars and be no worse than the oracle run in bf16 (the reference's own kind of bar,
    ref: perf/_checks.py:272-320).

    Seed 1001 holds an ill-conditioned row: position 192 of query head 1 is the first row of its chunk, its own key
    weighs (q.k)^2 ~ 7e-9, and the total weight of its whole history is 0.015 of the median row's -- its output is a
    ratio of two small sums over state entries that were rounded to 16 bits once per chunk, and 1/total multiplies
    that rounding in dQ of the row and, through the state, in dK and dlog_G of the keys it sees (the last keys of the
    chunk before).  Measured: that one row carries 2.9e-2 of dQ's 2.95e-2 (the oracle run in bf16: 1.5e-2 of 1.6e-2)
    and everything else is at 4e-3; the chained and the separate kernels agree to 1e-5 on it.  So the seed is checked
    in two parts at the FIXED bars: with the output gradient of the ill-conditioned rows (total weight below 2 % of
    the median; two of 1024 rows) zeroed in every run, all tensors; and dQ on all other rows with the full dO.  The
    ill-conditioned rows themselves are held to three times the bf16 oracle's error on the same rows."""
    names = ["Y", "dQ", "dK", "dV", "dlog_G"]
    fixed = [OUT_TOL] + [GRAD_TOL] * 4
    for chain in (True, False):
        seeds = [2000, 2001, 2002, 2003, 2004, 2005]
        mine, ref16 = [0.0] * 5, [0.0] * 5
        for seed in seeds:
            e, e16, _ = _short_d128_case(pra, seed, chain)
            mine = [a + x / len(seeds) for a, x in zip(mine, e)]
            ref16 = [a + x / len(seeds) for a, x in zip(ref16, e16)]
        for nm, a, r16, tol in zip(names, mine, ref16, fixed):
            print(f"  chain={chain} mean over seeds {nm}: {a:.3e} (bf16 oracle {r16:.3e})", flush=True)
            assert a <= tol and a <= 1.1 * r16, (nm, a, r16)

        Q, K, V, lg, _ = _short_d128_inputs(1001)
        L = _row_weight_totals(Q, K, lg, 2)                      # [b, hq, t]
        bad = (L < 0.02 * L.median()).permute(0, 2, 1)           # [b, t, hq]
        assert 1 <= int(bad.sum()) <= 4, int(bad.sum())
        e, e16, (got, r16, want) = _short_d128_case(pra, 1001, chain)
        for nm, a, b16 in zip(names, e, e16):
            print(f"  chain={chain} seed 1001, all rows {nm}: {a:.3e} (bf16 oracle {b16:.3e})", flush=True)
        keep = (~bad).unsqueeze(-1).float()
        dq, dq16, dqw = got[1].float().cpu(), r16[1].float(), want[1]
        a = rel_l2(dq * keep, dqw * keep)
        print(f"  chain={chain} seed 1001, dQ without the {int(bad.sum())} ill-conditioned rows: {a:.3e}", flush=True)
        assert a <= GRAD_TOL, a
        a, b16 = rel_l2(dq * (1 - keep), dqw * (1 - keep)), rel_l2(dq16 * (1 - keep), dqw * (1 - keep))
        print(f"  chain={chain} seed 1001, dQ on the ill-conditioned rows: {a:.3e} (bf16 oracle {b16:.3e})", flush=True)
        assert a <= max(GRAD_TOL, 3.0 * b16), (a, b16)
        e, e16, _ = _short_d128_case(pra, 1001, chain, dO_mask=~bad)
        for nm, a, b16, tol in zip(names, e, e16, fixed):
            print(f"  chain={chain} seed 1001, dO of those rows zeroed {nm}: {a:.3e} (bf16 oracle {b16:.3e})", flush=True)
            assert a <= tol, (nm, a, tol)


@pytest.mark.parametrize("chunk", [32, 96])
def test_chained_state_kernels_d128_short_stage(pra, chunk):
    """d = 128 stages 32 rows at a time, so chunks of 32 and 96 rows are whole stages there although they are not
    multiples of 64: the library's query and the two chained entry points must agree on that, and with 16 (batch,
    head) pairs the library picks the chained form by itself."""
    from retention_integration_amd import _lib
    lib = _lib.load()
    b, h, r, d = 4, 4, 1, 128
    t = chunk * 4
    assert lib.pr_state_chain_supported(b, t // chunk, chunk, h, r, d) >= 1
    _chained_case(pra, torch.bfloat16, b, t, h, r, d, chunk, True, 0.05)


def test_chunked_path_refuses_degree_4_and_quadratic_path_takes_it(pra):
    """deg = 4 has no state layout (ref: retention/_update_state/triton.py:310-311): both assemblies of the chunked
    path raise before launching anything; the quadratic form (attention only) computes it."""
    Q, K, V, lg = (x.to(DEV) for x in make_inputs(1, 256, 2, 1, 64, torch.bfloat16, True, seed=9))
    for fn in (pra.power_retention, pra.power_retention_composed):
        with pytest.raises(NotImplementedError):
            fn(Q, K, V, lg, deg=4, chunk_size=64)
    Y = pra.power_retention(Q, K, V, lg, deg=4, chunk_size=None)
    Yo = oracle.power_retention(Q.float().cpu(), K.float().cpu(), V.float().cpu(), lg.cpu(), deg=4, chunk_size=None)
    check("deg 4 quadratic", Y, Yo, OUT_TOL)


@pytest.mark.parametrize("dtype,b,t,h,r,d,chunk,gated,cut", [
    (torch.bfloat16, 2, 1024, 2, 1, 64, 128, True, 512),
    (torch.bfloat16, 1, 700, 2, 2, 64, 128, True, 300),      # neither part is a chunk multiple (padding inside)
    (torch.float16, 1, 512, 2, 1, 128, 64, False, 256),
    (torch.bfloat16, 1, 384, 2, 1, 32, None, True, 192),     # no chunk size: each call is one chunk
])
def test_state_carried_across_calls(pra, dtype, b, t, h, r, d, chunk, gated, cut):
    """initial_state / return_final_state: one call over t tokens == two calls chained through the returned
    (state, sum_of_keys), forward and backward, against the oracle's single call over everything; the final state
    against the oracle's."""
    std = 0.5 if dtype == torch.float16 else 1.0
    Q, K, V, lg = make_inputs(b, t, h, r, d, dtype, gated, seed=61 + d, std=std)
    dO = torch.randn(b, t, h * r, d, generator=torch.Generator().manual_seed(62)).to(dtype)
    sl = lambda x, a, e: None if x is None else x[:, a:e]  # noqa: E731
    xs = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    y1, st = pra.power_retention(*(sl(x, 0, cut) for x in xs), return_final_state=True, deg=2, chunk_size=chunk)
    y2, st2 = pra.power_retention(*(sl(x, cut, t) for x in xs), initial_state=st, return_final_state=True, deg=2,
                                  chunk_size=chunk)
    Y = torch.cat([y1, y2], 1)
    Y.backward(dO.to(DEV))
    xo = [x.float().clone().requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    Yo, sto = oracle.power_retention(*xo, return_final_state=True, deg=2, chunk_size=chunk or t)
    Yo.backward(dO.float())
    check("Y (two chained calls)", Y, Yo, OUT_TOL)
    check("final state", st2[0], sto[0], OUT_TOL)
    check("final sum_of_keys", st2[1], sto[1], OUT_TOL)
    for nm, a, o in zip(["dQ", "dK", "dV", "dlog_G"], xs, xo):
        if a is not None:
            check(nm, a.grad, o.grad, GRAD_TOL)
    # the same two calls through the operator composition (the carried state as one more entry in front of the chunk
    # states, ref: retention/power_retention_maker.py:158-172): same kernels, agreement at rounding level
    xc = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    c1, sc1 = pra.power_retention_composed(*(sl(x, 0, cut) for x in xc), return_final_state=True, deg=2, chunk_size=chunk)
    c2, sc2 = pra.power_retention_composed(*(sl(x, cut, t) for x in xc), initial_state=sc1, return_final_state=True,
                                           deg=2, chunk_size=chunk)
    torch.cat([c1, c2], 1).backward(dO.to(DEV))
    check("fused vs composed Y", Y, torch.cat([c1, c2], 1), 6e-3)
    check("fused vs composed final state", st2[0], sc2[0], 6e-3)
    check("fused vs composed final sum_of_keys", st2[1], sc2[1], 6e-3)
    for nm, a, o in zip(["dQ", "dK", "dV", "dlog_G"], xs, xc):
        if a is not None:
            check(f"fused vs composed {nm}", a.grad, o.grad, 8e-3)
    # and the inference function continues from the same pair
    q1 = torch.randn(b, 1, h * r, d, generator=torch.Generator().manual_seed(63)).to(dtype)
    Yi, _, _ = pra.power_retention_inference(q1.to(DEV), None, None, None, st2[0].detach(), st2[1].detach(), deg=2)
    Yio, _, _ = oracle.power_retention_inference(q1.float(), None, None, None, sto[0].detach(), sto[1].detach(), deg=2)
    # (one random query against the state alone: numerator and denominator are cancelling sums over 16-bit state
    # entries, so the 16-bit state's own rounding -- a few 1e-3 -- shows amplified; the bar only has to catch a wrong pair)
    check("inference from the returned state", Yi, Yio, 5e-2)


@pytest.mark.parametrize("b,t,h,r,d,chunk,gated,carried", [
    (2, 512, 2, 1, 64, 128, True, False),     # one full row block per (chunk, head)
    (1, 1024, 2, 1, 64, 256, True, True),     # two row blocks per chunk, a state in chunk 0 as well
    (1, 495, 1, 3, 64, 40, True, False),      # padded length, ragged row blocks, keys short of one tile
    (2, 384, 2, 2, 32, 96, False, False),     # d = 32, no gates, 1.5 key tiles
    (1, 128, 1, 16, 32, 16, True, True),      # 16 query heads per kv head on a quarter of a key tile
    (1, 4096, 2, 1, 64, 1024, True, False),   # the benchmark's chunk
])
def test_one_kernel_query_side_of_the_backward(pra, b, t, h, r, d, chunk, gated, carried):
    """The query side of the backward as one kernel (pr_chunk_bwd_dq) against the two kernels it replaces -- the query
    gradient through the state (sympow_grad) added in the attention kernel's epilogue -- and against the oracle: dQ and,
    through the row sums that feed the gate scan, dlog_G; dK, dV do not depend on the choice and must not move."""
    from retention_integration_amd import fused
    Q, K, V, lg = make_inputs(b, t, h, r, d, torch.bfloat16, gated, seed=77)
    dO = torch.randn(b, t, h * r, d, generator=torch.Generator().manual_seed(78)).to(torch.bfloat16)
    st0 = None
    if carried:
        Kp, Vp, lgp = (x[:, :2 * chunk] if x is not None else None for x in (K, V, lg))
        st0 = pra.power_retention(Q[:, :2 * chunk].to(DEV), Kp.to(DEV), Vp.to(DEV), None if lgp is None else lgp.to(DEV),
                                  deg=2, chunk_size=chunk, return_final_state=True)[1]
    outs = []
    try:
        for one in (True, False):
            fused.ONE_KERNEL_BWD_DQ = one
            xs = [x.to(DEV).requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
            Y = pra.power_retention(*xs, deg=2, chunk_size=chunk, initial_state=st0)
            Y.backward(dO.to(DEV))
            outs.append([Y] + [x.grad for x in xs if x is not None])
    finally:
        fused.ONE_KERNEL_BWD_DQ = True
    names = ["Y", "dQ", "dK", "dV", "dlog_G"]
    for nm, a, b_ in zip(names, *outs):
        if nm in ("Y", "dK", "dV"):
            assert torch.equal(a, b_), f"{nm} depends on the query side's kernels"
        else:
            check(f"one kernel vs two {nm}", a, b_, 5e-3)   # (the state part of dQ is not rounded to 16 bits on the way)
    So = None
    if carried:
        So = tuple(x.float().cpu() for x in st0)
    xo = [x.float().clone().requires_grad_(True) if x is not None else None for x in (Q, K, V, lg)]
    Yo = oracle.power_retention(*xo, deg=2, chunk_size=chunk, initial_state=So)
    Yo.backward(dO.float())
    for nm, a, b_ in zip(names, outs[0], [Yo] + [x.grad for x in xo if x is not None]):
        check(f"one kernel vs oracle {nm}", a, b_, OUT_TOL if nm == "Y" else GRAD_TOL)
