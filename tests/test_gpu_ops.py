"""GPU parity of the four HIP operators (through the C ABI) against the CPU oracle.

The oracle runs in fp32 on the same 16-bit-rounded inputs; the bar is the one the benchmark contract
states: relative L2 error <= 1e-2 on outputs and <= 2e-2 on gradients.
"""
import math

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

OUT_TOL, GRAD_TOL = 1e-2, 2e-2
DEV = "cuda"


def rel_l2(got, want):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def check(name, got, want, tol):
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    err = rel_l2(got, want)
    print(f"  {name}: rel-L2 {err:.3e}", flush=True)
    assert err <= tol, f"{name}: rel-L2 {err:.3e} > {tol}"


def rnd(*shape, dtype, scale=1.0, seed=None):
    g = torch.Generator().manual_seed(seed if seed is not None else hash(shape) % 2 ** 31)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def gates(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.nn.functional.logsigmoid(torch.randn(*shape, generator=g))


def dev(x, grad=False):
    if x is None:
        return None
    y = x.to(DEV)
    return y.requires_grad_(True) if grad else y


def gold(x, grad=False):
    if x is None:
        return None
    y = x.float().clone() if x.is_floating_point() else x.clone()
    return y.requires_grad_(True) if grad else y


@pytest.fixture(scope="module")
def pra():
    import retention_integration_amd as pra
    return pra


# ---------------------------------------------------------------- discumsum
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("keep_last", [True, False])
def test_discumsum(pra, dtype, keep_last):
    b, n, h, D, e = 2, 5, 3, 256, 16
    X, lg, dY = rnd(b, n, h, D, e, dtype=dtype, seed=1), gates(b, n, h, seed=2), None
    Xg, lgg = dev(X, True), dev(lg, True)
    Y = pra.discumsum(Xg, lgg, keep_last=keep_last)
    Xo, lgo = gold(X, True), gold(lg, True)
    Yo = oracle.discumsum(Xo, lgo)
    if not keep_last:
        Yo = Yo[:, :n]
    check("Y", Y, Yo, OUT_TOL if dtype != torch.float32 else 1e-5)
    dY = rnd(*Yo.shape, dtype=dtype, seed=3)
    Y.backward(dev(dY))
    Yo.backward(gold(dY))
    check("dX", Xg.grad, Xo.grad, GRAD_TOL if dtype != torch.float32 else 1e-5)
    check("dlog_G", lgg.grad, lgo.grad, GRAD_TOL if dtype != torch.float32 else 1e-4)


def test_discumsum_1d_features(pra):
    X, lg = rnd(1, 4, 2, 768, dtype=torch.float32, seed=4), gates(1, 4, 2, seed=5)
    check("Y", pra.discumsum(dev(X), dev(lg)), oracle.discumsum(X, lg), 1e-5)


@pytest.mark.parametrize("n_out_extra", [0, 1])
@pytest.mark.parametrize("dtype,F", [(torch.bfloat16, 768 * 32), (torch.float16, 2560 * 64)])
def test_state_scan_pair_equals_separate_scans(pra, dtype, F, n_out_extra):
    """The one-launch scan of (state, key sums) through the C ABI: same values as the two discumsum launches, and a
    gate gradient equal to the sum of theirs (ref: retention/power_retention_maker.py:167-170)."""
    from retention_integration_amd import _lib
    lib, st, p = _lib.load(), _lib.stream(), _lib.ptr
    b, n, h = 2, 6, 3
    F2 = F // (32 if F == 768 * 32 else 64)
    n_out = n + n_out_extra
    S, s, lg = dev(rnd(b, n, h, F, dtype=dtype, seed=11)), dev(rnd(b, n, h, F2, dtype=torch.float32, seed=12)), dev(gates(b, n, h, seed=13))
    code = _lib.dtype_code(dtype)
    Sc, sc = torch.empty(b, n_out, h, F, dtype=dtype, device=DEV), torch.empty(b, n_out, h, F2, device=DEV)
    Sc1, sc1 = torch.empty_like(Sc), torch.empty_like(sc)
    _lib.check(lib.pr_state_scan_fwd(p(S), p(s), p(lg), p(Sc), p(sc), None, None, None, None, b, n, n_out, h, F, F2, 0, code,
                                     st), "pair fwd")
    _lib.check(lib.pr_discumsum_fwd(p(S), p(lg), p(Sc1), b, n, n_out, h, F, code, st), "fwd")
    _lib.check(lib.pr_discumsum_fwd(p(s), p(lg), p(sc1), b, n, n_out, h, F2, _lib.PR_F32, st), "fwd")
    assert torch.equal(Sc, Sc1) and torch.equal(sc, sc1)

    dSc, dsc = dev(rnd(b, n_out, h, F, dtype=dtype, seed=14)), dev(rnd(b, n_out, h, F2, dtype=torch.float32, seed=15))
    u8 = torch.uint8
    dS, ds, dlg = torch.empty_like(S), torch.empty_like(s), torch.empty_like(lg)
    ws = torch.empty(lib.pr_state_scan_bwd_workspace(b, n, h, F, F2), dtype=u8, device=DEV)
    _lib.check(lib.pr_state_scan_bwd(p(dSc), p(Sc), p(dsc), p(sc), p(lg), p(dS), p(ds), p(dlg), p(ws), None, None, None,
                                     None, b, n, n_out, h, F, F2, 0, code, st), "pair bwd")
    dS1, ds1, dl1, dl2 = torch.empty_like(S), torch.empty_like(s), torch.empty_like(lg), torch.empty_like(lg)
    ws1 = torch.empty(max(lib.pr_discumsum_bwd_workspace(b, n, h, F, code),
                          lib.pr_discumsum_bwd_workspace(b, n, h, F2, _lib.PR_F32)), dtype=u8, device=DEV)
    _lib.check(lib.pr_discumsum_bwd(p(dSc), p(Sc), p(lg), p(dS1), p(dl1), p(ws1), b, n, n_out, h, F, code, st), "bwd")
    _lib.check(lib.pr_discumsum_bwd(p(dsc), p(sc), p(lg), p(ds1), p(dl2), p(ws1), b, n, n_out, h, F2, _lib.PR_F32, st), "bwd")
    assert torch.equal(dS, dS1) and torch.equal(ds, ds1)
    check("dlog_G", dlg, dl1 + dl2, 1e-5)


# ---------------------------------------------------------------- update_state
@pytest.mark.parametrize("dtype,d,c", [(torch.bfloat16, 64, 128), (torch.bfloat16, 32, 48), (torch.float16, 128, 64),
                                       (torch.float16, 64, 32), (torch.bfloat16, 128, 32)])
def test_update_state(pra, dtype, d, c):
    b, n, h = 1, 2, 2
    K, V = rnd(b, n, c, h, d, dtype=dtype, scale=d ** -0.25, seed=10), rnd(b, n, c, h, d, dtype=dtype, seed=11)
    Kg, Vg = dev(K, True), dev(V, True)
    S, s = pra.update_state(Kg, Vg, 2)
    Ko, Vo = gold(K, True), gold(V, True)
    So, so = oracle.update_state(Ko, Vo, 2)
    check("S", S, So, OUT_TOL)
    check("s", s, so, OUT_TOL)
    dS, ds = rnd(*So.shape, dtype=dtype, seed=12), rnd(*so.shape, dtype=torch.float32, seed=13)
    torch.autograd.backward([S, s], [dev(dS), dev(ds)])
    torch.autograd.backward([So, so], [gold(dS), gold(ds)])
    check("dK", Kg.grad, Ko.grad, GRAD_TOL)
    check("dV", Vg.grad, Vo.grad, GRAD_TOL)


def test_update_state_inference_form(pra):
    K, V = rnd(2, 40, 2, 64, dtype=torch.bfloat16, scale=0.35, seed=14), rnd(2, 40, 2, 64, dtype=torch.bfloat16, seed=15)
    S, s = pra.update_state(dev(K), dev(V), 2)
    So, so = oracle.update_state(gold(K), gold(V), 2)
    assert S.shape == (2, 2, 2560, 64) and s.shape == (2, 2, 2560)
    check("S", S, So, OUT_TOL)
    check("s", s, so, OUT_TOL)


# ---------------------------------------------------------------- query_state
@pytest.mark.parametrize("dtype,d,c,r,zis,attn", [
    (torch.bfloat16, 64, 128, 1, True, True), (torch.bfloat16, 32, 40, 2, False, True),
    (torch.float16, 128, 64, 1, True, True), (torch.bfloat16, 64, 256, 1, False, False),
    (torch.bfloat16, 64, 16, 4, False, True),
    # query-head ratios of the reference's own lists (ref: perf/tests/test_list.py:50-84 ratio 8, :189-218 ratio 16)
    (torch.bfloat16, 64, 64, 8, True, True), (torch.bfloat16, 32, 24, 16, False, True)])
def test_query_state(pra, dtype, d, c, r, zis, attn):
    b, n, h = 1, 2, 2
    D = oracle.expanded_dim(d)
    Q = rnd(b, n, c, h * r, d, dtype=dtype, seed=20)
    # a state that real keys produced, so the normaliser phi(Q).s = sum_j (q.k_j)^2 stays positive
    Ks = rnd(b, n, 48, h, d, dtype=torch.float32, scale=d ** -0.25, seed=21)
    Vs = rnd(b, n, 48, h, d, dtype=torch.float32, seed=22)
    S, s = oracle.update_state(Ks, Vs, 2)
    S = S.to(dtype)
    assert S.shape == (b, n, h, D, d)
    if zis:
        S[:, 0] = 0
        s[:, 0] = 0
    Ya = rnd(b, n, c, h * r, d, dtype=dtype, seed=23) if attn else None
    la = (rnd(b, n, c, h * r, dtype=torch.float32, seed=24).abs() + c) if attn else None
    rm = (rnd(b, n, c, h * r, dtype=torch.float32, seed=25).abs() * 3 + 1.0) if attn else None
    scale = 1.0 / math.sqrt(d)
    g_in = [dev(Q, True), dev(S, True), dev(s, True), dev(Ya, attn), dev(la, attn)]
    o_in = [gold(Q, True), gold(S, True), gold(s, True), gold(Ya, attn), gold(la, attn)]
    O = pra.query_state(*g_in, dev(rm), 2, scale, zis)
    Oo = oracle.query_state(*o_in, gold(rm), 2, scale, zis)
    check("O", O, Oo, OUT_TOL)
    dO = rnd(*Oo.shape, dtype=dtype, seed=26)
    O.backward(dev(dO))
    Oo.backward(gold(dO))
    names = ["dQ", "dS", "ds", "dY_attn", "dl_attn"]
    for nm, a, b_ in zip(names, g_in, o_in):
        if a is None:
            continue
        ga, gb = a.grad, b_.grad
        if zis and nm in ("dS", "ds"):  # chunk 0 state is declared zero: its gradient is not meaningful
            ga, gb = ga[:, 1:], gb[:, 1:]
        check(nm, ga, gb, GRAD_TOL)


@pytest.mark.parametrize("d,r", [(32, 1), (64, 1), (32, 16), (64, 16)])
def test_query_state_inference_form_gqa(pra, d, r):
    """The 4-D (inference) form at the reference's sizes: b = 32, 128 query positions, one or sixteen query heads per
    kv head, forward only (ref: perf/tests/test_list.py:189-218)."""
    b, c, h, dtype = 32, 128, 2, torch.bfloat16
    Q = rnd(b, c, h * r, d, dtype=dtype, seed=40)
    Ks = rnd(b, 48, h, d, dtype=torch.float32, scale=d ** -0.25, seed=41)
    Vs = rnd(b, 48, h, d, dtype=torch.float32, seed=42)
    S, s = oracle.update_state(Ks, Vs, 2)
    S = S.to(dtype)
    Ya = rnd(b, c, h * r, d, dtype=dtype, seed=43)
    la = rnd(b, c, h * r, dtype=torch.float32, seed=44).abs() + c
    rm = rnd(b, c, h * r, dtype=torch.float32, seed=45).abs() * 3 + 1.0
    scale = 1.0 / math.sqrt(d)
    O = pra.query_state(dev(Q), dev(S), dev(s), dev(Ya), dev(la), dev(rm), 2, scale, False)
    Oo = oracle.query_state(gold(Q), gold(S), gold(s), gold(Ya), gold(la), gold(rm), 2, scale, False)
    check("O", O, Oo, OUT_TOL)
    O2 = pra.query_state(dev(Q), dev(S), dev(s), None, None, None, 2, scale, False)
    Oo2 = oracle.query_state(gold(Q), gold(S), gold(s), None, None, None, 2, scale, False)
    check("O (state only)", O2, Oo2, OUT_TOL)


# ---------------------------------------------------------------- attention
@pytest.mark.parametrize("dtype,d,tq,tk,r,gated,norm,deg", [
    (torch.bfloat16, 64, 128, 128, 1, True, False, 2), (torch.bfloat16, 64, 200, 200, 1, False, True, 2),
    (torch.float16, 128, 96, 96, 1, True, False, 2), (torch.bfloat16, 32, 1, 130, 2, True, False, 2),
    (torch.bfloat16, 64, 70, 150, 2, True, True, 2), (torch.bfloat16, 64, 384, 384, 1, True, False, 2),
    (torch.bfloat16, 64, 1024, 1024, 1, True, False, 2), (torch.bfloat16, 64, 160, 160, 1, True, False, 4),
    (torch.bfloat16, 32, 128, 128, 2, False, True, 4),
    # query-head ratio 8 (ref: perf/tests/test_list.py:50-84, and its single-query "inference" cases) and 16
    (torch.bfloat16, 64, 128, 128, 8, True, False, 2), (torch.bfloat16, 32, 128, 128, 8, False, True, 4),
    (torch.bfloat16, 64, 1, 64, 8, True, True, 2), (torch.bfloat16, 64, 1, 64, 8, True, False, 4),
    (torch.bfloat16, 64, 1, 100, 16, True, False, 2), (torch.bfloat16, 64, 64, 64, 16, True, False, 2)])
def test_attention(pra, dtype, d, tq, tk, r, gated, norm, deg):
    b, h = 2, 2
    Q, K, V = (rnd(b, tq, h * r, d, dtype=dtype, seed=30), rnd(b, tk, h, d, dtype=dtype, seed=31),
               rnd(b, tk, h, d, dtype=dtype, seed=32))
    A = gates(b, tk, h, seed=33).cumsum(1) if gated else None
    scale = 1.0 / math.sqrt(d)
    g_in = [dev(Q, True), dev(K, True), dev(V, True), dev(A, gated)]
    o_in = [gold(Q, True), gold(K, True), gold(V, True), gold(A, gated)]
    out = pra.attention(*g_in, deg, scale=scale, norm=norm)
    ref = oracle.attention(*o_in, deg, scale=scale, norm=norm)
    if norm:
        check("Y", out, ref, OUT_TOL)
        dY = rnd(*ref.shape, dtype=dtype, seed=34)
        out.backward(dev(dY))
        ref.backward(gold(dY))
    else:
        check("rowmax", out[2], ref[2], 1e-3)
        check("l", out[1], ref[1], OUT_TOL)
        check("o", out[0], ref[0], OUT_TOL)
        dO, dl = rnd(*ref[0].shape, dtype=dtype, seed=35), rnd(*ref[1].shape, dtype=torch.float32, seed=36)
        torch.autograd.backward([out[0], out[1]], [dev(dO), dev(dl)])
        torch.autograd.backward([ref[0], ref[1]], [gold(dO), gold(dl)])
    for nm, a, b_ in zip(["dQ", "dK", "dV", "dG"], g_in, o_in):
        if a is not None:
            check(nm, a.grad, b_.grad, GRAD_TOL)


# ---------------------------------------------------------------- symmetric-state promise of the C ABI
def test_query_state_with_a_state_that_is_not_symmetric(pra):
    """The layout stores the pairs of a diagonal block in both orders.  The operator makes no assumption about them
    (ref: retention/_query_state/reference.py:27-31 expands every stored feature): a state whose two copies differ
    must give the oracle's output and gradients."""
    dtype, d, c, r = torch.bfloat16, 64, 128, 1
    b, n, h = 1, 2, 2
    Q = rnd(b, n, c, h * r, d, dtype=dtype, seed=40)
    Ks = rnd(b, n, 48, h, d, dtype=torch.float32, scale=d ** -0.25, seed=41)
    Vs = rnd(b, n, 48, h, d, dtype=torch.float32, seed=42)
    S, s = oracle.update_state(Ks, Vs, 2)
    S = (S + rnd(*S.shape, dtype=torch.float32, scale=S.std().item(), seed=43)).to(dtype)
    scale = 1.0 / math.sqrt(d)
    g_in = [dev(Q, True), dev(S, True), dev(s, True)]
    o_in = [gold(Q, True), gold(S, True), gold(s, True)]
    O = pra.query_state(*g_in, None, None, None, 2, scale, False)
    Oo = oracle.query_state(*o_in, None, None, None, 2, scale, False)
    check("O", O, Oo, OUT_TOL)
    dO = rnd(*Oo.shape, dtype=dtype, seed=44)
    O.backward(dev(dO))
    Oo.backward(gold(dO))
    for nm, a, b_ in zip(["dQ", "dS", "ds"], g_in, o_in):
        check(nm, a.grad, b_.grad, GRAD_TOL)


@pytest.mark.parametrize("dtype,d,c", [(torch.bfloat16, 64, 256), (torch.float16, 32, 128), (torch.bfloat16, 128, 128)])
def test_symmetric_state_flag_changes_nothing_for_a_symmetric_state(pra, dtype, d, c):
    """dS_symmetric / S_symmetric let the gradient kernels take one fold instead of two through the diagonal blocks
    and the two contractions over the state (query_state forward, dV of update_state backward) skip the mirrored
    quarter of every diagonal block.  For a state made by update_state (both copies of a pair are the same sum) the
    results with and without the promise agree to rounding, and the state produced by the forward kernel is
    symmetric bit for bit."""
    from retention_integration_amd import _lib, ops
    lib, st, p = _lib.load(), _lib.stream(), _lib.ptr
    b, n, h = 1, 3, 2
    std = 0.5 if dtype == torch.float16 else 1.0
    K = dev(rnd(b, n, c, h, d, dtype=dtype, scale=std, seed=50))
    V = dev(rnd(b, n, c, h, d, dtype=dtype, scale=std, seed=51))
    Q = dev(rnd(b, n, c, h, d, dtype=dtype, scale=std, seed=52))
    dO = dev(rnd(b, n, c, h, d, dtype=dtype, seed=53))
    S, s = ops.update_state_fwd(K, V)
    for y in range(d // 16):   # diagonal block y: features 128 y (y+1) + 256 y + 16 a + i  <->  pair (16y + a, 16y + i)
        f0 = 128 * y * (y + 1) + 256 * y
        blk = S[..., f0:f0 + 256, :].reshape(b, n, h, 16, 16, d)
        assert torch.equal(blk, blk.transpose(3, 4)), f"diagonal block {y} of the state is not symmetric"
    code = _lib.dtype_code(dtype)
    res = []
    for flag in (0, 1):
        dK, dV = torch.empty_like(K), torch.empty_like(V)
        _lib.check(lib.pr_update_state_bwd(p(K), p(V), p(S), p(s), None, None, None, None, p(dK), p(dV), b * n, c, h, d, 2,
                                           flag, 0, code, st),
                   "update_state_bwd")
        O, den = torch.empty_like(Q), torch.empty(b, n, c, h, dtype=torch.float32, device=DEV)
        _lib.check(lib.pr_query_state_fwd(p(Q), p(S), p(s), None, None, None, None, p(O), p(den), b * n, n, c, h, 1, d,
                                          1.0 / d, 2, 0, flag, code, st), "query_state_fwd")
        dQ, dS, ds = torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s)
        ws = torch.empty(lib.pr_query_state_bwd_workspace(b * n, c, h, 1, d, code), dtype=torch.uint8, device=DEV)
        _lib.check(lib.pr_query_state_bwd(p(Q), p(S), p(s), None, None, p(O), p(den), p(dO), p(dQ), p(dS), p(ds), None, None,
                                          None, p(ws), None, b * n, n, c, h, 1, d, 1.0 / d, 2, 0, flag, 0, code, st),
                   "query_state_bwd")
        res.append((dK, dV, dQ, dS, ds, O, den))
    for nm, a, b_ in zip(["dK", "dV", "dQ", "dS", "ds", "O", "den"], res[1], res[0]):
        check(f"{nm}: with the promise vs without", a, b_, 3e-3)
    assert torch.equal(res[0][3], res[1][3])
    Oo = oracle.query_state(gold(Q.cpu()), gold(S.cpu()), gold(s.cpu()), None, None, None, 2, 1.0 / math.sqrt(d), False)
    check("O with the promise vs the oracle", res[1][5], Oo, OUT_TOL)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_discumsum_without_gates_is_the_plain_cumsum(dtype):
    """log_G = None: the reference's other branch (ref: retention/_discumsum/reference.py:4-5), n entries."""
    import retention_integration_amd as pra
    g = torch.Generator().manual_seed(3)
    X = torch.randn(2, 6, 3, 40, 16, generator=g).to(dtype)
    Xg = X.to("cuda").requires_grad_(True)
    Y = pra.discumsum(Xg, None)
    Xo = X.float().clone().requires_grad_(True)
    Yo = oracle.discumsum(Xo, None)
    assert Y.shape == Yo.shape == X.shape
    W = torch.randn(X.shape, generator=g)
    (Y.float() * W.to("cuda")).sum().backward()
    (Yo * W).sum().backward()
    for nm, a, b in (("Y", Y, Yo), ("dX", Xg.grad, Xo.grad)):
        err = ((a.detach().float().cpu() - b.detach()).norm() / b.detach().norm()).item()
        print(f"  {nm}: rel-L2 {err:.3e}", flush=True)
        assert err <= (1e-2 if dtype == torch.bfloat16 else 1e-5)


def test_golden_update_state_d64_forward_and_backward():
    """The d = 64 layout and update_state's backward through the HIP kernels against the vector written from the
    reference (its hand-written backward, ref: retention/_update_state/reference.py:55-83).  The inputs are multiples of
    1/4 (exact in bf16); the upstream gradients are rounded to bf16 on the way in."""
    import os
    import numpy as np
    import retention_integration_amd as pra
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "update_state_d64_bwd.npz"))
    v = {k: torch.from_numpy(z[k]) for k in z.files}
    K = v["K"].to(torch.bfloat16).to("cuda").requires_grad_(True)
    V = v["V"].to(torch.bfloat16).to("cuda").requires_grad_(True)
    assert torch.equal(K.detach().float().cpu(), v["K"]) and torch.equal(V.detach().float().cpu(), v["V"])
    S, N = pra.update_state(K, V, 2)
    rel = lambda a, b: ((a.detach().float().cpu() - b).norm() / b.norm()).item()  # noqa: E731
    print(f"  S {rel(S, v['S']):.3e}  N {rel(N, v['N']):.3e}", flush=True)
    assert rel(S, v["S"]) <= 5e-3 and rel(N, v["N"]) <= 1e-6
    dS16 = (v["dS_u"][:, None] * v["dS_w"][None, :]).view(1, 1, 1, 2560, 64).to(torch.bfloat16)
    dK, dV = torch.autograd.grad((S, N), (K, V), (dS16.to("cuda"), v["dN"].to("cuda")))
    # the reference's gradients for the same (rounded) upstream gradient: linear in dS, so recompute the small
    # difference with the oracle, which the CPU suite pins to the reference's vector
    Ko, Vo = v["K"].clone().requires_grad_(True), v["V"].clone().requires_grad_(True)
    So, No = oracle.update_state(Ko, Vo, 2)
    dKo, dVo = torch.autograd.grad((So, No), (Ko, Vo), (dS16.float(), v["dN"]))
    print(f"  dK {rel(dK, dKo):.3e}  dV {rel(dV, dVo):.3e}", flush=True)
    assert rel(dK, dKo) <= 2e-2 and rel(dV, dVo) <= 2e-2


# ---------------------------------------------------------------- state handed across scans
@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.float16, 32)])
def test_state_scan_with_a_starting_value_and_a_final_entry(pra, dtype, d):
    """pr_state_scan_fwd / _bwd connected to the calls before and after (ref: retention/power_retention_maker.py:131-140,
    158-172): the scans start from (S_init, s_init) instead of zero and hand out entry n; the backward takes the
    gradient of that entry and hands out the gradient of the starting value.  Against the recurrence written out in
    fp32 with autograd."""
    from retention_integration_amd import _lib
    lib, st, p = _lib.load(), _lib.stream(), _lib.ptr
    code = _lib.dtype_code(dtype)
    b, n, h = 2, 5, 3
    D = oracle.expanded_dim(d)
    f32 = torch.float32
    S, s = rnd(b, n, h, D, d, dtype=dtype, seed=70), rnd(b, n, h, D, dtype=f32, seed=71)
    S0, s0 = rnd(b, h, D, d, dtype=dtype, seed=72), rnd(b, h, D, dtype=f32, seed=73)
    lg = gates(b, n, h, seed=74)
    dY, dy = rnd(b, n, h, D, d, dtype=dtype, seed=75), rnd(b, n, h, D, dtype=f32, seed=76)
    dYf, dyf = rnd(b, h, D, d, dtype=dtype, seed=77), rnd(b, h, D, dtype=f32, seed=78)
    E = lambda *shape, dt=dtype: torch.empty(*shape, dtype=dt, device=DEV)  # noqa: E731
    Y, y, Yf, yf = E(b, n, h, D, d), E(b, n, h, D, dt=f32), E(b, h, D, d), E(b, h, D, dt=f32)
    g = [dev(x) for x in (S, s, lg, S0, s0, dY, dy, dYf, dyf)]
    _lib.check(lib.pr_state_scan_fwd(p(g[0]), p(g[1]), p(g[2]), p(Y), p(y), p(g[3]), p(g[4]), p(Yf), p(yf), b, n, n, h,
                                     D * d, D, 0, code, st), "scan fwd")
    dX, dx, dlg, dY0, dy0 = E(b, n, h, D, d), E(b, n, h, D, dt=f32), E(b, n, h, dt=f32), E(b, h, D, d), E(b, h, D, dt=f32)
    ws = torch.empty(lib.pr_state_scan_bwd_workspace(b, n, h, D * d, D), dtype=torch.uint8, device=DEV)
    _lib.check(lib.pr_state_scan_bwd(p(g[5]), p(Y), p(g[6]), p(y), p(g[2]), p(dX), p(dx), p(dlg), p(ws), p(g[7]), p(g[8]),
                                     p(dY0), p(dy0), b, n, n, h, D * d, D, 0, code, st), "scan bwd")

    # the recurrence, in fp32 with autograd (the kernel rounds the running state only when it stores an entry)
    o = [gold(x, True) for x in (S, s, lg, S0, s0)]

    def scan(X, init, gates_):
        cur, out = init, []
        for k in range(n):
            out.append(cur)
            cur = cur * torch.exp(gates_[:, k]).reshape(b, h, *([1] * (X.dim() - 3))) + X[:, k]
        return torch.stack(out, 1), cur
    Yo, Yfo = scan(o[0], o[3], o[2])
    yo, yfo = scan(o[1], o[4], o[2])
    check("Y", Y, Yo, OUT_TOL)
    check("y", y, yo, 1e-5)
    check("Y_final", Yf, Yfo, OUT_TOL)
    check("y_final", yf, yfo, 1e-5)
    torch.autograd.backward([Yo, yo, Yfo, yfo], [gold(dY), gold(dy), gold(dYf), gold(dyf)])
    check("dX", dX, o[0].grad, GRAD_TOL)
    check("dx", dx, o[1].grad, 1e-5)
    check("dS_init", dY0, o[3].grad, GRAD_TOL)
    check("ds_init", dy0, o[4].grad, 1e-5)
    check("dlog_G", dlg, o[2].grad, GRAD_TOL)


# ---------------------------------------------------------------- one-kernel forward of the chunks
@pytest.mark.parametrize("d,c,r,gated,zis", [
    (64, 128, 1, True, True),      # one full row block per (chunk, head)
    (64, 256, 1, True, False),     # two row blocks, a state in every chunk
    (64, 40, 3, True, True),       # 120 folded rows: a ragged row block, keys short of one tile
    (32, 96, 2, True, False),      # d = 32; 192 folded rows (one full and one half row block), 1.5 key tiles
    (64, 192, 1, False, True),     # no gates
    (32, 16, 16, False, False),    # 16 query heads per kv head on a quarter of a key tile
    (64, 1024, 1, True, True),     # the benchmark's chunk
])
def test_chunk_fwd_in_one_kernel(pra, d, c, r, gated, zis):
    """pr_chunk_fwd against (a) the oracle's attention and query_state composed as the chunked algorithm composes them
    (ref: retention/power_retention_maker.py:176-190: attention without normalisation inside the chunk, the gated
    queries against the chunk's starting state, merged) and (b) the two library calls it replaces, whose rowmax and
    normaliser it must reproduce because the backward kernels take them as they are."""
    from retention_integration_amd import _lib
    lib, st, p = _lib.load(), _lib.stream(), _lib.ptr
    dtype = torch.bfloat16
    code = _lib.dtype_code(dtype)
    assert lib.pr_chunk_fwd_supported(d, 2, code) == 1
    assert lib.pr_chunk_fwd_supported(128, 2, code) == 0 and lib.pr_chunk_fwd_supported(d, 2, _lib.dtype_code(torch.float16)) == 0
    b, n, h = 2, 3, 2
    BN, hq = b * n, h * r
    D = oracle.expanded_dim(d)
    f32 = torch.float32
    scale = 1.0 / math.sqrt(d)
    Q, K, V = (rnd(BN, c, hq, d, dtype=dtype, seed=80), rnd(BN, c, h, d, dtype=dtype, seed=81),
               rnd(BN, c, h, d, dtype=dtype, seed=82))
    A = gates(BN, c, h, seed=83).cumsum(1) if gated else None
    # states that real keys produced (positive normaliser); chunk 0 of every batch entry zero when declared so
    Ks, Vs = rnd(BN, 64, h, d, dtype=f32, scale=1.0, seed=84), rnd(BN, 64, h, d, dtype=f32, seed=85)
    S, s = oracle.update_state(Ks, Vs, 2)
    S = S.to(dtype)
    if zis:
        S.view(b, n, h, D, d)[:, 0] = 0
        s.view(b, n, h, D)[:, 0] = 0

    E = lambda *shape, dt=dtype: torch.empty(*shape, dtype=dt, device=DEV)  # noqa: E731
    g = {k: dev(v) for k, v in dict(Q=Q, K=K, V=V, A=A, S=S, s=s).items()}
    pa = p(g["A"]) if gated else None
    O, rm, den = E(BN, c, hq, d), E(BN, c, hq, dt=f32), E(BN, c, hq, dt=f32)
    _lib.check(lib.pr_chunk_fwd(p(g["Q"]), p(g["K"]), p(g["V"]), pa, p(g["S"]), p(g["s"]), None, None, None, p(O), p(rm),
                                p(den), BN, n, c,
                                h, r, d, scale, 2, 1 if zis else 0, code, st), "chunk_fwd")
    # (b) the two calls
    Ya, la, rm2, O2, den2 = E(BN, c, hq, d), E(BN, c, hq, dt=f32), E(BN, c, hq, dt=f32), E(BN, c, hq, d), E(BN, c, hq, dt=f32)
    _lib.check(lib.pr_attention_fwd(p(g["Q"]), p(g["K"]), p(g["V"]), pa, p(Ya), p(la), p(rm2), BN, c, c, h, r, d, scale,
                                    2, 0, code, st), "attention_fwd")
    _lib.check(lib.pr_query_state_fwd(p(g["Q"]), p(g["S"]), p(g["s"]), p(Ya), p(la), p(rm2), pa, p(O2), p(den2), BN, n, c,
                                      h, r, d, scale ** 2, 2, 1 if zis else 0, 1, code, st), "query_state_fwd")
    torch.cuda.synchronize()
    check("rowmax vs two calls", rm, rm2, 1e-6)
    check("den vs two calls", den, den2, 2e-3)      # (the two calls take the attention sums through one more rounding)
    check("O vs two calls", O, O2, 5e-3)

    # (a) the oracle's composition, in fp32 on the same inputs; the query gate exp(A / 2) as the reference applies it
    Qo = gold(Q).view(b, n, c, hq, d)
    Ao = gold(A).view(b, n, c, h) if gated else None
    Ya_o, la_o, rm_o = oracle.attention(gold(Q), gold(K), gold(V), gold(A), 2, scale=scale, norm=False)
    if gated:
        Qo = Qo * torch.exp(Ao / 2).repeat_interleave(r, dim=3)[..., None]
    Oo = oracle.query_state(Qo, gold(S).view(b, n, h, D, d), gold(s).view(b, n, h, D), Ya_o.view(b, n, c, hq, d),
                            la_o.view(b, n, c, hq), rm_o.view(b, n, c, hq), 2, scale, zis)
    check("rowmax vs oracle", rm, rm_o, 1e-3)
    check("O vs oracle", O.view(b, n, c, hq, d), Oo, OUT_TOL)
    per_chunk = ((O.view(b, n, c, hq, d).float().cpu() - Oo).pow(2).sum((2, 4)).sqrt() / Oo.pow(2).sum((2, 4)).sqrt())
    print(f"  worst (batch, chunk, head): {per_chunk.max().item():.3e}", flush=True)
    assert per_chunk.max().item() <= OUT_TOL
