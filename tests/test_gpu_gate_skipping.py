"""Gate skipping: kernels leave out the key tiles, state sweeps, row blocks and scans whose every term the gates have
decayed to an exact zero (pr_set_gate_skipping, on by default).  The reference multiplies through those zeros
(retention/_attention/impl_triton.py visits every tile below the diagonal, retention/_query_state/impl_triton.py every
feature block, retention/_discumsum/reference.py:3-15 every chunk), so the bar is: not one bit of any output or gradient
changes between skipping on and off, whatever the gates, and both match the fp32 oracle as before.
"""
import math

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

DEV = "cuda"
OUT_TOL, GRAD_TOL = 1e-2, 2e-2


@pytest.fixture(scope="module")
def pra():
    import retention_integration_amd as pra
    return pra


@pytest.fixture()
def lib():
    from retention_integration_amd import _lib
    lib = _lib.load()
    yield lib
    lib.pr_set_gate_skipping(1)


def rel_l2(got, want):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def gates(kind, b, t, h, c, g):
    """log gates [b, t, h] fp32 of one of the regimes the skipping has to get right."""
    ls = torch.nn.functional.logsigmoid
    if kind == "strong":      # the benchmark contract's gates: about -0.8 per step, a chunk forgets what is 110 steps back
        return ls(torch.randn(b, t, h, generator=g))
    if kind == "weak":        # nothing ever decays to zero: skipping must change nothing, trivially
        return ls(6.9 + torch.randn(b, t, h, generator=g))
    if kind == "by_head":     # head 0 forgets, the others do not: per-(batch, head) decisions of the scans
        lg = ls(6.9 + torch.randn(b, t, h, generator=g))
        lg[:, :, 0] = ls(torch.randn(b, t, generator=g))
        return lg
    if kind == "by_chunk":    # every other chunk forgets: zero and non-zero carries alternate along a sequence
        lg = ls(6.9 + torch.randn(b, t, h, generator=g)).view(b, t // c, c, h)
        lg[:, 1::2] = ls(torch.randn(b, (t // c) // 2, c, h, generator=g))
        return lg.reshape(b, t, h).contiguous()
    if kind == "rising":      # log gates of both signs: gate sums that fall on average but rise by 3 now and then
        lg = torch.full((b, t, h), -1.0)
        lg[torch.rand(b, t, h, generator=g) < 0.05] = 3.0
        return lg
    if kind == "dead_start":  # the very first step of a chunk already forgets everything before it
        lg = ls(torch.randn(b, t, h, generator=g))
        lg.view(b, t // c, c, h)[:, :, 0] = -200.0
        return lg
    if kind == "burst":       # hardly any forgetting, except that one step in a hundred forgets everything: falls of
        lg = 0.01 * ls(1.0 + torch.randn(b, t, h, generator=g))   # 150 between two neighbouring keys of a tile
        lg[torch.rand(b, t, h, generator=g) < 0.01] = -150.0
        return lg
    if kind == "steep_head":  # head 0 forgets by e^-6 a step (96 over sixteen keys), the others hardly at all
        lg = ls(6.9 + torch.randn(b, t, h, generator=g))
        lg[:, :, 0] = ls(-6.0 + torch.randn(b, t, generator=g))
        return lg
    raise ValueError(kind)


def step(pra, Q, K, V, lg, dO, chunk):
    leaves = [x.detach().clone().requires_grad_(True) for x in (Q, K, V, lg)]
    Y = pra.power_retention(*leaves, deg=2, chunk_size=chunk)
    Y.backward(dO)
    torch.cuda.synchronize()
    return [Y.detach()] + [x.grad for x in leaves]


CASES = [
    # dtype, b, t, h, r, d, chunk, gates
    (torch.bfloat16, 1, 4096, 2, 1, 64, 1024, "strong"),      # the one-kernel readers; no carry survives: no scan
    (torch.bfloat16, 2, 2048, 2, 2, 64, 1024, "strong"),      # two sequences, GQA
    (torch.bfloat16, 1, 2048, 2, 4, 32, 512, "strong"),       # d = 32
    (torch.bfloat16, 1, 4096, 3, 1, 64, 1024, "by_head"),
    (torch.bfloat16, 1, 6144, 2, 1, 64, 1024, "by_chunk"),
    (torch.bfloat16, 1, 2048, 2, 1, 64, 1024, "rising"),
    (torch.bfloat16, 1, 2048, 2, 1, 64, 1024, "dead_start"),
    (torch.bfloat16, 1, 2048, 2, 1, 64, 1024, "weak"),
    (torch.bfloat16, 1, 1024, 2, 1, 128, 256, "strong"),      # the operator-by-operator path (d = 128) ...
    (torch.float16, 1, 1024, 2, 2, 64, 256, "strong"),        # ... and fp16
    (torch.bfloat16, 1, 1000, 2, 1, 64, 512, "strong"),       # padded last chunk
    (torch.bfloat16, 1, 1024, 2, 1, 64, None, "strong"),      # quadratic path: the attention kernels over the whole length
    (torch.bfloat16, 1, 2048, 2, 1, 64, 1024, "burst"),
    (torch.bfloat16, 1, 2048, 2, 2, 64, 512, "steep_head"),
]


@pytest.mark.parametrize("dtype,b,t,h,r,d,chunk,kind", CASES)
def test_skipping_changes_no_bit(pra, lib, dtype, b, t, h, r, d, chunk, kind):
    g = torch.Generator().manual_seed(1000 + t + d + r)
    std = 0.5 if dtype == torch.float16 else 1.0
    Q = (torch.randn(b, t, h * r, d, generator=g) * std).to(dtype).to(DEV)
    K = (torch.randn(b, t, h, d, generator=g) * std).to(dtype).to(DEV)
    V = (torch.randn(b, t, h, d, generator=g) * std).to(dtype).to(DEV)
    c_eff = chunk or t
    tg = (t + c_eff - 1) // c_eff * c_eff
    lg = gates(kind, b, tg, h, c_eff, g)[:, :t].contiguous().to(DEV)
    dO = torch.randn(b, t, h * r, d, generator=g).to(dtype).to(DEV)
    lib.pr_set_gate_skipping(1)
    assert lib.pr_get_gate_skipping() == 1
    on = step(pra, Q, K, V, lg, dO, chunk)
    lib.pr_set_gate_skipping(0)
    assert lib.pr_get_gate_skipping() == 0
    off = step(pra, Q, K, V, lg, dO, chunk)
    for name, x, y in zip(["Y", "dQ", "dK", "dV", "dlog_G"], on, off):
        assert torch.isfinite(x.float()).all(), f"{name}: non-finite values"
        assert torch.equal(x, y), f"{name}: skipping changed {int((x != y).sum())} values, " \
                                  f"largest difference {float((x.float() - y.float()).abs().max()):.3e}"


def test_skipping_against_the_oracle(pra, lib):
    """Strong gates, chunks of 1024, GQA, three chunks (so that no carry between chunks survives and the scans are left
    out): outputs and gradients against the fp32 oracle on the same rounded inputs, at the usual bar."""
    b, t, h, r, d, chunk = 1, 3072, 2, 2, 64, 1024
    g = torch.Generator().manual_seed(77)
    Q = torch.randn(b, t, h * r, d, generator=g).bfloat16()
    K = torch.randn(b, t, h, d, generator=g).bfloat16()
    V = torch.randn(b, t, h, d, generator=g).bfloat16()
    lg = gates("strong", b, t, h, chunk, g)
    dO = torch.randn(b, t, h * r, d, generator=g).bfloat16()
    lib.pr_set_gate_skipping(1)
    got = step(pra, *(x.to(DEV) for x in (Q, K, V, lg, dO)), chunk)
    oi = [x.float().clone().requires_grad_(True) for x in (Q, K, V, lg)]
    Yo = oracle.power_retention(*oi, deg=2, chunk_size=chunk)
    Yo.backward(dO.float())
    want = [Yo] + [x.grad for x in oi]
    for name, x, y, tol in zip(["Y", "dQ", "dK", "dV", "dlog_G"], got, want, [OUT_TOL] + [GRAD_TOL] * 4):
        err = rel_l2(x, y)
        print(f"  {name}: rel-L2 {err:.3e}", flush=True)
        assert err <= tol, f"{name}: rel-L2 {err:.3e} > {tol}"


STEEP_CASES = [
    # dtype, b, t, h, r, d, chunk, gates
    (torch.bfloat16, 1, 2048, 2, 1, 64, 1024, "burst"),       # the one-kernel readers
    (torch.bfloat16, 2, 256, 3, 1, 32, 128, "burst"),
    (torch.bfloat16, 1, 960, 2, 4, 64, 192, "steep_head"),
    (torch.float16, 1, 768, 2, 2, 64, 256, "steep_head"),     # the operator-by-operator path: fp16 ...
    (torch.bfloat16, 1, 512, 2, 1, 128, 128, "burst"),        # ... and d = 128
    (torch.bfloat16, 1, 700, 2, 2, 64, None, "burst"),        # quadratic path
]


@pytest.mark.parametrize("dtype,b,t,h,r,d,chunk,kind", STEEP_CASES)
def test_steep_gates_against_the_oracle(pra, lib, dtype, b, t, h, r, d, chunk, kind):
    """Gate sums that fall by more than the fp32 exponent range (87) inside one group of sixteen keys: the weight of a
    pair near the diagonal has to come from its own exponent G_q - G_k, as in the reference
    (retention/_attention/reference.py:38-44), not from a row factor and a key factor relative to a gate that a group
    shares -- those overflow and flush against each other and leave NaN or zeros where the weight is close to one."""
    g = torch.Generator().manual_seed(4242 + t + d)
    std = d ** -0.25 if dtype == torch.float16 else 1.0
    Q = (torch.randn(b, t, h * r, d, generator=g) * std).to(dtype)
    K = (torch.randn(b, t, h, d, generator=g) * std).to(dtype)
    V = (torch.randn(b, t, h, d, generator=g) * std).to(dtype)
    c_eff = chunk or t
    tg = (t + c_eff - 1) // c_eff * c_eff
    lg = gates(kind, b, tg, h, c_eff, g)[:, :t].contiguous()
    dO = torch.randn(b, t, h * r, d, generator=g).to(dtype)
    oi = [x.float().clone().requires_grad_(True) for x in (Q, K, V, lg)]
    Yo = oracle.power_retention(*oi, deg=2, chunk_size=chunk)
    Yo.backward(dO.float())
    want = [Yo] + [x.grad for x in oi]
    for skip in (1, 0):
        lib.pr_set_gate_skipping(skip)
        got = step(pra, *(x.to(DEV) for x in (Q, K, V, lg, dO)), chunk)
        for name, x, y, tol in zip(["Y", "dQ", "dK", "dV", "dlog_G"], got, want, [OUT_TOL] + [GRAD_TOL] * 4):
            assert torch.isfinite(x.float()).all(), f"{name} (skipping {skip}): non-finite values"
            err = rel_l2(x, y)
            print(f"  skipping {skip} {name}: rel-L2 {err:.3e}", flush=True)
            assert err <= tol, f"{name} (skipping {skip}): rel-L2 {err:.3e} > {tol}"


def test_live_rows_keep_their_promise(lib):
    """pr_chunk_prep_fwd's live_rows: every discounted key before live_rows[..., 0] is an exact zero, and from
    live_rows[..., 1] on the row-wise preparation of pr_query_state_bwd writes zeros for the scaled dO and the key-sum
    factor -- the two facts that pr_update_state_fwd / _bwd and pr_query_state_bwd rely on when they leave rows out.
    Weak gates leave every row alive."""
    from retention_integration_amd import _lib
    p, st = _lib.ptr, _lib.stream()
    BN, c, h, r, d = 6, 1024, 2, 2, 64
    D = oracle.expanded_dim(d)
    dt, f32 = torch.bfloat16, torch.float32
    code = _lib.dtype_code(dt)
    g = torch.Generator().manual_seed(5)
    K = torch.randn(BN, c, h, d, generator=g).to(dt).to(DEV)
    Q = torch.randn(BN, c, h * r, d, generator=g).to(dt).to(DEV)
    for kind in ("strong", "weak", "rising"):
        lg = gates(kind, BN, c, h, c, g).to(DEV)
        A, lcs = torch.empty(BN, c, h, device=DEV), torch.empty(BN, h, device=DEV)
        Kd = torch.empty_like(K)
        live = torch.full((BN, h, 2), -7, dtype=torch.int32, device=DEV)
        _lib.check(lib.pr_chunk_prep_fwd(p(lg), p(K), p(Q), p(A), p(lcs), p(Kd), None, p(live), BN, c, h, r, d, 2, code,
                                         st), "chunk_prep_fwd")
        torch.cuda.synchronize()
        assert torch.equal(A, lg.cumsum(1)) or rel_l2(A, lg.cumsum(1)) < 1e-6
        lo, hi = live[..., 0].long(), live[..., 1].long()
        assert (lo >= 0).all() and (lo < c).all() and (hi >= 0).all() and (hi <= c).all()
        t_idx = torch.arange(c, device=DEV).view(1, c, 1)
        dead_keys = t_idx < lo.view(BN, 1, h)
        assert (Kd.float().abs().amax(-1)[dead_keys] == 0).all(), f"{kind}: a discounted key before live_rows[0] is not zero"
        if kind == "weak":
            assert (lo == 0).all() and (hi == c).all()
        if kind == "strong":
            assert (lo > c // 2).all() and (hi < c // 2).all()   # (about 800 and 110 with these gates)

        # the query side: the preparation's outputs from live_rows[1] on
        rows = BN * c * h * r
        S = (torch.randn(BN, h, D, d, generator=g) * 0.1).to(dt).to(DEV)
        s = torch.rand(BN, h, D, generator=g).to(DEV) + 0.5
        O = torch.randn(BN, c, h * r, d, generator=g).to(dt).to(DEV)
        dO = torch.randn(BN, c, h * r, d, generator=g).to(dt).to(DEV)
        den = torch.rand(BN, c, h * r, generator=g).to(DEV) + 0.5
        rm = torch.randn(BN, c, h * r, generator=g).to(DEV)
        dla, dys = torch.empty_like(den), torch.empty_like(den)
        ws = torch.empty(lib.pr_query_state_bwd_workspace(BN, c, h, r, d, code), dtype=torch.uint8, device=DEV)
        _lib.check(lib.pr_query_state_bwd(p(Q), p(S), p(s), p(rm), p(A), p(O), p(den), p(dO), None, None, None, None,
                                          p(dla), p(dys), p(ws), None, BN, 1, c, h, r, d, 1.0 / d, 2, 0, 1, 0, code, st),
                   "query_state_bwd(prep)")
        torch.cuda.synchronize()
        off = (rows * d * 2 + 255) // 256 * 256
        dOs = ws[:rows * d * 2].view(dt).view(BN, c, h, r, d)
        cvec = ws[off:off + rows * 4].view(f32).view(BN, c, h, r)
        dead_q = (t_idx >= hi.view(BN, 1, h))
        assert (dOs.float().abs().amax(-1).amax(-1)[dead_q] == 0).all(), f"{kind}: scaled dO past live_rows[1] is not zero"
        assert (cvec.abs().amax(-1)[dead_q] == 0).all(), f"{kind}: key-sum factor past live_rows[1] is not zero"


def test_dS_only_call_leaves_the_dead_rows_of_the_workspace_unwritten_and_nobody_reads_them(lib):
    """pr_query_state_bwd with live_rows, as two calls: preparation + dS / ds, then dQ from the prepared workspace.  The
    first call does not store the scaled dO past the last live stage (the workspace is filled with NaN beforehand and
    keeps them there), the second, given the same live_rows, does not read those rows: dQ, dS, ds equal the one-call
    result without live_rows bit for bit."""
    from retention_integration_amd import _lib
    p, st = _lib.ptr, _lib.stream()
    BN, c, h, r, d = 4, 1024, 2, 2, 64
    D = oracle.expanded_dim(d)
    dt, f32 = torch.bfloat16, torch.float32
    code = _lib.dtype_code(dt)
    g = torch.Generator().manual_seed(15)
    K = torch.randn(BN, c, h, d, generator=g).to(dt).to(DEV)
    Q = torch.randn(BN, c, h * r, d, generator=g).to(dt).to(DEV)
    lg = gates("strong", BN, c, h, c, g).to(DEV)
    A, lcs = torch.empty(BN, c, h, device=DEV), torch.empty(BN, h, device=DEV)
    Kd = torch.empty_like(K)
    live = torch.empty((BN, h, 2), dtype=torch.int32, device=DEV)
    _lib.check(lib.pr_chunk_prep_fwd(p(lg), p(K), p(Q), p(A), p(lcs), p(Kd), None, p(live), BN, c, h, r, d, 2, code, st),
               "chunk_prep_fwd")
    S = (torch.randn(BN, h, D, d, generator=g) * 0.1).to(dt).to(DEV)
    s = torch.rand(BN, h, D, generator=g).to(DEV) + 0.5
    O = torch.randn(BN, c, h * r, d, generator=g).to(dt).to(DEV)
    dO = torch.randn(BN, c, h * r, d, generator=g).to(dt).to(DEV)
    den = torch.rand(BN, c, h * r, generator=g).to(DEV) + 0.5
    rm = torch.randn(BN, c, h * r, generator=g).to(DEV)
    rows = BN * c * h * r
    nbytes = lib.pr_query_state_bwd_workspace(BN, c, h, r, d, code)

    def call(ws, dQ, dS, ds, live_p, prepared):
        dla, dys = torch.empty_like(den), torch.empty_like(den)
        _lib.check(lib.pr_query_state_bwd(p(Q), p(S), p(s), p(rm), p(A), p(O), p(den), p(dO), dQ, dS, ds, None, p(dla),
                                          p(dys), p(ws), live_p, BN, 1, c, h, r, d, 1.0 / d, 2, 0, 0, prepared, code, st),
                   "query_state_bwd")

    lib.pr_set_gate_skipping(1)
    ws0 = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    dQ0, dS0, ds0 = torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s)
    call(ws0, p(dQ0), p(dS0), p(ds0), None, 0)
    ws1 = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=DEV)   # 0xFFFF is a NaN in both 16-bit types
    dQ1, dS1, ds1 = torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s)
    call(ws1, None, p(dS1), p(ds1), p(live), 0)
    call(ws1, p(dQ1), None, None, p(live), 1)
    torch.cuda.synchronize()
    assert torch.equal(dS1, dS0) and torch.equal(ds1, ds0) and torch.equal(dQ1, dQ0)
    hi = live[..., 1].long()
    assert (hi < c // 2).all()
    bound = (hi + 255) // 256 * 256
    t_idx = torch.arange(c, device=DEV).view(1, c, 1)
    unwritten = (t_idx >= bound.view(BN, 1, h)).view(BN, c, h, 1, 1).expand(BN, c, h, r, d)
    dOs0 = ws0[:rows * d * 2].view(dt).view(BN, c, h, r, d)
    dOs1 = ws1[:rows * d * 2].view(dt).view(BN, c, h, r, d)
    assert torch.isnan(dOs1.float()[unwritten]).all(), "a row of the scaled dO past the last live stage was written"
    assert torch.equal(dOs1[~unwritten], dOs0[~unwritten])


def test_scans_that_the_readers_make_unnecessary(lib):
    """pr_state_scan_fwd / _bwd with consumers_follow_gates: a (batch, head) whose every carry exp(log_G[k]), k >= 1, is
    zero is neither read nor written (its gate gradient is written as zero), every other one is scanned as without the
    promise; and where a carry is zero the scan's entry is its input entry next to it, bit for bit -- the fact the
    readers use (ref: retention/_discumsum/reference.py:3-15)."""
    from retention_integration_amd import _lib
    p, st = _lib.ptr, _lib.stream()
    b, n, h, F, F2 = 2, 6, 3, 4096, 256
    dt, f32 = torch.bfloat16, torch.float32
    code = _lib.dtype_code(dt)
    g = torch.Generator().manual_seed(9)
    S = torch.randn(b, n, h, F, generator=g).to(dt).to(DEV)
    s = torch.randn(b, n, h, F2, generator=g).to(DEV)
    lg = -torch.rand(b, n, h, generator=g)
    lg[:, :, 0] = -500.0                 # head 0: nothing is ever carried
    lg[:, 2, 1] = -500.0                 # head 1: one zero carry in the middle
    lg[0, 0, 0] = -0.5                   # (the factor of entry 0 multiplies the zero the scan starts from: irrelevant)
    lg = lg.to(DEV)

    def fwd(follow):
        Y = torch.full((b, n, h, F), 7.0, dtype=dt, device=DEV)
        y = torch.full((b, n, h, F2), 7.0, device=DEV)
        _lib.check(lib.pr_state_scan_fwd(p(S), p(s), p(lg), p(Y), p(y), None, None, None, None, b, n, n, h, F, F2, follow,
                                         code, st), "scan fwd")
        torch.cuda.synchronize()
        return Y, y
    Y0, y0 = fwd(0)
    Y1, y1 = fwd(1)
    assert (Y1[:, :, 0] == 7).all() and (y1[:, :, 0] == 7).all(), "head 0 was scanned"
    assert torch.equal(Y1[:, :, 1:], Y0[:, :, 1:]) and torch.equal(y1[:, :, 1:], y0[:, :, 1:])
    # what the readers use: entry k is input k - 1 where the carry into it is zero, and entry 1 always
    assert torch.equal(Y0[:, 1:, 0], S[:, :-1, 0]) and torch.equal(y0[:, 1:, 0], s[:, :-1, 0])
    assert torch.equal(Y0[:, 3, 1], S[:, 2, 1]) and torch.equal(Y0[:, 1], S[:, 0])

    dY = torch.randn(b, n, h, F, generator=g).to(dt).to(DEV)
    dy = torch.randn(b, n, h, F2, generator=g).to(DEV)
    ws = torch.empty(lib.pr_state_scan_bwd_workspace(b, n, h, F, F2), dtype=torch.uint8, device=DEV)

    def bwd(follow):
        dS = torch.full((b, n, h, F), 7.0, dtype=dt, device=DEV)
        ds = torch.full((b, n, h, F2), 7.0, device=DEV)
        dlg = torch.full((b, n, h), 7.0, device=DEV)
        _lib.check(lib.pr_state_scan_bwd(p(dY), p(Y0), p(dy), p(y0), p(lg), p(dS), p(ds), p(dlg), p(ws), None, None, None,
                                         None, b, n, n, h, F, F2, follow, code, st), "scan bwd")
        torch.cuda.synchronize()
        return dS, ds, dlg
    dS0, ds0, dl0 = bwd(0)
    dS1, ds1, dl1 = bwd(1)
    assert (dS1[:, :, 0] == 7).all() and (ds1[:, :, 0] == 7).all(), "head 0 was scanned"
    assert (dl1[:, :, 0] == 0).all() and (dl0[:, 1:, 0] == 0).all()
    assert torch.equal(dS1[:, :, 1:], dS0[:, :, 1:]) and torch.equal(ds1[:, :, 1:], ds0[:, :, 1:])
    assert torch.equal(dl1[:, :, 1:], dl0[:, :, 1:])
    # entry k is input k + 1 where the carry out of k + 1 is zero
    assert torch.equal(dS0[:, :-1, 0], dY[:, 1:, 0]) and torch.equal(ds0[:, :-1, 0], dy[:, 1:, 0])
    assert torch.equal(dS0[:, 1, 1], dY[:, 2, 1])

    # with skipping switched off the promise is not used
    lib.pr_set_gate_skipping(0)
    Y2, y2 = fwd(1)
    assert torch.equal(Y2, Y0) and torch.equal(y2, y0)


def test_switching_between_forward_and_backward_is_refused(pra, lib):
    """With skipping on, the forward leaves unwritten what its own readers leave out (dead rows of the discounted keys,
    scans that nothing survives); a backward that runs with the other setting would read them, so the node refuses."""
    g = torch.Generator().manual_seed(3)
    b, t, h, d, c = 1, 2048, 2, 64, 1024
    Q, K, V = (torch.randn(b, t, h, d, generator=g).bfloat16().to(DEV).requires_grad_(True) for _ in range(3))
    lg = gates("strong", b, t, h, c, g).to(DEV).requires_grad_(True)
    lib.pr_set_gate_skipping(1)
    Y = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=c)
    lib.pr_set_gate_skipping(0)
    with pytest.raises(RuntimeError, match="gate skipping was switched"):
        Y.sum().backward()
    lib.pr_set_gate_skipping(1)
    Y.sum().backward()          # (the same graph, with the forward's setting restored)
    assert torch.isfinite(Q.grad.float()).all()
