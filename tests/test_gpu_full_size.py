"""Parity at the benchmark contract's full sizes, against the fp32 CPU oracle.

The kernels' workgroup placement depends on how many (chunk, head) pairs a launch has (the causal blocks of the
attention kernels are dealt to (XCD, shader engine) groups pair by pair, the state kernels group the workgroups of a
pair on one XCD), so small shapes cannot stand in for the headline one: a mis-dealt block would be one chunk of one
head.  Heads are independent, so the oracle runs on slices of heads (bounded host memory) while the GPU launch keeps
all 512 pairs; errors are asserted per (chunk, head) as well as over each tensor.
(ref test strategy: perf/tests/common_tests.py:98-132, perf/tests/inference_tests.py:38-51)
"""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

OUT_TOL, GRAD_TOL = 1e-2, 2e-2   # rel-L2 vs the fp32 oracle on the same bf16-rounded inputs
DEV = "cuda"


@pytest.fixture(scope="module")
def pra():
    import retention_integration_amd as pra
    return pra


def _rel(got, want, dims):
    got, want = got.float(), want.float()
    num = (got - want).pow(2).sum(dims).sqrt()
    return num / want.pow(2).sum(dims).sqrt().clamp_min(1e-30)


def test_headline_shape_fwd_bwd_matches_the_oracle_per_chunk(pra):
    """b=1, t=65536, h=8, d=64, deg=2, chunk 1024, gated, bf16, dO ~ N(0,1): Y, dQ, dK, dV, dlog_G."""
    b, t, h, d, c = 1, 65536, 8, 64, 1024
    n = t // c
    g = torch.Generator().manual_seed(2024)
    Q, K, V = (torch.randn(b, t, h, d, generator=g).to(torch.bfloat16) for _ in range(3))
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g))
    dO = torch.randn(b, t, h, d, generator=g).to(torch.bfloat16)

    xs = [x.to(DEV).requires_grad_(True) for x in (Q, K, V, lg)]
    Y = pra.power_retention(*xs, deg=2, chunk_size=c)
    Y.backward(dO.to(DEV))
    torch.cuda.synchronize()
    got = {"Y": Y.detach().cpu(), "dQ": xs[0].grad.cpu(), "dK": xs[1].grad.cpu(), "dV": xs[2].grad.cpu(),
           "dlog_G": xs[3].grad.cpu()}
    del xs, Y
    torch.cuda.empty_cache()
    for v in got.values():
        assert torch.isfinite(v.float()).all()

    worst = {}
    for h0 in range(0, h, 2):          # two heads per oracle pass (a few GB of fp32 intermediates each)
        hs = slice(h0, h0 + 2)
        xo = [x[:, :, hs].float().clone().requires_grad_(True) for x in (Q, K, V, lg)]
        Yo = oracle.power_retention(*xo, deg=2, chunk_size=c)
        Yo.backward(dO[:, :, hs].float())
        want = {"Y": Yo.detach(), "dQ": xo[0].grad, "dK": xo[1].grad, "dV": xo[2].grad, "dlog_G": xo[3].grad}
        for nm, w in want.items():
            gsl = got[nm][:, :, hs]
            tol = OUT_TOL if nm == "Y" else GRAD_TOL
            whole = _rel(gsl, w, tuple(range(gsl.dim()))).item()
            # per (chunk, head): view [b, n, c, heads, ...] and reduce over everything but (n, heads)
            gv, wv = gsl.reshape(b, n, c, 2, -1), w.reshape(b, n, c, 2, -1)
            per = _rel(gv, wv, (0, 2, 4))                      # [n, heads]
            k = int(per.argmax())
            print(f"  heads {h0}-{h0 + 1} {nm}: rel-L2 {whole:.3e}, worst (chunk, head) {per.max().item():.3e} "
                  f"at chunk {k // 2} head {h0 + k % 2}", flush=True)
            worst[nm] = max(worst.get(nm, 0.0), per.max().item())
            assert whole <= tol, f"{nm} heads {h0}-{h0 + 1}: rel-L2 {whole:.3e} > {tol}"
            assert per.max().item() <= tol, \
                f"{nm}: chunk {k // 2} of head {h0 + k % 2} is off: rel-L2 {per.max().item():.3e} > {tol}"
        del xo, Yo, want
    print("  worst per-(chunk, head) rel-L2:", {k: f"{v:.3e}" for k, v in worst.items()}, flush=True)


def test_headline_shape_is_the_same_bit_for_bit_with_and_without_gate_skipping(pra):
    """The same step as above (which runs with the library's default, gate skipping on) once more with skipping off:
    every tile visited, every state swept, every chunk scanned.  All five tensors must agree bit for bit -- what is
    left out are products with exact zeros -- with all 512 (chunk, head) pairs in every launch."""
    from retention_integration_amd import _lib
    lib = _lib.load()
    b, t, h, d, c = 1, 65536, 8, 64, 1024
    g = torch.Generator().manual_seed(2024)
    Q, K, V = (torch.randn(b, t, h, d, generator=g).to(torch.bfloat16).to(DEV) for _ in range(3))
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g)).to(DEV)
    dO = torch.randn(b, t, h, d, generator=g).to(torch.bfloat16).to(DEV)

    def step():
        xs = [x.detach().clone().requires_grad_(True) for x in (Q, K, V, lg)]
        Y = pra.power_retention(*xs, deg=2, chunk_size=c)
        Y.backward(dO)
        torch.cuda.synchronize()
        return [Y.detach()] + [x.grad for x in xs]
    try:
        lib.pr_set_gate_skipping(1)
        on = step()
        lib.pr_set_gate_skipping(0)
        off = step()
    finally:
        lib.pr_set_gate_skipping(1)
    for nm, x, y in zip(["Y", "dQ", "dK", "dV", "dlog_G"], on, off):
        assert torch.isfinite(x.float()).all(), nm
        assert torch.equal(x, y), f"{nm}: {int((x != y).sum())} values differ, by up to " \
                                  f"{float((x.float() - y.float()).abs().max()):.3e}"


def test_inference_config_at_size_prefill_then_512_recurrent_steps(pra):
    """bf16, b=32, h=8, d=64: prefill with 2048 keys and switch_over_seq_len=1024 (state [32,8,2560,64], key sums
    [32,8,2560]), then 512 single-token steps that fold every token into the state in place of the previous one
    (switch_over_seq_len=1), the oracle carried alongside in fp32 on a slice of the batch.  Y is compared every 64
    steps, state and key sums at the end: 512 successive roundings of a 16-bit state must not drift."""
    b, h, d, tk, steps = 32, 8, 64, 2048, 512
    rows = [0, 1, 30, 31]
    g = torch.Generator().manual_seed(4)
    K, V = (torch.randn(b, tk, h, d, generator=g).to(torch.bfloat16) for _ in range(2))
    Q = torch.randn(b, 1, h, d, generator=g).to(torch.bfloat16)
    lg = torch.nn.functional.logsigmoid(torch.randn(b, tk, h, generator=g))
    Y, S, s = pra.power_retention_inference(Q.to(DEV), K.to(DEV), V.to(DEV), lg.to(DEV), None, None, deg=2,
                                            switch_over_seq_len=1024)
    assert S.shape == (b, h, pra.expanded_dim(d), d) and s.shape == (b, h, pra.expanded_dim(d))
    Yo, So, so = oracle.power_retention_inference(Q[rows].float(), K[rows].float(), V[rows].float(), lg[rows], None, None,
                                                  deg=2, switch_over_seq_len=1024)

    def check(name, got, want, tol=OUT_TOL):
        e = _rel(got.detach().cpu(), want, tuple(range(want.dim()))).item()
        print(f"  {name}: rel-L2 {e:.3e}", flush=True)
        assert torch.isfinite(got.float()).all() and e <= tol, f"{name}: rel-L2 {e:.3e} > {tol}"

    check("prefill Y", Y[rows], Yo)
    check("prefill state", S[rows], So)
    check("prefill sum_of_keys", s[rows], so)

    q = torch.randn(steps, b, 1, h, d, generator=g).to(torch.bfloat16)
    k = torch.randn(steps, b, 1, h, d, generator=g).to(torch.bfloat16)
    v = torch.randn(steps, b, 1, h, d, generator=g).to(torch.bfloat16)
    gl = torch.nn.functional.logsigmoid(torch.randn(steps, b, 1, h, generator=g))
    qd, kd, vd, gd = (x.to(DEV) for x in (q, k, v, gl))
    for i in range(steps):
        Y, S, s = pra.power_retention_inference(qd[i], kd[i], vd[i], gd[i], S, s, deg=2, switch_over_seq_len=1)
        Yo, So, so = oracle.power_retention_inference(q[i][rows].float(), k[i][rows].float(), v[i][rows].float(),
                                                      gl[i][rows], So, so, deg=2, switch_over_seq_len=1)
        if i % 64 == 63 or i == 0:
            check(f"step {i} Y", Y[rows], Yo)
    check("final state", S[rows], So)
    check("final sum_of_keys", s[rows], so)


@pytest.mark.parametrize("bi,hd", [(2, 5), (1, 11)])
def test_short_chunk_config_at_full_size_matches_the_oracle_on_a_slice(pra, bi, hd):
    """BASELINE configs[4] at its full size: fp16, b=4, t=16384, h=16, d=128, deg=2, chunk 128, no gating, inputs
    N(0,1) * 0.5, dO ~ N(0,1).  The GPU launch holds all 4 x 128 x 16 (batch, chunk, head) pairs (the library picks the
    chained state kernels there); batch entries and heads are independent, so the fp32 oracle runs on one head of one
    batch entry per case (0.6 GB of fp32 state, about a minute of host time).  Y, dQ, dK, dV per tensor and per chunk."""
    b, t, h, d, c = 4, 16384, 16, 128, 128
    n = t // c
    heads = [hd]
    g = torch.Generator().manual_seed(404)
    Q, K, V = ((0.5 * torch.randn(b, t, h, d, generator=g)).to(torch.float16) for _ in range(3))
    dO = torch.randn(b, t, h, d, generator=g).to(torch.float16)
    xs = [x.to(DEV).requires_grad_(True) for x in (Q, K, V)]
    Y = pra.power_retention(*xs, None, deg=2, chunk_size=c)
    Y.backward(dO.to(DEV))
    torch.cuda.synchronize()
    got = {"Y": Y.detach()[bi][:, heads].cpu(), "dQ": xs[0].grad[bi][:, heads].cpu(), "dK": xs[1].grad[bi][:, heads].cpu(),
           "dV": xs[2].grad[bi][:, heads].cpu()}
    for x in [Y] + [x.grad for x in xs]:
        assert torch.isfinite(x).all()
    del xs, Y
    torch.cuda.empty_cache()

    worst = {}
    for j, hd in enumerate(heads):     # one head per oracle pass
        xo = [x[bi:bi + 1, :, hd:hd + 1].float().clone().requires_grad_(True) for x in (Q, K, V)]
        Yo = oracle.power_retention(*xo, None, deg=2, chunk_size=c)
        Yo.backward(dO[bi:bi + 1, :, hd:hd + 1].float())
        want = {"Y": Yo.detach()[0, :, 0], "dQ": xo[0].grad[0, :, 0], "dK": xo[1].grad[0, :, 0], "dV": xo[2].grad[0, :, 0]}
        for nm, w in want.items():
            gsl = got[nm][:, j]
            tol = OUT_TOL if nm == "Y" else GRAD_TOL
            whole = _rel(gsl, w, (0, 1)).item()
            per = _rel(gsl.reshape(n, c, d), w.reshape(n, c, d), (1, 2))     # [n]
            k = int(per.argmax())
            print(f"  batch {bi} head {hd} {nm}: rel-L2 {whole:.3e}, worst chunk {per.max().item():.3e} at chunk {k}",
                  flush=True)
            worst[nm] = max(worst.get(nm, 0.0), per.max().item())
            assert whole <= tol, f"{nm} head {hd}: rel-L2 {whole:.3e} > {tol}"
            assert per.max().item() <= tol, f"{nm}: chunk {k} of head {hd} is off: rel-L2 {per.max().item():.3e} > {tol}"
        del xo, Yo, want
    print("  worst per-(chunk, head) rel-L2:", {k: f"{v:.3e}" for k, v in worst.items()}, flush=True)
