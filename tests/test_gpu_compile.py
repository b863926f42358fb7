"""The custom operators under torch.compile and torch.library.opcheck.

Mirrors the reference's generic operator checks (ref: perf/tests/common_tests.py:64-82 with
perf/_checks.py:185-214): a compiled function returns what the eager one returns, forward and backward, and the
operator registrations (schema, fake implementation, autograd) are consistent.  The reference skips opcheck
("have not yet figured out how to make opcheck pass", common_tests.py:78); here it runs.

The compiled runs use the ``aot_eager`` backend: graph capture, fake tensors and the autograd registration are
what is under test; no code generator is involved in this package.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"
OPCHECKS = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic")


def _qkv(b, t, h, r, d, dtype, gated, seed=0, grad=True):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV).requires_grad_(grad)  # noqa: E731
    Q, K, V = mk(b, t, h * r, d), mk(b, t, h, d), mk(b, t, h, d)
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g)).to(DEV).requires_grad_(grad) if gated else None
    return Q, K, V, lg


@pytest.fixture(scope="module")
def pra():
    import retention_integration_amd as pra
    return pra


@pytest.mark.parametrize("gated", [True, False])
def test_opcheck_chunked(pra, gated):
    from retention_integration_amd import fused
    Q, K, V, lg = _qkv(1, 256, 2, 2, 32, torch.bfloat16, gated)
    torch.library.opcheck(fused.chunked_fwd, (Q, K, V, lg, 2, 0.25, 64), test_utils=OPCHECKS)


def test_opcheck_operators(pra):
    from retention_integration_amd import ops
    b, n, c, h, d = 1, 2, 64, 2, 32
    Q, K, V, lg = _qkv(b * n, c, h, 1, d, torch.bfloat16, True, seed=1)
    A = lg.detach().cumsum(1).requires_grad_(True)
    torch.library.opcheck(ops.attention_fwd, (Q, K, V, A, 2, 0.25, False), test_utils=OPCHECKS)
    K5, V5, Q5 = (x.detach().view(b, n, c, h, d).requires_grad_(True) for x in (K, V, Q))
    torch.library.opcheck(ops.update_state_fwd, (K5, V5), test_utils=OPCHECKS)
    S, s = ops.update_state_fwd(K5.detach(), V5.detach())
    lcs = lg.detach().view(b, n, c, h).sum(2).contiguous().requires_grad_(True)
    torch.library.opcheck(ops.discumsum_fwd, (S.detach().requires_grad_(True), lcs, n + 1), test_utils=OPCHECKS)
    # every chunk gets a non-zero state (a zero state without an attention part is 0/0 by definition)
    S1, s1 = S.detach().requires_grad_(True), s.detach().requires_grad_(True)
    torch.library.opcheck(ops.query_state_fwd, (Q5, S1, s1, None, None, None, 0.0625, False), test_utils=OPCHECKS)
    Ya, la, rm = ops.attention_fwd(Q.detach(), K.detach(), V.detach(), A.detach(), 2, 0.25, False)
    Ya5, la5, rm5 = Ya.view(b, n, c, h, d).requires_grad_(True), la.view(b, n, c, h).requires_grad_(True), rm.view(b, n, c, h)
    Sc = ops.discumsum_fwd(S, lcs.detach(), n).requires_grad_(True)
    sc = ops.discumsum_fwd(s, lcs.detach(), n).requires_grad_(True)
    torch.library.opcheck(ops.query_state_fwd, (Q5, Sc, sc, Ya5, la5, rm5, 0.0625, True), test_utils=OPCHECKS)
    # the accumulated gates of the quadratic branch (ref: log_G.cumsum(1), retention/power_retention_maker.py:129)
    lg3 = lg.detach().clone().requires_grad_(True)
    torch.library.opcheck(ops.gate_cumsum, (lg3,), test_utils=OPCHECKS)
    dA = torch.randn_like(lg3)
    (g_lib,) = torch.autograd.grad(ops.gate_cumsum(lg3), lg3, dA)
    (g_ref,) = torch.autograd.grad(lg3.cumsum(1), lg3, dA)
    assert torch.allclose(ops.gate_cumsum(lg3), lg3.cumsum(1), rtol=1e-5, atol=1e-5)
    assert torch.allclose(g_lib, g_ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("chunk", [64, None])
def test_compiled_matches_eager(pra, chunk):
    Q, K, V, lg = _qkv(2, 256, 2, 2, 32, torch.bfloat16, True, seed=2)
    dO = torch.randn_like(Q)

    def fwd_bwd():
        for x in (Q, K, V, lg):
            x.grad = None
        Y = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=chunk)
        Y.backward(dO)
        return [Y.detach()] + [x.grad.clone() for x in (Q, K, V, lg)]

    want = fwd_bwd()
    compiled = torch.compile(fwd_bwd, backend="aot_eager")
    for _ in range(2):
        got = compiled()
    for a, b_ in zip(got, want):
        assert a.shape == b_.shape and a.dtype == b_.dtype
        assert torch.equal(a, b_), "the compiled function must run the same kernels on the same data"
    torch._dynamo.reset()


def test_compiled_forward_has_no_graph_break(pra):
    Q, K, V, lg = _qkv(1, 256, 2, 1, 64, torch.float16, True, seed=3, grad=False)
    f = torch.compile(lambda q, k, v, g: pra.power_retention(q, k, v, g, deg=2, chunk_size=128),
                      backend="aot_eager", fullgraph=True)
    with torch.no_grad():
        want = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=128)
        got = f(Q, K, V, lg)
    assert torch.equal(got, want)
    torch._dynamo.reset()
