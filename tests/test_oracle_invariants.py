"""Pins the CPU oracle with checks that do not retype its formulas: the O(t^2)
closed form evaluated by explicit loops in fp64, textbook special cases, and the
algebraic invariants the reference's own tests rely on
(ref: perf/tests/chunk_consistency_tests.py:21-45, perf/tests/inference_tests.py:38-51,
perf/tests/gqa_tests.py:72-129)."""
import math

import numpy as np
import pytest
import torch

import oracle

torch.manual_seed(0)


def closed_form(Q, K, V, log_G, scale, deg=2):
    """out_i = sum_{j<=i} w_ij v_j / sum_{j<=i} w_ij with
    w_ij = (scale q_i.k_j)^deg * exp(sum_{j<m<=i} log_G_m); plain loops, fp64 numpy."""
    Q, K, V = (x.double().numpy() for x in (Q, K, V))
    lg = None if log_G is None else log_G.double().numpy()
    b, t, hq, d = Q.shape
    h = K.shape[2]
    r = hq // h
    out = np.zeros((b, t, hq, V.shape[-1]))
    for bi in range(b):
        for hi in range(hq):
            kv = hi // r
            for i in range(t):
                num = np.zeros(V.shape[-1]); den = 0.0
                for j in range(i + 1):
                    w = (scale * float(Q[bi, i, hi] @ K[bi, j, kv])) ** deg
                    if lg is not None:
                        w *= math.exp(lg[bi, j + 1:i + 1, kv].sum())
                    num += w * V[bi, j, kv]; den += w
                out[bi, i, hi] = num / den
    return torch.from_numpy(out)


def inputs(b, t, h, r, d, gated, dtype=torch.float64):
    Q = torch.randn(b, t, h * r, d, dtype=dtype)
    K = torch.randn(b, t, h, d, dtype=dtype)
    V = torch.randn(b, t, h, d, dtype=dtype)
    G = torch.nn.functional.logsigmoid(torch.randn(b, t, h, dtype=dtype)) if gated else None
    return Q, K, V, G


def test_expanded_dim_values():
    assert [oracle.expanded_dim(d) for d in (16, 32, 64, 128)] == [256, 768, 2560, 9216]


@pytest.mark.parametrize("d", [16, 32, 64])
def test_phi_inner_product_is_squared_dot(d):
    q, k = torch.randn(5, d, dtype=torch.float64), torch.randn(5, d, dtype=torch.float64)
    lhs = (oracle.expand_queries(q) * oracle.expand_keys(k)).sum(-1)
    torch.testing.assert_close(lhs, (q * k).sum(-1) ** 2)


def test_feature_table_is_a_bijection_onto_lower_tiles():
    x, w, m = oracle.state_feature_table(64)
    pairs = set(zip(x.tolist(), w.tolist()))
    assert len(pairs) == 2560
    expect = {(a, c) for a in range(64) for c in range(64) if a // 16 <= c // 16}
    assert pairs == expect
    assert all((mm == 2.0) == (a // 16 < c // 16) for a, c, mm in zip(x.tolist(), w.tolist(), m.tolist()))


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("r", [1, 2])
def test_quadratic_and_chunked_match_closed_form(gated, r):
    Q, K, V, G = inputs(1, 24, 2, r, 16, gated)
    want = closed_form(Q, K, V, G, scale=0.25)
    for cs in (None, 8):
        got = oracle.power_retention(Q, K, V, G, deg=2, scale=0.25, chunk_size=cs)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)  # eps terms of the reference are <= 1e-6 relative


def test_padding_matches_closed_form():
    Q, K, V, G = inputs(1, 21, 1, 1, 16, True)
    want = closed_form(Q, K, V, G, scale=0.25)
    got = oracle.power_retention(Q, K, V, G, deg=2, scale=0.25, chunk_size=8)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_gradients_chunked_equal_quadratic():
    Q, K, V, G = inputs(1, 16, 1, 2, 16, True)
    grads = []
    for cs in (None, 4):
        xs = [x.clone().requires_grad_(True) for x in (Q, K, V, G)]
        Y = oracle.power_retention(*xs, deg=2, scale=0.25, chunk_size=cs)
        grads.append(torch.autograd.grad(Y, xs, torch.cos(torch.arange(Y.numel(), dtype=Y.dtype)).view_as(Y)))
    for a, b_ in zip(*grads):
        # fp32 intermediates (l, log_G) and the 1e-6 / 1e-7 guards bound the agreement; the
        # reference's own check uses atol 1e-2 (perf/tests/chunk_consistency_tests.py:44)
        torch.testing.assert_close(a, b_, rtol=1e-4, atol=2e-5)


def test_attention_ungated_deg2_is_squared_scores():
    Q, K, V, _ = inputs(2, 9, 2, 1, 16, False)
    got = oracle.attention(Q, K, V, None, 2, scale=0.3, norm=True)
    s = torch.einsum("bihd,bjhd->bhij", Q, K) * 0.3
    w = torch.tril(s ** 2)
    want = torch.einsum("bhij,bjhe->bihe", w / w.sum(-1, keepdim=True), V)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_attention_triple_is_consistent():
    Q, K, V, G = inputs(1, 7, 1, 1, 16, True)
    A = G.cumsum(1)
    o, l, m = oracle.attention(Q, K, V, A, 2, scale=0.5, norm=False)
    torch.testing.assert_close(o / l[..., None].double(), oracle.attention(Q, K, V, A, 2, scale=0.5, norm=True))
    assert (l >= 1.0).all()  # the row maximum contributes exp(0)


def test_update_state_is_sum_of_outer_products():
    K, V = torch.randn(1, 1, 5, 1, 32, dtype=torch.float64), torch.randn(1, 1, 5, 1, 32, dtype=torch.float64)
    S, N = oracle.update_state(K, V, 2)
    x, w, m = oracle.state_feature_table(32)
    Sb = torch.zeros(768, 32, dtype=torch.float64); Nb = torch.zeros(768, dtype=torch.float64)
    for t in range(5):
        for f in range(768):
            p = m[f] * K[0, 0, t, 0, x[f]] * K[0, 0, t, 0, w[f]]
            Sb[f] += p * V[0, 0, t, 0]; Nb[f] += p
    torch.testing.assert_close(S[0, 0, 0], Sb)
    torch.testing.assert_close(N[0, 0, 0].double(), Nb, rtol=1e-5, atol=1e-5)


def test_discumsum_closed_form_and_plain_cumsum():
    X = torch.randn(2, 6, 3, 4, dtype=torch.float64)
    lg = torch.nn.functional.logsigmoid(torch.randn(2, 6, 3, dtype=torch.float64))
    Y = oracle.discumsum(X, lg)
    assert Y.shape == (2, 7, 3, 4) and (Y[:, 0] == 0).all()
    for k in range(1, 7):
        want = sum(X[:, j] * torch.exp(lg[:, j + 1:k].sum(1))[..., None] for j in range(k))
        torch.testing.assert_close(Y[:, k], want)
    Y0 = oracle.discumsum(X, torch.zeros_like(lg))
    torch.testing.assert_close(Y0[:, 1:], X.cumsum(1))


def test_query_state_limits_and_gamma_independence():
    b, n, c, h, d = 1, 2, 3, 1, 16
    D = oracle.expanded_dim(d)
    Q = torch.randn(b, n, c, h, d, dtype=torch.float64)
    S = torch.randn(b, n, h, D, d, dtype=torch.float64)
    s = torch.randn(b, n, h, D, dtype=torch.float64).abs() + 3
    Ya = torch.randn(b, n, c, h, d, dtype=torch.float64)
    la = torch.randn(b, n, c, h, dtype=torch.float64).abs() + 3
    rm = torch.randn(b, n, c, h, dtype=torch.float64)
    phi = oracle.expand_queries(Q.transpose(2, 3))
    # no attention part: phi(Q) S / phi(Q) s
    O = oracle.query_state(Q, S, s, None, None, None, 2, 0.5, False)
    want = (phi @ S) / (phi @ s.unsqueeze(-1))
    torch.testing.assert_close(O, want.transpose(2, 3), rtol=1e-5, atol=1e-5)  # l is accumulated in fp32
    # zero state: attention alone
    O = oracle.query_state(Q, torch.zeros_like(S), torch.zeros_like(s), Ya, la, rm, 2, 0.5, True)
    torch.testing.assert_close(O, Ya / la[..., None])
    # the gamma/alpha rescaling cancels
    a = oracle.query_state(Q, S, s, Ya, la, rm, 2, 0.5, True)
    b_ = oracle.query_state(Q, S, s, Ya, la, rm, 2, 0.5, False)
    torch.testing.assert_close(a, b_, rtol=1e-5, atol=1e-5)
    e = torch.exp(rm)
    want = (Ya * e[..., None] + 0.25 * (phi @ S).transpose(2, 3)) / (la * e + 0.25 * (phi @ s.unsqueeze(-1)).squeeze(-1).transpose(2, 3))[..., None]
    torch.testing.assert_close(a, want, rtol=1e-5, atol=1e-5)


def test_gqa_equals_repeated_kv_heads():
    Q, K, V, G = inputs(1, 12, 2, 3, 16, True)
    a = oracle.power_retention(Q, K, V, G, deg=2, chunk_size=4)
    b_ = oracle.power_retention(Q, K.repeat_interleave(3, 2), V.repeat_interleave(3, 2), G.repeat_interleave(3, 2),
                                deg=2, chunk_size=4)
    torch.testing.assert_close(a, b_)


@pytest.mark.parametrize("gated", [False, True])
def test_inference_decode_equals_closed_form_over_history(gated):
    t0, steps = 6, 3
    Q, K, V, G = inputs(1, t0 + steps, 1, 2, 16, gated)
    want = closed_form(Q, K, V, G, scale=0.25)
    Y, st, sk = oracle.power_retention_inference(Q[:, :t0], K[:, :t0], V[:, :t0], None if G is None else G[:, :t0],
                                                 None, None, deg=2, switch_over_seq_len=t0)
    torch.testing.assert_close(Y, want[:, :t0], rtol=1e-5, atol=1e-6)
    for i in range(t0, t0 + steps):  # pure recurrent decode: query + rank-1 update every step
        Y, st, sk = oracle.power_retention_inference(Q[:, i:i + 1], K[:, i:i + 1], V[:, i:i + 1],
                                                     None if G is None else G[:, i:i + 1], st, sk,
                                                     deg=2, switch_over_seq_len=1)
        torch.testing.assert_close(Y, want[:, i:i + 1], rtol=1e-5, atol=1e-6)


def test_inference_state_parity():
    Q, K, V, _ = inputs(1, 9, 2, 2, 16, False)
    Y, st, sk = oracle.power_retention_inference(Q[:, -1:], K, V, None, None, None, deg=2, switch_over_seq_len=9)
    Y2, st2, sk2 = oracle.power_retention_inference(Q[:, -1:], None, None, None, st, sk, deg=2, switch_over_seq_len=9)
    torch.testing.assert_close(Y, Y2, rtol=1e-5, atol=1e-6)
    assert st2 is st and sk2 is sk


# --------------------------------------------------------------------------
# state carried across calls (initial_state / return_final_state): the product's own definition, pinned by the
# closed form over the whole history and by the state the (golden-pinned) inference function forms
# --------------------------------------------------------------------------
@pytest.mark.parametrize("gated,r,chunk", [(True, 1, 8), (False, 2, 8), (True, 2, None)])
def test_two_chained_calls_equal_the_closed_form_over_the_whole_sequence(gated, r, chunk):
    b, t, h, d = 2, 32, 2, 16
    Q, K, V, G = inputs(b, t, h, r, d, gated)
    scale = 1.0 / math.sqrt(d)
    want = closed_form(Q, K, V, G, scale)
    half = t // 2
    sl = lambda x, a, e: None if x is None else x[:, a:e]  # noqa: E731
    y1, st = oracle.power_retention(Q[:, :half], K[:, :half], V[:, :half], sl(G, 0, half), return_final_state=True,
                                    deg=2, chunk_size=chunk)
    y2, st2 = oracle.power_retention(Q[:, half:], K[:, half:], V[:, half:], sl(G, half, t), initial_state=st,
                                     return_final_state=True, deg=2, chunk_size=chunk)
    torch.testing.assert_close(torch.cat([y1, y2], 1), want, rtol=1e-5, atol=1e-6)   # the eps terms are ~1e-6 relative
    # one call over everything returns the same final state, and so does the inference function's prefill
    _, st_all = oracle.power_retention(Q, K, V, G, return_final_state=True, deg=2, chunk_size=chunk or t)
    _, S_inf, s_inf = oracle.power_retention_inference(Q[:, -1:], K, V, G, None, None, deg=2, switch_over_seq_len=t)
    for a, b_, c_ in zip(st2, st_all, (S_inf, s_inf)):
        # (the scan's first entry passes through fp32, as in the reference: retention/_discumsum/reference.py:10)
        torch.testing.assert_close(a, b_, rtol=1e-5, atol=1e-5)
        # (the training function rounds the gates to fp32 as the reference does, the inference function does not)
        torch.testing.assert_close(a.double(), c_.double(), rtol=1e-5, atol=1e-5)


def test_chained_calls_with_ragged_lengths_and_gradients():
    """Padding must not touch the carried state, and gradients flow through it: the gradient of a loss over both
    calls equals the gradient of the same loss over one call."""
    b, t, h, r, d, chunk = 1, 27, 2, 2, 16, 8
    Q, K, V, G = inputs(b, t, h, r, d, True)
    W = torch.randn(b, t, h * r, d, dtype=torch.float64)
    xs = [x.clone().requires_grad_(True) for x in (Q, K, V, G)]
    (oracle.power_retention(*xs, deg=2, chunk_size=chunk) * W).sum().backward()
    ys = [x.clone().requires_grad_(True) for x in (Q, K, V, G)]
    cut = 13   # neither part is a chunk multiple
    y1, st = oracle.power_retention(*(x[:, :cut] for x in ys), return_final_state=True, deg=2, chunk_size=chunk)
    y2 = oracle.power_retention(*(x[:, cut:] for x in ys), initial_state=st, deg=2, chunk_size=chunk)
    (torch.cat([y1, y2], 1) * W).sum().backward()
    for a, b_ in zip(xs, ys):
        # (the chunk boundaries differ between the two runs, and with them where the 1e-6 / 1e-7 terms enter)
        torch.testing.assert_close(b_.grad, a.grad, rtol=1e-3, atol=1e-5)


def test_discumsum_without_gates_is_the_inclusive_cumsum():
    X = torch.randn(2, 5, 3, 4, 6, dtype=torch.float64)
    torch.testing.assert_close(oracle.discumsum(X, None), X.cumsum(1))
    torch.testing.assert_close(oracle.discumsum(X, torch.zeros(2, 5, 3, dtype=torch.float64))[:, 1:], X.cumsum(1))
