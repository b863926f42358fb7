"""Pure-PyTorch CPU restatement of the reference's power-retention path.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  All functions are ordinary
differentiable torch code, so gradients come from autograd; they run in any
float dtype (fp64 for pinning, fp32 as "gold", bf16/fp16 as "ref").

Notation: b batch, t time, h kv heads, r = hq // h query heads per kv head,
d key dim, e value dim, c chunk, n chunks, D expanded state dim.
"""
from __future__ import annotations

import math
from functools import lru_cache

import torch

TILE = 16  # side of the square feature tiles of the state layout

LOG_EPS = 1e-7  # added to |s| inside the log   (ref: retention/_attention/reference.py:46)
SUM_EPS = 1e-6  # added to the row sum l         (ref: retention/_attention/reference.py:55)


# --------------------------------------------------------------------------
# state layout
# --------------------------------------------------------------------------
def expanded_dim(d: int, deg: int = 2) -> int:
    """Size D of the degree-2 state (ref: retention/_utils.py:5-8,18-19).

    The d x d matrix of pair products is cut into 16x16 tiles; the tiles on or
    below the block diagonal are kept whole, so D = 256 * T(T+1)/2, T = d/16.
    """
    if deg != 2:
        raise NotImplementedError("only deg=2 has a state layout")
    assert d % TILE == 0, f"head dim must be a multiple of {TILE}: {d}"
    tiles = d // TILE
    return TILE * TILE * tiles * (tiles + 1) // 2


@lru_cache(maxsize=None)
def _feature_table(d: int):
    D = expanded_dim(d)
    lo = torch.empty(D, dtype=torch.long)
    hi = torch.empty(D, dtype=torch.long)
    mult = torch.empty(D, dtype=torch.float64)
    for y in range(d // TILE):
        base = 128 * y * (y + 1)
        for x in range(TILE * (y + 1)):
            for i in range(TILE):
                f = base + TILE * x + i
                lo[f] = x
                hi[f] = TILE * y + i
                mult[f] = 2.0 if x < TILE * y else 1.0
    return lo, hi, mult


def state_feature_table(d: int):
    """(x[f], w[f], m[f]) for every state feature f.

    Feature f = 128*y*(y+1) + 16*x + i  (y in [0,d/16), x in [0,16(y+1)),
    i in [0,16)) is the product of key coordinates x and w = 16*y + i; the key
    side multiplies by m = 2 when the pair lies in a tile strictly below the
    block diagonal (x < 16*y) and by 1 inside a diagonal tile, where both
    (a,b) and (b,a) are stored.  Derived from the loops of
    ref: retention/_update_state/reference.py:16-28 (keys, 8-wide outer block,
    16-wide inner block) and ref: retention/_query_state/reference.py:19-32
    (queries, 1-wide outer block), which enumerate the same order.
    """
    return _feature_table(d)


def expand_keys(K: torch.Tensor) -> torch.Tensor:
    """phi(K) over the last axis, with the off-diagonal factor 2.

    ref: retention/_update_state/reference.py:5-29 -- the pair product is
    rounded to K.dtype before the (exact) multiplication by 1 or 2.
    """
    lo, hi, mult = _feature_table(K.shape[-1])
    prod = (K[..., lo] * K[..., hi]).to(K.dtype)
    return (prod * mult.to(K.dtype)).to(K.dtype)


def expand_queries(Q: torch.Tensor) -> torch.Tensor:
    """phi(Q) over the last axis, all multipliers 1.

    ref: retention/_query_state/reference.py:11-33.
    """
    lo, hi, _ = _feature_table(Q.shape[-1])
    return (Q[..., lo] * Q[..., hi]).to(Q.dtype)


# --------------------------------------------------------------------------
# operators
# --------------------------------------------------------------------------
def attention(Q, K, V, log_G, deg, causal=True, head_first=False, scale=1.0, norm=False, use_log2=False):
    """Power attention on [b, t, h, d] tensors.

    ref: retention/_attention/reference.py:10-69.  log_G is the *accumulated*
    log gate [b, tk, h]; queries are aligned to the end of the keys (:29,:45);
    r query heads share a kv head (:35).  Returns o/l if ``norm`` else
    (o, l, rowmax) with o = sum_j exp(z - rowmax) v_j, l = sum_j exp(.) + 1e-6,
    z = deg*log(|s| + 1e-7) + G_q - G_k, rowmax detached (:50).
    """
    assert causal and not head_first and not use_log2, "only the configuration used by the maker is restated"
    assert isinstance(deg, int) and deg % 2 == 0, "deg must be a positive even integer"
    b, tq, hq, d = Q.shape
    _, tk, h, e = V.shape
    assert hq % h == 0
    r = hq // h
    q = Q.reshape(b, tq, h, r, d)
    s = torch.einsum("bihrd,bjhd->bhrij", q, K) * scale  # [b,h,r,tq,tk]
    i_idx = torch.arange(tq, device=Q.device)[:, None] + (tk - tq)
    j_idx = torch.arange(tk, device=Q.device)[None, :]
    allowed = i_idx >= j_idx
    z = float(deg) * torch.where(allowed, torch.log(s.abs() + LOG_EPS), torch.full_like(s, -float("inf")))
    if log_G is not None:
        assert log_G.shape == (b, tk, h)
        Gk = log_G.permute(0, 2, 1)  # [b,h,tk]
        Gq = Gk[..., tk - tq:]
        z = z + (Gq[:, :, None, :, None] - Gk[:, :, None, None, :])
    rowmax = z.max(dim=-1, keepdim=True).values.detach()
    p = torch.exp(z - rowmax).to(V.dtype)  # even degree: sign of s is ignored (:51-54)
    l = p.sum(dim=-1).to(torch.float32) + SUM_EPS  # [b,h,r,tq]
    o = torch.einsum("bhrij,bjhe->bihre", p, V).reshape(b, tq, hq, e)
    l = l.permute(0, 3, 1, 2).reshape(b, tq, hq)
    rowmax = rowmax.squeeze(-1).permute(0, 3, 1, 2).reshape(b, tq, hq)
    if norm:
        return (o / l[..., None]).to(V.dtype)
    return o, l, rowmax.to(torch.float32)


def update_state(K, V, deg):
    """Chunk states S = phi(K)^T V and key sums N = sum_t phi(K_t).

    ref: retention/_update_state/reference.py:33-52 (forward), :86-94 (4-D
    inference form).  K, V: [b, n, c, h, d] -> S [b, n, h, D, e] in K.dtype,
    N [b, n, h, D] fp32.
    """
    if K.dim() == 4:
        S, N = update_state(K.unsqueeze(1), V.unsqueeze(1), deg)
        return S.squeeze(1), N.squeeze(1)
    assert deg == 2
    phi = expand_keys(K.transpose(2, 3))  # [b,n,h,c,D]
    N = phi.to(torch.float32).sum(dim=-2)
    S = torch.einsum("bnhcf,bnchv->bnhfv", phi, V)
    return S, N


def discumsum(X, log_G):
    """Gated exclusive scan over the chunk axis.

    ref: retention/_discumsum/reference.py:3-15.  X [b, n, h, ...],
    log_G [b, n, h] -> Y [b, n+1, h, ...] with Y[0] = 0, Y[1] = X[0] and
    Y[k+1] = Y[k] * exp(log_G[k]) + X[k]; the decayed state is rounded to
    X.dtype before the add (:13).  log_G[0] never scales anything.
    """
    if log_G is None:
        return X.cumsum(dim=1, dtype=X.dtype)
    n = log_G.shape[1]
    g = torch.exp(log_G)
    g = g.reshape(*g.shape, *([1] * (X.dim() - 3)))
    first = X[:, 0].to(torch.float32) + 0 * g[:, 0]
    out = [torch.zeros_like(first).to(X.dtype), first.to(X.dtype)]
    run = first
    for k in range(1, n):
        run = (run * g[:, k]).to(X.dtype) + X[:, k]
        out.append(run)
    return torch.stack(out, dim=1)


def query_state(Q, S, s, Y_attn, l_attn, rowmax, deg, scale, zero_initial_state):
    """Query the chunk state and merge with the intra-chunk attention.

    ref: retention/_query_state/reference.py:36-96 (math), :166-191 (4-D
    inference form, GQA folding).  Q [b,n,c,hq,d], S [b,n,h,D,e], s [b,n,h,D],
    Y_attn [b,n,c,hq,e], l_attn / rowmax [b,n,c,hq] -> O [b,n,c,hq,e].

        gamma = sqrt(D)  (1 for chunk 0 when zero_initial_state)
        alpha = max(gamma, exp(rowmax))
        num = Y_attn*exp(rowmax)/alpha + phi(Q)(S/gamma) * scale^deg * gamma/alpha
        den = l_attn*exp(rowmax)/alpha + phi(Q)(s/gamma) * scale^deg * gamma/alpha
        O = num / den
    """
    if Q.dim() == 4:
        un = lambda x: None if x is None else x.unsqueeze(1)  # noqa: E731
        O = query_state(un(Q), un(S), un(s), un(Y_attn), un(l_attn), un(rowmax), deg, scale, zero_initial_state)
        return O.squeeze(1)
    b, n, c, hq, d = Q.shape
    _, _, h, D, e = S.shape
    assert hq % h == 0
    r = hq // h
    scale_p = scale ** deg
    gamma = torch.full((n,), math.sqrt(float(D)), dtype=torch.float32, device=Q.device)
    if zero_initial_state:
        gamma[0] = 1.0
    g_state = gamma.view(1, n, 1, 1, 1)
    Sg = (S / g_state).to(S.dtype)
    sg = s / gamma.view(1, n, 1, 1)
    phi = expand_queries(Q.reshape(b, n, c, h, r, d))  # [b,n,c,h,r,D]
    Y_qs = torch.einsum("bnchrf,bnhfv->bnchrv", phi.to(Q.dtype), Sg.to(Q.dtype)).to(Q.dtype).reshape(b, n, c, hq, e)
    l_qs = torch.einsum("bnchrf,bnhf->bnchr", phi.to(torch.float32), sg.to(torch.float32)).reshape(b, n, c, hq)
    if Y_attn is not None:
        g_row = gamma.view(1, n, 1, 1)
        alpha = torch.maximum(g_row, torch.exp(rowmax))
        w_attn = torch.exp(rowmax) / alpha
        w_qs = g_row / alpha
        num = Y_attn * w_attn.unsqueeze(-1) + Y_qs * scale_p * w_qs.unsqueeze(-1)
        den = l_attn * w_attn + l_qs * scale_p * w_qs
    else:
        num, den = Y_qs, l_qs
    return (num.to(torch.float32) / den.unsqueeze(-1)).to(Y_qs.dtype).contiguous()


# --------------------------------------------------------------------------
# composed functions
# --------------------------------------------------------------------------
def power_retention(Q, K, V, log_G=None, initial_state=None, return_final_state=False,
                    deg=2, scale=None, chunk_size=None, switch_over_seq_len=None):
    """Training-path power retention.

    ref: retention/power_retention_maker.py:71-90 (padding), :96-197 (body),
    wired as in ref: retention/reference.py:8.

    ``initial_state`` / ``return_final_state`` do NOT follow the reference
    (:131-140, :158-160, :168-172), whose handling is unfinished there: the
    returned tensor is the state at the start of the last chunk, the carried
    state is not decayed by the gates (":158 TODO") and no key sums travel with
    it.  Here they carry the definition the product documents: the state is
    the pair (S [b,h,D,d], sum_of_keys [b,h,D]) AFTER the last token, decayed
    like any chunk state, so that two chained calls equal one call.  That
    definition is pinned by exactly this property and by equality with the
    state ``power_retention_inference`` forms over the same tokens
    (tests/test_oracle_invariants.py), not by the reference.
    """
    assert deg % 2 == 0, f"deg must be even: {deg=}"
    with_state = initial_state is not None or return_final_state
    t_orig = Q.shape[1]
    pad = 0
    if chunk_size is not None and t_orig % chunk_size != 0:
        pad = chunk_size - t_orig % chunk_size
        zp = lambda x: torch.nn.functional.pad(x, (0, 0, 0, 0, 0, pad))  # noqa: E731
        Q, K, V = zp(Q), zp(K), zp(V)
        if log_G is not None:
            log_G = torch.nn.functional.pad(log_G, (0, 0, 0, pad))
    assert Q.dtype == K.dtype == V.dtype
    dtype = Q.dtype
    b, t, hq, d = Q.shape
    h = K.shape[2]
    assert hq % h == 0
    r = hq // h
    if chunk_size is not None:
        c, n = chunk_size, t // chunk_size
        if switch_over_seq_len is None:
            switch_over_seq_len = chunk_size
    else:
        c, n = t, 1
    gating = log_G is not None
    if gating:
        log_G = log_G.to(torch.float32)
    if not scale:
        scale = 1.0 / d ** 0.5

    if (switch_over_seq_len is None or t <= switch_over_seq_len) and not with_state:
        A = log_G.cumsum(1) if gating else None
        out = attention(Q, K, V, A, deg, scale=scale, norm=True)
        return out[:, :t_orig] if pad else out

    Qc, Kc, Vc = Q.view(b, n, c, hq, d), K.view(b, n, c, h, d), V.view(b, n, c, h, d)
    if gating:
        A = log_G.view(b, n, c, h).cumsum(2)
        w = torch.exp((A[:, :, c - 1:c] - A) / deg)
        Kd = Kc * w.unsqueeze(-1).to(K.dtype)
        lcs = A[:, :, -1].contiguous()
    else:
        A = None
        Kd = Kc
        lcs = torch.zeros(b, n, h, dtype=torch.float32, device=Q.device)
    S, s = update_state(Kd.contiguous(), Vc.contiguous(), deg)
    first = 0
    if initial_state is not None:  # one more scan entry in front; chunk k's gate sum decays it like a chunk state
        S0, s0 = initial_state
        S = torch.cat([S0.unsqueeze(1).to(S.dtype), S], dim=1)
        s = torch.cat([s0.unsqueeze(1).to(s.dtype), s], dim=1)
        lcs = torch.cat([torch.zeros_like(lcs[:, :1]), lcs], dim=1)
        first = 1
    S, s = discumsum(S, lcs), discumsum(s, lcs)
    final = (S[:, first + n], s[:, first + n])
    S, s = S.narrow(1, first, n), s.narrow(1, first, n)

    Ya, la, rm = attention(Qc.reshape(b * n, c, hq, d), Kc.reshape(b * n, c, h, d), Vc.reshape(b * n, c, h, d),
                           A.reshape(b * n, c, h) if gating else None, deg, scale=scale, norm=False)
    Ya, la, rm = (x.view(b, n, *x.shape[1:]) for x in (Ya, la, rm))
    if gating:
        Aq = A.repeat_interleave(r, dim=3) if r > 1 else A
        Qg = Qc * torch.exp(Aq / deg).unsqueeze(-1).to(Q.dtype)
    else:
        Qg = Qc
    Y = query_state(Qg.contiguous(), S.contiguous(), s.contiguous(), Ya.contiguous(), la.contiguous(),
                    rm.contiguous(), deg, scale, initial_state is None)
    out = Y.contiguous().view(b, t, hq, d).to(dtype)
    out = out[:, :t_orig] if pad else out
    return (out, final) if return_final_state else out


def power_retention_inference(Q, K, V, log_G=None, initial_state=None, sum_of_keys=None,
                              deg=2, scale=None, switch_over_seq_len=512):
    """Prefill / decode step with an explicit state.

    ref: retention/power_retention_maker.py:287-390 with
    ``fused_normalizer=False`` (ref: retention/reference.py:9).
    Returns (Y, state, sum_of_keys).
    """
    has_cache = K is not None and V is not None
    assert has_cache or initial_state is not None
    b, tq, hq, d = Q.shape
    if has_cache:
        assert Q.dtype == K.dtype == V.dtype
        assert K.shape[1] == V.shape[1]
        tk, hk = K.shape[1], K.shape[2]
        assert log_G is None or log_G.shape[:3] == K.shape[:3]
    else:
        assert sum_of_keys is not None
        tk, hk = 0, initial_state.shape[1]
    scale = 1.0 / d ** 0.5 if scale is None else scale
    A = log_G.cumsum(1) if log_G is not None else None
    r = hq // hk
    if initial_state is None:
        Y = attention(Q, K, V, A, deg, scale=scale, norm=True)
    else:
        assert initial_state.shape[0] == b and initial_state.shape[1] == hk
        if tk > 0:
            Ya, la, rm = attention(Q, K, V, A, deg, scale=scale, norm=False)
        else:
            Ya = la = rm = None
        Qs = Q
        if A is not None:
            Qs = Q * torch.exp(A[:, -1:] / deg).repeat_interleave(r, dim=-1).unsqueeze(-1).to(Q.dtype)
        Y = query_state(Qs, initial_state, sum_of_keys, Ya, la, rm, deg, scale, False)

    if switch_over_seq_len is not None and tk >= switch_over_seq_len:
        Kd = K
        if A is not None:
            Kd = (K * torch.exp((A[:, -1:] - A) / deg).unsqueeze(-1)).to(K.dtype)
        dS, ds = update_state(Kd.contiguous(), V.contiguous(), deg)
        if initial_state is None:
            new_S, new_s = dS, ds
        elif A is None:
            new_S, new_s = initial_state + dS, sum_of_keys + ds
        else:
            decay = torch.exp(A[:, -1, :])
            new_S = initial_state * decay[..., None, None].to(initial_state.dtype) + dS
            new_s = sum_of_keys * decay[..., None].to(sum_of_keys.dtype) + ds
    else:
        new_S, new_s = initial_state, sum_of_keys
    return Y, new_S, new_s
