"""Composition of the four operators into ``power_retention`` and ``power_retention_inference``.

Mirrors the reference's plugin boundary: a backend is four callables injected into
``make_power_retention(update_state, query_state, discumsum, attention)`` and three into
``make_power_retention_inference(update_state, query_state, attention)``
(ref: retention/power_retention_maker.py:92, 284; wiring: retention/reference.py:8-9).
Signatures, defaults, tensor layouts and the conditions that raise are the reference's.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def _pad_time(x, pad, dims_after):
    return F.pad(x, (0, 0) * dims_after + (0, pad))


def make_power_retention(update_state_impl, query_state_impl, discumsum_impl, attention_impl, *,
                         scan_keeps_last=True, chunked_impl=None, full_scan_impl=None, gate_cumsum_impl=None):
    """Build ``power_retention`` from operator implementations.

    ``scan_keeps_last=False`` declares that ``discumsum_impl(X, log_G)`` already returns only the first n
    entries of the scan (the composed path never reads the last one).  ``chunked_impl(Q, K, V, log_G, deg,
    scale, chunk_size)``, when given, replaces the composition of the four operators on the chunked branch
    (same result; used for the fused single-node path).  ``full_scan_impl(X, log_G)`` must return all n + 1
    entries; it is needed for ``return_final_state`` when ``discumsum_impl`` drops the last one.
    ``gate_cumsum_impl(log_G)``, when given, stands in for ``log_G.cumsum(1)`` on the quadratic branch (fp32
    ``[b, t, h]``; it may return None for shapes it does not take).

    State across calls.  ``initial_state`` is a pair ``(state [b,h,D,d], sum_of_keys [b,h,D])`` -- what
    ``power_retention_inference`` takes and returns -- and ``return_final_state=True`` returns
    ``(out, (state, sum_of_keys))`` with the state AFTER the last token of this call, every chunk's decay
    applied to what came before it.  One call over t tokens therefore equals two calls over t/2 chained
    through the returned pair.  This departs from the reference on purpose: there the returned tensor is the
    state at the START of the last chunk, the initial state is not decayed by the gates ("TODO", ref:
    retention/power_retention_maker.py:158, 168-172) and no key sums travel with it, so its normaliser
    forgets the earlier call.
    """
    if full_scan_impl is None and scan_keeps_last:
        full_scan_impl = discumsum_impl

    def power_retention(Q, K, V, log_G=None, initial_state=None, return_final_state=False,
                        deg=2, scale=None, chunk_size=None, switch_over_seq_len=None):
        # ref: retention/power_retention_maker.py:71-90 -- pad the time axis to a chunk multiple (gate pad = log 1)
        t_in = Q.shape[1]
        pad = 0
        if chunk_size is not None and t_in % chunk_size != 0:
            pad = chunk_size - t_in % chunk_size
            Q, K, V = _pad_time(Q, pad, 2), _pad_time(K, pad, 2), _pad_time(V, pad, 2)
            if log_G is not None:
                log_G = _pad_time(log_G, pad, 1)
        out = _body(Q, K, V, log_G, initial_state, return_final_state, deg, scale, chunk_size, switch_over_seq_len)
        if not pad:
            return out
        if return_final_state:   # (padded keys are zero and padded gates are log 1: the state is not touched by them)
            return out[0][:, :t_in], out[1]
        return out[:, :t_in]

    def _body(Q, K, V, log_G, initial_state, return_final_state, deg, scale, chunk_size, switch_over_seq_len):
        # ref: retention/power_retention_maker.py:96-197
        assert deg % 2 == 0, f"deg must be even: {deg=}"
        assert Q.dtype == K.dtype == V.dtype, f"dtypes of inputs must match: {Q.dtype=}, {K.dtype=}, {V.dtype=}"
        dtype = Q.dtype
        b, t, hq, d = Q.shape
        h = K.shape[2]
        assert hq % h == 0, f"Q heads must be a multiple of KV heads: {hq=} {h=}"
        r = hq // h
        if chunk_size is not None:
            assert t % chunk_size == 0, f"{t=} not evenly divisible by {chunk_size=}"
            c, n = chunk_size, t // chunk_size
            if switch_over_seq_len is None:
                switch_over_seq_len = chunk_size
        else:
            c, n = t, 1
        gated = log_G is not None
        if gated:
            log_G = log_G.to(torch.float32)
        if not scale:
            scale = 1.0 / d ** 0.5
        with_state = initial_state is not None or return_final_state
        if initial_state is not None:
            assert isinstance(initial_state, (tuple, list)) and len(initial_state) == 2, \
                "initial_state must be the pair (state [b,h,D,d], sum_of_keys [b,h,D])"
            S0, s0 = initial_state
            assert S0.dim() == 4 and S0.shape[:2] == (b, h) and S0.shape[3] == d and s0.shape == S0.shape[:3], \
                f"initial_state shapes {tuple(S0.shape)}, {tuple(s0.shape)} do not fit {b=} {h=} {d=}"
            assert S0.dtype == dtype, f"initial_state dtype {S0.dtype} must match the inputs' {dtype}"

        if (switch_over_seq_len is None or t <= switch_over_seq_len) and not with_state:   # quadratic form (:128-140)
            A = None
            if gated:   # (ref: retention/power_retention_maker.py:129)
                A = gate_cumsum_impl(log_G) if gate_cumsum_impl is not None else None
                if A is None:
                    A = log_G.cumsum(1)
            return attention_impl(Q, K, V, A, deg, scale=scale, norm=True)

        # Everything below goes through the state, which exists for degree 2 only: refuse here, before anything is
        # launched, whichever implementation follows (ref: retention/_update_state/triton.py:310-311).
        if deg != 2:
            raise NotImplementedError(f"the chunked algorithm needs the degree-2 state layout (got deg={deg})")

        if chunked_impl is not None:
            # one autograd node; a carried state enters the scan as its starting value and the state after the last
            # token leaves it as the scan's last entry (no copy of the chunk states, no second path)
            if not with_state:
                return chunked_impl(Q.contiguous(), K.contiguous(), V.contiguous(),
                                    log_G.contiguous() if gated else None, deg, scale, c)
            return chunked_impl(Q.contiguous(), K.contiguous(), V.contiguous(), log_G.contiguous() if gated else None,
                                deg, scale, c, initial_state, return_final_state)

        Qc, Kc, Vc = Q.view(b, n, c, hq, d), K.view(b, n, c, h, d), V.view(b, n, c, h, d)
        if gated:
            A = log_G.view(b, n, c, h).cumsum(2)                       # (:147-148)
            A_last = A[:, :, c - 1]
            Kd = Kc * torch.exp((A_last.unsqueeze(2) - A) / deg).unsqueeze(-1).to(dtype)   # (:151-153)
            lcs = A_last.contiguous()
        else:
            A, Kd = None, Kc
            lcs = torch.zeros(b, n, h, device=Q.device, dtype=torch.float32)              # (:166)
        S, s = update_state_impl(Kd.contiguous(), Vc.contiguous(), deg)                    # (:156)
        final = None
        if with_state:
            if full_scan_impl is None:
                raise NotImplementedError("initial_state / return_final_state need a scan that keeps its last entry")
            first = 0
            if initial_state is not None:
                # the carried state is one more entry in front of the chunk states; its own gate is never applied
                # (entry 0 of the scan is zero), and chunk k's gate sum then decays it like any other chunk's state
                S = torch.cat([S0.unsqueeze(1), S], 1)
                s = torch.cat([s0.unsqueeze(1).to(s.dtype), s], 1)
                lcs = torch.cat([torch.zeros_like(lcs[:, :1]), lcs], 1)
                first = 1
            S, s = full_scan_impl(S, lcs), full_scan_impl(s, lcs)
            if return_final_state:
                final = (S[:, first + n], s[:, first + n])
            S, s = S.narrow(1, first, n), s.narrow(1, first, n)
        else:
            S, s = discumsum_impl(S, lcs), discumsum_impl(s, lcs)                          # (:167-170)
            if scan_keeps_last:
                S, s = S.narrow(1, 0, n), s.narrow(1, 0, n)

        flat = lambda x: x.reshape(b * n, *x.shape[2:])  # noqa: E731
        Ya, la, rm = attention_impl(flat(Qc), flat(Kc), flat(Vc), flat(A) if gated else None, deg,
                                    scale=scale, norm=False)                               # (:180)
        Ya, la, rm = (x.view(b, n, *x.shape[1:]) for x in (Ya, la, rm))
        if gated:                                                                          # (:183-186)
            Aq = A.repeat_interleave(r, dim=3) if r > 1 else A
            Qg = Qc * torch.exp(Aq / deg).unsqueeze(-1).to(dtype)
        else:
            Qg = Qc
        Y = query_state_impl(Qg.contiguous(), S.contiguous(), s.contiguous(), Ya.contiguous(), la.contiguous(),
                             rm.contiguous(), deg, scale, initial_state is None)           # (:190)
        out = Y.contiguous().view(b, t, hq, d).to(dtype)
        return (out, final) if return_final_state else out

    return power_retention


def make_power_retention_inference(update_state_impl, query_state_impl, attention_impl, fused_normalizer=False):
    """Build ``power_retention_inference`` (ref: retention/power_retention_maker.py:284-395).

    Only the explicit-normaliser form (``fused_normalizer=False``, ref: retention/reference.py:9) exists here.
    """
    if fused_normalizer:
        raise NotImplementedError("the fused-normaliser state layout belongs to a backend this build does not provide")

    def power_retention_inference(Q, K, V, log_G=None, initial_state=None, sum_of_keys=None,
                                  deg=2, scale=None, switch_over_seq_len=512):
        has_cache = K is not None and V is not None
        assert has_cache or initial_state is not None, "initial_state or cache must be provided for inference"
        assert not has_cache or Q.dtype == K.dtype == V.dtype, "dtypes of inputs must match"
        assert not has_cache or Q.shape[0] == K.shape[0] == V.shape[0], "batch sizes of inputs must match"
        assert not has_cache or K.shape[1] == V.shape[1], "key and value must have the same seq_len"
        assert initial_state is None or not has_cache or initial_state.shape[0] == K.shape[0], \
            "initial_state must have a batch size of the same as the key"
        assert initial_state is None or not has_cache or initial_state.shape[1] == K.shape[2], \
            "initial_state must have the same number of kv heads as the key"
        assert log_G is None or not has_cache or log_G.shape[:3] == K.shape[:3], \
            "log_gating must have a batch size, seq_len, and head count of the same as the key"
        b, tq, hq, d = Q.shape
        if has_cache:
            tk, hk = K.shape[1], K.shape[2]
        else:
            assert sum_of_keys is not None, "sum_of_keys must be provided for inference"
            tk, hk = 0, initial_state.shape[1]
        scale = 1.0 / d ** 0.5 if scale is None else scale
        A = log_G.to(torch.float32).cumsum(1) if log_G is not None else None               # (:347)
        r = hq // hk
        if initial_state is None:
            Y = attention_impl(Q, K, V, A, deg, scale=scale, norm=True)                    # (:350)
        else:
            assert initial_state.shape[0] == b, "initial_state must have a batch size of the same as the query"
            assert initial_state.shape[1] == hk, "initial_state must have the same number of kv heads as the key"
            if tk > 0:
                Ya, la, rm = attention_impl(Q, K, V, A, deg, scale=scale, norm=False)      # (:355)
            else:
                Ya = la = rm = None
            Qs = Q
            if A is not None:                                                              # (:358-359)
                Qs = Q * torch.exp(A[:, -1:] / deg).repeat_interleave(r, dim=-1).unsqueeze(-1).to(Q.dtype)
            Y = query_state_impl(Qs, initial_state, sum_of_keys, Ya, la, rm, deg, scale, False)   # (:363)

        if switch_over_seq_len is not None and tk >= switch_over_seq_len:                  # (:366-382)
            Kd = K
            if A is not None:
                Kd = (K * torch.exp((A[:, -1:] - A) / deg).unsqueeze(-1)).to(K.dtype)
            dS, ds = update_state_impl(Kd.contiguous(), V.contiguous(), deg)
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

    return power_retention_inference
