"""The four power-retention operators on MI355X, as PyTorch custom ops over the HIP library.

Same call signatures, argument meaning and tensor layouts as the reference's operator backends
(ref: retention/_attention/reference.py:10, retention/_update_state/reference.py:86,
retention/_discumsum/reference.py:3, retention/_query_state/reference.py:166), so they can be handed to
``make_power_retention`` / ``make_power_retention_inference`` like any other backend.  Registration follows
the custom-op convention of the reference's CUDA wrappers (ref: retention/_attention/cuda.py:10-43,129-245):
one ``torch.library.custom_op`` per kernel, a fake implementation for shapes and dtypes, autograd
registered in Python.

PyTorch only supplies device memory and the current stream; all arithmetic happens in the library.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib

_HALF = (torch.bfloat16, torch.float16)


def expanded_dim(d: int, deg: int = 2) -> int:
    """State size D for head dim d (ref: retention/_utils.py:18-19)."""
    assert deg == 2, "only deg=2 has a state layout"
    assert d % 16 == 0
    t = d // 16
    return 128 * t * (t + 1)


def _cont(x):
    return None if x is None else x.contiguous()


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------
@torch.library.custom_op("pr::attention_fwd", mutates_args=(), device_types="cuda")
def attention_fwd(Q: Tensor, K: Tensor, V: Tensor, G: Optional[Tensor], deg: int, scale: float,
                  norm: bool) -> Tuple[Tensor, Tensor, Tensor]:
    b, tq, hq, d = Q.shape
    _, tk, h, _ = K.shape
    O = torch.empty_like(Q)
    l = torch.empty((b, tq, hq), dtype=torch.float32, device=Q.device)
    rowmax = torch.empty((b, tq, hq), dtype=torch.float32, device=Q.device)
    lib = _lib.load()
    _lib.check(lib.pr_attention_fwd(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(G), _lib.ptr(O), _lib.ptr(l),
                                    _lib.ptr(rowmax), b, tq, tk, h, hq // h, d, float(scale), int(deg), int(norm),
                                    _lib.dtype_code(Q.dtype), _lib.stream()), "attention_fwd")
    return O, l, rowmax


@attention_fwd.register_fake
def _(Q, K, V, G, deg, scale, norm):
    b, tq, hq, _ = Q.shape
    return (torch.empty_like(Q), Q.new_empty((b, tq, hq), dtype=torch.float32),
            Q.new_empty((b, tq, hq), dtype=torch.float32))


@torch.library.custom_op("pr::attention_bwd", mutates_args=(), device_types="cuda")
def attention_bwd(Q: Tensor, K: Tensor, V: Tensor, G: Optional[Tensor], rowmax: Tensor, dO: Tensor,
                  dl: Optional[Tensor], dO_scale: Optional[Tensor], deg: int,
                  scale: float) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    b, tq, hq, d = Q.shape
    _, tk, h, _ = K.shape
    r = hq // h
    dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)
    dGq = dGk = None
    if G is not None:
        dGq = torch.empty((b, tq, hq), dtype=torch.float32, device=Q.device)
        dGk = torch.empty((b, tk, h), dtype=torch.float32, device=Q.device)
    lib = _lib.load()
    _lib.check(lib.pr_attention_bwd(_lib.ptr(Q), _lib.ptr(K), _lib.ptr(V), _lib.ptr(G), _lib.ptr(rowmax),
                                    _lib.ptr(dO), _lib.ptr(dl), _lib.ptr(dO_scale), _lib.ptr(dQ), _lib.ptr(dK),
                                    _lib.ptr(dV),
                                    _lib.ptr(dGq), _lib.ptr(dGk), b, tq, tk, h, r, d, float(scale), int(deg),
                                    _lib.dtype_code(Q.dtype), _lib.stream()), "attention_bwd")
    if G is None:
        dG = torch.empty((0,), dtype=torch.float32, device=Q.device)
    else:
        dG = dGk
        dG[:, tk - tq:] += dGq.view(b, tq, h, r).sum(-1)
    return dQ, dK, dV, dG


@attention_bwd.register_fake
def _(Q, K, V, G, rowmax, dO, dl, dO_scale, deg, scale):
    dG = Q.new_empty((0,), dtype=torch.float32) if G is None else torch.empty_like(G)
    return torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V), dG


def _attention_setup(ctx, inputs, output):
    Q, K, V, G, deg, scale, norm = inputs
    O, l, rowmax = output
    ctx.save_for_backward(Q, K, V, G, O, l, rowmax)
    ctx.deg, ctx.scale, ctx.norm = deg, scale, norm


def _attention_backward(ctx, dO, dl, drowmax):
    Q, K, V, G, O, l, rowmax = ctx.saved_tensors
    if ctx.norm:  # O = o / l: chain back to the unnormalised pair (o, l); the 1/l on dO is applied in the kernel
        osc = 1.0 / l
        dlu = -(dO.float() * O.float()).sum(-1) * osc
    else:
        dlu, osc = dl, None
    dQ, dK, dV, dG = attention_bwd(Q, K, V, G, rowmax, dO.contiguous(), _cont(dlu), _cont(osc), ctx.deg, ctx.scale)
    return dQ, dK, dV, (dG if G is not None else None), None, None, None


torch.library.register_autograd("pr::attention_fwd", _attention_backward, setup_context=_attention_setup)


def attention(Q, K, V, log_G, deg, causal=True, head_first=False, scale=1.0, norm=False, use_log2=False):
    """Power attention; ``log_G`` is the accumulated log gate [b, tk, h] (fp32) or None.

    Returns ``o / l`` when ``norm`` else ``(o, l, rowmax)`` (ref: retention/_attention/reference.py:10-69).
    Only the configuration the composed functions use is provided: causal, time-major, natural log.
    """
    assert causal and not head_first and not use_log2, "only causal=True, head_first=False, use_log2=False"
    assert isinstance(deg, int) and deg > 0 and deg % 2 == 0, "deg must be a positive even integer"
    assert Q.dtype == K.dtype == V.dtype and Q.dtype in _HALF, f"Q, K, V must share a dtype in {_HALF}"
    assert Q.dim() == 4 and K.shape == V.shape and Q.shape[0] == K.shape[0] and Q.shape[3] == K.shape[3]
    assert Q.shape[2] % K.shape[2] == 0, "query heads must be a multiple of kv heads"
    assert Q.shape[1] <= K.shape[1], "queries are aligned to the end of the keys: tq <= tk"
    if log_G is not None:
        assert log_G.shape == K.shape[:3], "log_G must be [b, tk, h]"
        log_G = log_G.to(torch.float32).contiguous()
    O, l, rowmax = attention_fwd(Q.contiguous(), K.contiguous(), V.contiguous(), log_G, deg, float(scale), bool(norm))
    if norm:
        return O
    return O, l, rowmax


# ----------------------------------------------------------------------------
# update_state
# ----------------------------------------------------------------------------
@torch.library.custom_op("pr::update_state_fwd", mutates_args=(), device_types="cuda")
def update_state_fwd(K: Tensor, V: Tensor) -> Tuple[Tensor, Tensor]:
    b, n, c, h, d = K.shape
    D = expanded_dim(d)
    S = torch.empty((b, n, h, D, d), dtype=K.dtype, device=K.device)
    s = torch.empty((b, n, h, D), dtype=torch.float32, device=K.device)
    lib = _lib.load()
    _lib.check(lib.pr_update_state_fwd(_lib.ptr(K), _lib.ptr(V), _lib.ptr(S), _lib.ptr(s), None, b * n, c, h, d, 2, 0,
                                       _lib.dtype_code(K.dtype), _lib.stream()), "update_state_fwd")
    return S, s


@update_state_fwd.register_fake
def _(K, V):
    b, n, c, h, d = K.shape
    D = expanded_dim(d)
    return K.new_empty((b, n, h, D, d)), K.new_empty((b, n, h, D), dtype=torch.float32)


@torch.library.custom_op("pr::update_state_bwd", mutates_args=(), device_types="cuda")
def update_state_bwd(K: Tensor, V: Tensor, dS: Tensor, ds: Tensor) -> Tuple[Tensor, Tensor]:
    b, n, c, h, d = K.shape
    dK, dV = torch.empty_like(K), torch.empty_like(V)
    lib = _lib.load()
    _lib.check(lib.pr_update_state_bwd(_lib.ptr(K), _lib.ptr(V), _lib.ptr(dS), _lib.ptr(ds), None, None, None, None,
                                       _lib.ptr(dK),
                                       _lib.ptr(dV), b * n, c, h, d, 2, 0, 0, _lib.dtype_code(K.dtype), _lib.stream()),
               "update_state_bwd")
    return dK, dV


@update_state_bwd.register_fake
def _(K, V, dS, ds):
    return torch.empty_like(K), torch.empty_like(V)


def _update_state_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _update_state_backward(ctx, dS, ds):
    K, V = ctx.saved_tensors
    return update_state_bwd(K, V, dS.contiguous(), ds.contiguous())


torch.library.register_autograd("pr::update_state_fwd", _update_state_backward, setup_context=_update_state_setup)


def update_state(K, V, deg):
    """Chunk states: K, V [b, n, c, h, d] (or [b, c, h, d]) -> S [b, n, h, D, d], s [b, n, h, D] fp32
    (ref: retention/_update_state/reference.py:33-52, 86-94)."""
    if deg != 2:
        raise NotImplementedError("update_state: only deg=2 has a state layout")
    if K.dim() == 4:
        S, s = update_state(K.unsqueeze(1), V.unsqueeze(1), deg)
        return S.squeeze(1), s.squeeze(1)
    assert K.dim() == 5 and K.shape == V.shape and K.dtype == V.dtype and K.dtype in _HALF
    return update_state_fwd(K.contiguous(), V.contiguous())


# ----------------------------------------------------------------------------
# discumsum
# ----------------------------------------------------------------------------
def _flat(X):
    b, n, h = X.shape[:3]
    F = 1
    for x in X.shape[3:]:
        F *= x
    return b, n, h, F


@torch.library.custom_op("pr::discumsum_fwd", mutates_args=(), device_types="cuda")
def discumsum_fwd(X: Tensor, log_G: Tensor, n_out: int) -> Tensor:
    b, n, h, F = _flat(X)
    Y = torch.empty((b, n_out, *X.shape[2:]), dtype=X.dtype, device=X.device)
    lib = _lib.load()
    _lib.check(lib.pr_discumsum_fwd(_lib.ptr(X), _lib.ptr(log_G), _lib.ptr(Y), b, n, n_out, h, F,
                                    _lib.dtype_code(X.dtype), _lib.stream()), "discumsum_fwd")
    return Y


@discumsum_fwd.register_fake
def _(X, log_G, n_out):
    return X.new_empty((X.shape[0], n_out, *X.shape[2:]))


@torch.library.custom_op("pr::discumsum_bwd", mutates_args=(), device_types="cuda")
def discumsum_bwd(dY: Tensor, Y: Tensor, log_G: Tensor) -> Tuple[Tensor, Tensor]:
    b, n, h = log_G.shape
    n_out = Y.shape[1]
    F = 1
    for x in Y.shape[3:]:
        F *= x
    dX = torch.empty((b, n, *Y.shape[2:]), dtype=Y.dtype, device=Y.device)
    dlg = torch.empty_like(log_G)
    lib = _lib.load()
    code = _lib.dtype_code(Y.dtype)
    ws = torch.empty((lib.pr_discumsum_bwd_workspace(b, n, h, F, code),), dtype=torch.uint8, device=Y.device)
    _lib.check(lib.pr_discumsum_bwd(_lib.ptr(dY), _lib.ptr(Y), _lib.ptr(log_G), _lib.ptr(dX), _lib.ptr(dlg),
                                    _lib.ptr(ws), b, n, n_out, h, F, code, _lib.stream()), "discumsum_bwd")
    return dX, dlg


@discumsum_bwd.register_fake
def _(dY, Y, log_G):
    return Y.new_empty((Y.shape[0], log_G.shape[1], *Y.shape[2:])), torch.empty_like(log_G)


def _discumsum_setup(ctx, inputs, output):
    X, log_G, n_out = inputs
    ctx.save_for_backward(log_G, output)


def _discumsum_backward(ctx, dY):
    log_G, Y = ctx.saved_tensors
    dX, dlg = discumsum_bwd(dY.contiguous(), Y, log_G)
    return dX, dlg, None


torch.library.register_autograd("pr::discumsum_fwd", _discumsum_backward, setup_context=_discumsum_setup)


def discumsum(X, log_G, keep_last=True):
    """Gated exclusive scan over axis 1: X [b, n, h, ...], log_G [b, n, h] fp32 -> [b, n+1, h, ...]
    (ref: retention/_discumsum/reference.py:3-15).  ``keep_last=False`` returns only the first n entries,
    which is what the composed function keeps (ref: retention/power_retention_maker.py:167-170).
    ``log_G=None`` is the reference's other branch (:4-5): the plain inclusive cumulative sum, n entries --
    the same scan with every gate log 1, minus its leading zero."""
    assert X.dim() >= 4 and X.dtype in (*_HALF, torch.float32)
    if log_G is None:
        zeros = torch.zeros(X.shape[:3], dtype=torch.float32, device=X.device)
        return discumsum_fwd(X.contiguous(), zeros, X.shape[1] + 1)[:, 1:]
    assert log_G.shape == X.shape[:3]
    n = X.shape[1]
    return discumsum_fwd(X.contiguous(), log_G.to(torch.float32).contiguous(), n + 1 if keep_last else n)


# ----------------------------------------------------------------------------
# query_state
# ----------------------------------------------------------------------------
@torch.library.custom_op("pr::query_state_fwd", mutates_args=(), device_types="cuda")
def query_state_fwd(Q: Tensor, S: Tensor, s: Tensor, Y_attn: Optional[Tensor], l_attn: Optional[Tensor],
                    rowmax: Optional[Tensor], scale_p: float, zero_initial_state: bool) -> Tuple[Tensor, Tensor]:
    b, n, c, hq, d = Q.shape
    h = S.shape[2]
    O = torch.empty_like(Q)
    den = torch.empty((b, n, c, hq), dtype=torch.float32, device=Q.device)
    lib = _lib.load()
    _lib.check(lib.pr_query_state_fwd(_lib.ptr(Q), _lib.ptr(S), _lib.ptr(s), _lib.ptr(Y_attn), _lib.ptr(l_attn),
                                      _lib.ptr(rowmax), None, _lib.ptr(O), _lib.ptr(den), b * n, n, c, h, hq // h, d,
                                      float(scale_p), 2, int(zero_initial_state), 0, _lib.dtype_code(Q.dtype),
                                      _lib.stream()), "query_state_fwd")
    return O, den


@query_state_fwd.register_fake
def _(Q, S, s, Y_attn, l_attn, rowmax, scale_p, zero_initial_state):
    return torch.empty_like(Q), Q.new_empty(Q.shape[:4], dtype=torch.float32)


@torch.library.custom_op("pr::query_state_bwd", mutates_args=(), device_types="cuda")
def query_state_bwd(Q: Tensor, S: Tensor, s: Tensor, rowmax: Optional[Tensor], O: Tensor, den: Tensor, dO: Tensor,
                    scale_p: float, zero_initial_state: bool) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    b, n, c, hq, d = Q.shape
    h = S.shape[2]
    r = hq // h
    dQ, dS, ds = torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s)
    has_attn = rowmax is not None
    dYa = torch.empty_like(Q) if has_attn else None
    dla = torch.empty_like(den) if has_attn else None
    lib = _lib.load()
    code = _lib.dtype_code(Q.dtype)
    ws = torch.empty((lib.pr_query_state_bwd_workspace(b * n, c, h, r, d, code),), dtype=torch.uint8, device=Q.device)
    _lib.check(lib.pr_query_state_bwd(_lib.ptr(Q), _lib.ptr(S), _lib.ptr(s), _lib.ptr(rowmax), None, _lib.ptr(O),
                                      _lib.ptr(den), _lib.ptr(dO), _lib.ptr(dQ), _lib.ptr(dS), _lib.ptr(ds),
                                      _lib.ptr(dYa), _lib.ptr(dla), None, _lib.ptr(ws), None, b * n, n, c, h, r, d,
                                      float(scale_p), 2, int(zero_initial_state), 0, 0, code, _lib.stream()),
               "query_state_bwd")
    if not has_attn:
        dYa = torch.empty((0,), dtype=Q.dtype, device=Q.device)
        dla = torch.empty((0,), dtype=torch.float32, device=Q.device)
    return dQ, dS, ds, dYa, dla


@query_state_bwd.register_fake
def _(Q, S, s, rowmax, O, den, dO, scale_p, zero_initial_state):
    if rowmax is None:
        return (torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s), Q.new_empty((0,)),
                Q.new_empty((0,), dtype=torch.float32))
    return torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s), torch.empty_like(Q), torch.empty_like(den)


def _query_state_setup(ctx, inputs, output):
    Q, S, s, Y_attn, l_attn, rowmax, scale_p, zis = inputs
    O, den = output
    ctx.save_for_backward(Q, S, s, rowmax, O, den)
    ctx.scale_p, ctx.zis = scale_p, zis


def _query_state_backward(ctx, dO, dden):
    Q, S, s, rowmax, O, den = ctx.saved_tensors
    dQ, dS, ds, dYa, dla = query_state_bwd(Q, S, s, rowmax, O, den, dO.contiguous(), ctx.scale_p, ctx.zis)
    if rowmax is None:
        dYa = dla = None
    return dQ, dS, ds, dYa, dla, None, None, None


torch.library.register_autograd("pr::query_state_fwd", _query_state_backward, setup_context=_query_state_setup)


def query_state(Q, S, s, Y_attn, l_attn, rowmax, deg, scale, zero_initial_state):
    """Query the state and merge with the attention part: Q [b, n, c, hq, d] (already gated),
    S [b, n, h, D, d], s [b, n, h, D] fp32, Y_attn / l_attn / rowmax from ``attention(norm=False)`` or all
    None -> O [b, n, c, hq, d]; 4-D inputs are the inference form
    (ref: retention/_query_state/reference.py:36-96, 166-191)."""
    if deg != 2:
        raise NotImplementedError("query_state: only deg=2 has a state layout")
    if Q.dim() == 4:
        un = lambda x: None if x is None else x.unsqueeze(1)  # noqa: E731
        return query_state(un(Q), un(S), un(s), un(Y_attn), un(l_attn), un(rowmax), deg, scale,
                           zero_initial_state).squeeze(1)
    assert Q.dim() == 5 and S.dim() == 5 and Q.dtype == S.dtype and Q.dtype in _HALF
    assert Q.shape[3] % S.shape[2] == 0, "query heads must be a multiple of kv heads"
    assert S.shape[3] == expanded_dim(Q.shape[4]) and S.shape[4] == Q.shape[4]
    assert (Y_attn is None) == (l_attn is None) == (rowmax is None)
    f32 = lambda x: None if x is None else x.to(torch.float32).contiguous()  # noqa: E731
    O, _den = query_state_fwd(Q.contiguous(), S.contiguous(), f32(s), _cont(Y_attn), f32(l_attn), f32(rowmax),
                              float(scale) ** deg, bool(zero_initial_state))
    return O


@torch.library.custom_op("pr::gate_cumsum", mutates_args=(), device_types="cuda")
def gate_cumsum(log_G: Tensor) -> Tensor:
    """log_G [b, t, h] fp32 contiguous, t <= 8192 -> cumulative sum over t (ref: log_G.cumsum(1),
    retention/power_retention_maker.py:129, 348-349)."""
    b, t, h = log_G.shape
    A = torch.empty_like(log_G)
    _lib.check(_lib.load().pr_gate_cumsum(_lib.ptr(log_G), _lib.ptr(A), b, t, h, _lib.stream()), "gate_cumsum")
    return A


@gate_cumsum.register_fake
def _(log_G):
    return torch.empty_like(log_G)


def _gate_cumsum_backward(ctx, dA):
    # the adjoint of a running sum is the running sum from the other end
    return gate_cumsum(dA.flip(1).contiguous()).flip(1)


torch.library.register_autograd("pr::gate_cumsum", _gate_cumsum_backward)


def gate_cumsum_or_none(log_G: Tensor):
    """The accumulated gates through the library's kernel where it takes the shape (fp32 on the GPU, t <= 8192: one
    workgroup per (batch, head) with the sequence in LDS; torch's scan along a middle axis takes 1.4 ms at t = 8192
    where this takes 10 us), else None."""
    if log_G.is_cuda and log_G.dtype == torch.float32 and log_G.dim() == 3 and log_G.shape[1] <= 8192:
        return gate_cumsum(log_G.contiguous())
    return None


# ----------------------------------------------------------------------------
# single-token inference step on the state (no autograd: inference only)
# ----------------------------------------------------------------------------
@torch.library.custom_op("pr::decode_step", mutates_args=(), device_types="cuda")
def decode_step(Q: Tensor, gq: Optional[Tensor], S: Tensor, s: Tensor, Y_attn: Optional[Tensor],
                l_attn: Optional[Tensor], rowmax: Optional[Tensor], K_new: Optional[Tensor], V_new: Optional[Tensor],
                log_decay: Optional[Tensor], scale_p: float, attend_new: bool = False) -> Tuple[Tensor, Tensor, Tensor]:
    """Q [b, tq, hq, d] (tq * hq/h <= 16), gq [b, h] fp32 or None, S [b, h, D, d], s [b, h, D] fp32, attention part or
    None, and optionally one new token K_new, V_new [b, h, d] with log_decay [b, h] -> (out [b, tq, hq, d],
    S_new, s_new); without a new token S_new, s_new are empty tensors.  attend_new: the attention part is the new
    token attending to itself (tq == 1, no Y_attn)."""
    b, tq, hq, d = Q.shape
    h = S.shape[1]
    out = torch.empty_like(Q)
    lib = _lib.load()
    ws = torch.empty(lib.pr_decode_step_workspace(b, tq, h, hq // h, d), dtype=torch.uint8, device=Q.device)
    if K_new is not None:
        S_new, s_new = torch.empty_like(S), torch.empty_like(s)
    else:
        S_new, s_new = S.new_empty(0), s.new_empty(0)
    _lib.check(lib.pr_decode_step(_lib.ptr(Q), _lib.ptr(gq), _lib.ptr(S), _lib.ptr(s), _lib.ptr(Y_attn),
                                  _lib.ptr(l_attn), _lib.ptr(rowmax), _lib.ptr(K_new), _lib.ptr(V_new),
                                  _lib.ptr(log_decay), _lib.ptr(S_new) if K_new is not None else None,
                                  _lib.ptr(s_new) if K_new is not None else None, _lib.ptr(out), _lib.ptr(ws),
                                  b, tq, h, hq // h, d, float(scale_p), 2, _lib.dtype_code(Q.dtype), int(attend_new),
                                  _lib.stream()),
               "decode_step")
    return out, S_new, s_new


@decode_step.register_fake
def _(Q, gq, S, s, Y_attn, l_attn, rowmax, K_new, V_new, log_decay, scale_p, attend_new=False):
    if K_new is not None:
        return torch.empty_like(Q), torch.empty_like(S), torch.empty_like(s)
    return torch.empty_like(Q), S.new_empty(0), s.new_empty(0)
