"""``power_retention_inference`` with the single-token step fused (ref: retention/power_retention_maker.py:284-395).

Same signature, results and state layout as the maker-assembled function; calls with a state and at most 16 query
rows per (batch, kv head) -- the decode step -- go through one pass over the state (query, and the fold of a
single new token when ``switch_over_seq_len`` is reached with a one-token cache) instead of the operator chain.
Everything else is delegated to the composed function.
"""
import torch

from . import ops


def _direct(op):
    """The Python function behind a custom op.  The decode step needs no autograd, and outside ``torch.compile`` the
    dispatcher's per-call cost (tens of microseconds per operator) is most of a step's host time."""
    return getattr(op, "_init_fn", op)


def _impls(*tensors):
    traced = torch.compiler.is_compiling() or (torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in tensors))
    if traced:
        return ops.attention_fwd, ops.decode_step, ops.gate_cumsum
    return _direct(ops.attention_fwd), _direct(ops.decode_step), _direct(ops.gate_cumsum)


def make_fused_inference(composed):
    def power_retention_inference(Q, K, V, log_G=None, initial_state=None, sum_of_keys=None, deg=2, scale=None,
                                  switch_over_seq_len=512):
        has_cache = K is not None and V is not None
        fast = (initial_state is not None and sum_of_keys is not None and deg == 2 and Q.dim() == 4
                and Q.dtype in (torch.bfloat16, torch.float16) and initial_state.dtype == Q.dtype
                and Q.shape[1] * (Q.shape[2] // initial_state.shape[1]) <= 16
                and Q.shape[3] in (32, 64, 128))
        if has_cache:
            fast = fast and K.shape[1] >= Q.shape[1] and K.dtype == Q.dtype == V.dtype and K.shape[0] == Q.shape[0] \
                and K.shape[2] == initial_state.shape[1] and K.shape == V.shape and K.shape[3] == Q.shape[3] \
                and Q.shape[2] % K.shape[2] == 0 and (log_G is None or log_G.shape == K.shape[:3])
        if not fast:
            return composed(Q, K, V, log_G, initial_state, sum_of_keys, deg, scale, switch_over_seq_len)
        b, tq, hq, d = Q.shape
        assert initial_state.shape[0] == b, "initial_state must have a batch size of the same as the query"
        scale = 1.0 / d ** 0.5 if scale is None else scale
        tk = K.shape[1] if has_cache else 0
        attention_fwd, decode_step, gate_cumsum = _impls(Q, K, V, log_G, initial_state, sum_of_keys)
        fold = switch_over_seq_len is not None and tk >= switch_over_seq_len
        if fold and tk == 1:   # (then tq == 1 as well)
            # the recurrent loop (every token folded as it arrives): the new token attends to itself, queries the old
            # state and is folded, all in one pass over the state
            g1 = log_G.to(torch.float32)[:, 0].contiguous() if log_G is not None else None
            Y, new_S, new_s = decode_step(Q.contiguous(), g1, initial_state.contiguous(),
                                              sum_of_keys.to(torch.float32).contiguous(), None, None, None,
                                              K[:, 0].contiguous(), V[:, 0].contiguous(), g1, float(scale) ** deg, True)
            return Y, new_S, new_s.to(sum_of_keys.dtype)
        A = None
        if log_G is not None and has_cache:
            lg32 = log_G.to(torch.float32).contiguous()
            A = gate_cumsum(lg32) if (tk <= 8192 and not lg32.requires_grad) else lg32.cumsum(1)
        Ya = la = rm = None
        if tk > 0:
            Ya, la, rm = attention_fwd(Q.contiguous(), K.contiguous(), V.contiguous(), A, deg, float(scale), False)
        a_last = A[:, -1].contiguous() if A is not None else None
        S32 = sum_of_keys.to(torch.float32).contiguous()
        Y, _, _ = decode_step(Q.contiguous(), a_last, initial_state.contiguous(), S32, Ya, la, rm, None, None,
                                  None, float(scale) ** deg)
        if not fold:
            return Y, initial_state, sum_of_keys
        # fold of a longer cache: the operator chain of the composed function
        Kd = K
        if A is not None:
            Kd = (K * torch.exp((A[:, -1:] - A) / deg).unsqueeze(-1)).to(K.dtype)
        dS, ds = ops.update_state(Kd.contiguous(), V.contiguous(), deg)
        if A is None:
            return Y, initial_state + dS, sum_of_keys + ds
        decay = torch.exp(A[:, -1, :])
        return (Y, initial_state * decay[..., None, None].to(initial_state.dtype) + dS,
                sum_of_keys * decay[..., None].to(sum_of_keys.dtype) + ds)

    return power_retention_inference
