"""Preallocated K / V / gate / state cache for the decode loop, and the decode step over it.

The reference's caller keeps one cache layer per attention layer holding ``keys, values, gatings, state,
sum_of_keys`` (ref: deploy/models/powercoder/kvgs_dynamic_cache.py:26-34, 111-172): every step concatenates the new
token to three tensors (``update_kv``), hands the WHOLE cache to ``power_retention_inference`` and, once the cache
holds ``switch_over_seq_len`` tokens, replaces it by the returned state (``clean_kv`` + ``update_state``,
ref: deploy/models/powercoder/modeling_powercoder.py:161-196).  ``RetentionCache`` is that layer with fixed buffers:

* ``keys, values [b, capacity, h, d]`` and the ACCUMULATED log gates ``[b, capacity, h]`` fp32 are written in place by
  one append kernel (``pr_cache_append``; no ``torch.cat``, no cumulative sum over the cache per step);
* ``state [b, h, D, d]``, ``sum_of_keys [b, h, D]`` fp32 live in buffers that are updated in place;
* ``step(q, k, v, log_g)`` is the caller's whole per-token sequence (append, attention over the cache, query of the
  state, merge; fold + clearing at the switch-over) with every output buffer preallocated -- three library calls per
  token and no allocation, so a loop of steps can also be captured in a HIP graph;
* ``update_kv / update_state / clean_kv / reset / get_seq_length`` keep the reference layer's method names.

Inference only (no autograd).
"""
from __future__ import annotations

import torch

from . import _lib
from .ops import expanded_dim


class RetentionCache:
    def __init__(self, batch, kv_heads, head_dim, capacity, dtype=torch.bfloat16, device="cuda", q_heads=None):
        assert dtype in (torch.bfloat16, torch.float16) and head_dim in (32, 64, 128)
        self.b, self.h, self.d, self.capacity = batch, kv_heads, head_dim, capacity
        self.hq = q_heads or kv_heads
        assert self.hq % kv_heads == 0, "query heads must be a multiple of kv heads"
        # the single-pass decode kernel takes up to 16 query rows per kv head; wider groups run the state query as the
        # query_state operator over the same preallocated buffers (a few more launches per token, same results)
        self._fused_step = self.hq // kv_heads <= 16
        self.dtype, self.device = dtype, torch.device(device)
        D = expanded_dim(head_dim)
        f32 = torch.float32
        self.keys = torch.empty(batch, capacity, kv_heads, head_dim, dtype=dtype, device=device)
        self.values = torch.empty_like(self.keys)
        self.gatings = torch.empty(batch, capacity, kv_heads, dtype=f32, device=device)     # accumulated log gates
        self.state = torch.zeros(batch, kv_heads, D, head_dim, dtype=dtype, device=device)
        self.sum_of_keys = torch.zeros(batch, kv_heads, D, dtype=f32, device=device)
        self.has_state = False
        self.length = 0
        # outputs and scratch of a step (never reallocated)
        self._ya = torch.empty(batch, 1, self.hq, head_dim, dtype=dtype, device=device)
        self._la = torch.empty(batch, 1, self.hq, dtype=f32, device=device)
        self._rm = torch.empty(batch, 1, self.hq, dtype=f32, device=device)
        self._out = torch.empty(batch, 1, self.hq, head_dim, dtype=dtype, device=device)
        self._gq = torch.empty(batch, kv_heads, dtype=f32, device=device)   # accumulated gate at the newest position
        self._lib = _lib.load()
        self._code = _lib.dtype_code(dtype)
        ws = self._lib.pr_decode_step_workspace(batch, 1, kv_heads, self.hq // kv_heads, head_dim) if self._fused_step else 0
        self._ws = torch.empty(max(ws, 16), dtype=torch.uint8, device=device)

    # ---- the reference layer's interface ---------------------------------------------------------------------
    def get_seq_length(self):
        return self.length

    def update_kv(self, key_states, value_states, gate_states):
        """Append ``key_states, value_states [b, t_new, h, d]`` and ``gate_states [b, t_new, h]`` (log gates, fp32, or
        None) in place; returns views of the filled part ``(keys, values, accumulated_gates, state, sum_of_keys)``
        (state entries None while there is no state).  Note the third entry: ACCUMULATED log gates since the start of
        the cache, i.e. what the reference computes from its ``gatings`` with ``cumsum(1)``."""
        t_new = key_states.shape[1]
        assert key_states.shape == (self.b, t_new, self.h, self.d) and value_states.shape == key_states.shape
        assert key_states.dtype == self.dtype and value_states.dtype == self.dtype, \
            f"the cache holds {self.dtype}; got {key_states.dtype} / {value_states.dtype}"
        assert key_states.device == self.keys.device and value_states.device == self.keys.device
        assert gate_states is None or gate_states.shape == (self.b, t_new, self.h)
        if self.length + t_new > self.capacity:
            raise ValueError(f"cache capacity {self.capacity} exceeded ({self.length} + {t_new})")
        p = _lib.ptr
        g = None if gate_states is None else gate_states.to(torch.float32).contiguous()
        _lib.check(self._lib.pr_cache_append(p(self.keys), p(self.values), p(self.gatings), p(key_states.contiguous()),
                                             p(value_states.contiguous()), p(g), p(self._gq), self.b, self.capacity, self.length,
                                             t_new, self.h, self.d, self._code, _lib.stream()), "cache_append")
        self.length += t_new
        n = self.length
        st = (self.state, self.sum_of_keys) if self.has_state else (None, None)
        return self.keys[:, :n], self.values[:, :n], self.gatings[:, :n], *st

    def update_state(self, state, sum_of_keys):
        """Adopt a state (copied into the cache's own buffers unless it already is them)."""
        if state is not self.state:
            self.state.copy_(state)
        if sum_of_keys is not self.sum_of_keys:
            self.sum_of_keys.copy_(sum_of_keys)
        self.has_state = True
        return self.state, self.sum_of_keys

    def clean_kv(self):
        self.length = 0

    def reset(self):
        self.length = 0
        self.has_state = False
        self.state.zero_()
        self.sum_of_keys.zero_()

    # ---- the decode step ---------------------------------------------------------------------------------------
    def step(self, q, k, v, log_g=None, scale=None, switch_over_seq_len=512, out=None):
        """One token: ``q [b, 1, hq, d]``, ``k, v [b, 1, h, d]``, ``log_g [b, 1, h]`` fp32 or None -> ``[b, 1, hq, d]``,
        written to ``out`` (contiguous, same shape and dtype as q) or, without it, to a buffer of the cache that the next
        step overwrites.  Same arithmetic as the reference caller's sequence
        ``update_kv -> power_retention_inference(whole cache, state) -> clean_kv + update_state at the switch-over``."""
        lib, p, stream = self._lib, _lib.ptr, _lib.stream()
        assert q.shape == (self.b, 1, self.hq, self.d) and q.dtype == self.dtype and q.device == self.keys.device
        assert k.shape == (self.b, 1, self.h, self.d) and v.shape == k.shape and k.dtype == self.dtype and v.dtype == self.dtype
        if out is None:
            out = self._out
        else:
            assert out.shape == q.shape and out.dtype == q.dtype and out.is_contiguous()
        scale = float(scale) if scale else 1.0 / self.d ** 0.5
        r = self.hq // self.h
        fold = switch_over_seq_len is not None and self.length + 1 >= switch_over_seq_len
        if self.has_state and fold and self.length == 0 and self._fused_step:
            # one-token cache folded at once (switch_over_seq_len = 1): the recurrent step, one pass over the state
            g = None if log_g is None else log_g.to(torch.float32).reshape(self.b, self.h).contiguous()
            _lib.check(lib.pr_decode_step(p(q.contiguous()), p(g), p(self.state), p(self.sum_of_keys), None, None, None,
                                          p(k.reshape(self.b, self.h, self.d).contiguous()),
                                          p(v.reshape(self.b, self.h, self.d).contiguous()), p(g), p(self.state),
                                          p(self.sum_of_keys), p(out), p(self._ws), self.b, 1, self.h, r, self.d,
                                          scale ** 2, 2, self._code, 1, stream), "decode_step")
            return out
        self.update_kv(k, v, log_g)
        n = self.length
        if not self.has_state:
            # no state yet: normalised attention over the cache
            _lib.check(lib.pr_cache_attention_fwd(p(q.contiguous()), p(self.keys), p(self.values), p(self.gatings),
                                                  p(out), p(self._la), p(self._rm), self.b, 1, n, self.capacity,
                                                  self.h, r, self.d, scale, 2, 1, self._code, stream), "cache_attention_fwd")
        else:
            _lib.check(lib.pr_cache_attention_fwd(p(q.contiguous()), p(self.keys), p(self.values), p(self.gatings),
                                                  p(self._ya), p(self._la), p(self._rm), self.b, 1, n, self.capacity,
                                                  self.h, r, self.d, scale, 2, 0, self._code, stream), "cache_attention_fwd")
            if not self._fused_step:
                # more query rows per kv head than the single-pass kernel holds: the state query as the operator
                # (ref: retention/power_retention_maker.py:358-363), gated by the accumulated gate at the newest position
                from . import ops
                qg = q
                if log_g is not None:
                    qg = (q * torch.exp(self._gq / 2).repeat_interleave(r, dim=-1)[:, None, :, None]).to(self.dtype)
                out.copy_(ops.query_state(qg.contiguous(), self.state, self.sum_of_keys, self._ya, self._la, self._rm, 2,
                                          scale, False))
                if fold:
                    self._fold()
                return out
            # (the query is gated by the accumulated gate at the newest cache position, which the append left in _gq)
            _lib.check(lib.pr_decode_step(p(q.contiguous()), p(self._gq), p(self.state), p(self.sum_of_keys), p(self._ya),
                                          p(self._la), p(self._rm), None, None, None, None, None, p(out),
                                          p(self._ws), self.b, 1, self.h, r, self.d, scale ** 2, 2, self._code, 0,
                                          stream), "decode_step")
        if fold:
            self._fold()
        return out

    def _fold(self):
        """Compress the cache into the state and clear it (ref: retention/power_retention_maker.py:366-382 and
        deploy/models/powercoder/modeling_powercoder.py:195-196).  Happens once per switch_over_seq_len tokens."""
        from . import ops
        n = self.length
        K, V, A = self.keys[:, :n], self.values[:, :n], self.gatings[:, :n]
        Kd = (K * torch.exp((A[:, -1:] - A) / 2).unsqueeze(-1)).to(self.dtype)
        dS, ds = ops.update_state(Kd.contiguous(), V.contiguous(), 2)
        if self.has_state:
            decay = torch.exp(A[:, -1, :])
            self.state.mul_(decay[..., None, None].to(self.dtype)).add_(dS)
            self.sum_of_keys.mul_(decay[..., None]).add_(ds)
        else:
            self.state.copy_(dS)
            self.sum_of_keys.copy_(ds)
            self.has_state = True
        self.clean_kv()
