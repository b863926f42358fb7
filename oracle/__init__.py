"""CPU oracle for symmetric power retention.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this; it is
used by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline``
leg of ``bench.py`` as the checker / reported baseline, never as the thing that
is shipped or measured as the product.

It restates, in plain PyTorch on the CPU, the reference's pure-torch backend
(``retention/reference.py`` and the four ``retention/_*/reference.py``
operators wired through ``retention/power_retention_maker.py``).  Each function
cites the reference lines it follows.

How each function is pinned (see tests/test_oracle_*.py):

* ``state_feature_table`` / ``expand_keys`` / ``expand_queries``: layout pinned
  by golden vectors written from the reference itself
  (tests/golden/make_golden.py -> tests/golden/*.npz) and by the invariant
  phi(q).phi(k) == (q.k)^2.
* ``attention``: brute-force fp64 loops of the closed form (independent code),
  special cases (ungated deg=2 -> s^2 weights), golden vectors.
* ``update_state``: definition S = sum_t phi(k_t) v_t^T by explicit loops,
  golden vectors.
* ``discumsum``: closed form of the linear recurrence, log_G = 0 -> exclusive
  cumsum, golden vectors.
* ``query_state``: gamma/alpha independence, limits (no attention part; zero
  state), golden vectors.
* ``power_retention``: O(t^2) fp64 closed form, chunked == quadratic, golden
  vectors.
* ``power_retention_inference``: state-parity invariant, decode == closed form
  over the full history, golden vectors.
"""
from .power_retention_oracle import (  # noqa: F401
    expanded_dim,
    state_feature_table,
    expand_keys,
    expand_queries,
    attention,
    update_state,
    discumsum,
    query_state,
    power_retention,
    power_retention_inference,
)
