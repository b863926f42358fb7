"""Host-side behaviour that needs no GPU: the conditions that must raise before anything is launched
(ref: retention/power_retention_maker.py:98-114, retention/_update_state/triton.py:310-311)."""
import pytest
import torch

import retention_integration_amd as pra


def _cpu_inputs(b=1, t=64, h=2, r=1, d=32):
    g = torch.Generator().manual_seed(0)
    Q = torch.randn(b, t, h * r, d, generator=g).to(torch.bfloat16)
    K, V = (torch.randn(b, t, h, d, generator=g).to(torch.bfloat16) for _ in range(2))
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g))
    return Q, K, V, lg


@pytest.mark.parametrize("fn", [pra.power_retention, pra.power_retention_composed])
def test_chunked_path_refuses_degrees_without_a_state_layout_before_any_launch(fn):
    """CPU tensors: reaching a kernel would fail differently, so NotImplementedError proves the refusal comes first."""
    Q, K, V, lg = _cpu_inputs()
    with pytest.raises(NotImplementedError):
        fn(Q, K, V, lg, deg=4, chunk_size=16)
    with pytest.raises(NotImplementedError):
        fn(Q, K, V, lg, deg=4, chunk_size=None, return_final_state=True)


@pytest.mark.parametrize("fn", [pra.power_retention, pra.power_retention_composed])
def test_argument_checks_of_the_composed_function(fn):
    Q, K, V, lg = _cpu_inputs()
    with pytest.raises(AssertionError):
        fn(Q, K, V, lg, deg=3, chunk_size=16)                       # odd degree
    with pytest.raises(AssertionError):
        fn(Q, K.float(), V, lg, deg=2, chunk_size=16)               # dtypes differ
    with pytest.raises(AssertionError):
        fn(Q[:, :, :1].repeat(1, 1, 3, 1), K, V, lg, deg=2, chunk_size=16)   # 3 query heads over 2 kv heads
    with pytest.raises(AssertionError):
        fn(Q, K, V, lg, deg=2, chunk_size=16, initial_state=torch.zeros(1, 2, 768, 32))   # not the (S, s) pair


def test_fused_chunked_node_refuses_degree_4_itself():
    from retention_integration_amd.fused import chunked_power_retention
    Q, K, V, lg = _cpu_inputs()
    with pytest.raises(NotImplementedError):
        chunked_power_retention(Q, K, V, lg, 4, 0.125, 16)


def test_operators_refuse_degree_4_state():
    Q, K, V, _ = _cpu_inputs()
    with pytest.raises(NotImplementedError):
        pra.update_state(K.view(1, 4, 16, 2, 32), V.view(1, 4, 16, 2, 32), 4)
    with pytest.raises(NotImplementedError):
        pra.query_state(Q.view(1, 4, 16, 2, 32), None, None, None, None, None, 4, 0.125, True)


class _RecordingLibrary:
    """Stands in for the shared library: every entry point returns success and is recorded, so the cache layer's
    bookkeeping (ref: deploy/models/powercoder/kvgs_dynamic_cache.py:111-172) can be exercised without a GPU."""

    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def entry(*args):
            self.calls.append((name, args))
            return 16 if name.endswith("_workspace") else 0
        return entry


@pytest.fixture
def cpu_cache(monkeypatch):
    from retention_integration_amd import _lib
    lib = _RecordingLibrary()
    monkeypatch.setattr(_lib, "load", lambda: lib)
    monkeypatch.setattr(_lib, "stream", lambda: None)
    cache = pra.RetentionCache(batch=2, kv_heads=2, head_dim=32, capacity=4, dtype=torch.bfloat16, device="cpu", q_heads=4)
    return cache, lib


def test_cache_layer_bookkeeping(cpu_cache):
    cache, lib = cpu_cache
    k = torch.zeros(2, 3, 2, 32, dtype=torch.bfloat16)
    g = torch.zeros(2, 3, 2)
    keys, values, gates, state, sk = cache.update_kv(k, k, g)
    assert cache.get_seq_length() == 3 and keys.shape == (2, 3, 2, 32) and gates.shape == (2, 3, 2)
    assert state is None and sk is None
    name, args = lib.calls[-1]
    assert name == "pr_cache_append" and args[7:14] == (2, 4, 0, 3, 2, 32, 0)   # B, capacity, pos, t_new, h, d, bf16
    with pytest.raises(ValueError):                       # 3 + 3 tokens do not fit a capacity of 4
        cache.update_kv(k, k, g)
    assert cache.get_seq_length() == 3
    with pytest.raises(AssertionError):                   # the cache holds bf16
        cache.update_kv(k[:, :1].half(), k[:, :1].half(), g[:, :1])
    cache.update_kv(k[:, :1], k[:, :1], None)             # ungated append at position 3
    assert lib.calls[-1][1][9] == 3 and cache.get_seq_length() == 4
    cache.clean_kv()
    assert cache.get_seq_length() == 0 and not cache.has_state
    S = torch.ones_like(cache.state)
    cache.update_state(S, torch.ones_like(cache.sum_of_keys))
    assert cache.has_state and torch.equal(cache.state, S)
    assert cache.update_kv(k[:, :1], k[:, :1], g[:, :1])[3] is cache.state
    cache.reset()
    assert cache.get_seq_length() == 0 and not cache.has_state and float(cache.state.abs().sum()) == 0.0


def test_cache_layer_takes_wide_query_groups_and_refuses_ragged_ones(monkeypatch):
    """Up to 16 query heads per kv head use the single-pass decode kernel, wider groups the operator chain (the
    reference's own lists go to 16: perf/tests/test_list.py:189-218); a head count that is no multiple is refused."""
    from retention_integration_amd import _lib
    monkeypatch.setattr(_lib, "load", lambda: _RecordingLibrary())
    assert pra.RetentionCache(batch=1, kv_heads=1, head_dim=32, capacity=4, device="cpu", q_heads=16)._fused_step
    assert not pra.RetentionCache(batch=1, kv_heads=1, head_dim=32, capacity=4, device="cpu", q_heads=24)._fused_step
    with pytest.raises(AssertionError):
        pra.RetentionCache(batch=1, kv_heads=2, head_dim=32, capacity=4, device="cpu", q_heads=5)
