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
