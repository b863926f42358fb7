"""The training step of the fused node inside a HIP graph: the node forks its backward onto a second stream and joins
it again with events, so a capture has to take both streams in and a replay has to reproduce the eager step exactly.
(Replayed several times with the process's own eager work and synchronisations in between, every replay checked.)"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def pra():
    import retention_integration_amd as pra
    return pra


@pytest.mark.parametrize("b,t,h,r,d,chunk,gated", [(1, 2048, 2, 1, 64, 256, True), (2, 512, 2, 2, 32, 128, False)])
def test_training_step_captured_in_a_graph_replays_the_eager_step(pra, b, t, h, r, d, chunk, gated):
    g = torch.Generator(device=DEV).manual_seed(5)
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV).bfloat16()  # noqa: E731
    Q, K, V = mk(b, t, h * r, d).requires_grad_(True), mk(b, t, h, d).requires_grad_(True), mk(b, t, h, d).requires_grad_(True)
    lg = torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g, device=DEV)).requires_grad_(True) if gated else None
    dO = mk(b, t, h * r, d)
    leaves = [x for x in (Q, K, V, lg) if x is not None]

    def step():
        Y = pra.power_retention(Q, K, V, lg, deg=2, chunk_size=chunk)
        grads = torch.autograd.grad(Y, leaves, dO)
        return (Y,) + grads

    # warm-up on a side stream, as a capture wants it (allocator pools, the node's second stream)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for trial in range(3):
        with torch.no_grad():      # new inputs in the captured tensors
            for x in (Q, K, V, dO):
                x.copy_(mk(*x.shape))
            if gated:
                lg.copy_(torch.nn.functional.logsigmoid(torch.randn(b, t, h, generator=g, device=DEV)))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = step()              # the same step, eager, between two replays
        torch.cuda.synchronize()
        for nm, a, w in zip(["Y", "dQ", "dK", "dV", "dlog_G"], got, want):
            assert torch.isfinite(a.float()).all(), f"replay {trial}: {nm} is not finite"
            assert torch.equal(a, w), f"replay {trial}: {nm} differs from the eager step"
