"""The preallocated decode cache (RetentionCache) against the reference caller's sequence -- concatenate, call
power_retention_inference with the whole cache, clear at the switch-over
(ref: deploy/models/powercoder/modeling_powercoder.py:161-196, kvgs_dynamic_cache.py:131-172) -- run through the
maker-assembled function and through the CPU oracle; and the recurrent step captured in a HIP graph."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"
OUT_TOL = 1e-2


def rel_l2(got, want):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def check(name, got, want, tol=OUT_TOL):
    e = rel_l2(got, want)
    print(f"  {name}: rel-L2 {e:.3e}", flush=True)
    assert torch.isfinite(got.float()).all() and e <= tol, f"{name}: rel-L2 {e:.3e} > {tol}"


def tokens(b, n, h, r, d, dtype, seed, gated=True):
    g = torch.Generator().manual_seed(seed)
    std = 0.5 if dtype == torch.float16 else 1.0
    q = (torch.randn(n, b, 1, h * r, d, generator=g) * std).to(dtype)
    k = (torch.randn(n, b, 1, h, d, generator=g) * std).to(dtype)
    v = (torch.randn(n, b, 1, h, d, generator=g) * std).to(dtype)
    lg = torch.nn.functional.logsigmoid(torch.randn(n, b, 1, h, generator=g) + 2.0) if gated else None
    return q, k, v, lg


@pytest.mark.parametrize("dtype,b,h,r,d,sw,gated", [
    (torch.bfloat16, 3, 2, 2, 64, 8, True),      # several switch-overs in 30 steps
    (torch.float16, 2, 2, 1, 128, 5, True),
    (torch.bfloat16, 2, 1, 4, 32, 7, False),     # no gates
    (torch.bfloat16, 2, 2, 8, 64, 6, True),      # 8 query heads per kv head
    (torch.bfloat16, 1, 2, 16, 32, 6, True),     # 16: still one pass over the state
    (torch.bfloat16, 1, 1, 24, 32, 6, True),     # 24: the state query runs as the operator over the same buffers
])
def test_cache_step_follows_the_reference_callers_sequence(dtype, b, h, r, d, sw, gated):
    """30 tokens through RetentionCache.step and through the caller's loop over the maker-assembled function and over
    the oracle: growing cache without a state, compression at the switch-over, growing cache on top of a state, the
    next switch-over (state decayed and updated) -- every output, and the final state."""
    import retention_integration_amd as pra
    n = 30
    q, k, v, lg = tokens(b, n, h, r, d, dtype, seed=3 + d, gated=gated)
    cache = pra.RetentionCache(b, h, d, capacity=sw, dtype=dtype, device=DEV, q_heads=h * r)
    # the caller's loop, on the GPU (composed function) and on the CPU (oracle, fp32)
    Kc = Vc = Gc = None
    S = s = None
    Ko = Vo = Go = None
    So = so = None
    cat = lambda a, x: x if a is None else torch.cat([a, x], 1)  # noqa: E731
    for i in range(n):
        gi = None if lg is None else lg[i]
        out = cache.step(q[i].to(DEV), k[i].to(DEV), v[i].to(DEV), None if gi is None else gi.to(DEV),
                         switch_over_seq_len=sw).clone()
        Kc, Vc = cat(Kc, k[i].to(DEV)), cat(Vc, v[i].to(DEV))
        Gc = None if gi is None else cat(Gc, gi.to(DEV))
        Y, S2, s2 = pra.power_retention_inference_composed(q[i].to(DEV), Kc, Vc, Gc, S, s, deg=2, switch_over_seq_len=sw)
        Ko, Vo = cat(Ko, k[i].float()), cat(Vo, v[i].float())
        Go = None if gi is None else cat(Go, gi)
        Yo, So2, so2 = oracle.power_retention_inference(q[i].float(), Ko, Vo, Go, So, so, deg=2, switch_over_seq_len=sw)
        check(f"step {i} vs composed", out, Y, 6e-3)
        check(f"step {i} vs oracle", out, Yo)
        if Kc.shape[1] >= sw:      # the caller's clean_kv + update_state
            Kc = Vc = Gc = Ko = Vo = Go = None
            S, s, So, so = S2, s2, So2, so2
            assert cache.get_seq_length() == 0 and cache.has_state
            check(f"state after step {i} vs oracle", cache.state, So)
            check(f"sum_of_keys after step {i} vs oracle", cache.sum_of_keys, so)
        else:
            assert cache.get_seq_length() == Kc.shape[1]


def test_update_kv_appends_in_place_and_accumulates_the_gates():
    import retention_integration_amd as pra
    b, h, d = 2, 3, 64
    cache = pra.RetentionCache(b, h, d, capacity=16, device=DEV)
    g = torch.Generator().manual_seed(0)
    ks, vs, gs = [], [], []
    ptr0 = cache.keys.data_ptr()
    for t_new in (1, 3, 1, 5):
        k = torch.randn(b, t_new, h, d, generator=g).to(torch.bfloat16).to(DEV)
        v = torch.randn(b, t_new, h, d, generator=g).to(torch.bfloat16).to(DEV)
        lg = torch.nn.functional.logsigmoid(torch.randn(b, t_new, h, generator=g)).to(DEV)
        K, V, A, S, s = cache.update_kv(k, v, lg)
        ks.append(k); vs.append(v); gs.append(lg)
        assert S is None and s is None and K.data_ptr() == ptr0
        assert torch.equal(K, torch.cat(ks, 1)) and torch.equal(V, torch.cat(vs, 1))
        torch.testing.assert_close(A, torch.cat(gs, 1).cumsum(1), rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        cache.update_kv(torch.zeros(b, 7, h, d, dtype=torch.bfloat16, device=DEV),
                        torch.zeros(b, 7, h, d, dtype=torch.bfloat16, device=DEV), None)


def test_recurrent_steps_captured_in_a_hip_graph_equal_the_eager_loop():
    """64 recurrent steps (switch_over_seq_len = 1: every token folded, state updated in place) captured as ONE graph and
    replayed three times, with eager work and synchronisations between the replays: outputs and final state equal the
    eager loop bit for bit on every replay."""
    import retention_integration_amd as pra
    b, h, r, d, n = 32, 8, 1, 64, 64
    q, k, v, lg = (x.to(DEV) for x in tokens(b, n, h, r, d, torch.bfloat16, seed=11))
    g = torch.Generator().manual_seed(1)
    S0 = (torch.randn(b, h, pra.expanded_dim(d), d, generator=g) * 0.3).to(torch.bfloat16).to(DEV)
    s0 = (torch.rand(b, h, pra.expanded_dim(d), generator=g) + 0.5).to(DEV)
    cache = pra.RetentionCache(b, h, d, capacity=4, device=DEV)
    outs = torch.empty(n, b, 1, h * r, d, dtype=torch.bfloat16, device=DEV)

    def run():
        for i in range(n):
            cache.step(q[i], k[i], v[i], lg[i], switch_over_seq_len=1, out=outs[i])

    cache.update_state(S0, s0)
    run()
    torch.cuda.synchronize()
    want = (outs.clone(), cache.state.clone(), cache.sum_of_keys.clone())

    cache.update_state(S0, s0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    cache.update_state(S0, s0)
    with torch.cuda.graph(graph):
        run()
    for replay in range(3):
        cache.update_state(S0, s0)              # eager work between the replays
        outs.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(outs, want[0]), f"replay {replay}: outputs differ from the eager loop"
        assert torch.equal(cache.state, want[1]) and torch.equal(cache.sum_of_keys, want[2]), f"replay {replay}: state"
