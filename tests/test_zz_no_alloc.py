"""pr_decode_step_noalloc -- the single-token step whose partial sums live in the library's own per-GPU array --
against pr_decode_step with a caller's workspace, through the C ABI: same kernels, so every output must be equal bit
for bit.  Two calls in a row share the array, the second on a smaller input (fewer sequences, fewer slices): stale
partial sums of the first call must not leak into it.  (Collected last: a failure here must not hide other tests.)"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(lib, _lib, B, h, r, tq, d, dtype, mode, seed):
    """Runs both entry points on the same inputs (out of place and in place) and compares."""
    p, st = _lib.ptr, _lib.stream()
    code = _lib.dtype_code(dtype)
    D = lib.pr_expanded_dim(d, 2)
    g = torch.Generator().manual_seed(seed)
    hq = h * r
    S = (torch.randn(B, h, D, d, generator=g) * 0.3).to(dtype).to(DEV)
    s = (torch.rand(B, h, D, generator=g) + 0.5).to(DEV)
    Q = torch.randn(B, tq, hq, d, generator=g).to(dtype).to(DEV)
    K, V = (torch.randn(B, h, d, generator=g).to(dtype).to(DEV) for _ in range(2))
    lg = torch.nn.functional.logsigmoid(torch.randn(B, h, generator=g)).to(DEV)
    Ya = torch.randn(B, tq, hq, d, generator=g).to(dtype).to(DEV)
    la = (torch.rand(B, tq, hq, generator=g) + 0.5).to(DEV)
    rm = torch.randn(B, tq, hq, generator=g).to(DEV)
    scale_p = 1.0 / d
    if mode == "new":       # query + fold of the new token, which attends to itself
        att, new, attend = (None, None, None), (K, V, lg), 1
    elif mode == "cache":   # query only, merged with an attention part
        att, new, attend = (Ya, la, rm), (None, None, None), 0
    else:                   # fold with a separate attention part
        att, new, attend = (Ya, la, rm), (K, V, lg), 0
    upd = new[0] is not None

    def run(noalloc):
        S_out, s_out = (torch.empty_like(S), torch.empty_like(s)) if upd else (None, None)
        out = torch.empty_like(Q)
        head = (p(Q), p(lg), p(S), p(s), p(att[0]), p(att[1]), p(att[2]), p(new[0]), p(new[1]), p(new[2]), p(S_out),
                p(s_out), p(out))
        tail = (B, tq, h, r, d, scale_p, 2, code, attend, st)
        if noalloc:
            _lib.check(lib.pr_decode_step_noalloc(*head, *tail), "decode_step_noalloc")
        else:
            ws = torch.empty(lib.pr_decode_step_workspace(B, tq, h, r, d), dtype=torch.uint8, device=DEV)
            _lib.check(lib.pr_decode_step(*head, p(ws), *tail), "decode_step")
        torch.cuda.synchronize()
        return out, S_out, s_out

    want = run(False)
    got = run(True)
    for nm, a, b in zip(("out", "S_out", "s_out"), got, want):
        if b is not None:
            assert torch.isfinite(a.float()).all(), nm
            assert torch.equal(a, b), f"{nm} differs (B={B} h={h} r={r} tq={tq} d={d} {mode})"


def test_noalloc_decode_step_equals_the_workspace_form_on_two_calls_in_a_row():
    from retention_integration_amd import _lib
    lib = _lib.load()
    assert lib.pr_decode_step_noalloc_max_workspace() == 8 << 20
    mem0 = torch.cuda.memory_allocated()
    # big first (16 pairs x 16 slices x 4 rows), then smaller inputs that reuse the front of the array
    _case(lib, _lib, 8, 2, 2, 2, 64, torch.bfloat16, "cache", 1)
    _case(lib, _lib, 3, 2, 2, 1, 64, torch.bfloat16, "new", 2)
    _case(lib, _lib, 2, 1, 1, 1, 128, torch.float16, "both", 3)
    _case(lib, _lib, 5, 3, 4, 2, 32, torch.bfloat16, "cache", 4)      # 8 query rows
    _case(lib, _lib, 32, 8, 1, 1, 64, torch.bfloat16, "new", 5)       # one workgroup per pair: no partial sums at all
    assert torch.cuda.memory_allocated() == mem0


def test_noalloc_decode_step_refuses_what_does_not_fit():
    from retention_integration_amd import _lib
    lib = _lib.load()
    # up to 1024 slices x 8 rows x 129 floats x 4 B = 4.2 MB always fits; 2200 (batch, kv head) pairs with 8 query rows
    # each at d = 128 need 9.1 MB
    B, h, r, tq, d = 1100, 2, 8, 1, 128
    assert lib.pr_decode_step_workspace(B, tq, h, r, d) > lib.pr_decode_step_noalloc_max_workspace()
    x = torch.zeros(64, device=DEV)
    rc = lib.pr_decode_step_noalloc(x.data_ptr(), None, x.data_ptr(), x.data_ptr(), None, None, None, None, None, None,
                                    None, None, x.data_ptr(), B, tq, h, r, d, 1.0 / d, 2, 0, 0, _lib.stream())
    assert rc == -3 and b"partial sums" in lib.pr_last_error()


def test_noalloc_decode_step_captured_in_a_hip_graph_replays_bit_for_bit():
    """The entry point is meant for callers under stream capture: after the set-up call (which takes the array's
    address on this GPU) a recurrent step is captured, and every replay -- with eager work and synchronisations in
    between -- must give the eager result of the same step bit for bit (state updated in place, so each replay is
    compared with an eager step from the same starting state)."""
    from retention_integration_amd import _lib
    lib = _lib.load()
    assert lib.pr_decode_step_noalloc_max_workspace() == 8 << 20   # set-up call: resolves the array on this GPU
    p = _lib.ptr
    B, h, r, d, dtype = 4, 2, 2, 64, torch.bfloat16
    code = _lib.dtype_code(dtype)
    D = lib.pr_expanded_dim(d, 2)
    g = torch.Generator().manual_seed(11)
    S0 = (torch.randn(B, h, D, d, generator=g) * 0.3).to(dtype).to(DEV)
    s0 = (torch.rand(B, h, D, generator=g) + 0.5).to(DEV)
    Q = torch.randn(B, 1, h * r, d, generator=g).to(dtype).to(DEV)
    K, V = (torch.randn(B, h, d, generator=g).to(dtype).to(DEV) for _ in range(2))
    lg = torch.nn.functional.logsigmoid(torch.randn(B, h, generator=g)).to(DEV)

    def step(S, s, out, stream, noalloc):
        head = (p(Q), p(lg), p(S), p(s), None, None, None, p(K), p(V), p(lg), p(S), p(s), p(out))
        tail = (B, 1, h, r, d, 1.0 / d, 2, code, 1, stream)
        if noalloc:
            _lib.check(lib.pr_decode_step_noalloc(*head, *tail), "decode_step_noalloc")
        else:
            ws = torch.empty(lib.pr_decode_step_workspace(B, 1, h, r, d), dtype=torch.uint8, device=DEV)
            _lib.check(lib.pr_decode_step(*head, p(ws), *tail), "decode_step")

    # eager trajectory of three steps with the workspace form
    S, s = S0.clone(), s0.clone()
    want = []
    for _ in range(3):
        out = torch.empty_like(Q)
        step(S, s, out, _lib.stream(), False)
        torch.cuda.synchronize()
        want.append((out.clone(), S.clone(), s.clone()))

    Sg, sg, outg = S0.clone(), s0.clone(), torch.empty_like(Q)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(Sg, sg, outg, side.cuda_stream, True)   # warm-up on the capture stream
        torch.cuda.synchronize()
        Sg.copy_(S0)
        sg.copy_(s0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        step(Sg, sg, outg, torch.cuda.current_stream().cuda_stream, True)
    for k in range(3):
        graph.replay()
        torch.cuda.synchronize()
        (torch.ones(1024, device=DEV) * 2).sum().item()   # eager work and a synchronisation between the replays
        assert torch.equal(outg, want[k][0]), f"replay {k}: out differs"
        assert torch.equal(Sg, want[k][1]) and torch.equal(sg, want[k][2]), f"replay {k}: state differs"
