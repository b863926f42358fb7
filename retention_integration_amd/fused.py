"""The chunked power-retention path as ONE autograd node over the HIP library.

Same arithmetic as composing the four operators through ``make_power_retention``
(ref: retention/power_retention_maker.py:142-197), but the glue between the operators (chunk-local
cumsum of the gates, key discounting, query gating, and their gradients) runs inside fused HIP kernels
instead of a dozen elementwise launches, and only the first n entries of the scans are produced.

Forward and backward are ``torch.library.custom_op``s (``pr::chunked_fwd`` / ``pr::chunked_bwd``) with fake
implementations, like the per-kernel operators (the convention of the reference's CUDA wrappers,
ref: retention/_attention/cuda.py:10-43,129-245), so the node survives ``torch.compile`` without a graph break.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib
from .ops import expanded_dim


# The state kernels chained with the scan over the chunk axis (short chunks, many batch elements x heads).
# None: where the library says it is the faster form; True: wherever the shape allows it; False: never.
CHAIN = None


def _chained(lib, b, n, c, h, r, d):
    if CHAIN is False:
        return False
    return lib.pr_state_chain_supported(b, n, c, h, r, d) >= (1 if CHAIN else 2)


# The two kernels of the attention backward (key side, query side) read the same Q, K, V, dO of every (chunk, head) and
# deal their workgroups to the XCDs pair by pair in the same order: launched side by side on two streams of the same
# priority they share those rows in L2 instead of fetching them twice (12 us of a training step at the headline shape).
ATTN_BWD_TWO_STREAMS = True
# Forward: the attention kernel needs only the gate sums, so it runs next to  key discount -> chunk states -> scan.
FWD_TWO_STREAMS = True
# The same for the whole query side of the backward: the query gradient through the state depends only on the
# row-wise preparation, so it can run next to the chain  dS -> reverse scan -> dK, dV  instead of in front of it.
BWD_TWO_STREAMS = True
# Forward: attention inside the chunks, the query of the scanned states and their merge as one kernel where the library
# has it (pr_chunk_fwd_supported); False runs the attention kernel and the state query with its merge epilogue.
ONE_KERNEL_FWD = True
# Backward, query side: the query gradient through the state and the query side of the attention backward as one kernel
# where the library has it (pr_chunk_bwd_dq_supported); False runs sympow_grad and then the attention kernel, which adds
# the former's result in its epilogue.
ONE_KERNEL_BWD_DQ = True
_SIDE = {}


def _side_stream(device):
    key = str(device)
    if key not in _SIDE:
        _SIDE[key] = torch.cuda.Stream(device=device)
    return _SIDE[key]


def _follows_gates(lib, d, deg, code):
    """True when both readers of the scanned chunk states are the one-kernel ones, which take a chunk's own sum in
    place of the scan's entry wherever the gates make the two equal (and gate skipping is on)."""
    return bool(ONE_KERNEL_FWD and ONE_KERNEL_BWD_DQ and lib.pr_get_gate_skipping()
                and lib.pr_chunk_fwd_supported(d, deg, code) and lib.pr_chunk_bwd_dq_supported(d, deg, code))


def _empty(shape, dtype, device):
    return torch.empty(shape, dtype=dtype, device=device)


@torch.library.custom_op("pr::chunked_fwd", mutates_args=(), device_types="cuda")
def chunked_fwd(Q: Tensor, K: Tensor, V: Tensor, log_G: Optional[Tensor], deg: int, scale: float, c: int,
                S0: Optional[Tensor] = None, s0: Optional[Tensor] = None, want_final: bool = False
                ) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor,
                           Tensor]:
    """-> O, what the backward needs: A, lcs, Kd (empty when ungated), Sc, sc, rowmax, den, the state after the
    last token (Sf [b,h,D,d], sf [b,h,D]; empty unless want_final), and for the backward again the rows of every chunk
    that the gates have not decayed to exact zeros (live [BN,h,2] int32; empty when ungated) and the per-chunk sums S, s
    that the scan turned into Sc, sc (empty unless the readers of Sc, sc follow the gates, see below).

    S0 [b,h,D,d], s0 [b,h,D] fp32: the state the sequence starts from (the pair a previous call returned), in the
    reference layout; chunk k then sees it decayed by the gates of chunks 0..k-1 like any chunk state, and the final
    state is the scan's entry n (ref: retention/power_retention_maker.py:131-140,158-172 carries a state of the same
    shape but returns the one at the START of the last chunk and leaves the carried one undecayed).

    The gated queries Q * exp(A / deg) (ref: retention/power_retention_maker.py:183-186) are never formed: the state part
    is homogeneous of degree deg in the query, so the gate is a per-row factor exp(A) on it, applied where the state
    part is merged with the attention part (and, in the backward, in the per-row factor of dO)."""
    lib = _lib.load()
    st = _lib.stream()
    b, t, hq, d = Q.shape
    h = K.shape[2]
    r = hq // h
    n = t // c
    BN = b * n
    dev, dt = Q.device, Q.dtype
    code = _lib.dtype_code(dt)
    f32 = torch.float32
    gated = log_G is not None
    carried = S0 is not None
    p = _lib.ptr
    chained = _chained(lib, b, n, c, h, 1, d) and not carried and not want_final
    D = expanded_dim(d)

    if gated:
        A, lcs = _empty((BN, c, h), f32, dev), _empty((BN, h), f32, dev)
        Kd = torch.empty_like(K)
        live = _empty((BN, h, 2), torch.int32, dev)
        # (the sums first: the attention kernel needs nothing else; the discounted keys follow below)
        _lib.check(lib.pr_chunk_prep_fwd(p(log_G), p(K), p(Q), p(A), p(lcs), None, None, p(live), BN, c, h, r, d, deg,
                                         code, st), "chunk_prep_fwd(sums)")
        Kd_ = Kd
    else:
        A, Kd = _empty((0,), f32, dev), _empty((0,), dt, dev)
        live = _empty((0,), torch.int32, dev)
        Kd_ = K
        lcs = torch.zeros((BN, h), dtype=f32, device=dev)

    one_kernel = ONE_KERNEL_FWD and bool(lib.pr_chunk_fwd_supported(d, deg, code))
    rm = _empty((BN, c, hq), f32, dev)
    if not one_kernel:
        Ya, la = torch.empty_like(Q), _empty((BN, c, hq), f32, dev)

    def attention(stream):
        _lib.check(lib.pr_attention_fwd(p(Q), p(K), p(V), p(A) if gated else None, p(Ya), p(la), p(rm), BN, c, c, h, r,
                                        d, scale, deg, 0, code, stream), "attention_fwd")
    two_streams = FWD_TWO_STREAMS and not one_kernel
    if two_streams:
        main, side = torch.cuda.current_stream(), _side_stream(dev)
        side.wait_stream(main)
        attention(side.cuda_stream)

    if gated:
        # (every reader of Kd below and in the backward is handed `live`: its dead rows need not be written)
        _lib.check(lib.pr_chunk_prep_fwd(None, p(K), p(Q), p(A), p(lcs), p(Kd), None, None if chained else p(live), BN, c,
                                         h, r, d, deg, code, st), "chunk_prep_fwd(keys)")
    Sc, sc = _empty((BN, h, D, d), dt, dev), _empty((BN, h, D), f32, dev)
    Sf, sf = _empty((0,), dt, dev), _empty((0,), f32, dev)
    S, s = _empty((0,), dt, dev), _empty((0,), f32, dev)
    follow = False
    if chained:
        # short chunks: the chunk states are scanned as they are formed and never written on their own
        _lib.check(lib.pr_update_state_scan_fwd(p(Kd_), p(V), p(lcs) if gated else None, p(Sc), p(sc), b, n, c, h, d,
                                                deg, code, st), "update_state_scan_fwd")
    else:
        S, s = torch.empty_like(Sc), torch.empty_like(sc)
        # Where the gates let nothing through from one chunk to the next (exp(lcs) == 0), the scan's entry k IS the sum
        # of chunk k-1: the kernels that read a chunk's state then take that sum directly (they are handed both), and a
        # sequence of a head whose every carry is zero is not scanned at all.  Only with the one-kernel readers, which
        # know the rule, on both sides of the step.
        follow = bool(gated and not carried and not want_final and _follows_gates(lib, d, deg, code))
        # (the last chunk's own state is only needed for the state after the last token)
        # (... or when the sums themselves are handed to the backward: an output of the node holds no unwritten memory)
        _lib.check(lib.pr_update_state_fwd(p(Kd_), p(V), p(S), p(s), p(live) if gated else None, BN, c, h, d, deg,
                                           0 if want_final or follow else n, code, st), "update_state_fwd")
        s0f = s0.to(f32).contiguous() if carried else None
        if want_final:
            Sf, sf = _empty((b, h, D, d), dt, dev), _empty((b, h, D), f32, dev)
        # the carried state is the scan's starting value, the state after the last token its entry n
        _lib.check(lib.pr_state_scan_fwd(p(S), p(s), p(lcs), p(Sc), p(sc), p(S0) if carried else None, p(s0f),
                                         p(Sf) if want_final else None, p(sf) if want_final else None, b, n, n, h,
                                         D * d, D, 1 if follow else 0, code, st), "state_scan_fwd")
        if not follow:
            S, s = _empty((0,), dt, dev), _empty((0,), f32, dev)

    O, den = torch.empty_like(Q), _empty((BN, c, hq), f32, dev)
    if one_kernel:
        _lib.check(lib.pr_chunk_fwd(p(Q), p(K), p(V), p(A) if gated else None, p(Sc), p(sc), p(S) if follow else None,
                                    p(s) if follow else None, p(lcs) if follow else None, p(O), p(rm), p(den), BN, n,
                                    c, h, r, d, scale, deg, 0 if carried else 1, code, st), "chunk_fwd")
        return O, A, lcs, Kd, Sc, sc, rm, den, Sf, sf, live, S, s
    if two_streams:
        main.wait_stream(side)
    else:
        attention(st)
    _lib.check(lib.pr_query_state_fwd(p(Q), p(Sc), p(sc), p(Ya), p(la), p(rm), p(A) if gated else None, p(O), p(den),
                                      BN, n, c, h, r, d, scale ** deg, deg, 0 if carried else 1, 1, code, st),
               "query_state_fwd")
    return O, A, lcs, Kd, Sc, sc, rm, den, Sf, sf, live, S, s


@chunked_fwd.register_fake
def _(Q, K, V, log_G, deg, scale, c, S0=None, s0=None, want_final=False):
    b, t, hq, d = Q.shape
    h = K.shape[2]
    BN = b * (t // c)
    D = Dr = expanded_dim(d)
    f32 = torch.float32
    gated = log_G is not None
    lib = _lib.load()
    follow = bool(gated and S0 is None and not want_final and not _chained(lib, b, t // c, c, h, 1, d)
                  and _follows_gates(lib, d, deg, _lib.dtype_code(Q.dtype)))
    A = Q.new_empty((BN, c, h) if gated else (0,), dtype=f32)
    return (torch.empty_like(Q), A, Q.new_empty((BN, h), dtype=f32),
            torch.empty_like(K) if gated else K.new_empty((0,)),
            Q.new_empty((BN, h, D, d)), Q.new_empty((BN, h, D), dtype=f32), Q.new_empty((BN, c, hq), dtype=f32),
            Q.new_empty((BN, c, hq), dtype=f32),
            Q.new_empty((b, h, Dr, d) if want_final else (0,)), Q.new_empty((b, h, Dr) if want_final else (0,), dtype=f32),
            Q.new_empty((BN, h, 2) if gated else (0,), dtype=torch.int32),
            Q.new_empty((BN, h, D, d) if follow else (0,)), Q.new_empty((BN, h, D) if follow else (0,), dtype=f32))


@torch.library.custom_op("pr::chunked_bwd", mutates_args=(), device_types="cuda")
def chunked_bwd(Q: Tensor, K: Tensor, V: Tensor, A: Tensor, lcs: Tensor, Kd: Tensor, Sc: Tensor,
                sc: Tensor, rm: Tensor, O: Tensor, den: Tensor, dO: Tensor, deg: int, scale: float, c: int,
                gated: bool, carried: bool = False, dSf: Optional[Tensor] = None, dsf: Optional[Tensor] = None,
                live: Optional[Tensor] = None, S: Optional[Tensor] = None, s: Optional[Tensor] = None
                ) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> dQ, dK, dV, dlog_G (empty when ungated), and the gradient of the state the sequence started from
    (dS0 [b,h,D,d], ds0 [b,h,D]; empty unless carried).  dSf, dsf: gradient of the returned final state, or None.
    live: the forward's array of the rows that the gates left alive, or None.  S, s: the per-chunk sums, given when the
    forward's scan counted on readers that follow the gates (the backward then does the same, and must)."""
    if not gated:
        Kd = K
    qgate = _lib.ptr(A) if gated else None
    live_p = _lib.ptr(live) if gated and live is not None and live.numel() else None
    follow = S is not None and S.numel() > 0
    lib = _lib.load()
    st = _lib.stream()
    b, t, hq, d = Q.shape
    h = K.shape[2]
    r = hq // h
    n = t // c
    BN = b * n
    D = expanded_dim(d)
    dev, dt = Q.device, Q.dtype
    code = _lib.dtype_code(dt)
    f32, u8 = torch.float32, torch.uint8
    p = _lib.ptr
    dO = dO.contiguous()
    dQg = torch.empty_like(Q)
    # the attention part's output gradient is dO times a per-row factor: the attention backward applies it on the fly
    dla, dys = torch.empty_like(den), torch.empty_like(den)
    dS, ds = torch.empty_like(Sc), torch.empty_like(sc)
    dlcs = torch.empty_like(lcs)   # gate gradient of both scans
    dS0, ds0 = _empty((0,), dt, dev), _empty((0,), f32, dev)
    has_dfin = dSf is not None or dsf is not None
    two_streams = dq_one_kernel = False
    if not carried and not has_dfin and _chained(lib, b, n, c, h, r, d):
        ws = _empty((lib.pr_query_state_scan_bwd_workspace(b, n, c, h, r, d, code),), u8, dev)
        _lib.check(lib.pr_query_state_scan_bwd(p(Q), p(Sc), p(sc), p(rm), qgate, p(O), p(den), p(dO),
                                               p(lcs) if gated else None, p(dQg), p(dS), p(ds), None, p(dla), p(dys),
                                               p(dlcs) if gated else None, p(ws), b, n, c, h, r, d, scale ** deg, deg,
                                               code, st), "query_state_scan_bwd")
    else:
        dSc, dsc = torch.empty_like(Sc), torch.empty_like(sc)
        qws = _empty((lib.pr_query_state_bwd_workspace(BN, c, h, r, d, code),), u8, dev)
        zis = 0 if carried else 2   # (2 = chunk 0 sees no state and nobody wants its gradient; 0 = it sees the carried one)

        def qs_bwd(dQ_, dS_, ds_, prepared, stream):
            _lib.check(lib.pr_query_state_bwd(p(Q), p(Sc), p(sc), p(rm), qgate, p(O), p(den), p(dO), dQ_, dS_, ds_, None,
                                              p(dla), p(dys), p(qws), live_p, BN, n, c, h, r, d, scale ** deg, deg, zis,
                                              1, prepared, code, stream), "query_state_bwd")
        dq_one_kernel = ONE_KERNEL_BWD_DQ and bool(lib.pr_chunk_bwd_dq_supported(d, deg, code))
        if follow and not (dq_one_kernel and lib.pr_get_gate_skipping()):
            raise RuntimeError("the forward left out scans that this backward would read: keep ONE_KERNEL_BWD_DQ and "
                               "gate skipping as they were for the forward")
        dQa = torch.empty_like(Q)
        dGq = _empty((BN, c, hq), f32, dev) if gated else None

        def query_side(stream):
            # (the workspace of pr_query_state_bwd: the scaled dO, then the row vector of the key-sum term)
            cvec = qws.data_ptr() + (BN * c * hq * d * 2 + 255) // 256 * 256
            _lib.check(lib.pr_chunk_bwd_dq(p(Q), p(K), p(V), qgate, p(rm), p(den), p(dO), p(dla), p(dys), cvec, p(Sc),
                                           p(sc), p(S) if follow else None, p(s) if follow else None,
                                           p(lcs) if follow else None, p(dQa), p(dGq), BN, n, c, h, r, d, scale, deg,
                                           0 if carried else 1, code, stream), "chunk_bwd_dq")
        if dq_one_kernel:
            qs_bwd(None, p(dSc), p(dsc), 0, st)          # preparation and dS; the query side follows further down
            if not BWD_TWO_STREAMS:
                query_side(st)
        elif BWD_TWO_STREAMS:
            # The query gradient through the state (and, after it, the query side of the attention backward) depends
            # only on the row-wise preparation: it runs on a second stream next to the chain dS -> scan -> dK, dV.
            main, side = torch.cuda.current_stream(), _side_stream(dev)
            qs_bwd(None, None, None, 0, st)              # preparation only
            side.wait_stream(main)
            qs_bwd(p(dQg), None, None, 1, side.cuda_stream)
            qs_bwd(None, p(dSc), p(dsc), 1, st)
        else:
            qs_bwd(p(dQg), p(dSc), p(dsc), 0, st)
        dSf_ = dsf_ = None
        if has_dfin:   # the gradient that arrived through the returned final state enters the reverse scan as entry n
            dSf_ = (dSf if dSf is not None else torch.zeros((b, h, D, d), dtype=dt, device=dev)).contiguous()
            dsf_ = (dsf.to(f32) if dsf is not None else torch.zeros((b, h, D), dtype=f32, device=dev)).contiguous()
        if carried:
            dS0, ds0 = _empty((b, h, D, d), dt, dev), _empty((b, h, D), f32, dev)
        sws = _empty((lib.pr_state_scan_bwd_workspace(b, n, h, D * d, D),), u8, dev)
        _lib.check(lib.pr_state_scan_bwd(p(dSc), p(Sc), p(dsc), p(sc), p(lcs), p(dS), p(ds), p(dlcs), p(sws), p(dSf_),
                                         p(dsf_), p(dS0) if carried else None, p(ds0) if carried else None, b, n, n, h,
                                         D * d, D, 1 if follow else 0, code, st), "state_scan_bwd")
        two_streams = BWD_TWO_STREAMS
    dKd, dVs = torch.empty_like(K), torch.empty_like(V)
    # (where the reverse scan lets nothing through, its entry k IS its input entry k + 1: the kernels are handed both)
    scan_in = (p(dSc), p(dsc), p(lcs)) if follow else (None, None, None)
    # (dS comes from the kernels above, so both orders of a pair hold the same sum: the symmetry flag says so; the last
    # chunk's dS is zero unless a gradient arrived through the final state)
    if two_streams and dq_one_kernel:
        # The one-kernel query side needs only the row-wise preparation, so where it runs is a matter of what it runs
        # beside: started after dV, next to dK and the key side of the attention backward, the step is 15-25 us shorter
        # than with it next to dS and the reverse scan (measured at every point of the chain).
        def usb(dk_, dv_):
            _lib.check(lib.pr_update_state_bwd(p(Kd), p(V), p(dS), p(ds), *scan_in, live_p, dk_, dv_, BN, c, h, d, deg, 1,
                                               0 if has_dfin else n, code, st), "update_state_bwd")
        main, side = torch.cuda.current_stream(), _side_stream(dev)
        usb(None, p(dVs))
        side.wait_stream(main)
        query_side(side.cuda_stream)
        usb(p(dKd), None)
    else:
        _lib.check(lib.pr_update_state_bwd(p(Kd), p(V), p(dS), p(ds), *scan_in, live_p, p(dKd), p(dVs), BN, c, h, d, deg,
                                           1, 0 if has_dfin else n, code, st), "update_state_bwd")

    # the attention backward adds the state-path gradients in its epilogue and writes the final dQ, dK, dV
    dKa, dVa = torch.empty_like(K), torch.empty_like(V)
    if not dq_one_kernel:
        dQa = torch.empty_like(Q)
        dGq = _empty((BN, c, hq), f32, dev) if gated else None
    dGk = _empty((b, t, h), f32, dev) if gated else None
    dotk = _empty((BN, c, h), f32, dev) if gated else None
    Ag = p(A) if gated else None
    if dq_one_kernel:
        # the query side is done (or running on the second stream): the key side alone
        _lib.check(lib.pr_chunk_attention_bwd(p(Q), p(K), p(V), Ag, p(rm), p(dO), p(dla), p(dys), None, p(dKd), p(dVs),
                                              live_p, None, p(dKa), p(dVa), None, p(dGk), p(dotk), BN, c, h, r, d, scale, deg, 1,
                                              code, st), "chunk_attention_bwd(dK, dV)")
        if two_streams:
            torch.cuda.current_stream().wait_stream(_side_stream(dev))
    elif two_streams or ATTN_BWD_TWO_STREAMS:
        # the key side on the launch stream, the query side next to it on the second stream (which, with
        # BWD_TWO_STREAMS, already holds the state part of the query gradient)
        main, side = torch.cuda.current_stream(), _side_stream(dev)
        if not two_streams:
            side.wait_stream(main)
        _lib.check(lib.pr_chunk_attention_bwd(p(Q), p(K), p(V), Ag, p(rm), p(dO), p(dla), p(dys), p(dQg), None, None,
                                              None, p(dQa), None, None, p(dGq), None, None, BN, c, h, r, d, scale, deg, 1,
                                              code, side.cuda_stream), "chunk_attention_bwd(dQ)")
        _lib.check(lib.pr_chunk_attention_bwd(p(Q), p(K), p(V), Ag, p(rm), p(dO), p(dla), p(dys), None, p(dKd), p(dVs),
                                              live_p, None, p(dKa), p(dVa), None, p(dGk), p(dotk), BN, c, h, r, d, scale, deg, 1,
                                              code, st), "chunk_attention_bwd(dK, dV)")
        main.wait_stream(side)
    else:
        _lib.check(lib.pr_chunk_attention_bwd(p(Q), p(K), p(V), Ag, p(rm), p(dO), p(dla), p(dys), p(dQg), p(dKd),
                                              p(dVs), live_p, p(dQa), p(dKa), p(dVa), p(dGq), p(dGk), p(dotk), BN, c, h, r, d,
                                              scale, deg, 1, code, st), "chunk_attention_bwd")
    dlg = _empty((0,), f32, dev)
    if gated:
        dlg = dGk
        _lib.check(lib.pr_chunk_gate_scan_bwd(p(dlg), p(dGq), p(dotk), p(dlcs), None, BN, c, h, r, deg, st),
                   "chunk_gate_scan_bwd")
    return dQa, dKa, dVa, dlg, dS0, ds0


@chunked_bwd.register_fake
def _(Q, K, V, A, lcs, Kd, Sc, sc, rm, O, den, dO, deg, scale, c, gated, carried=False, dSf=None, dsf=None, live=None,
      S=None, s=None):
    b, t, _, d = Q.shape
    h = K.shape[2]
    Dr = expanded_dim(d)
    return (torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V),
            Q.new_empty((b, t, h) if gated else (0,), dtype=torch.float32),
            Q.new_empty((b, h, Dr, d) if carried else (0,)),
            Q.new_empty((b, h, Dr) if carried else (0,), dtype=torch.float32))


def _chunked_setup(ctx, inputs, output):
    Q, K, V, log_G, deg, scale, c, S0, s0, want_final = inputs
    O, A, lcs, Kd, Sc, sc, rm, den, Sf, sf, live, S, s = output
    ctx.save_for_backward(Q, K, V, A, lcs, Kd, Sc, sc, rm, O, den, live, S, s)
    ctx.meta = (deg, scale, c, log_G is not None, S0 is not None, None if s0 is None else s0.dtype, bool(want_final),
                int(_lib.load().pr_get_gate_skipping()))
    ctx.set_materialize_grads(False)


def _chunked_backward(ctx, dO, dA, dlcs, dKd, dSc, dsc, drm, dden, dSf, dsf, dlive, dS_, ds_):
    Q, K, V, A, lcs, Kd, Sc, sc, rm, O, den, live, S, s = ctx.saved_tensors
    deg, scale, c, gated, carried, s0_dtype, want_final, skipping = ctx.meta
    if gated and skipping != int(_lib.load().pr_get_gate_skipping()):
        # (with skipping on, the forward leaves unwritten what its own readers leave out -- dead rows of the discounted
        # keys, scans that nothing survives -- and a backward with skipping off would read them)
        raise RuntimeError("gate skipping was switched between this forward and its backward (pr_set_gate_skipping): "
                           "keep the setting for the whole step")
    if not want_final:   # (the placeholders returned in place of a final state carry no gradient)
        dSf = dsf = None
    if dO is None and dSf is None and dsf is None:
        return (None,) * 10
    if dO is None:
        dO = torch.zeros_like(O)
    dQ, dK, dV, dlg, dS0, ds0 = chunked_bwd(Q, K, V, A, lcs, Kd, Sc, sc, rm, O, den, dO, deg, scale, c, gated, carried,
                                            dSf, dsf, live, S, s)
    return (dQ, dK, dV, (dlg if gated else None), None, None, None, dS0 if carried else None,
            ds0.to(s0_dtype) if carried else None, None)


torch.library.register_autograd("pr::chunked_fwd", _chunked_backward, setup_context=_chunked_setup)


def chunked_power_retention(Q, K, V, log_G, deg, scale, chunk_size, initial_state=None, return_final_state=False):
    """Q [b,t,hq,d], K, V [b,t,h,d] contiguous, t a multiple of chunk_size, log_G [b,t,h] fp32 or None;
    initial_state = (state [b,h,D,d], sum_of_keys [b,h,D]) or None -> out, or (out, (state, sum_of_keys)) with
    return_final_state.  Only deg = 2 has a state (ref: retention/_update_state/triton.py:310-311 raises the same way)."""
    if deg != 2:
        raise NotImplementedError(f"the chunked algorithm needs the degree-2 state layout (got deg={deg})")
    S0, s0 = (None, None) if initial_state is None else (initial_state[0].contiguous(), initial_state[1].contiguous())
    out = chunked_fwd(Q, K, V, log_G, int(deg), float(scale), int(chunk_size), S0, s0, bool(return_final_state))
    if return_final_state:
        return out[0], (out[8], out[9])
    return out[0]
