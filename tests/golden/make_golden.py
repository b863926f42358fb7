"""Writes tests/golden/*.npz: input/output vectors of the reference's pure-torch
backend for the functions whose element order no mathematical invariant pins
(the state layout of update_state / query_state / the inference tuple), plus
whole-path vectors as a belt-and-braces check of the same layout end to end.

Runs ONLY in the build container, where the reference tree is mounted
read-only at /root/reference.  The reference package's __init__ files import
its Triton/vidrial backends, so the pure-torch files are loaded under empty
namespace packages instead; nothing from the reference is copied here.

    python tests/golden/make_golden.py
"""
import importlib
import os
import sys
import types

import numpy as np
import torch

REF = os.environ.get("REFERENCE_ROOT", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def _namespace(name, path):
    m = types.ModuleType(name)
    m.__path__ = [path]
    sys.modules[name] = m
    return m


def load_reference():
    _namespace("retention", os.path.join(REF, "retention"))
    for sub in ("_attention", "_update_state", "_discumsum", "_query_state"):
        _namespace(f"retention.{sub}", os.path.join(REF, "retention", sub))
    return importlib.import_module("retention.reference")


def npz(name, **arrays):
    out = {}
    for k, v in arrays.items():
        if v is None:
            continue
        out[k] = v.detach().cpu().numpy() if isinstance(v, torch.Tensor) else np.asarray(v)
    np.savez_compressed(os.path.join(HERE, name), **out)
    print("wrote", name, {k: tuple(a.shape) for k, a in out.items()})


def main():
    ref = load_reference()
    from retention._update_state.reference import update_state
    from retention._query_state.reference import query_state_reference
    from retention._discumsum.reference import discumsum_reference
    from retention._attention.reference import attention
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(1234)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)  # noqa: E731

    # update_state: d=32 has one off-diagonal tile (multiplier 2) and two diagonal tiles
    K, V = rn(1, 2, 8, 1, 32), rn(1, 2, 8, 1, 32)
    S, N = update_state(K, V, 2)
    npz("update_state_d32.npz", K=K, V=V, S=S, N=N)

    # update_state at d=64 (four diagonal tiles, six below them: D = 2560) together with the one hand-written backward
    # the reference's pure-torch backend has (SymmetricPowerUpdateStateReference.backward).  Inputs are multiples of
    # 1/4, so every product and sum is exact in fp32 (and the file compresses); the upstream gradient of S is the outer
    # product u w^T of two stored vectors, so it need not be stored itself.
    g64 = torch.Generator().manual_seed(4321)   # (its own stream: the vectors below keep their values)
    q4 = lambda *s: (torch.randn(*s, generator=g64, dtype=torch.float32) * 4).round().clamp(-8, 8) / 4  # noqa: E731
    K64, V64 = q4(1, 1, 4, 1, 64).requires_grad_(True), q4(1, 1, 4, 1, 64).requires_grad_(True)
    S64, N64 = update_state(K64, V64, 2)
    u, wv, dN = q4(2560), q4(64), q4(1, 1, 1, 2560)
    dS = (u[:, None] * wv[None, :]).view(1, 1, 1, 2560, 64)
    dK64, dV64 = torch.autograd.grad((S64, N64), (K64, V64), (dS, dN))
    npz("update_state_d64_bwd.npz", K=K64, V=V64, S=S64, N=N64, dS_u=u, dS_w=wv, dN=dN, dK=dK64, dV=dV64)

    # query_state with GQA ratio 2, second chunk uses gamma = sqrt(D)
    Q = rn(1, 2, 4, 2, 32)
    S_in = rn(1, 2, 1, 768, 32)
    s_in = rn(1, 2, 1, 768).abs() + 4.0
    Ya, la, rm = rn(1, 2, 4, 2, 32), rn(1, 2, 4, 2).abs() + 4.0, rn(1, 2, 4, 2).abs() + 1.0
    for zis in (True, False):
        O = query_state_reference(Q, S_in, s_in, Ya, la, rm, 2, 0.25, zis)
        npz(f"query_state_d32_zis{int(zis)}.npz", Q=Q, S=S_in, s=s_in, Y_attn=Ya, l_attn=la, rowmax=rm,
            scale=0.25, O=O)

    # discumsum with a varying gate
    X = rn(2, 5, 3, 4, 2)
    lg = F.logsigmoid(rn(2, 5, 3))
    npz("discumsum.npz", X=X, log_G=lg, Y=discumsum_reference(X, lg))

    # attention: tq < tk, GQA ratio 2, accumulated gate
    Qa, Ka, Va = rn(2, 5, 4, 16), rn(2, 12, 2, 16), rn(2, 12, 2, 16)
    Ga = F.logsigmoid(rn(2, 12, 2)).cumsum(1)
    o, l, m = attention(Qa, Ka, Va, Ga, 2, scale=0.25, norm=False)
    on = attention(Qa, Ka, Va, Ga, 2, scale=0.25, norm=True)
    npz("attention_gqa.npz", Q=Qa, K=Ka, V=Va, log_G_accum=Ga, scale=0.25, o=o, l=l, rowmax=m, o_norm=on)

    # whole path, chunked, padded (t=40, c=16), GQA ratio 2, gated
    Qp, Kp, Vp = rn(1, 40, 2, 32), rn(1, 40, 1, 32), rn(1, 40, 1, 32)
    Gp = F.logsigmoid(rn(1, 40, 1))
    Y = ref.power_retention(Qp, Kp, Vp, Gp, deg=2, scale=None, chunk_size=16)
    Yq = ref.power_retention(Qp, Kp, Vp, Gp, deg=2, scale=None, chunk_size=None)
    npz("power_retention_d32.npz", Q=Qp, K=Kp, V=Vp, log_G=Gp, Y_chunked=Y, Y_quadratic=Yq)

    # inference: prefill that compresses the cache, then one decode step on the state
    Qi, Ki, Vi = rn(1, 1, 2, 32), rn(1, 24, 1, 32), rn(1, 24, 1, 32)
    Gi = F.logsigmoid(2.0 + rn(1, 24, 1))
    Y0, st, sk = ref.power_retention_inference(Qi, Ki, Vi, Gi, None, None, deg=2, scale=None, switch_over_seq_len=16)
    Q1, K1, V1 = rn(1, 1, 2, 32), rn(1, 3, 1, 32), rn(1, 3, 1, 32)
    G1 = F.logsigmoid(2.0 + rn(1, 3, 1))
    Y1, st1, sk1 = ref.power_retention_inference(Q1, K1, V1, G1, st, sk, deg=2, scale=None, switch_over_seq_len=3)
    npz("inference_d32.npz", Q0=Qi, K0=Ki, V0=Vi, log_G0=Gi, Y0=Y0, state0=st, sum_of_keys0=sk,
        Q1=Q1, K1=K1, V1=V1, log_G1=G1, Y1=Y1, state1=st1, sum_of_keys1=sk1)


if __name__ == "__main__":
    main()
