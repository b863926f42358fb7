"""The CPU oracle against vectors written from the reference's pure-torch
backend (tests/golden/make_golden.py).  fp32 in, fp32 out: equality up to
summation order."""
import os

import numpy as np
import pytest
import torch

import oracle

G = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    z = np.load(os.path.join(G, name))
    return {k: torch.from_numpy(z[k]) if z[k].ndim else float(z[k]) for k in z.files}


def close(a, b, rtol=2e-5, atol=2e-5):
    torch.testing.assert_close(a, b, rtol=rtol, atol=atol)


def test_update_state_layout():
    v = load("update_state_d32.npz")
    S, N = oracle.update_state(v["K"], v["V"], 2)
    close(S, v["S"])
    close(N, v["N"])


@pytest.mark.parametrize("zis", [0, 1])
def test_query_state(zis):
    v = load(f"query_state_d32_zis{zis}.npz")
    O = oracle.query_state(v["Q"], v["S"], v["s"], v["Y_attn"], v["l_attn"], v["rowmax"], 2, v["scale"], bool(zis))
    close(O, v["O"], rtol=1e-4, atol=1e-5)


def test_discumsum():
    v = load("discumsum.npz")
    close(oracle.discumsum(v["X"], v["log_G"]), v["Y"])


def test_attention_gqa_unaligned():
    v = load("attention_gqa.npz")
    o, l, m = oracle.attention(v["Q"], v["K"], v["V"], v["log_G_accum"], 2, scale=v["scale"], norm=False)
    close(o, v["o"]); close(l, v["l"]); close(m, v["rowmax"])
    close(oracle.attention(v["Q"], v["K"], v["V"], v["log_G_accum"], 2, scale=v["scale"], norm=True), v["o_norm"])


def test_power_retention_chunked_and_quadratic():
    v = load("power_retention_d32.npz")
    Y = oracle.power_retention(v["Q"], v["K"], v["V"], v["log_G"], deg=2, chunk_size=16)
    close(Y, v["Y_chunked"], rtol=1e-4, atol=1e-5)
    Yq = oracle.power_retention(v["Q"], v["K"], v["V"], v["log_G"], deg=2, chunk_size=None)
    close(Yq, v["Y_quadratic"], rtol=1e-4, atol=1e-5)


def test_inference_prefill_then_decode():
    v = load("inference_d32.npz")
    Y0, st, sk = oracle.power_retention_inference(v["Q0"], v["K0"], v["V0"], v["log_G0"], None, None,
                                                  deg=2, switch_over_seq_len=16)
    close(Y0, v["Y0"], rtol=1e-4, atol=1e-5); close(st, v["state0"]); close(sk, v["sum_of_keys0"])
    Y1, st1, sk1 = oracle.power_retention_inference(v["Q1"], v["K1"], v["V1"], v["log_G1"], v["state0"],
                                                    v["sum_of_keys0"], deg=2, switch_over_seq_len=3)
    close(Y1, v["Y1"], rtol=1e-4, atol=1e-5); close(st1, v["state1"]); close(sk1, v["sum_of_keys1"])


def test_update_state_d64_forward_and_the_references_hand_written_backward():
    """d = 64: ten feature tiles (four on the diagonal), and the gradients of the one backward the reference's
    pure-torch backend writes by hand (ref: retention/_update_state/reference.py:55-83) against the oracle's autograd.
    The inputs are multiples of 1/4, so both sides are exact in fp32."""
    v = load("update_state_d64_bwd.npz")
    K, V = v["K"].clone().requires_grad_(True), v["V"].clone().requires_grad_(True)
    S, N = oracle.update_state(K, V, 2)
    assert torch.equal(S, v["S"]) and torch.equal(N, v["N"])
    dS = (v["dS_u"][:, None] * v["dS_w"][None, :]).view(1, 1, 1, 2560, 64)
    dK, dV = torch.autograd.grad((S, N), (K, V), (dS, v["dN"]))
    close(dK, v["dK"], rtol=1e-6, atol=1e-4)
    close(dV, v["dV"], rtol=1e-6, atol=1e-4)
