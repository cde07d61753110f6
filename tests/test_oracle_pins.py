"""Pins for the CPU oracle (no GPU).  None of these re-types the oracle's formulas: they use
torch.nn library cells, an un-stabilised float64 recurrence, closed forms and autograd."""
import math

import pytest
import torch

from oracle import (FUNCTIONS, flashrnn_oracle, flashrnn_oracle_backward,
                    flashrnn_oracle_fwbw_manual, make_inputs)

torch.manual_seed(0)
DT = torch.float64


def _nn_cells(kind, N, D, G):
    """N independent torch.nn cells with input size G*D and identity-free random weights."""
    cls = {"lstm": torch.nn.LSTM, "gru": torch.nn.GRU, "elman": torch.nn.RNN}[kind]
    cells = [cls(G * D, D, num_layers=1, bias=True, batch_first=True).to(DT) for _ in range(N)]
    for c in cells:
        with torch.no_grad():
            # input projection = identity: the cell's x IS our Wx, so x.grad pins dWx fully
            c.weight_ih_l0.copy_(torch.eye(G * D, dtype=DT))
            c.weight_hh_l0.normal_(0, 1.0 / math.sqrt(D))  # non-symmetric
            c.bias_ih_l0.normal_(0, 0.3)
            c.bias_hh_l0.normal_(0, 0.3)
    return cells


@pytest.mark.parametrize("N", [1, 3])
def test_lstm_matches_torch_nn_lstm(N):
    B, T, D = 3, 7, 5
    cells = _nn_cells("lstm", N, D, 4)
    x = torch.randn(B, T, 4, N, D, dtype=DT, requires_grad=True)
    h0 = torch.randn(B, N, D, dtype=DT, requires_grad=True)
    c0 = torch.randn(B, N, D, dtype=DT, requires_grad=True)
    cot_h = torch.randn(B, T, N, D, dtype=DT)
    cot_c = torch.randn(B, N, D, dtype=DT)
    hs, cs = [], []
    for n, cell in enumerate(cells):
        out, (hn, cn) = cell(x[:, :, :, n].reshape(B, T, 4 * D),
                             (h0[None, :, n].contiguous(), c0[None, :, n].contiguous()))
        hs.append(out)
        cs.append(cn[0])
    h_ref = torch.stack(hs, 2)
    c_ref = torch.stack(cs, 1)
    loss = (h_ref * cot_h).sum() + (c_ref * cot_c).sum()
    gx, gh0, gc0 = torch.autograd.grad(loss, [x, h0, c0], retain_graph=True)
    gR = torch.stack([torch.autograd.grad(loss, c.weight_hh_l0, retain_graph=True)[0].reshape(4, D, D)
                      for c in cells], 1)
    gb = torch.stack([torch.autograd.grad(loss, c.bias_hh_l0, retain_graph=True)[0].reshape(4, D)
                      for c in cells], 1)

    R = torch.stack([c.weight_hh_l0.detach().reshape(4, D, D) for c in cells], 1)
    b = torch.stack([(c.bias_ih_l0 + c.bias_hh_l0).detach().reshape(4, D) for c in cells], 1)
    s0 = torch.stack([h0.detach(), c0.detach()], 0)[:, :, None]
    ds = torch.zeros(2, B, T, N, D, dtype=DT)
    ds[0] = cot_h
    ds[1, :, -1] = cot_c
    out, (dWx, dR, db, ds0) = flashrnn_oracle_backward(x.detach(), R, b, s0, "lstm", ds)
    assert torch.allclose(out[0], h_ref, atol=1e-12)
    assert torch.allclose(out[1, :, -1], c_ref, atol=1e-12)
    assert torch.allclose(dWx, gx, atol=1e-11)
    assert torch.allclose(dR, gR, atol=1e-11)
    assert torch.allclose(db, gb, atol=1e-11)
    assert torch.allclose(ds0[0, :, 0], gh0, atol=1e-11)
    assert torch.allclose(ds0[1, :, 0], gc0, atol=1e-11)


def test_lstm_reference_known_answer_fp32():
    """The reference's only known-answer test (flashrnn/tests/test_lstm.py:70-115): N=1, fp32,
    Wx = x W_ih^T, R = W_hh.reshape(4,1,D,D), b = b_ih + b_hh, atol 1e-3 / rtol 2e-3."""
    B, T, D = 2, 3, 32
    lstm = torch.nn.LSTM(D, D, num_layers=1, bias=True, batch_first=True)
    x = torch.randn(B, T, D)
    with torch.no_grad():
        Wx = (x @ lstm.weight_ih_l0.T).reshape(B, T, 4, 1, D)
        R = lstm.weight_hh_l0.reshape(4, 1, D, D)
        b = (lstm.bias_hh_l0 + lstm.bias_ih_l0).reshape(4, 1, D)
        got = flashrnn_oracle(Wx, R, b, None, "lstm")[0][0, :, :, 0]
        want = lstm(x)[0]
    assert torch.allclose(got, want, atol=1e-3, rtol=2e-3)
    assert torch.allclose(got, want, atol=2e-6)


@pytest.mark.parametrize("N", [1, 2])
def test_gru_matches_torch_nn_gru(N):
    B, T, D = 3, 6, 4
    cells = _nn_cells("gru", N, D, 3)
    x = torch.randn(B, T, 3, N, D, dtype=DT, requires_grad=True)
    h0 = torch.randn(B, N, D, dtype=DT, requires_grad=True)
    cot = torch.randn(B, T, N, D, dtype=DT)
    h_ref = torch.stack([cell(x[:, :, :, n].reshape(B, T, 3 * D), h0[None, :, n].contiguous())[0]
                         for n, cell in enumerate(cells)], 2)
    loss = (h_ref * cot).sum()
    gx, gh0 = torch.autograd.grad(loss, [x, h0], retain_graph=True)
    # torch gate order (r, z, n); ours: R gates [g(=n-recurrent), r, z], b gates [g, r, z, n]
    Rl, bl, gRl, gbl = [], [], [], []
    for c in cells:
        W = c.weight_hh_l0.detach().reshape(3, D, D)
        bi, bh = c.bias_ih_l0.detach().reshape(3, D), c.bias_hh_l0.detach().reshape(3, D)
        Rl.append(torch.stack([W[2], W[0], W[1]], 0))
        bl.append(torch.stack([bh[2], bi[0] + bh[0], bi[1] + bh[1], bi[2]], 0))
        gW = torch.autograd.grad(loss, c.weight_hh_l0, retain_graph=True)[0].reshape(3, D, D)
        gbi = torch.autograd.grad(loss, c.bias_ih_l0, retain_graph=True)[0].reshape(3, D)
        gbh = torch.autograd.grad(loss, c.bias_hh_l0, retain_graph=True)[0].reshape(3, D)
        gRl.append(torch.stack([gW[2], gW[0], gW[1]], 0))
        gbl.append(torch.stack([gbh[2], gbh[0], gbh[1], gbi[2]], 0))
    R, b = torch.stack(Rl, 1), torch.stack(bl, 1)
    ds = cot[None]
    out, (dWx, dR, db, ds0) = flashrnn_oracle_backward(x.detach(), R, b, h0.detach()[None, :, None], "gru", ds)
    assert torch.allclose(out[0], h_ref, atol=1e-12)
    assert torch.allclose(dWx, gx, atol=1e-11)
    assert torch.allclose(dR, torch.stack(gRl, 1), atol=1e-11)
    assert torch.allclose(db, torch.stack(gbl, 1), atol=1e-11)
    assert torch.allclose(ds0[0, :, 0], gh0, atol=1e-11)


def test_elman_matches_torch_nn_rnn():
    B, T, D, N = 4, 9, 6, 2
    cells = _nn_cells("elman", N, D, 1)
    x = torch.randn(B, T, 1, N, D, dtype=DT, requires_grad=True)
    h0 = torch.randn(B, N, D, dtype=DT, requires_grad=True)
    cot = torch.randn(B, T, N, D, dtype=DT)
    h_ref = torch.stack([cell(x[:, :, 0, n], h0[None, :, n].contiguous())[0]
                         for n, cell in enumerate(cells)], 2)
    loss = (h_ref * cot).sum()
    gx, gh0 = torch.autograd.grad(loss, [x, h0], retain_graph=True)
    gR = torch.stack([torch.autograd.grad(loss, c.weight_hh_l0, retain_graph=True)[0] for c in cells], 0)[None]
    gb = torch.stack([torch.autograd.grad(loss, c.bias_hh_l0, retain_graph=True)[0] for c in cells], 0)[None]
    R = torch.stack([c.weight_hh_l0.detach() for c in cells], 0)[None]
    b = torch.stack([(c.bias_ih_l0 + c.bias_hh_l0).detach() for c in cells], 0)[None]
    out, (dWx, dR, db, ds0) = flashrnn_oracle_backward(x.detach(), R, b, h0.detach()[None, :, None], "elman", cot[None])
    assert torch.allclose(out[0], h_ref, atol=1e-12)
    assert torch.allclose(dWx, gx, atol=1e-11)
    assert torch.allclose(dR, gR, atol=1e-11)
    assert torch.allclose(db, gb, atol=1e-11)
    assert torch.allclose(ds0[0, :, 0], gh0, atol=1e-11)


def test_slstm_matches_unstabilised_float64_recurrence():
    """C_t = sig(f) C + e^i tanh z,  N_t = sig(f) N + e^i,  h = sig(o) C/N  (no stabiliser),
    c_t = C_t e^{-m_t}, n_t = N_t e^{-m_t};  m_t = max_s<=t ( i_s + sum_{r=s+1..t} logsig f_r )."""
    B, T, N, D = 2, 12, 2, 3
    inp = make_inputs("slstm", B, T, N, D, seed=5)
    Wx, R, b = inp["Wx"].to(DT), inp["R"].to(DT) * 2.0, inp["b"].to(DT)
    out, last = flashrnn_oracle(Wx, R, b, None, "slstm")
    C = torch.zeros(B, N, D, dtype=DT)
    Nn = torch.zeros_like(C)
    h = torch.zeros_like(C)
    paths = []  # candidates i_s + sum of later log-sigmoid(f)
    for t in range(T):
        raw = Wx[:, t] + torch.einsum("bnp,gndp->bgnd", h, R) + b[None]
        i, f, z, o = raw.unbind(1)
        sf = 1.0 / (1.0 + torch.exp(-f))
        C = sf * C + torch.exp(i) * torch.tanh(z)
        Nn = sf * Nn + torch.exp(i)
        h = C / Nn / (1.0 + torch.exp(-o))
        paths = [p + torch.log(sf) for p in paths] + [i]
        m = torch.stack(paths, 0).max(0).values
        assert torch.allclose(out[0, :, t], h, atol=1e-12), t
        assert torch.allclose(out[3, :, t], m, atol=1e-12), t
        assert torch.allclose(out[1, :, t] * torch.exp(m), C, rtol=1e-11), t
        assert torch.allclose(out[2, :, t] * torch.exp(m), Nn, rtol=1e-11), t
    assert (out[2] >= 1.0).all()
    assert torch.equal(last, out[:, :, -1:])


def test_slstm_closed_form_single_step():
    B, N, D = 3, 2, 4
    inp = make_inputs("slstm", B, 1, N, D, seed=9)
    Wx, b = inp["Wx"].to(DT), inp["b"].to(DT)
    R = torch.randn(4, N, D, D, dtype=DT)  # irrelevant: h0 = 0
    out, _ = flashrnn_oracle(Wx, R, b, None, "slstm")
    raw = Wx[:, 0] + b[None]
    i, f, z, o = raw.unbind(1)
    assert torch.allclose(out[3, :, 0], i)
    assert torch.allclose(out[2, :, 0], torch.ones_like(i))
    assert torch.allclose(out[1, :, 0], torch.tanh(z), atol=1e-14)
    assert torch.allclose(out[0, :, 0], torch.tanh(z) / (1 + torch.exp(-o)), atol=1e-14)


def test_slstm_first_step_branch_is_whole_tensor():
    """vanilla/slstm.py:21 tests all(n == 0) over the whole tensor; with every n non-zero the
    per-element test of the native kernels agrees with it."""
    inp = make_inputs("slstm", 2, 3, 1, 4, seed=2, init="randn")
    a = flashrnn_oracle(inp["Wx"], inp["R"], inp["b"], inp["states"], "slstm")[0]
    c = flashrnn_oracle(inp["Wx"], inp["R"], inp["b"], inp["states"], "slstm",
                        slstm_per_element_first_step=True)[0]
    assert torch.equal(a, c)
    z = make_inputs("slstm", 2, 3, 1, 4, seed=2)
    a = flashrnn_oracle(z["Wx"], z["R"], z["b"], z["states"], "slstm")[0]
    c = flashrnn_oracle(z["Wx"], z["R"], z["b"], z["states"], "slstm",
                        slstm_per_element_first_step=True)[0]
    assert torch.equal(a, c)


@pytest.mark.parametrize("function", ["lstm", "gru", "elman", "slstm"])
@pytest.mark.parametrize("init", ["zeros", "randn"])
def test_manual_reverse_scan_matches_autograd(function, init):
    B, T, N, D = 3, 6, 2, 5
    inp = make_inputs(function, B, T, N, D, seed=11, init=init,
                      grad_on="h" if function == "slstm" else "all")
    Wx, R, b, s0, ds = (inp[k].to(DT) for k in ("Wx", "R", "b", "states", "dstates"))
    out_a, (gWx, gR, gb, gs0) = flashrnn_oracle_backward(Wx, R, b, s0, function, ds,
                                                        **({"slstm_per_element_first_step": True}
                                                           if function == "slstm" else {}))
    out_m, (dWx, dR, db, ds0) = flashrnn_oracle_fwbw_manual(Wx, R, b, s0, function, ds)
    assert torch.allclose(out_m, out_a, atol=1e-12)
    assert torch.allclose(dWx, gWx, atol=1e-10)
    assert torch.allclose(dR, gR, atol=1e-10)
    assert torch.allclose(db, gb, atol=1e-10)
    S = FUNCTIONS[function][4]
    # sLSTM: the kernels hold the stabiliser m constant, so d/dm0 is reported as 0 by design
    # (slstm_pointwise.cu:205); autograd's d/dc0, d/dn0 hold m0 fixed too and must agree.
    keep = [0, 1, 2] if function == "slstm" else list(range(S))
    if function == "slstm" and init == "zeros":
        keep = [0, 1]  # n0 == 0 sits on the kink of max(.,1) and of the n==0 branch
    for k in keep:
        assert torch.allclose(ds0[k], gs0[k], atol=1e-10), k


@pytest.mark.parametrize("function", ["lstm", "gru", "elman", "slstm"])
def test_chunked_sequence_invariant(function):
    B, T, N, D = 2, 10, 2, 4
    inp = make_inputs(function, B, T, N, D, seed=3)
    Wx, R, b = (inp[k].to(DT) for k in ("Wx", "R", "b"))
    full, last = flashrnn_oracle(Wx, R, b, None, function)
    a, la = flashrnn_oracle(Wx[:, :4], R, b, None, function)
    c, lc = flashrnn_oracle(Wx[:, 4:], R, b, la, function)
    assert torch.allclose(torch.cat([a, c], 2), full, atol=1e-13)
    assert torch.allclose(lc, last, atol=1e-13)


def test_heads_are_independent_and_R_orientation():
    """Ry[b,g,n,d] = sum_p R[g,n,d,p] h[b,n,p]: a one-hot R must route unit p of head n only."""
    B, N, D = 1, 2, 3
    Wx = torch.zeros(B, 2, 1, N, D, dtype=DT)
    Wx[0, 0, 0, 1, 2] = 0.7  # step 0: excites head 1, unit 2
    R = torch.zeros(1, N, D, D, dtype=DT)
    R[0, 1, 0, 2] = 1.0  # head 1: output unit 0 listens to previous unit 2
    b = torch.zeros(1, N, D, dtype=DT)
    out, _ = flashrnn_oracle(Wx, R, b, None, "elman")
    h1 = math.tanh(0.7)
    want = torch.zeros(B, N, D, dtype=DT)
    want[0, 1, 0] = math.tanh(h1)
    assert torch.allclose(out[0, :, 1], want)
