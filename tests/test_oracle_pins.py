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


# ---- clip / cut options -----------------------------------------------------------------------
def _scalar_elman(w, r, b, h0):
    """A 1-unit Elman cell over T = len(w) steps, written out: h_t = tanh(w_t + r h_{t-1} + b)."""
    import math

    h = [h0]
    for wt in w:
        h.append(math.tanh(wt + r * h[-1] + b))
    return h


def test_gradient_clip_and_cut_closed_form_scalar_elman():
    """Loss = h_3 on a scalar Elman cell, T = 3.  By hand: dpre_3 = 1 - h_3^2; the cotangent sent
    back to h_2 is r*dpre_3, to h_1 r*dpre_2, ...; the clip clamps exactly those carried values,
    the cut replaces them by 0; the cotangent of h_0 is never clamped."""
    w, r, b, h0 = [0.3, -0.2, 0.5], 2.5, 0.1, 0.4
    h = _scalar_elman(w, r, b, h0)
    d = [1 - x * x for x in h]  # tanh' at h_t
    Wx = torch.tensor(w, dtype=torch.float64).reshape(1, 3, 1, 1, 1)
    R = torch.tensor([[[[r]]]], dtype=torch.float64)
    bb = torch.tensor([[[b]]], dtype=torch.float64)
    s0 = torch.tensor(h0, dtype=torch.float64).reshape(1, 1, 1, 1, 1)
    ds = torch.zeros(1, 1, 3, 1, 1, dtype=torch.float64)
    ds[0, 0, 2] = 1.0
    clamp = lambda x, c: max(-c, min(c, x))
    for c in (0.05, 0.7, 100.0):
        dpre3 = d[3]
        dpre2 = clamp(r * dpre3, c) * d[2]
        dpre1 = clamp(r * dpre2, c) * d[1]
        want_dWx = [dpre1, dpre2, dpre3]
        want_ds0 = r * dpre1  # not clamped
        want_dR = dpre1 * h[0] + dpre2 * h[1] + dpre3 * h[2]
        for run in (lambda: flashrnn_oracle_backward(Wx, R, bb, s0, "elman", ds, gradient_recurrent_clipval=c)[1],
                    lambda: flashrnn_oracle_fwbw_manual(Wx, R, bb, s0, "elman", ds, gradient_recurrent_clipval=c)[1]):
            dWx, dR, db, ds0 = run()
            assert torch.allclose(dWx.flatten(), torch.tensor(want_dWx, dtype=torch.float64), atol=1e-14)
            assert abs(float(ds0) - want_ds0) < 1e-14 and abs(float(dR) - want_dR) < 1e-14
            assert abs(float(db) - sum(want_dWx)) < 1e-14
    # cut: nothing flows back through r
    for run in (lambda: flashrnn_oracle_backward(Wx, R, bb, s0, "elman", ds, gradient_recurrent_cut=True)[1],
                lambda: flashrnn_oracle_fwbw_manual(Wx, R, bb, s0, "elman", ds, gradient_recurrent_cut=True)[1]):
        dWx, dR, db, ds0 = run()
        assert torch.allclose(dWx.flatten(), torch.tensor([0.0, 0.0, d[3]], dtype=torch.float64), atol=1e-14)
        assert float(ds0) == 0.0 and abs(float(dR) - d[3] * h[2]) < 1e-14


def test_forward_clip_closed_form_scalar_elman():
    """h is clamped before it is stored and fed back; the gradient is the unclamped one evaluated
    on the clamped trajectory (straight-through)."""
    import math

    w, r, b, h0, c = [1.5, -0.2], 0.8, 0.0, 0.0, 0.6
    g1 = math.tanh(w[0] + r * h0 + b)
    h1 = max(-c, min(c, g1))
    assert h1 == c  # the clamp is active at step 1
    g2 = math.tanh(w[1] + r * h1 + b)
    Wx = torch.tensor(w, dtype=torch.float64).reshape(1, 2, 1, 1, 1)
    R = torch.tensor([[[[r]]]], dtype=torch.float64)
    bb = torch.zeros(1, 1, 1, dtype=torch.float64)
    s0 = torch.zeros(1, 1, 1, 1, 1, dtype=torch.float64)
    ds = torch.zeros(1, 1, 2, 1, 1, dtype=torch.float64)
    ds[0, 0, 1] = 1.0
    out, (dWx, dR, db, ds0) = flashrnn_oracle_backward(Wx, R, bb, s0, "elman", ds, forward_clipval=c)
    assert abs(float(out[0, 0, 0]) - c) < 1e-15 and abs(float(out[0, 0, 1]) - g2) < 1e-15
    dpre2 = 1 - g2 * g2
    dpre1 = r * dpre2 * (1 - g1 * g1)  # tanh' of the unclamped gate value, as the native kernels cache it
    assert torch.allclose(dWx.flatten(), torch.tensor([dpre1, dpre2], dtype=torch.float64), atol=1e-14)
    out2, (dWx2, _, _, _) = flashrnn_oracle_fwbw_manual(Wx, R, bb, s0, "elman", ds, forward_clipval=c)
    assert torch.equal(out, out2) and torch.allclose(dWx, dWx2, atol=1e-14)


@pytest.mark.parametrize("function", ["lstm", "gru", "elman", "slstm"])
def test_options_autograd_and_explicit_scan_agree(function):
    """Two independent statements of every option: a clamp-the-cotangent node / detach /
    straight-through clamp under autograd against the explicit reverse scan."""
    inp = make_inputs(function, 3, 7, 2, 8, 21, init="randn", grad_on="h" if function == "slstm" else "all")
    a = [inp[k].double() for k in ("Wx", "R", "b", "states")]
    a[1] = a[1] * 3  # a recurrent gradient large enough for the clamp to bite
    ds = inp["dstates"].double()
    base = {"slstm_per_element_first_step": True} if function == "slstm" else {}
    plain = flashrnn_oracle_backward(*a, function, ds, **base)[1]
    cases = [dict(gradient_recurrent_clipval=0.05), dict(gradient_recurrent_cut=True),
             dict(gradient_recurrent_clipval=0.05, gradient_recurrent_cut=True)]
    if function != "slstm":  # the native sLSTM adjoint reads the clamped h: only the explicit scan states that
        cases += [dict(forward_clipval=0.3), dict(forward_clipval=0.3, gradient_recurrent_clipval=0.05)]
    for kw in cases:
        o1, g1 = flashrnn_oracle_backward(*a, function, ds, **base, **kw)
        o2, g2 = flashrnn_oracle_fwbw_manual(*a, function, ds, **kw)
        assert torch.allclose(o1, o2, atol=1e-12)
        for k, (x, y) in enumerate(zip(g1, g2)):
            if function == "slstm" and k == 3:
                x, y = x[:3], y[:3]  # the stabiliser's cotangent is 0 by design in the explicit scan
            assert torch.allclose(x, y, atol=1e-10), (kw, k, float((x - y).abs().max()))
        assert float((g1[0] - plain[0]).abs().max()) > 1e-3, kw  # the option did change something


@pytest.mark.parametrize("function", ["lstm", "gru", "elman", "slstm"])
def test_options_noop_limits(function):
    """A clip value above every carried value changes nothing; with R = 0 the cut changes nothing."""
    inp = make_inputs(function, 2, 5, 2, 8, 22, init="randn", grad_on="h" if function == "slstm" else "all")
    a = [inp[k].double() for k in ("Wx", "R", "b", "states")]
    ds = inp["dstates"].double()
    base = {"slstm_per_element_first_step": True} if function == "slstm" else {}
    o0, g0 = flashrnn_oracle_backward(*a, function, ds, **base)
    o1, g1 = flashrnn_oracle_backward(*a, function, ds, **base, gradient_recurrent_clipval=1e9, forward_clipval=1e9)
    assert torch.equal(o0, o1) and all(torch.allclose(x, y, atol=1e-13) for x, y in zip(g0, g1))
    a0 = [a[0], torch.zeros_like(a[1]), a[2], a[3]]
    _, g2 = flashrnn_oracle_backward(*a0, function, ds, **base)
    _, g3 = flashrnn_oracle_backward(*a0, function, ds, **base, gradient_recurrent_cut=True)
    for k, (x, y) in enumerate(zip(g2, g3)):
        if k == 1:
            continue  # dR itself is not zero when R is
        assert torch.allclose(x, y, atol=1e-13), k
    # forward clamp: every stored h lies inside the interval and the untouched steps are unchanged
    o4, _ = flashrnn_oracle_backward(*a, function, ds, **base, forward_clipval=0.25)
    assert float(o4[0].abs().max()) <= 0.25 + 1e-15
