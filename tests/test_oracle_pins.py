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


# ---- sLSTM: what the native adjoint does beyond plain autograd -------------------------------------
def test_slstm_adjoint_for_cotangents_on_c_and_n_is_autograd_with_the_stabiliser_held_constant():
    """The explicit reverse scan (the native adjoint, slstm_fused_pointwise.cuh:117-186) with cotangents on
    every state equals float64 autograd of the forward with the stabiliser m detached, and differs from
    plain autograd, which also differentiates exp(-m) in c and n.  For a cotangent on h alone the two
    autograd variants agree (h does not depend on m).  Initial n > 1 keeps max(., 1) away from its kink."""
    B, T, N, D = 3, 6, 2, 5
    inp = make_inputs("slstm", B, T, N, D, seed=31, init="randn", grad_on="all")
    Wx, R, b, s0, ds = (inp[k].to(DT) for k in ("Wx", "R", "b", "states", "dstates"))
    ds[3] = 0  # m itself gets no cotangent anywhere in the native path
    kw = dict(slstm_per_element_first_step=True)
    out_d, g_det = flashrnn_oracle_backward(Wx, R, b, s0, "slstm", ds, slstm_detach_m=True, **kw)
    out_p, g_plain = flashrnn_oracle_backward(Wx, R, b, s0, "slstm", ds, **kw)
    out_m, g_man = flashrnn_oracle_fwbw_manual(Wx, R, b, s0, "slstm", ds)
    assert torch.equal(out_d, out_p) and torch.allclose(out_m, out_d, atol=1e-12)
    for k, (x, y) in enumerate(zip(g_man, g_det)):
        assert torch.allclose(x, y, atol=1e-10), (k, float((x - y).abs().max()))
    assert float(g_det[3][3].abs().max()) == 0.0 and float(g_man[3][3].abs().max()) == 0.0   # d/dm0 = 0
    assert float((g_plain[0] - g_det[0]).abs().max()) > 1e-2   # plain autograd is a different function here
    # zero initial state: n' = max(0 + 1, 1) ties at the first step; the native adjoint (and the detached
    # autograd, whose guard is transparent) takes slope 1 there, so even d/dn0 agrees
    z0 = torch.zeros_like(s0)
    _, gz_det = flashrnn_oracle_backward(Wx, R, b, z0, "slstm", ds, slstm_detach_m=True, **kw)
    _, gz_man = flashrnn_oracle_fwbw_manual(Wx, R, b, z0, "slstm", ds)
    for k, (x, y) in enumerate(zip(gz_man, gz_det)):
        assert torch.allclose(x, y, atol=1e-10), ("zero init", k, float((x - y).abs().max()))
    ds_h = ds.clone()
    ds_h[1:] = 0
    _, a = flashrnn_oracle_backward(Wx, R, b, s0, "slstm", ds_h, slstm_detach_m=True, **kw)
    _, c = flashrnn_oracle_backward(Wx, R, b, s0, "slstm", ds_h, **kw)
    for k in range(3):
        assert torch.allclose(a[k], c[k], atol=1e-10), k


def test_slstm_backward_through_carried_state_of_two_chunks():
    """Truncated sequences carry (h, c, n, m) from chunk to chunk; the gradient of the whole equals the
    chunk-wise reverse scan in which the second chunk's ds0 is the first chunk's extra cotangent on its
    last states (c and n included: the path that only a cotangent on c, n exercises)."""
    B, T, N, D = 2, 8, 1, 4
    inp = make_inputs("slstm", B, T, N, D, seed=32, init="randn", grad_on="h")
    Wx, R, b, s0, ds = (inp[k].to(DT) for k in ("Wx", "R", "b", "states", "dstates"))
    _, (dWx, dR, db, ds0) = flashrnn_oracle_fwbw_manual(Wx, R, b, s0, "slstm", ds)
    T1 = 5
    out1, _ = flashrnn_oracle_fwbw_manual(Wx[:, :T1], R, b, s0, "slstm", ds[:, :, :T1])
    mid = out1[:, :, -1:]
    _, (dWx2, dR2, db2, dmid) = flashrnn_oracle_fwbw_manual(Wx[:, T1:], R, b, mid, "slstm", ds[:, :, T1:])
    ds1 = ds[:, :, :T1].clone()
    ds1[:, :, -1] += dmid[:, :, 0]
    _, (dWx1, dR1, db1, ds0c) = flashrnn_oracle_fwbw_manual(Wx[:, :T1], R, b, s0, "slstm", ds1)
    assert float(dmid[1].abs().max()) > 0 and float(dmid[2].abs().max()) > 0
    assert torch.allclose(torch.cat([dWx1, dWx2], 1), dWx, atol=1e-11)
    assert torch.allclose(dR1 + dR2, dR, atol=1e-11) and torch.allclose(db1 + db2, db, atol=1e-11)
    assert torch.allclose(ds0c, ds0, atol=1e-11)


def test_slstm_backward_under_forward_clip_closed_form_scalar_cell():
    """A scalar sLSTM cell, zero initial state, two steps, forward_clipval active at step 1.  Every quantity
    is written out by hand from the native definitions: the forward pass clamps h after the cache is taken
    (slstm_fused_pointwise.cuh:96-109) and the adjoint reads the stored, clamped h where the unclamped
    derivative has o c / n (:154-166: dn -= dy/n * h, do = (1 - o) h dy), while dc keeps o/n."""
    sig = lambda x: 1.0 / (1.0 + math.exp(-x))
    lsig = lambda x: -math.log1p(math.exp(-x))
    clamp = lambda x, v: max(-v, min(v, x))
    v = 0.3
    w1, w2 = [0.4, 1.1, 1.7, 2.0], [-0.3, 0.6, -0.9, 0.5]      # Wx of the gates i, f, z, o at steps 1 and 2
    r, bb = [0.7, -0.5, 1.3, 0.9], [0.1, 0.2, -0.1, 0.05]     # recurrent weight and bias per gate
    g1, g2 = 0.8, -1.2                                         # cotangents of h_1, h_2
    # step 1: h_0 = 0, n_0 = 0 -> m_1 = i_1, ig = 1, c_1 = z_1, n_1 = 1
    i1, f1 = w1[0] + bb[0], w1[1] + bb[1]
    z1, o1 = math.tanh(w1[2] + bb[2]), sig(w1[3] + bb[3])
    m1, ig1, fg1 = i1, 1.0, math.exp(lsig(f1) - i1)
    c1, n1 = z1, 1.0
    y1 = o1 * c1 / n1
    h1 = clamp(y1, v)
    assert h1 == v and y1 > v                                  # the clamp is active
    # step 2
    i2, f2 = w2[0] + r[0] * h1 + bb[0], w2[1] + r[1] * h1 + bb[1]
    z2, o2 = math.tanh(w2[2] + r[2] * h1 + bb[2]), sig(w2[3] + r[3] * h1 + bb[3])
    lfm = lsig(f2) + m1
    m2 = max(i2, lfm)
    ig2, fg2 = math.exp(i2 - m2), math.exp(lfm - m2)
    c2 = fg2 * c1 + ig2 * z2
    n2 = max(fg2 * n1 + ig2, 1.0)
    y2 = o2 * c2 / n2
    h2 = clamp(y2, v)
    # reverse step 2
    dy = g2
    dc, dn = dy / n2 * o2, -dy / n2 * h2
    dg2 = [ig2 * (z2 * dc + dn), fg2 * (dc * c1 + dn * n1) * (1 - sig(f2)), dc * ig2 * (1 - z2 * z2), (1 - o2) * h2 * dy]
    dc1, dn1 = fg2 * dc, fg2 * dn
    dh1 = sum(rg * d for rg, d in zip(r, dg2))
    # reverse step 1 (c_0 = n_0 = 0, n_1 = 1)
    dy = g1 + dh1
    dc, dn = dc1 + dy * o1, dn1 - dy * h1
    dg1 = [ig1 * (z1 * dc + dn), 0.0, dc * ig1 * (1 - z1 * z1), (1 - o1) * h1 * dy]
    want_dR = [d * h1 for d in dg2]                            # h_0 = 0: only step 2 contributes
    want_db = [a + c for a, c in zip(dg1, dg2)]
    want_ds0 = [sum(rg * d for rg, d in zip(r, dg1)), fg1 * dc, fg1 * dn, 0.0]

    t = lambda x: torch.tensor(x, dtype=torch.float64)
    Wx = t([w1, w2]).reshape(1, 2, 4, 1, 1)
    R = t(r).reshape(4, 1, 1, 1)
    b = t(bb).reshape(4, 1, 1)
    s0 = torch.zeros(4, 1, 1, 1, 1, dtype=torch.float64)
    ds = torch.zeros(4, 1, 2, 1, 1, dtype=torch.float64)
    ds[0, 0, 0], ds[0, 0, 1] = g1, g2
    out, (dWx, dR, db, ds0) = flashrnn_oracle_fwbw_manual(Wx, R, b, s0, "slstm", ds, forward_clipval=v)
    assert torch.allclose(out[:, 0, 0].flatten(), t([h1, c1, n1, m1]), atol=1e-14)
    assert torch.allclose(out[:, 0, 1].flatten(), t([h2, c2, n2, m2]), atol=1e-14)
    assert torch.allclose(dWx.flatten(), t(dg1 + dg2), atol=1e-13)
    assert torch.allclose(dR.flatten(), t(want_dR), atol=1e-13)
    assert torch.allclose(db.flatten(), t(want_db), atol=1e-13)
    assert torch.allclose(ds0.flatten(), t(want_ds0), atol=1e-13)
    # and the clamp does matter for the gradient: with the unclamped h in the adjoint dWx differs
    _, (dWx_plain, _, _, _) = flashrnn_oracle_fwbw_manual(Wx, R, b, s0, "slstm", ds)
    assert float((dWx_plain - dWx).abs().max()) > 1e-3


def test_slstm_first_step_branch_mixed_initial_n_differs_between_native_and_vanilla():
    """vanilla/slstm.py:21 takes m' = i only when EVERY n is zero; the native kernels (and the HIP kernels)
    decide per element (slstm_fused_pointwise.cuh:54-62).  With some initial n zero and some not the two
    differ, exactly at the elements whose n is zero: there vanilla uses max(i, logsig(f) + m)."""
    inp = make_inputs("slstm", 2, 2, 1, 4, seed=33, init="randn")
    s0 = inp["states"].clone()
    s0[:, 0, 0, 0, :2] = 0.0            # two elements of batch row 0 start fresh: h = c = n = m = 0
    inp["Wx"][0, 0, 0, 0, :2] = -4.0    # their input gate is far below log sigmoid(f) + m
    whole, _ = flashrnn_oracle(inp["Wx"], inp["R"], inp["b"], s0, "slstm")
    per, _ = flashrnn_oracle(inp["Wx"], inp["R"], inp["b"], s0, "slstm", slstm_per_element_first_step=True)
    diff = (whole - per).abs()[:, :, 0]                       # first step, [S,B,N,D]
    raw = inp["Wx"][:, 0] + torch.einsum("bnp,gndp->bgnd", s0[0, :, 0], inp["R"]) + inp["b"][None]
    fresh_and_lfm_wins = (s0[2, :, 0] == 0) & (torch.nn.functional.logsigmoid(raw[:, 1]) + s0[3, :, 0] > raw[:, 0])
    assert bool(fresh_and_lfm_wins.any())
    assert bool((diff[3] > 0)[fresh_and_lfm_wins].all())       # m' differs where the fresh element's i loses
    assert float(diff[3][~fresh_and_lfm_wins].max()) == 0.0    # and nowhere else
    # h differs there too: n' = max(ig, 1) = 1 hides the scale exp(i - m') < 1 that c' = ig tanh(z) carries
    i, f, z, o = raw.unbind(1)
    fresh = fresh_and_lfm_wins
    h_native = torch.sigmoid(o) * torch.tanh(z)                # the closed form of a first step: m' = i, ig = 1
    h_vanilla = h_native * torch.exp(i - torch.nn.functional.logsigmoid(f))   # m' = logsig(f) + 0, ig = exp(i - m')
    assert torch.allclose(per[0, :, 0][fresh], h_native[fresh], atol=1e-6)
    assert torch.allclose(whole[0, :, 0][fresh], h_vanilla[fresh], atol=1e-6)
