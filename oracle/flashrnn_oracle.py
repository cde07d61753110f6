"""CPU restatement of the FlashRNN recurrence (the ``vanilla`` backend of the reference).

TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the timed CPU baseline.
The shipped package never imports this file.

What follows the reference, and where:

* ``flashrnn_oracle``          -- the time loop of flashrnn/flashrnn/vanilla/__init__.py:20-70
  (only state 0 feeds the recurrence, ``Ry[b,g,n,d] = sum_p h[b,n,p] R[g,n,d,p]``) behind
  the public layouts of flashrnn/flashrnn/flashrnn.py:1114-1135 (``Wx [B,T,G_w,N,D]``,
  ``R [G_r,N,D,P]``, ``b [G_t,N,D]``, ``states [S,B,1,N,D]`` -> ``([S,B,T,N,D], [S,B,1,N,D])``).
* ``_pw_lstm``                 -- flashrnn/flashrnn/vanilla/lstm.py:16-29
* ``_pw_gru``                  -- flashrnn/flashrnn/vanilla/gru.py:16-32
* ``_pw_elman``                -- flashrnn/flashrnn/vanilla/elman.py:16-23
* ``_pw_slstm``                -- flashrnn/flashrnn/vanilla/slstm.py:15-35
* ``FUNCTIONS``                -- flashrnn/flashrnn/flashrnn.py:49-71
* ``zero_state``               -- flashrnn/flashrnn/flashrnn.py:927-954
* ``flashrnn_oracle_fwbw_manual`` -- the hand-written reverse scan the native kernels run:
  sequence loop flashrnn/flashrnn/vanilla_fwbw/bw.py:19-97; per-function adjoints
  flashrnn/flashrnn/alternating/lstm_pointwise.cu:117-186, gru_pointwise.cu:120-193,
  slstm_pointwise.cu:135-214, elman_pointwise.cu:80-120 (and what each forward caches,
  same files, forward kernels).

* options ``forward_clipval`` / ``gradient_recurrent_clipval`` / ``gradient_recurrent_cut``
  -- what the native pointwise functions do under FLASHRNN_FORWARD_CLIPVAL_VALID and
  FLASHRNN_GRADIENT_RECURRENT_CLIPVAL_VALID (flashrnn/flashrnn/fused/lstm_fused_pointwise.cuh:75-80,
  115-121 and the same lines of the gru/elman/slstm files) and what ``backward_cut`` leaves out
  (flashrnn/flashrnn/fused/flashrnn_fused_backward_cut.cu:89-178: no ``dg R^T`` term).  Each option
  has its own value here; the reference feeds ``gradient_recurrent_clipval`` into both defines
  (flashrnn/flashrnn/flashrnn.py:361-382).

Pinning (tests/test_oracle_*.py, none of them re-types these formulas):
  LSTM / GRU / Elman forward and all gradients against torch.nn.LSTM / GRU / RNN;
  sLSTM forward against an un-stabilised float64 brute-force recurrence, the T=1 closed
  form and its invariants; every manual adjoint against float64 autograd of the forward;
  recurrence glue by the chunked-sequence invariant and non-symmetric R with N > 1;
  the three options by hand-derived closed forms on a scalar Elman cell, by the agreement of
  the autograd formulation (identity-forward / clamp-backward node, detach) with the explicit
  reverse scan, and by their no-op limits (huge clip value, R = 0).
  the sLSTM backward under ``forward_clipval`` (the native adjoint reads the stored, clamped h,
  slstm_fused_pointwise.cuh:117-186, which only ``flashrnn_oracle_fwbw_manual`` restates) by a closed
  form derived by hand on a scalar cell over two steps with the clamp active;
  the sLSTM adjoint for cotangents on c and n (stabiliser held constant) by float64 autograd with the
  stabiliser detached.
  The reference holds no golden vectors for this path (its only known-answer test is
  flashrnn/tests/test_lstm.py:70-115, LSTM vs torch.nn.LSTM, which is reproduced).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

# function -> (G_r, G_w, G_i, G_t, S)        flashrnn/flashrnn/flashrnn.py:49-71
FUNCTIONS = {
    "slstm": (4, 4, 4, 4, 4),
    "lstm": (4, 4, 4, 4, 2),
    "gru": (3, 3, 4, 4, 1),
    "elman": (1, 1, 1, 1, 1),
}


def zero_state(function: str, Wx: torch.Tensor) -> torch.Tensor:
    """Default initial state ``[S,B,1,N,D]`` of zeros (flashrnn.py:927-954)."""
    S = FUNCTIONS[function][4]
    B, _, _, N, D = Wx.shape
    return torch.zeros((S, B, 1, N, D), dtype=Wx.dtype, device=Wx.device)


# ----------------------------------------------------------------------------------------
# pointwise forward, one time step.  Wx_t [B,G_w,N,D], Ry [B,G_r,N,D], b [G_t,N,D],
# s: tuple of S tensors [B,N,D].  Returns tuple of S new states.
# ----------------------------------------------------------------------------------------
def _pw_lstm(Wx_t, Ry, b, s):
    raw = Wx_t + Ry + b[None]
    i, f, z, o = raw.unbind(1)
    c = s[1]
    c_new = torch.sigmoid(f) * c + torch.sigmoid(i) * torch.tanh(z)
    h_new = torch.sigmoid(o) * torch.tanh(c_new)
    return (h_new, c_new)


def _pw_gru(Wx_t, Ry, b, s):
    # R gates [g, r, z]; Wx gates [r, z, n]; b gates [g, r, z, n]
    g = Ry[:, 0] + b[0]
    r = torch.sigmoid(Wx_t[:, 0] + Ry[:, 1] + b[1])
    z = torch.sigmoid(Wx_t[:, 1] + Ry[:, 2] + b[2])
    n = Wx_t[:, 2] + b[3]
    h = s[0]
    return (z * h + (1 - z) * torch.tanh(n + r * g),)


def _pw_elman(Wx_t, Ry, b, s):
    return (torch.tanh(Wx_t[:, 0] + Ry[:, 0] + b[0]),)


def _pw_slstm(Wx_t, Ry, b, s, per_element_first_step=False, detach_m=False):
    raw = Wx_t + Ry + b[None]
    i, f, z, o = raw.unbind(1)
    _, c, n, m = s
    if detach_m:
        # the native adjoint holds the stabiliser constant: no cotangent enters m_t or leaves through
        # m_{t-1} (slstm_fused_pointwise.cuh:117-186 differentiates exp(i - m') and exp(logsig(f) + m - m')
        # with m, m' fixed and returns ds[3] = 0).  For a loss on h this is the full gradient (h does not
        # depend on m); for a loss on c or n, which scale with exp(-m), it is not.
        m = m.detach()
    lfm = F.logsigmoid(f) + m
    if per_element_first_step:
        # what the native kernels test (slstm_fused_pointwise.cuh:54-62)
        m_new = torch.where(n == 0.0, i, torch.maximum(i, lfm))
    elif bool(torch.all(n == 0.0)):  # over the whole tensor: vanilla/slstm.py:21
        m_new = i
    else:
        m_new = torch.maximum(i, lfm)
    if detach_m:
        m_new = m_new.detach()
    ig = torch.exp(i - m_new)
    fg = torch.exp(lfm - m_new)
    c_new = fg * c + ig * torch.tanh(z)
    n_raw = fg * n + ig
    n_new = torch.maximum(n_raw, torch.ones_like(n))
    if detach_m:
        # the native adjoint differentiates n' = fg n + ig and ignores the guard max(., 1), which is never
        # strictly active on reachable states ("n cannot get smaller than one by construction",
        # slstm_fused_pointwise.cuh:90-92) but ties at the very first step (n' = 0 + 1), where autograd
        # would halve the slope
        n_new = n_raw + (n_new - n_raw).detach()
    h_new = torch.sigmoid(o) * c_new / n_new
    return (h_new, c_new, n_new, m_new)


_PW = {"lstm": _pw_lstm, "gru": _pw_gru, "elman": _pw_elman, "slstm": _pw_slstm}


class _ClampGrad(torch.autograd.Function):
    """Identity whose cotangent is clamped to [-c, c]: the clip the native backward pointwise
    functions apply to the gradient carried into h_t from step t+1 (lstm_fused_pointwise.cuh:115-121)."""

    @staticmethod
    def forward(ctx, x, c):
        ctx.c = c
        return x.view_as(x)

    @staticmethod
    def backward(ctx, g):
        return g.clamp(-ctx.c, ctx.c), None


def flashrnn_oracle(
    Wx: torch.Tensor,
    R: torch.Tensor,
    b: torch.Tensor,
    states: Optional[torch.Tensor] = None,
    function: str = "lstm",
    slstm_per_element_first_step: bool = False,
    slstm_detach_m: bool = False,
    forward_clipval: Optional[float] = None,
    gradient_recurrent_clipval: Optional[float] = None,
    gradient_recurrent_cut: bool = False,
):
    """Differentiable CPU forward in the arithmetic of ``Wx.dtype``.

    ``forward_clipval``: the new h of every step is clamped to [-v, v]; the backward pass does not
    see the clamp (straight-through), as the native backward pointwise functions do not.
    ``slstm_detach_m``: differentiation as the native adjoint does it (values unchanged): the stabiliser
    state is held constant and the guard max(., 1) on n is transparent.
    ``gradient_recurrent_clipval``: the cotangent that step t+1 sends to h_t (through R and through
    the pointwise carry) is clamped before the upstream cotangent of h_t is added; the cotangent
    of the initial state is not clamped.  ``gradient_recurrent_cut``: no gradient through R h.

    Returns ``(all_states [S,B,T,N,D], last_states [S,B,1,N,D])``.
    """
    Gr, Gw, _, Gt, S = FUNCTIONS[function]
    B, T, gw, N, D = Wx.shape
    assert gw == Gw and tuple(R.shape) == (Gr, N, D, D) and tuple(b.shape) == (Gt, N, D)
    if states is None:
        states = zero_state(function, Wx)
    assert tuple(states.shape) == (S, B, 1, N, D)
    s = tuple(states[k, :, 0] for k in range(S))
    # [N, P, G_r*D]: one batched matmul per step, as vanilla/__init__.py:53-61
    Rm = R.permute(1, 3, 0, 2).reshape(N, D, Gr * D)
    pw = _PW[function]
    outs = []
    # one unbind instead of Wx[:, t] per step: the same values, but the backward of T selects builds T
    # full-size zero tensors (quadratic in T; 16x slower at T = 2048), that of unbind one stack
    Wx_t = Wx.unbind(1)
    for t in range(T):
        s_in = s
        if gradient_recurrent_clipval is not None and t > 0:
            s_in = (_ClampGrad.apply(s[0], float(gradient_recurrent_clipval)),) + tuple(s[1:])
        h_rec = s_in[0].detach() if gradient_recurrent_cut else s_in[0]
        Ry = torch.matmul(h_rec.transpose(0, 1), Rm)  # [N,B,G_r*D]
        Ry = Ry.reshape(N, B, Gr, D).permute(1, 2, 0, 3)  # [B,G_r,N,D]
        if function == "slstm":
            s = pw(Wx_t[t], Ry, b, s_in, slstm_per_element_first_step, slstm_detach_m)
        else:
            s = pw(Wx_t[t], Ry, b, s_in)
        if forward_clipval is not None:
            h = s[0]
            s = (h + (h.clamp(-forward_clipval, forward_clipval) - h).detach(),) + tuple(s[1:])
        outs.append(torch.stack(s, 0))  # [S,B,N,D]
    all_states = torch.stack(outs, 2)  # [S,B,T,N,D]
    return all_states, all_states[:, :, -1:]


def flashrnn_oracle_backward(Wx, R, b, states, function, dstates, **kw):
    """Autograd gradients of ``sum(all_states * dstates)`` w.r.t. (Wx, R, b, states)."""
    leaves = [x.detach().clone().requires_grad_(True) for x in (Wx, R, b, states)]
    out, _ = flashrnn_oracle(leaves[0], leaves[1], leaves[2], leaves[3], function, **kw)
    grads = torch.autograd.grad(out, leaves, grad_outputs=dstates, allow_unused=True)
    # a leaf without a path to the output (the initial state of an Elman cell under
    # gradient_recurrent_cut) has a zero gradient
    grads = tuple(torch.zeros_like(x) if g is None else g for g, x in zip(grads, leaves))
    return out.detach(), grads


# ----------------------------------------------------------------------------------------
# The explicit forward-with-cache + reverse scan that the native kernels implement.
# ----------------------------------------------------------------------------------------
def _fw_cache(function, Wx_t, Ry, b, s):
    """One step; returns (new states tuple, cache tuple) with the kernels' cache contents."""
    if function == "lstm":
        raw = Wx_t + Ry + b[None]
        i, f, z, o = (torch.sigmoid(raw[:, 0]), torch.sigmoid(raw[:, 1]),
                      torch.tanh(raw[:, 2]), torch.sigmoid(raw[:, 3]))
        c_new = f * s[1] + i * z
        return (o * torch.tanh(c_new), c_new), (i, f, z, o)
    if function == "slstm":
        raw = Wx_t + Ry + b[None]
        i, f, zr, orr = raw.unbind(1)
        _, c, n, m = s
        lfm = F.logsigmoid(f) + m
        m_new = torch.where(n == 0.0, i, torch.maximum(i, lfm))
        ig, fg = torch.exp(i - m_new), torch.exp(lfm - m_new)
        z, o = torch.tanh(zr), torch.sigmoid(orr)
        c_new = fg * c + ig * z
        n_new = torch.maximum(fg * n + ig, torch.ones_like(n))
        return (o * c_new / n_new, c_new, n_new, m_new), (ig, f, z, o)
    if function == "gru":
        g = Ry[:, 0] + b[0]
        r = torch.sigmoid(Wx_t[:, 0] + Ry[:, 1] + b[1])
        z = torch.sigmoid(Wx_t[:, 1] + Ry[:, 2] + b[2])
        n = Wx_t[:, 2] + b[3]
        return (z * s[0] + (1 - z) * torch.tanh(n + r * g),), (g, r, z, n)
    if function == "elman":
        h = torch.tanh(Wx_t[:, 0] + Ry[:, 0] + b[0])
        return (h,), (h,)
    raise KeyError(function)


def _bw_pointwise(function, cache, s_prev, s_new, ds_out, ds_run):
    """One reverse step.  Returns (dg_r list, dg_w list, dg_b list, new running ds list);
    the recurrent term R^T dg_r is added to ds[0] by the caller."""
    dy = ds_out[0] + ds_run[0]
    zero = torch.zeros_like(dy)
    if function == "lstm":
        i, f, z, o = cache
        dc = ds_out[1] + ds_run[1]
        tc = torch.tanh(s_new[1])
        dc = dc + (1 - tc * tc) * o * dy
        dg = [i * (1 - i) * z * dc, f * (1 - f) * s_prev[1] * dc,
              (1 - z * z) * i * dc, o * (1 - o) * tc * dy]
        return dg, dg, dg, [zero, f * dc]
    if function == "slstm":
        ig, fraw, z, o = cache
        dc = ds_out[1] + ds_run[1]
        dn = ds_out[2] + ds_run[2]
        y_new, n_new, m_new = s_new[0], s_new[2], s_new[3]
        c_cur, n_cur, m_cur = s_prev[1], s_prev[2], s_prev[3]
        fg = torch.exp(F.logsigmoid(fraw) + m_cur - m_new)
        fsig = torch.sigmoid(fraw)
        dyi = dy / n_new
        dc = dc + dyi * o
        dn = dn - dyi * y_new
        dg = [ig * (z * dc + dn), fg * (dc * c_cur + dn * n_cur) * (1 - fsig),
              dc * ig * (1 - z * z), (1 - o) * y_new * dy]
        return dg, dg, dg, [zero, fg * dc, fg * dn, zero]
    if function == "gru":
        g, r, z, nraw = cache
        nval = torch.tanh(nraw + r * g)
        dz = z * (1 - z) * dy * (s_prev[0] - nval)
        dn = dy * (1 - z) * (1 - nval * nval)
        dr = dn * g * r * (1 - r)
        dgg = dn * r
        return [dgg, dr, dz], [dr, dz, dn], [dgg, dr, dz, dn], [z * dy]
    if function == "elman":
        (y,) = cache
        dg = [(1 - y * y) * dy]
        return dg, dg, dg, [zero]
    raise KeyError(function)


def flashrnn_oracle_fwbw_manual(Wx, R, b, states, function, dstates, forward_clipval=None,
                                gradient_recurrent_clipval=None, gradient_recurrent_cut=False):
    """Forward with gate cache, then the explicit reverse scan; no autograd.

    Returns ``(all_states [S,B,T,N,D], (dWx, dR, db, dstates0 [S,B,1,N,D]))``.
    """
    Gr, Gw, _, Gt, S = FUNCTIONS[function]
    B, T, _, N, D = Wx.shape
    with torch.no_grad():
        s = tuple(states[k, :, 0] for k in range(S))
        traj, caches = [s], []
        for t in range(T):
            Ry = torch.einsum("bnp,gndp->bgnd", s[0], R)
            s, cache = _fw_cache(function, Wx[:, t], Ry, b, s)
            if forward_clipval is not None:  # after the cache is taken: the cache holds unclipped gates
                s = (s[0].clamp(-forward_clipval, forward_clipval),) + tuple(s[1:])
            traj.append(s)
            caches.append(cache)
        out = torch.stack([torch.stack(x, 0) for x in traj[1:]], 2)
        ds = [torch.zeros_like(s[0]) for _ in range(S)]
        dWx = torch.zeros_like(Wx)
        dR = torch.zeros_like(R)
        db = torch.zeros_like(b)
        for t in range(T - 1, -1, -1):
            ds_out = [dstates[k, :, t] for k in range(S)]
            if gradient_recurrent_clipval is not None:
                ds[0] = ds[0].clamp(-gradient_recurrent_clipval, gradient_recurrent_clipval)
            dg_r, dg_w, dg_b, ds = _bw_pointwise(function, caches[t], traj[t], traj[t + 1], ds_out, ds)
            dg_r = torch.stack(dg_r, 1)  # [B,G_r,N,D]
            if not gradient_recurrent_cut:
                ds[0] = ds[0] + torch.einsum("bgnd,gndp->bnp", dg_r, R)
            dR += torch.einsum("bgnd,bnp->gndp", dg_r, traj[t][0])
            dWx[:, t] = torch.stack(dg_w, 1)
            db += torch.stack(dg_b, 1).sum(0)
        ds0 = torch.stack(ds, 0)[:, :, None]
    return out, (dWx, dR, db, ds0)


# ----------------------------------------------------------------------------------------
# Seeded synthetic inputs: one generator, fixed draw order Wx, R, b, states, cotangents.
# ----------------------------------------------------------------------------------------
def make_inputs(function, B, T, N, D, seed, init="zeros", round_to=None, grad_on="all",
                forget_bias_linspace=False):
    """fp32 CPU tensors: Wx ~ N(0,1), R ~ N(0,1/D), b ~ N(0, std 0.1), states zeros or N(0,1),
    cotangent ~ N(0,1) on all states ("all") or on h only ("h").  ``round_to=torch.bfloat16``
    rounds every tensor to bf16-representable values (still stored as fp32) so that a bf16
    kernel and the fp32 oracle see identical inputs."""
    Gr, Gw, _, Gt, S = FUNCTIONS[function]
    g = torch.Generator(device="cpu").manual_seed(seed)
    Wx = torch.randn((B, T, Gw, N, D), generator=g)
    R = torch.randn((Gr, N, D, D), generator=g) / (D ** 0.5)
    b = torch.randn((Gt, N, D), generator=g) * 0.1
    s0 = torch.randn((S, B, 1, N, D), generator=g)
    ds = torch.randn((S, B, T, N, D), generator=g)
    if init == "zeros":
        s0 = torch.zeros_like(s0)
    elif function == "slstm":
        # a reachable sLSTM state: n >= 1 (vanilla/slstm.py:29), any m
        s0[2] = s0[2].abs() + 1.0
    if grad_on == "h":
        ds[1:] = 0
    if forget_bias_linspace:
        b[1] = torch.linspace(3.0, 6.0, N * D).reshape(N, D)
    if round_to is not None:
        Wx, R, b, s0, ds = (x.to(round_to).float() for x in (Wx, R, b, s0, ds))
    return dict(Wx=Wx, R=R, b=b, states=s0, dstates=ds)
