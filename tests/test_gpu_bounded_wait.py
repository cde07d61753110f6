"""The waits between the workgroups of a head are bounded: when one runs out, every kernel still
ends normally, the status word says so and the affected outputs are NaN.  The condition is forced
from the host with a spin limit below zero (a wait then gives up after its first unsuccessful
probe); nothing on the GPU faults or hangs."""
import pytest
import torch

from oracle import make_inputs

pytestmark = pytest.mark.gpu


def _call(gpu, inp, grad):
    from flashrnn_amd import flashrnn

    Wx = inp["Wx"].to(gpu, torch.bfloat16).requires_grad_(grad)
    st, _ = flashrnn(Wx, inp["R"].to(gpu, torch.bfloat16), inp["b"].to(gpu, torch.bfloat16), None,
                     function="lstm", backend="hip_fused", dtype="bfloat16")
    dWx = None
    if grad:
        (dWx,) = torch.autograd.grad(st, [Wx], grad_outputs=torch.ones_like(st))
    torch.cuda.synchronize()
    return st.detach().float(), dWx


@pytest.mark.parametrize("grad", [False, True])
def test_expired_wait_ends_the_kernels_and_is_reported(gpu, monkeypatch, grad):
    from flashrnn_amd.flashrnn import last_status

    B, T, N, D = 8, 64, 1, 256   # 4 workgroups per head: every step has a wait
    print(f"case bounded-wait lstm B{B} T{T} N{N} D{D} grad={grad}", flush=True)
    inp = make_inputs("lstm", B, T, N, D, 5, init="zeros", round_to=torch.bfloat16)
    good, good_dWx = _call(gpu, inp, grad)
    assert last_status("forward") == 0 and torch.isfinite(good).all()

    monkeypatch.setenv("FRNN_SPIN_LIMIT", "-1")
    bad, bad_dWx = _call(gpu, inp, grad)               # returns: every wave left its time loop
    fwd_status = last_status("forward")
    assert fwd_status in (0, 1)
    if fwd_status == 1:
        assert torch.isnan(bad[0]).any()               # h of the workgroups that gave up
    else:                                              # every first probe found its data: a normal run
        assert torch.equal(bad, good)
    if grad:
        bwd_status = last_status("backward")
        assert bwd_status in (0, 1)
        if fwd_status == 0 and bwd_status == 0:
            assert torch.equal(bad_dWx, good_dWx)
    # over 64 steps and 16 waves some first probe comes too early
    assert fwd_status == 1 or (grad and last_status("backward") == 1)

    monkeypatch.delenv("FRNN_SPIN_LIMIT")
    again, again_dWx = _call(gpu, inp, grad)           # the next call starts clean
    assert last_status("forward") == 0 and torch.equal(again, good)
    if grad:
        assert last_status("backward") == 0 and torch.equal(again_dWx, good_dWx)
