"""The waits between the workgroups of a head are bounded: when one runs out, every kernel still
ends normally, the status word says so and the affected outputs are NaN.  The condition is forced
from the host with FRNN_SPIN_LIMIT=-2 (every wait then gives up at once, before its first probe);
nothing on the GPU faults or hangs."""
import pytest
import torch

from oracle import make_inputs

pytestmark = pytest.mark.gpu


def _call(gpu, inp, grad):
    from flashrnn_amd import flashrnn

    Wx = inp["Wx"].to(gpu, torch.bfloat16).requires_grad_(grad)
    b = inp["b"].to(gpu, torch.bfloat16).requires_grad_(grad)
    st, _ = flashrnn(Wx, inp["R"].to(gpu, torch.bfloat16), b, None,
                     function="lstm", backend="hip_fused", dtype="bfloat16")
    grads = None
    if grad:
        grads = torch.autograd.grad(st, [Wx, b], grad_outputs=torch.ones_like(st))
    torch.cuda.synchronize()
    return st.detach().float(), grads


@pytest.mark.parametrize("grad", [False, True])
def test_expired_wait_ends_the_kernels_and_is_reported(gpu, monkeypatch, grad):
    from flashrnn_amd.flashrnn import last_status

    B, T, N, D = 8, 64, 1, 256   # 4 workgroups per head: every step has a wait
    print(f"case bounded-wait lstm B{B} T{T} N{N} D{D} grad={grad}", flush=True)
    inp = make_inputs("lstm", B, T, N, D, 5, init="zeros", round_to=torch.bfloat16)
    good, good_g = _call(gpu, inp, grad)
    assert last_status("forward") == 0 and torch.isfinite(good).all()

    monkeypatch.setenv("FRNN_SPIN_LIMIT", "-2")
    bad, bad_g = _call(gpu, inp, grad)               # returns: every wave left its time loop
    assert last_status("forward") == 1
    assert torch.isnan(bad[0]).all()                   # h of every workgroup: all of them gave up
    if grad:
        assert last_status("backward") == 1 and torch.isnan(bad_g[1].float()).all()   # db of every workgroup

    monkeypatch.delenv("FRNN_SPIN_LIMIT")
    again, again_g = _call(gpu, inp, grad)           # the next call starts clean
    assert last_status("forward") == 0 and torch.equal(again, good)
    if grad:
        assert last_status("backward") == 0 and all(torch.equal(x, y) for x, y in zip(again_g, good_g))
