"""The waits between the workgroups of a head are bounded: when one runs out, every kernel still
ends normally, the status word says so, the affected outputs are NaN and the Python layer raises
RuntimeError at the next call or at check_status().  The condition is forced from the host with
FRNN_SPIN_LIMIT=-2 (every wait then gives up at once, before its first probe); nothing on the GPU
faults or hangs."""
import pytest
import torch

from oracle import make_inputs

pytestmark = pytest.mark.gpu


def _forward(gpu, inp, grad):
    from flashrnn_amd import flashrnn

    Wx = inp["Wx"].to(gpu, torch.bfloat16).requires_grad_(grad)
    b = inp["b"].to(gpu, torch.bfloat16).requires_grad_(grad)
    st, _ = flashrnn(Wx, inp["R"].to(gpu, torch.bfloat16), b, None,
                     function="lstm", backend="hip_fused", dtype="bfloat16")
    return Wx, b, st


def _call(gpu, inp, grad):
    Wx, b, st = _forward(gpu, inp, grad)
    grads = torch.autograd.grad(st, [Wx, b], grad_outputs=torch.ones_like(st)) if grad else None
    torch.cuda.synchronize()
    return st.detach().float(), grads


def test_expired_wait_in_forward_raises_at_the_next_call(gpu, monkeypatch):
    from flashrnn_amd import check_status, last_status

    B, T, N, D = 8, 64, 1, 256   # 4 workgroups per head: every step has a wait
    print(f"case bounded-wait forward lstm B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs("lstm", B, T, N, D, 5, init="zeros", round_to=torch.bfloat16)
    good, _ = _call(gpu, inp, False)
    check_status()
    assert torch.isfinite(good).all()

    monkeypatch.setenv("FRNN_SPIN_LIMIT", "-2")
    bad, _ = _call(gpu, inp, False)                    # returns: every wave left its time loop
    assert torch.isnan(bad[0]).all()                   # h of every workgroup: all of them gave up
    assert last_status("forward") == 1
    monkeypatch.delenv("FRNN_SPIN_LIMIT")
    with pytest.raises(RuntimeError, match="bounded wait"):
        _call(gpu, inp, False)                         # the next call finds the failed one (it has finished)
    check_status()                                     # reported once
    again, _ = _call(gpu, inp, False)                  # and the call after that is clean
    check_status()
    assert torch.equal(again, good)


def test_expired_wait_in_backward_is_reported_by_check_status(gpu, monkeypatch):
    from flashrnn_amd import check_status, last_status

    B, T, N, D = 8, 64, 1, 256
    print(f"case bounded-wait backward lstm B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs("lstm", B, T, N, D, 5, init="zeros", round_to=torch.bfloat16)
    good, good_g = _call(gpu, inp, True)
    check_status()

    Wx, b, st = _forward(gpu, inp, True)               # a good forward
    torch.cuda.synchronize()
    monkeypatch.setenv("FRNN_SPIN_LIMIT", "-2")
    grads = torch.autograd.grad(st, [Wx, b], grad_outputs=torch.ones_like(st))   # a backward whose waits give up
    monkeypatch.delenv("FRNN_SPIN_LIMIT")
    torch.cuda.synchronize()
    assert last_status("forward") == 0 and last_status("backward") == 1
    assert torch.isnan(grads[1].float()).all()         # db of every workgroup
    with pytest.raises(RuntimeError, match="backward of lstm B8 T64 N1 D256"):
        check_status()
    again, again_g = _call(gpu, inp, True)
    check_status()
    assert torch.equal(again, good) and all(torch.equal(x, y) for x, y in zip(again_g, good_g))
