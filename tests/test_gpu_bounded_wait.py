"""The waits between the workgroups of a head are bounded: when one runs out, every kernel still
ends normally, the status word says so, the affected outputs are NaN and the Python layer raises
RuntimeError at the next call or at check_status().  The condition is forced from the host with
FRNN_SPIN_LIMIT=-2 (every wait then gives up at once, before its first probe); nothing on the GPU
faults or hangs."""
import pytest
import torch

from oracle import make_inputs

pytestmark = pytest.mark.gpu


KDT = {"bfloat16": torch.bfloat16, "float32": torch.float32}
# (the fp32 case and bf16 D = 1024: the kernels whose waves work in pairs, 14 and 32 workgroups per head, where the second
# wave of a pair takes part in every barrier of the first and must leave the time loop with it)
SHAPES = [("bfloat16", 256), ("float32", 448), ("bfloat16", 1024), ("float32", 1024)]


def _forward(gpu, inp, grad, dtype="bfloat16"):
    from flashrnn_amd import flashrnn

    Wx = inp["Wx"].to(gpu, KDT[dtype]).requires_grad_(grad)
    b = inp["b"].to(gpu, KDT[dtype]).requires_grad_(grad)
    st, _ = flashrnn(Wx, inp["R"].to(gpu, KDT[dtype]), b, None,
                     function="lstm", backend="hip_fused", dtype=dtype)
    return Wx, b, st


def _call(gpu, inp, grad, dtype="bfloat16"):
    Wx, b, st = _forward(gpu, inp, grad, dtype)
    grads = torch.autograd.grad(st, [Wx, b], grad_outputs=torch.ones_like(st)) if grad else None
    torch.cuda.synchronize()
    return st.detach().float(), grads


@pytest.mark.parametrize("dtype,D", SHAPES)
def test_expired_wait_in_forward_raises_at_the_next_call(gpu, monkeypatch, dtype, D):
    from flashrnn_amd import check_status, last_status

    B, T, N = 8, 64, 1   # 4 (14) workgroups per head: every step has a wait
    print(f"case bounded-wait forward lstm {dtype} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs("lstm", B, T, N, D, 5, init="zeros", round_to=torch.bfloat16)
    good, _ = _call(gpu, inp, False, dtype)
    check_status()
    assert torch.isfinite(good).all()

    monkeypatch.setenv("FRNN_SPIN_LIMIT", "-2")
    bad, _ = _call(gpu, inp, False, dtype)             # returns: every wave left its time loop
    assert torch.isnan(bad[0]).all()                   # h of every workgroup: all of them gave up
    assert last_status("forward") == 1
    monkeypatch.delenv("FRNN_SPIN_LIMIT")
    with pytest.raises(RuntimeError, match="bounded wait"):
        _call(gpu, inp, False, dtype)                  # the next call finds the failed one (it has finished)
    check_status()                                     # reported once
    again, _ = _call(gpu, inp, False, dtype)           # and the call after that is clean
    check_status()
    assert torch.equal(again, good)


@pytest.mark.parametrize("dtype,D", SHAPES)
def test_expired_wait_in_backward_is_reported_by_check_status(gpu, monkeypatch, dtype, D):
    from flashrnn_amd import check_status, last_status

    B, T, N = 8, 64, 1
    print(f"case bounded-wait backward lstm {dtype} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs("lstm", B, T, N, D, 5, init="zeros", round_to=torch.bfloat16)
    good, good_g = _call(gpu, inp, True, dtype)
    check_status()

    Wx, b, st = _forward(gpu, inp, True, dtype)        # a good forward
    torch.cuda.synchronize()
    monkeypatch.setenv("FRNN_SPIN_LIMIT", "-2")
    grads = torch.autograd.grad(st, [Wx, b], grad_outputs=torch.ones_like(st))   # a backward whose waits give up
    monkeypatch.delenv("FRNN_SPIN_LIMIT")
    torch.cuda.synchronize()
    assert last_status("forward") == 0 and last_status("backward") == 1
    assert torch.isnan(grads[1].float()).all()         # db of every workgroup
    with pytest.raises(RuntimeError, match=f"backward of lstm B8 T64 N1 D{D}"):
        check_status()
    again, again_g = _call(gpu, inp, True, dtype)
    check_status()
    assert torch.equal(again, good) and all(torch.equal(x, y) for x, y in zip(again_g, good_g))
