"""Fused calls that overlap on one device.  The workgroups of a head that spans several of them wait for each
other and a launch is sized to the device, so two such kernels running at once could starve each other; the
library orders multi-workgroup launches of different streams behind each other on the device (an event wait,
nothing blocks on the host).  No environment variable is set here: this is the default behaviour."""
import pytest
import torch

from oracle import make_inputs

pytestmark = pytest.mark.gpu


def _leaves(gpu, inp):
    return [inp[k].to(gpu, torch.bfloat16).requires_grad_(True) for k in ("Wx", "R", "b", "states")]


def _fwd_bwd(leaves, ds):
    from flashrnn_amd import flashrnn

    out, _ = flashrnn(*leaves, function="lstm", backend="hip_fused", dtype="bfloat16")
    return (out,) + tuple(torch.autograd.grad(out, leaves, grad_outputs=ds))


@pytest.mark.parametrize("B,T,N,D", [
    (8, 1024, 3, 256),    # the metric configuration: 24 workgroups per kernel
    (256, 64, 3, 256),    # 192 workgroups per kernel: two kernels do not fit the device together
])
def test_two_streams_get_the_single_stream_bits(gpu, B, T, N, D):
    from flashrnn_amd import check_status

    print(f"case overlap lstm B{B} T{T} N{N} D{D}", flush=True)
    inps = [make_inputs("lstm", B, T, N, D, 40 + i, init="randn", round_to=torch.bfloat16) for i in range(2)]
    leaves = [_leaves(gpu, inp) for inp in inps]
    ds = [inp["dstates"].to(gpu, torch.bfloat16) for inp in inps]
    ref = [_fwd_bwd(leaves[i], ds[i]) for i in range(2)]          # one after the other on the current stream
    torch.cuda.synchronize()
    check_status()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        got = [None, None]
        for i in (0, 1):                                           # both issued before either is waited for
            with torch.cuda.stream(streams[i]):
                got[i] = _fwd_bwd(leaves[i], ds[i])
        torch.cuda.synchronize()
        check_status()
        for i in (0, 1):
            for name, a, r in zip(("states", "dWx", "dR", "db", "ds0"), got[i], ref[i]):
                assert torch.equal(a, r), f"repetition {rep}, stream {i}: {name} differs from the single-stream run"


def test_two_threads_two_streams(gpu):
    """The same from two host threads (forward on the calling thread, backward on autograd's)."""
    import threading

    from flashrnn_amd import check_status

    B, T, N, D = 64, 128, 3, 256
    print(f"case overlap threads lstm B{B} T{T} N{N} D{D}", flush=True)
    inps = [make_inputs("lstm", B, T, N, D, 50 + i, init="randn", round_to=torch.bfloat16) for i in range(2)]
    leaves = [_leaves(gpu, inp) for inp in inps]
    ds = [inp["dstates"].to(gpu, torch.bfloat16) for inp in inps]
    ref = [_fwd_bwd(leaves[i], ds[i]) for i in range(2)]
    torch.cuda.synchronize()
    got, errs = [None, None], []

    def work(i):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for _ in range(4):
                    got[i] = _fwd_bwd(leaves[i], ds[i])
                torch.cuda.current_stream().synchronize()
        except Exception as e:  # surfaced on the main thread below
            errs.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errs, errs
    torch.cuda.synchronize()
    check_status()
    for i in (0, 1):
        for name, a, r in zip(("states", "dWx", "dR", "db", "ds0"), got[i], ref[i]):
            assert torch.equal(a, r), f"thread {i}: {name} differs from the single-stream run"
