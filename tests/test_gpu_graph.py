"""The entry points under HIP graph capture: a captured call (forward, or forward + backward through
autograd) replayed several times on new inputs, with eager calls and synchronisations in between, gives
bit for bit what the eager call gives.  The library launches kernels only (its workspace is cleared by a
fill kernel, not by a memset), reads the environment at capture time and allocates nothing, so a captured
sequence is self-contained."""
import pytest
import torch

pytestmark = pytest.mark.gpu

GATES = {"lstm": (4, 4, 2), "slstm": (4, 4, 4), "gru": (3, 4, 1), "elman": (1, 1, 1)}  # G_w = G_r, G_t, S

CASES = [
    ("lstm", 8, 1, 3, 256, "hip_fused", False),   # single-step decode, 4 workgroups per head
    ("lstm", 8, 1, 3, 256, "hip", False),
    ("lstm", 8, 16, 3, 256, "hip_fused", True),
    ("gru", 5, 9, 2, 128, "hip_fused", True),     # ragged batch, one workgroup per head
    ("slstm", 16, 8, 1, 768, "hip_fused", True),  # 12 workgroups per head, dynamic LDS in the reverse kernel
    ("elman", 16, 8, 1, 512, "hip", True),
]


@pytest.mark.parametrize("function,B,T,N,D,backend,bwd", CASES)
def test_captured_call_replays_like_eager(gpu, function, B, T, N, D, backend, bwd):
    from flashrnn_amd import flashrnn

    print(f"case graph {function} B{B} T{T} N{N} D{D} {backend} bwd={bwd}", flush=True)
    G, Gt, S = GATES[function]
    gen = torch.Generator(device="cpu").manual_seed(4242)
    mk = lambda *s: torch.randn(*s, generator=gen).to(gpu, torch.bfloat16)
    Wx = mk(B, T, G, N, D).requires_grad_(bwd)
    R = (mk(G, N, D, D).float() / D ** 0.5).to(torch.bfloat16).requires_grad_(bwd)
    b = (mk(Gt, N, D).float() * 0.1).to(torch.bfloat16).requires_grad_(bwd)
    s0 = mk(S, B, 1, N, D).requires_grad_(bwd)
    ds = mk(S, B, T, N, D)

    def step():
        out, _ = flashrnn(Wx, R, b, s0, function=function, backend=backend)
        if bwd:
            return (out,) + torch.autograd.grad(out, [Wx, R, b, s0], grad_outputs=ds)
        return (out,)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for i in range(4):
        with torch.no_grad():
            Wx.copy_(mk(B, T, G, N, D))
            s0.copy_(mk(S, B, 1, N, D))
            ds.copy_(mk(S, B, T, N, D))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.detach().clone() for o in outs]
        ref = step()   # the program's own eager work between replays
        torch.cuda.synchronize()
        for k, (a, r) in enumerate(zip(got, ref)):
            assert torch.isfinite(a.float()).all(), (i, k)
            assert torch.equal(a, r.detach()), (i, k, float((a.float() - r.detach().float()).abs().max()))
