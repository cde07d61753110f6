"""frnn_fused_forward_static: the forward entry point that allocates nothing (its workspace is a static
array in device memory that belongs to the library).  Called through the C ABI with raw pointers and
checked bit for bit against frnn_fused_forward_opt, which takes the caller's workspace: two calls in a
row, the second with a smaller input, so that what the first call left in the shared array is still there
when the second starts.  Both use heads that span several workgroups, so the array's exchange slots are
in use."""
import ctypes
import os

import pytest
import torch

from oracle import FUNCTIONS, make_inputs

pytestmark = pytest.mark.gpu

FN = {"lstm": 0, "slstm": 1, "gru": 2, "elman": 3}
DT = {"bfloat16": 0, "float32": 1, "float16": 2}


class Options(ctypes.Structure):
    _fields_ = [("struct_size", ctypes.c_uint), ("forward_clipval", ctypes.c_float),
                ("gradient_recurrent_clipval", ctypes.c_float), ("gradient_recurrent_cut", ctypes.c_int),
                ("recompute", ctypes.c_int), ("batch_stride", ctypes.c_int)]


def _open():
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.environ.get("FLASHRNN_HIP_LIBRARY") or os.path.join(here, "flashrnn_amd", "libflashrnn_hip.so"))
    i, p, z = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
    lib.frnn_last_error.restype = ctypes.c_char_p
    lib.frnn_fused_cache_bytes.restype = z
    lib.frnn_fused_cache_bytes.argtypes = [i] * 6
    lib.frnn_fused_workspace_bytes.restype = z
    lib.frnn_fused_workspace_bytes.argtypes = [i] * 7
    lib.frnn_fused_forward_opt.argtypes = [i] * 7 + [p] * 7 + [z, p, ctypes.POINTER(Options)]
    lib.frnn_fused_forward_static.argtypes = [i] * 7 + [p] * 7 + [ctypes.POINTER(Options)]
    lib.frnn_fused_forward_static_max_bytes.restype = z
    return lib


def _both(lib, gpu, function, B, T, N, D, dtype, seed):
    """One training forward through each entry point on the same inputs; returns (states, cache) of each."""
    Gr, Gw, _, Gt, S = FUNCTIONS[function]
    kdt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    inp = make_inputs(function, B, T, N, D, seed, init="randn", round_to=kdt if kdt != torch.float32 else None)
    dev = lambda x: x.to(gpu, kdt).contiguous()
    Wx, R, b = dev(inp["Wx"]), dev(inp["R"]), dev(inp["b"])
    s0 = dev(inp["states"].reshape(S, B, N, D))
    f, d = FN[function], DT[dtype]
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cache_bytes = max(int(lib.frnn_fused_cache_bytes(f, d, B, T, N, D)), 256)
    ws_bytes = int(lib.frnn_fused_workspace_bytes(f, d, B, T, N, D, 0))
    assert 256 < ws_bytes <= lib.frnn_fused_forward_static_max_bytes(), "the case must use the exchange slots"
    # outputs of both entry points are allocated before either call: the static call itself allocates nothing
    out = [(torch.full((S, B, T, N, D), float("nan"), dtype=kdt, device=gpu),
            torch.zeros(cache_bytes, dtype=torch.uint8, device=gpu)) for _ in range(2)]
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=gpu)
    torch.cuda.synchronize()
    rc = lib.frnn_fused_forward_opt(f, d, 1, B, T, N, D, vp(Wx), vp(R), vp(b), vp(s0), vp(out[0][0]), vp(out[0][1]),
                                    vp(ws), ws.numel(), stream, None)
    assert rc == 0, lib.frnn_last_error().decode()
    rc = lib.frnn_fused_forward_static(f, d, 1, B, T, N, D, vp(Wx), vp(R), vp(b), vp(s0), vp(out[1][0]), vp(out[1][1]),
                                       stream, None)
    assert rc == 0, lib.frnn_last_error().decode()
    torch.cuda.synchronize()
    assert int(ws[:4].view(torch.int32).item()) == 0
    return out


def test_static_forward_matches_the_workspace_forward_twice(gpu):
    lib = _open()
    # first call: 4 workgroups per head, 3 heads x 5 batch tiles; second call: smaller in every extent, and a
    # different cell, so that its exchange slots overlay what the first call wrote there
    for k, (function, B, T, N, D, dtype) in enumerate([("lstm", 20, 24, 3, 256, "bfloat16"),
                                                       ("gru", 6, 9, 1, 256, "bfloat16")]):
        print(f"case static forward call {k}: {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
        (st_ws, ca_ws), (st_static, ca_static) = _both(lib, gpu, function, B, T, N, D, dtype, seed=31 + k)
        assert torch.isfinite(st_ws.float()).all()
        assert torch.equal(st_ws, st_static), f"call {k}: states differ"
        assert torch.equal(ca_ws, ca_static), f"call {k}: gate cache differs"


def test_static_forward_refuses_what_does_not_fit(gpu):
    lib = _open()
    f, d = FN["lstm"], DT["float32"]
    B, T, N, D = 4096, 2, 8, 256   # fp32 exchange slots of 8 heads x 256 batch tiles: far beyond 4 MiB
    assert lib.frnn_fused_workspace_bytes(f, d, B, T, N, D, 0) > lib.frnn_fused_forward_static_max_bytes()
    fake = ctypes.c_void_p(0x1000)  # never dereferenced: the size check comes first
    rc = lib.frnn_fused_forward_static(f, d, 0, B, T, N, D, fake, fake, fake, fake, fake, None, None, None)
    assert rc == -5 and b"static scratch" in lib.frnn_last_error()
