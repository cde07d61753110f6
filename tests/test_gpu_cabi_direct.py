"""The C ABI on its own, as a binding on the reference's side would use it: a private ctypes handle with
its own argtypes, raw device pointers, caller-allocated outputs, cache and workspace, the caller's stream;
nothing of the package's Python layer.  Checked against the CPU oracle."""
import ctypes
import os

import pytest
import torch

from oracle import FUNCTIONS, make_inputs
from parity import assert_close, oracle_run

pytestmark = pytest.mark.gpu

FN = {"lstm": 0, "slstm": 1, "gru": 2, "elman": 3}   # FRNN_LSTM ... of include/flashrnn_hip.h
DT = {"bfloat16": 0, "float32": 1, "float16": 2}     # FRNN_BF16, FRNN_F32, FRNN_F16


def _open():
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ctypes.CDLL(os.environ.get("FLASHRNN_HIP_LIBRARY") or os.path.join(here, "flashrnn_amd", "libflashrnn_hip.so"))
    i, p, z = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
    lib.frnn_last_error.restype = ctypes.c_char_p
    for pre in ("frnn_fused_", "frnn_alt_"):
        getattr(lib, pre + "cache_bytes").restype = z
        getattr(lib, pre + "cache_bytes").argtypes = [i] * 6
        getattr(lib, pre + "workspace_bytes").restype = z
        getattr(lib, pre + "workspace_bytes").argtypes = [i] * 7
        getattr(lib, pre + "forward").argtypes = [i] * 7 + [p] * 7 + [z, p]
        getattr(lib, pre + "backward").argtypes = [i] * 6 + [p] * 11 + [z, p]
    return lib


@pytest.mark.parametrize("function,B,T,N,D,dtype,pre", [
    ("lstm", 8, 12, 3, 256, "bfloat16", "frnn_fused_"),
    ("gru", 5, 9, 2, 128, "bfloat16", "frnn_fused_"),
    ("slstm", 3, 6, 2, 64, "float32", "frnn_fused_"),
    ("elman", 16, 7, 1, 512, "bfloat16", "frnn_alt_"),
])
def test_entry_points_with_raw_pointers(gpu, function, B, T, N, D, dtype, pre):
    print(f"case raw C ABI {pre} {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    lib = _open()
    Gr, Gw, _, Gt, S = FUNCTIONS[function]
    kdt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    inp = make_inputs(function, B, T, N, D, 5, init="randn", round_to=kdt if kdt != torch.float32 else None)
    if function == "slstm":
        inp["dstates"][3] = 0  # the stabiliser gets no cotangent in the native path
    dev = lambda x: x.to(gpu, kdt).contiguous()
    Wx, R, b = dev(inp["Wx"]), dev(inp["R"]), dev(inp["b"])
    s0 = dev(inp["states"].reshape(S, B, N, D))
    ds = dev(inp["dstates"])
    f, d = FN[function], DT[dtype]
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    nbytes = lambda name, *a: getattr(lib, pre + name)(f, d, B, T, N, D, *a)
    new = lambda n: torch.empty(max(int(n), 256), dtype=torch.uint8, device=gpu)
    states = torch.empty((S, B, T, N, D), dtype=kdt, device=gpu)
    cache, ws_f, ws_b = new(nbytes("cache_bytes")), new(nbytes("workspace_bytes", 0)), new(nbytes("workspace_bytes", 1))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = getattr(lib, pre + "forward")(f, d, 1, B, T, N, D, vp(Wx), vp(R), vp(b), vp(s0), vp(states), vp(cache),
                                        vp(ws_f), ws_f.numel(), stream)
    assert rc == 0, lib.frnn_last_error().decode()
    dWx = torch.empty((B, T, Gw, N, D), dtype=kdt, device=gpu)
    ds0 = torch.empty((S, B, N, D), dtype=kdt, device=gpu)
    dR = torch.empty((Gr, N, D, D), dtype=torch.float32, device=gpu)
    db = torch.empty((Gt, N, D), dtype=torch.float32, device=gpu)
    rc = getattr(lib, pre + "backward")(f, d, B, T, N, D, vp(R), vp(b), vp(s0), vp(states), vp(cache), vp(ds),
                                         vp(dWx), vp(ds0), vp(dR), vp(db), vp(ws_b), ws_b.numel(), stream)
    assert rc == 0, lib.frnn_last_error().decode()
    torch.cuda.synchronize()
    if pre == "frnn_fused_":
        assert int(ws_f[:4].view(torch.int32).item()) == 0 and int(ws_b[:4].view(torch.int32).item()) == 0
    ref_out, ref_g = oracle_run(function, inp, dtype, True, None)
    out = states.float().cpu()
    for k in range(S):
        assert_close(f"state {k}", out[k], ref_out[k], dtype, "h" if k == 0 else "state")
    assert_close("dWx", dWx.float().cpu(), ref_g[0], dtype, "token")
    assert_close("dR", dR.cpu(), ref_g[1], dtype, "sum")
    assert_close("db", db.cpu(), ref_g[2], dtype, "sum")
    for k in range(S):
        if function == "slstm" and k == 3:
            continue  # the stabiliser's cotangent is reported as 0 by design
        assert_close(f"ds0[{k}]", ds0[k].float().cpu().reshape(B, 1, N, D), ref_g[3][k], dtype, "token")
