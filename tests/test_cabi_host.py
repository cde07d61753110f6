"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares, and rejects bad arguments with the documented codes before any launch."""
import ctypes
import os
import re

import pytest
import torch

from flashrnn_amd import FlashRNNConfig, flashrnn, load_library
from flashrnn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flashrnn_hip.h")
FAKE = ctypes.c_void_p(0x1000)  # non-null, 16-byte aligned; never dereferenced: every call below fails earlier


@pytest.fixture(scope="module")
def lib():
    return load_library()


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(frnn_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = _declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(_lib.EXPORTED_SYMBOLS)
    assert b"gfx950" in lib.frnn_version()


def test_function_dims_mirror_the_registry(lib):
    from flashrnn_amd import rnn_function_registry

    for name, fid in _lib.FUNCTION_IDS.items():
        vals = [ctypes.c_int() for _ in range(5)]
        assert lib.frnn_function_dims(fid, *[ctypes.byref(v) for v in vals]) == 0
        gr, gw, gi, gt, s = rnn_function_registry[name]["gates_states"]
        assert [v.value for v in vals[:4]] == [gr, gw, gt, s]
    assert lib.frnn_function_dims(9, None, None, None, None, None) == _lib.E_ARG


def test_supported_table(lib):
    L, S, G, E = (_lib.FUNCTION_IDS[k] for k in ("lstm", "slstm", "gru", "elman"))
    for f in (L, S, G, E):
        for D in (32, 64, 96, 128, 160, 192, 256, 320, 384, 448, 512, 640):
            assert lib.frnn_fused_supported(f, 0, 8, 3, D) == 0, (f, D)
    for f in (L, S, G, E):
        assert lib.frnn_fused_supported(f, 0, 8, 1, 768) == 0, f
    assert lib.frnn_fused_supported(E, 0, 32, 1, 1024) == 0 and lib.frnn_fused_supported(G, 0, 32, 1, 1024) == 0
    assert lib.frnn_fused_supported(L, 0, 8, 1, 1024) == 0
    assert lib.frnn_fused_supported(L, 0, 8, 1, 2048) == _lib.E_UNSUPPORTED  # too large to keep on chip
    # fp32: R is twice the size: the gated cells run every head dim of the 16-bit list (the reference's test grid,
    # tests/test_lstm.py:9-46, has 32, 64, 512 and 1024; beyond 512 a head takes 40 to 64 workgroups, spread over the device)
    for f in (L, S, G, E):
        for D in (32, 64, 96, 128, 160, 192, 256, 320, 384, 448, 512):
            assert lib.frnn_fused_supported(f, 1, 8, 1, D) == 0, (f, D)
    for f in (L, S, G):
        for D in (640, 768, 1024):
            assert lib.frnn_fused_supported(f, 1, 8, 2, D) == 0, (f, D)
    assert lib.frnn_fused_supported(L, 1, 8, 1, 896) == _lib.E_UNSUPPORTED
    assert lib.frnn_fused_supported(E, 1, 8, 1, 768) == 0 and lib.frnn_fused_supported(E, 1, 8, 1, 1024) == 0
    assert lib.frnn_fused_supported(L, 0, 8, 1, 48) == _lib.E_UNSUPPORTED
    assert b"head dim" in lib.frnn_last_error()
    assert lib.frnn_alt_supported(L, 0, 8, 1, 1024) == 0
    assert lib.frnn_alt_supported(L, 0, 8, 1, 48) == _lib.E_UNSUPPORTED
    assert lib.frnn_fused_supported(7, 0, 8, 1, 64) == _lib.E_ARG
    assert lib.frnn_fused_supported(L, 5, 8, 1, 64) == _lib.E_ARG
    assert lib.frnn_fused_supported(L, 0, 0, 1, 64) == _lib.E_ARG


def test_plan_and_sizes(lib):
    L = _lib.FUNCTION_IDS["lstm"]
    out = [ctypes.c_int() for _ in range(4)]
    assert lib.frnn_fused_plan(L, 0, 8, 3, 256, 0, *[ctypes.byref(o) for o in out]) == 0
    waves, utw, kw, active = (o.value for o in out)
    # workgroups = heads x batch tiles (of 4, 8 or 16 rows, by the compute units at hand) x kw
    assert 16 * waves * utw * kw == 256 and active in (3 * kw, 6 * kw)
    # gate cache: T * N * B * D * values (padded to whole dwords: sLSTM bf16 5 -> 6, the sixth carries c_(t-1)) * bytes
    assert lib.frnn_fused_cache_bytes(L, 0, 8, 1024, 3, 256) == 1024 * 3 * 8 * 256 * 4 * 2
    assert lib.frnn_fused_cache_bytes(_lib.FUNCTION_IDS["slstm"], 0, 8, 16, 3, 256) == 16 * 3 * 8 * 256 * 6 * 2
    assert lib.frnn_fused_cache_bytes(_lib.FUNCTION_IDS["slstm"], 1, 8, 16, 3, 256) == 16 * 3 * 8 * 256 * 5 * 4
    assert lib.frnn_alt_cache_bytes(L, 0, 8, 1024, 3, 256) == 1024 * 3 * 8 * 256 * 4 * 2
    assert lib.frnn_fused_cache_bytes(_lib.FUNCTION_IDS["elman"], 0, 8, 16, 3, 256) == 0
    assert lib.frnn_fused_workspace_bytes(L, 0, 8, 1024, 3, 256, 0) >= 256
    assert lib.frnn_fused_workspace_bytes(L, 0, 8, 1024, 3, 256, 1) > lib.frnn_fused_workspace_bytes(L, 0, 8, 1024, 3, 256, 0)
    assert lib.frnn_fused_workspace_bytes(L, 0, 8, 1024, 3, 2048, 0) == 0  # unsupported


def test_small_batches_get_the_tiling_with_more_workgroups_per_head(lib):
    """Where the table has a small-batch alternative for a head dim (gru bf16 D = 192 backward: 3 workgroups of 4
    waves instead of one of 12), it is used while all groups of the call fit one launch with 4-row tiles, and the
    workspace size follows the choice."""
    G = _lib.FUNCTION_IDS["gru"]
    out = [ctypes.c_int() for _ in range(4)]
    plan = lambda B, backward: (lib.frnn_fused_plan(G, 0, B, 4, 192, backward, *[ctypes.byref(o) for o in out]),
                                [o.value for o in out])[1]
    assert plan(16, 1)[:3] == [4, 1, 3] and plan(1024, 1)[:3] == [12, 1, 1]
    assert plan(16, 0)[:3] == [12, 1, 1]  # forward: one tiling
    ws = lambda B: lib.frnn_fused_workspace_bytes(G, 0, B, 64, 4, 192, 1)
    assert ws(16) > 256 + 64 * 1024  # exchange buffers of the 3-workgroup tiling
    assert lib.frnn_fused_workspace_bytes(G, 0, 16, 64, 4, 192, 0) <= 1024  # one workgroup per head: the status word only


def _fwd(lib, entry, function=0, dtype=0, B=8, T=4, N=1, D=64, Wx=FAKE, R=FAKE, b=FAKE, s0=FAKE, states=FAKE,
         cache=FAKE, ws=FAKE, ws_bytes=0, training=1, opt=None):
    args = [function, dtype, training, B, T, N, D, Wx, R, b, s0, states, cache, ws, ws_bytes, None]
    if entry.endswith("_opt"):
        args.append(ctypes.byref(opt) if opt is not None else None)
    return getattr(lib, entry)(*args)


@pytest.mark.parametrize("entry", ["frnn_fused_forward", "frnn_alt_forward"])
def test_forward_rejects_bad_arguments_before_launch(lib, entry):
    assert _fwd(lib, entry, function=4) == _lib.E_ARG
    assert _fwd(lib, entry, dtype=3) == _lib.E_ARG
    assert _fwd(lib, entry, T=0) == _lib.E_ARG
    assert _fwd(lib, entry, D=40) == _lib.E_UNSUPPORTED
    assert _fwd(lib, entry, Wx=None) == _lib.E_NULL
    assert b"Wx" in lib.frnn_last_error()
    assert _fwd(lib, entry, cache=None) == _lib.E_NULL          # training needs the cache
    assert _fwd(lib, entry, R=ctypes.c_void_p(0x1004)) == _lib.E_ALIGN
    assert _fwd(lib, entry, ws_bytes=16) == _lib.E_WORKSPACE    # smaller than *_workspace_bytes
    assert b"workspace" in lib.frnn_last_error()


@pytest.mark.parametrize("entry", ["frnn_fused_backward", "frnn_alt_backward"])
def test_backward_rejects_bad_arguments_before_launch(lib, entry):
    fn = getattr(lib, entry)

    def call(function=0, dtype=0, B=8, T=4, N=1, D=64, ptrs=None, ws_bytes=0):
        p = [FAKE] * 11 if ptrs is None else ptrs
        return fn(function, dtype, B, T, N, D, *p, ws_bytes, None)

    assert call(function=-1) == _lib.E_ARG
    assert call(D=24) == _lib.E_UNSUPPORTED
    for i in (0, 2, 3, 5, 6, 7, 8, 9, 10):  # R, s0, states, dstates, dWx, ds0, dR, db, workspace
        p = [FAKE] * 11
        p[i] = None
        assert call(ptrs=p) == _lib.E_NULL, i
    p = [FAKE] * 11
    p[8] = ctypes.c_void_p(0x1008)
    assert call(ptrs=p) == _lib.E_ALIGN
    assert call(ws_bytes=64) == _lib.E_WORKSPACE


def test_fused_refuses_tensors_of_2_gib(lib):
    # 32-bit byte offsets inside the fused kernels: B*T*N*D*G_w*2 bytes must stay below 2 GiB
    # (a code of its own, so that a binding can tell "split the batch" from a bad argument)
    assert _fwd(lib, "frnn_fused_forward", B=64, T=16384, N=4, D=256) == _lib.E_TOO_LARGE
    assert b"2 GiB" in lib.frnn_last_error()
    L, S = _lib.FUNCTION_IDS["lstm"], _lib.FUNCTION_IDS["slstm"]
    T, N, D = 1024, 12, 64
    row = T * N * D * 2                                          # bytes of one batch row of one bf16 plane
    lim = (1 << 31) - 1
    # each call on tensors of its own: Wx (4 gates) and the gate cache (4 values) bound an LSTM call, 341 rows
    assert lib.frnn_fused_max_batch(L, 0, T, N, D, 0, 1, None) == lim // (4 * row) == 341
    # ranges of a batch of 512 rows used in place: the c plane starts 512 rows behind the h plane
    assert lib.frnn_fused_max_batch(L, 0, T, N, D, 512, 1, None) == min(341, (lim - 512 * row) // row) == 341
    assert lib.frnn_fused_max_batch(L, 0, T, N, D, 1200, 1, None) == (lim - 1200 * row) // row == 165
    # sLSTM: four planes; at 512 rows the fourth lies beyond 2 GiB from the first: no row fits in place
    assert lib.frnn_fused_max_batch(S, 0, T, N, D, 512, 1, None) == 0
    assert lib.frnn_fused_max_batch(S, 0, T, N, D, 0, 1, None) == lim // (6 * row) == 227   # (its cache: 5 values padded to 6)
    o = _lib.Options(0.0, 0.0, 0, 0, 512)
    assert _fwd(lib, "frnn_fused_forward_opt", B=341, T=T, N=N, D=D, opt=o) != _lib.E_TOO_LARGE
    assert _fwd(lib, "frnn_fused_forward_opt", B=342, T=T, N=N, D=D, opt=o) == _lib.E_TOO_LARGE
    o = _lib.Options(0.0, 0.0, 0, 0, 100)
    assert _fwd(lib, "frnn_fused_forward_opt", B=128, T=8, N=2, D=64, opt=o) == _lib.E_ARG   # stride smaller than the call's rows


def test_python_api_argument_errors():
    with pytest.raises(ValueError):
        FlashRNNConfig(backend="vanilla")  # the torch loop is the test oracle, not a backend
    with pytest.raises(ValueError):
        FlashRNNConfig(function="rnn")
    with pytest.raises(ValueError):
        FlashRNNConfig(dtype="float64")
    assert FlashRNNConfig(dtype="float16").dtype == "float16"
    with pytest.raises(ValueError):
        FlashRNNConfig(gradient_recurrent_clipval=-1.0)
    assert FlashRNNConfig(gradient_recurrent_cut=True, forward_clipval=2.0).gradient_recurrent_cut
    cfg = FlashRNNConfig(function="gru", head_dim=64, num_heads=3)
    assert (cfg.num_gates_r, cfg.num_gates_w, cfg.num_gates_t, cfg.num_states, cfg.hidden_dim) == (3, 3, 4, 1, 192)
    Wx = torch.zeros(2, 3, 4, 1, 32)
    R = torch.zeros(4, 1, 32, 32)
    b = torch.zeros(4, 1, 32)
    with pytest.raises(ValueError):
        flashrnn(Wx, R[:3], b, function="lstm")
    with pytest.raises(ValueError):
        flashrnn(Wx, R, b, states=torch.zeros(2, 2, 1, 1, 16), function="lstm")
    with pytest.raises(ValueError):
        flashrnn(Wx[:, :, :3], R, b, function="lstm")
    # no CPU path: a CPU tensor is refused, loudly
    with pytest.raises(RuntimeError, match="GPU only"):
        flashrnn(Wx, R, b, function="lstm")


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    monkeypatch.setenv("FLASHRNN_HIP_LIBRARY", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_LIB", None)
    with pytest.raises(RuntimeError, match="missing"):
        _lib.load_library()


def test_options_are_validated_before_launch(lib):
    """frnn_options: negative or NaN clip values are argument errors; forward_clipval is accepted for every cell
    (elman then needs a gate cache for the unclamped h, which the size query reports)."""
    import math

    def fwd(entry, function=0, **opt):
        o = _lib.Options(opt.get("f", 0.0), opt.get("g", 0.0), opt.get("cut", 0))
        return getattr(lib, entry)(function, 0, 1, 8, 4, 1, 64, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 0, None,
                                   ctypes.byref(o))

    for entry in ("frnn_fused_forward_opt", "frnn_alt_forward_opt"):
        assert fwd(entry, f=-1.0) == _lib.E_ARG
        assert fwd(entry, g=math.nan) == _lib.E_ARG
        assert fwd(entry, function=_lib.FUNCTION_IDS["elman"], f=0.5) == _lib.E_WORKSPACE
        assert fwd(entry, f=0.5) == _lib.E_WORKSPACE  # options accepted: the next check is the workspace size
    el, clip = _lib.FUNCTION_IDS["elman"], _lib.Options(0.5, 0.0, 0)
    for pre, per_elem in (("frnn_fused_", 2 * 2), ("frnn_alt_", 2)):  # fused: values padded to whole dwords
        assert getattr(lib, pre + "cache_bytes_opt")(el, 0, 8, 4, 1, 64, None) == 0
        assert getattr(lib, pre + "cache_bytes_opt")(el, 0, 8, 4, 1, 64, ctypes.byref(clip)) == 8 * 4 * 64 * per_elem
        assert getattr(lib, pre + "cache_bytes_opt")(0, 0, 8, 4, 1, 64, ctypes.byref(clip)) == \
            getattr(lib, pre + "cache_bytes")(0, 0, 8, 4, 1, 64)
    for entry in ("frnn_fused_backward_opt", "frnn_alt_backward_opt"):
        o = _lib.Options(0.0, -2.0, 0)
        assert getattr(lib, entry)(0, 0, 8, 4, 1, 64, *([FAKE] * 11), 0, None, ctypes.byref(o)) == _lib.E_ARG
        assert getattr(lib, entry)(0, 0, 8, 4, 1, 64, *([FAKE] * 11), 0, None, None) == _lib.E_WORKSPACE


def test_layout_options_and_initial_state():
    """The reference's public layout options (flashrnn.py:163-173, permute_to :100-110) and the default
    initial state with `initial_val` (:927-954), checked on CPU tensors (no kernel involved)."""
    from flashrnn_amd.flashrnn import _permuted, _zero_state, permute_to

    assert permute_to("ABC", "BAC") == (1, 0, 2) and permute_to("GHD", "GHD") is None
    cfg = FlashRNNConfig(function="slstm", head_dim=4, num_heads=2, input_shape="TBGHD", output_shape="STBHD",
                         recurrent_shape="HPGD", bias_shape="HDG", initial_val=[0.0, 1.0, 2.0, 3.0])
    Wx = torch.arange(5 * 3 * 4 * 2 * 4, dtype=torch.float32).reshape(5, 3, 4, 2, 4)      # T B G H D
    x = _permuted(Wx, cfg.input_shape, "BTGHD")
    assert x.shape == (3, 5, 4, 2, 4) and x[1, 2, 3, 1, 0] == Wx[2, 1, 3, 1, 0]
    R = torch.arange(2 * 4 * 4 * 4, dtype=torch.float32).reshape(2, 4, 4, 4)               # H P G D
    r = _permuted(R, cfg.recurrent_shape, "GHDP")
    assert r.shape == (4, 2, 4, 4) and r[3, 1, 2, 0] == R[1, 0, 3, 2]
    z = _zero_state(cfg, x)
    assert z.shape == (4, 3, 1, 2, 4) and [float(z[k].unique()) for k in range(4)] == [0.0, 1.0, 2.0, 3.0]
    z = _zero_state(FlashRNNConfig(function="lstm", head_dim=4, num_heads=2, initial_val=0.5), x)
    assert z.shape == (2, 3, 1, 2, 4) and float(z.unique()) == 0.5
    back = _permuted(_permuted(z, "SBTHD", "STBHD"), "STBHD", "SBTHD")
    assert torch.equal(back, z)
    with pytest.raises(ValueError):
        FlashRNNConfig(input_shape="BTGH")
    with pytest.raises(ValueError):
        FlashRNNConfig(output_shape="SBTHX")


def test_decode_session_arguments_are_checked_before_any_launch(lib):
    L, G = _lib.FUNCTION_IDS["lstm"], _lib.FUNCTION_IDS["gru"]
    # mailbox: control block + exchange area (heads of several workgroups) + slots x (inbox + outbox) of tagged records
    small = lib.frnn_fused_decode_mailbox_bytes(L, 0, 8, 2, 64, 4)     # one workgroup per head: no exchange area
    assert small == 256 + 4 * (8 * 2 * 64 * 16) + 4 * (8 * 2 * 64 * 8)
    big = lib.frnn_fused_decode_mailbox_bytes(L, 0, 8, 3, 256, 4)
    assert big > 256 + 4 * (8 * 3 * 256 * 24)
    assert lib.frnn_fused_decode_mailbox_bytes(G, 1, 4, 2, 64, 2) == 256 + 2 * (4 * 2 * 64 * 32) + 2 * (4 * 2 * 64 * 8)  # fp32: 8 bytes a value
    off = [ctypes.c_size_t() for _ in range(4)]
    assert lib.frnn_fused_decode_mailbox_layout(L, 0, 8, 2, 64, 4, *[ctypes.byref(o) for o in off]) == 0
    assert [o.value for o in off] == [256, 8 * 2 * 64 * 16, 256 + 4 * 8 * 2 * 64 * 16, 8 * 2 * 64 * 8]
    assert lib.frnn_fused_decode_mailbox_bytes(L, 0, 8, 2, 64, 3) == 0 and b"slots" in lib.frnn_last_error()
    assert lib.frnn_fused_decode_mailbox_layout(L, 0, 8, 2, 80, 4, None, None, None, None) == _lib.E_UNSUPPORTED
    # more groups than can stay on the device at once: 2000 heads x 1 batch tile
    assert lib.frnn_fused_decode_mailbox_layout(L, 0, 4, 2000, 64, 4, None, None, None, None) == _lib.E_UNSUPPORTED
    assert b"fit" in lib.frnn_last_error()
    mb = ctypes.c_void_p(0x10000)
    s1, s2 = ctypes.c_void_p(0x100), ctypes.c_void_p(0x200)
    args = lambda **kw: [L, 0, 8, 2, 64, kw.get("R", FAKE), FAKE, FAKE, None, kw.get("mb", mb), kw.get("bytes", small),
                         kw.get("slots", 4), kw.get("max_tokens", 100), kw.get("idle", 1000), s1, kw.get("ks", s2), None]
    assert lib.frnn_fused_decode_open(*args(R=None)) == _lib.E_NULL
    assert lib.frnn_fused_decode_open(*args(mb=ctypes.c_void_p(0x10010))) == _lib.E_ALIGN
    assert lib.frnn_fused_decode_open(*args(bytes=small - 1)) == _lib.E_WORKSPACE
    assert lib.frnn_fused_decode_open(*args(max_tokens=0)) == _lib.E_ARG
    assert lib.frnn_fused_decode_open(*args(idle=0)) == _lib.E_ARG
    assert lib.frnn_fused_decode_open(*args(ks=s1)) == _lib.E_ARG and b"stream of its own" in lib.frnn_last_error()
    step = lambda count, wx=FAKE: lib.frnn_fused_decode_step(L, 0, 8, 2, 64, count, wx, FAKE, mb, small, 4, s1)
    assert step(0) == _lib.E_ARG and step(5) == _lib.E_ARG and step(1, None) == _lib.E_NULL
    assert lib.frnn_fused_decode_close(None, s1, s2) == _lib.E_NULL
    assert lib.frnn_fused_decode_close(mb, s1, s1) == _lib.E_ARG
    assert lib.frnn_streams_overlap(s1, s1) == 0


def test_options_carry_their_size(lib):
    """frnn_options starts with struct_size, so that fields can be appended: a caller that knows fewer fields is served
    with the later ones off, one that does not set the size is refused."""
    L = _lib.FUNCTION_IDS["lstm"]
    o = _lib.Options(0.5, 0.0, 0, 0)
    assert o.struct_size == ctypes.sizeof(_lib.Options) == 24
    assert lib.frnn_fused_cache_bytes_opt(L, 0, 4, 8, 2, 64, ctypes.byref(o)) > 0
    o.struct_size = 0
    assert lib.frnn_fused_cache_bytes_opt(L, 0, 4, 8, 2, 64, ctypes.byref(o)) == 0 and b"struct_size" in lib.frnn_last_error()
    o = _lib.Options(0.0, 0.0, 0, 1)            # recompute on ...
    assert lib.frnn_fused_cache_bytes_opt(L, 0, 4, 8, 2, 64, ctypes.byref(o)) == 0
    o.struct_size = 16                          # ... but the caller's build ends before that field: it is not read
    assert lib.frnn_fused_cache_bytes_opt(L, 0, 4, 8, 2, 64, ctypes.byref(o)) > 0
