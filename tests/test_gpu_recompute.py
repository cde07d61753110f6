"""Recompute mode of the fused backend (FlashRNNConfig.recompute_gates, frnn_fused_backward_recompute): the
training forward writes no gate cache and the reverse scan rebuilds the gates from Wx, b and R h_(t-1).
Same parity bar as the cached path; in fp32 the rebuilt gates of lstm and gru are the cached ones bit for bit."""
import ctypes

import pytest
import torch

from oracle import make_inputs
from parity import check_case

pytestmark = pytest.mark.gpu
RC = {"recompute_gates": True}

CASES = [
    # function, B, T, N, D, dtype
    ("lstm", 3, 5, 2, 32, "bfloat16"),
    ("lstm", 9, 7, 2, 64, "bfloat16"),       # ragged batch over three 4-row tiles
    ("lstm", 1, 1, 1, 64, "bfloat16"),       # a single step: only the prologue rebuild runs
    ("lstm", 5, 2, 1, 96, "bfloat16"),
    ("lstm", 20, 6, 2, 128, "bfloat16"),     # 2 workgroups per head in this mode
    ("lstm", 7, 9, 1, 192, "bfloat16"),      # 3 workgroups per head
    ("lstm", 8, 16, 3, 256, "bfloat16"),     # 4 workgroups per head
    ("lstm", 33, 4, 1, 256, "float16"),
    ("lstm", 6, 7, 1, 320, "bfloat16"),      # 5 workgroups per head: the largest head whose two operands fit the registers
    ("lstm", 9, 5, 1, 320, "float16"),
    ("lstm", 5, 9, 2, 64, "float32"),
    ("lstm", 4, 6, 1, 32, "float32"),
    ("gru", 5, 9, 2, 64, "bfloat16"),
    ("gru", 16, 8, 4, 128, "bfloat16"),
    ("gru", 6, 5, 1, 192, "bfloat16"),
    ("gru", 7, 5, 1, 256, "bfloat16"),
    ("gru", 5, 6, 1, 320, "bfloat16"),
    ("gru", 10, 5, 1, 384, "bfloat16"),      # (three gate rows: one head dim further than the 4-gate cells)
    ("gru", 3, 6, 2, 32, "float32"),
    ("slstm", 8, 6, 2, 64, "bfloat16"),
    ("slstm", 6, 7, 1, 96, "bfloat16"),
    ("slstm", 16, 12, 2, 192, "bfloat16"),
    ("slstm", 12, 5, 2, 256, "bfloat16"),
    ("slstm", 7, 6, 1, 320, "bfloat16"),
    ("slstm", 5, 8, 1, 64, "float32"),
    ("elman", 16, 7, 2, 128, "bfloat16"),    # nothing is cached for elman: the flag changes nothing
]


@pytest.mark.parametrize("function,B,T,N,D,dtype", CASES)
@pytest.mark.parametrize("init", ["zeros", "randn"])
def test_recompute_matches_oracle(gpu, function, B, T, N, D, dtype, init):
    print(f"case recompute {function} B{B} T{T} N{N} D{D} {dtype} init={init}", flush=True)
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=81, init=init, options=RC)


@pytest.mark.parametrize("function,B,T,N,D,dtype", [
    ("lstm", 21, 6, 2, 256, "bfloat16"), ("gru", 20, 7, 2, 128, "bfloat16"), ("slstm", 18, 8, 2, 192, "bfloat16"),
    ("lstm", 19, 5, 1, 64, "float32"), ("slstm", 9, 6, 3, 64, "bfloat16"),
])
@pytest.mark.parametrize("tile_rows", [4, 8, 16])
def test_recompute_every_batch_tiling(gpu, monkeypatch, tile_rows, function, B, T, N, D, dtype):
    print(f"case recompute tiling rows={tile_rows} {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    monkeypatch.setenv("FRNN_TILE_ROWS", str(tile_rows))
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=82, init="randn", options=RC)


@pytest.mark.parametrize("options", [
    dict(gradient_recurrent_clipval=0.5), dict(gradient_recurrent_cut=True), dict(forward_clipval=0.4),
    dict(forward_clipval=0.4, gradient_recurrent_clipval=0.5, gradient_recurrent_cut=True),
], ids=lambda o: "+".join(sorted(o)))
@pytest.mark.parametrize("function,B,T,N,D,dtype", [
    ("lstm", 8, 12, 3, 256, "bfloat16"), ("gru", 6, 8, 2, 128, "bfloat16"), ("slstm", 7, 10, 2, 192, "bfloat16"),
    ("lstm", 5, 9, 2, 64, "float32"),
])
def test_recompute_with_clip_and_cut(gpu, options, function, B, T, N, D, dtype):
    print(f"case recompute options {options} {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=83, init="randn", options=dict(options, **RC))


@pytest.mark.parametrize("function", ["lstm", "gru"])
@pytest.mark.parametrize("tile_rows", [8, 4])
def test_recompute_in_fp32_gives_the_bits_of_the_cached_path(gpu, function, tile_rows, monkeypatch):
    """fp32 storage: the stored h is what the forward pass fed to its product.  With 8-row tiles the rebuild runs the
    same MFMA chain and the same gate math as the forward pass, so every gradient must come out bit for bit as with
    the cache.  With 4-row tiles the forward product runs on the 4x4x1 instruction (another summation order) and
    the rebuild on the 16x16x4 one: equal to fp32 rounding.  (Both reverse kernels on the tiling that the two modes
    share, one workgroup per head: a small call with the cache would otherwise run as 2 workgroups per head, which
    sum the recurrent cotangent in another order.)"""
    from flashrnn_amd import FlashRNNConfig, flashrnn

    B, T, N, D = 7, 33, 2, 64
    print(f"case recompute bits {function} rows {tile_rows}", flush=True)
    monkeypatch.setenv("FRNN_TILE_ROWS", str(tile_rows))
    monkeypatch.setenv("FRNN_FUSED_VARIANT", "1")  # (no such entry: the table's default tiling, no switching)
    inp = make_inputs(function, B, T, N, D, 84, init="randn")
    res = []
    for rc in (False, True):
        leaves = [inp[k].to(gpu).requires_grad_(True) for k in ("Wx", "R", "b", "states")]
        cfg = FlashRNNConfig(backend="hip_fused", function=function, dtype="float32", head_dim=D, num_heads=N,
                             recompute_gates=rc)
        out, _ = flashrnn(*leaves, config=cfg)
        res.append((out,) + torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"].to(gpu)))
    torch.cuda.synchronize()
    for name, a, c in zip(("states", "dWx", "dR", "db", "ds0"), *res):
        if tile_rows == 8:
            assert torch.equal(a, c), f"{name}: max diff {(a - c).abs().max().item():.3e}"
        else:
            assert float((a - c).abs().max()) <= 1e-5 * max(1.0, float(c.abs().max())), name


def test_recompute_has_no_cache_and_refuses_what_it_cannot_do(gpu):
    from flashrnn_amd import FlashRNNConfig, _lib, flashrnn

    lib = _lib.load_library()
    on = _lib.Options(0.0, 0.0, 0, 1)
    for f in ("lstm", "gru", "slstm"):
        fid = _lib.FUNCTION_IDS[f]
        assert lib.frnn_fused_cache_bytes_opt(fid, 0, 8, 1024, 3, 256, ctypes.byref(on)) == 0
        assert lib.frnn_fused_cache_bytes_opt(fid, 0, 8, 1024, 3, 256, None) > 0
        assert lib.frnn_fused_recompute_supported(fid, 0, 8, 3, 256) == 0
        assert lib.frnn_fused_recompute_supported(fid, 0, 8, 1, 512) == _lib.E_UNSUPPORTED
    cfg = FlashRNNConfig(backend="hip_fused", function="lstm", dtype="bfloat16", head_dim=512, num_heads=1,
                         recompute_gates=True)
    Wx = torch.zeros(2, 3, 4, 1, 512, device=gpu, requires_grad=True)
    with pytest.raises(ValueError, match="recompute"):
        flashrnn(Wx, torch.zeros(4, 1, 512, 512, device=gpu), torch.zeros(4, 1, 512, device=gpu), config=cfg)


# ---- the benchmark configurations in recompute mode, full size ---------------------------------------
def test_config2_recompute_full_size(gpu):
    print("case C2 recompute full", flush=True)
    check_case(gpu, "lstm", 8, 1024, 3, 256, "bfloat16", "hip_fused", seed=1002, init="randn", options=RC,
               vs_bf16_vanilla=True)


def test_config3_recompute_full_size(gpu):
    print("case C3 recompute full", flush=True)
    check_case(gpu, "gru", 16, 2048, 4, 128, "bfloat16", "hip_fused", seed=1003, init="zeros", options=RC,
               vs_bf16_vanilla=True)


def test_config4_recompute_full_size(gpu):
    print("case C4 recompute full", flush=True)
    check_case(gpu, "slstm", 16, 4096, 4, 192, "bfloat16", "hip_fused", seed=1004, init="zeros",
               forget_bias_linspace=True, grad_on="h", options=RC, vs_bf16_vanilla=True)
