"""Parity of the HIP path (through the C ABI) with the CPU oracle on the same seeded inputs."""
import pytest
import torch

from parity import check_case

pytestmark = pytest.mark.gpu

FUSED_SMALL = [
    # function, B, T, N, D, dtype
    ("lstm", 4, 8, 1, 64, "float32"),
    ("lstm", 3, 5, 2, 32, "bfloat16"),
    ("lstm", 1, 1, 1, 32, "bfloat16"),       # single step, single row
    ("lstm", 9, 3, 2, 64, "bfloat16"),       # ragged batch: one row over two 4-row tiles
    ("lstm", 20, 6, 2, 128, "bfloat16"),     # two batch tiles, second ragged
    ("lstm", 8, 16, 3, 256, "bfloat16"),     # 4 workgroups per head
    ("lstm", 16, 9, 1, 256, "bfloat16"),
    ("lstm", 33, 4, 1, 256, "bfloat16"),     # 3 batch tiles x 4 workgroups
    ("lstm", 16, 5, 1, 512, "bfloat16"),     # 8 workgroups per head
    ("lstm", 4, 6, 1, 256, "float32"),       # fp32, 4 workgroups per head
    ("lstm", 5, 7, 2, 128, "float32"),
    ("gru", 5, 9, 2, 64, "bfloat16"),
    ("gru", 16, 8, 4, 128, "bfloat16"),
    ("gru", 7, 5, 1, 256, "bfloat16"),
    ("gru", 3, 6, 2, 32, "float32"),
    ("gru", 16, 4, 1, 192, "bfloat16"),
    ("elman", 16, 7, 2, 128, "bfloat16"),
    ("elman", 32, 6, 1, 512, "bfloat16"),
    ("elman", 16, 4, 1, 1024, "bfloat16"),   # 16 workgroups per head
    ("elman", 6, 9, 3, 64, "float32"),
    ("slstm", 8, 6, 2, 64, "bfloat16"),
    ("slstm", 16, 12, 2, 192, "bfloat16"),   # D not a power of two, 3 workgroups per head
    ("slstm", 5, 8, 1, 192, "float32"),
    ("slstm", 12, 5, 2, 256, "bfloat16"),
    ("lstm", 7, 6, 2, 96, "bfloat16"),       # 6 waves, 3 k-steps
    ("lstm", 5, 5, 1, 96, "float32"),
    ("gru", 9, 5, 1, 96, "bfloat16"),
    ("slstm", 6, 7, 1, 96, "bfloat16"),
    ("elman", 10, 6, 2, 96, "bfloat16"),
    ("lstm", 9, 7, 1, 384, "bfloat16"),      # 6 workgroups per head
    ("gru", 6, 5, 1, 384, "bfloat16"),
    ("slstm", 5, 6, 1, 384, "bfloat16"),
    ("elman", 12, 6, 1, 384, "bfloat16"),    # 3 workgroups of 8 waves
    ("lstm", 6, 7, 1, 768, "bfloat16"),      # 12 workgroups per head; backward keeps part of R^T in LDS
    ("gru", 9, 5, 1, 768, "bfloat16"),
    ("slstm", 5, 6, 1, 768, "bfloat16"),
    ("lstm", 17, 4, 1, 768, "float16"),
    ("elman", 11, 6, 1, 768, "bfloat16"),
    ("gru", 7, 5, 1, 1024, "bfloat16"),      # 16 workgroups per head
    ("lstm", 6, 7, 1, 1024, "bfloat16"),     # 32 workgroups of two wave pairs per head (k / the destinations split over a pair)
    ("slstm", 5, 5, 1, 1024, "bfloat16"),
    ("lstm", 18, 4, 1, 1024, "float16"),
    ("lstm", 6, 5, 2, 160, "bfloat16"),      # 10 waves
    ("slstm", 9, 6, 1, 160, "bfloat16"),
    ("gru", 5, 7, 1, 320, "bfloat16"),       # 5 workgroups per head
    ("lstm", 10, 6, 1, 320, "float16"),
    ("elman", 7, 5, 2, 320, "bfloat16"),
    ("lstm", 5, 6, 1, 448, "bfloat16"),      # 7 workgroups per head
    ("elman", 9, 5, 1, 448, "bfloat16"),
    ("lstm", 7, 5, 1, 640, "bfloat16"),      # 10 workgroups per head
    ("slstm", 4, 6, 1, 640, "bfloat16"),
    ("gru", 6, 4, 1, 640, "bfloat16"),
    ("elman", 12, 5, 1, 640, "bfloat16"),
    # fp32 beyond D = 256 (5 to 16 workgroups per head; gated cells from 384 on: workgroups of two wave pairs, the waves
    # of a pair split k (forward) or the destination workgroups (backward) between them)
    ("lstm", 6, 5, 1, 160, "float32"),
    ("gru", 5, 6, 2, 160, "float32"),
    ("elman", 9, 5, 1, 160, "float32"),      # 10 waves
    ("lstm", 5, 6, 1, 320, "float32"),
    ("slstm", 7, 5, 1, 320, "float32"),
    ("gru", 4, 5, 1, 320, "float32"),
    ("lstm", 9, 4, 1, 384, "float32"),
    ("gru", 6, 5, 1, 384, "float32"),
    ("elman", 5, 6, 1, 384, "float32"),
    ("slstm", 7, 6, 2, 384, "float32"),      # 12 workgroups per head: 3 groups of 4 destinations, 2 + 1 over a wave pair
    ("lstm", 5, 5, 1, 448, "float32"),       # 14 workgroups per head
    ("gru", 7, 4, 1, 448, "float32"),
    ("slstm", 3, 5, 1, 448, "float32"),
    ("lstm", 6, 6, 1, 512, "float32"),       # 16 workgroups per head
    ("slstm", 4, 5, 1, 512, "float32"),
    ("gru", 9, 4, 1, 512, "float32"),
    ("elman", 7, 5, 1, 768, "float32"),
    ("elman", 10, 4, 1, 1024, "float32"),
    ("lstm", 6, 5, 1, 1024, "float32"),      # 64 workgroups per head, spread over the device; 4 waves split k / the destinations
    ("slstm", 9, 4, 1, 1024, "float32"),     # 3 groups, the last with one valid row
    ("gru", 17, 3, 1, 1024, "float32"),      # 5 groups: two launches
    ("lstm", 3, 4, 2, 1024, "float32"),
    ("lstm", 7, 4, 1, 640, "float32"),       # 40 workgroups per head: 10 groups of 4 destinations, 3 + 3 + 2 + 2 over the waves
    ("slstm", 5, 5, 1, 768, "float32"),      # 48 workgroups per head
    ("gru", 25, 3, 1, 768, "float32"),       # 7 groups: two launches of at most 5
    ("slstm", 4, 4, 1, 640, "float32"),
    ("lstm", 37, 4, 1, 512, "float32"),      # 10 groups of 4 rows, the last with one valid row
    ("gru", 70, 4, 1, 384, "float32"),       # 18 groups of 12 workgroups: two launches
    # elman fp32 from D = 128 on: D / 64 workgroups of one tile per wave
    ("elman", 6, 5, 2, 128, "float32"),
    ("elman", 21, 4, 1, 192, "float32"),
    ("elman", 9, 6, 2, 256, "float32"),
    ("elman", 40, 4, 1, 512, "float32"),
    # head dims with a small-batch tiling (more workgroups per head while the call fits one launch at 4-row tiles):
    # these run on it, test_default_tiling_of_head_dims_with_a_small_batch_one on the other
    ("gru", 14, 5, 2, 192, "bfloat16"),
    ("lstm", 10, 5, 2, 160, "bfloat16"),
    ("lstm", 9, 6, 3, 64, "float32"),
    ("gru", 11, 5, 2, 64, "float32"),
    ("elman", 8, 5, 1, 96, "float32"),
    ("lstm", 12, 5, 1, 96, "float32"), ("gru", 70, 4, 2, 96, "float32"),   # backward: 3 workgroups of 2 waves
]


@pytest.mark.parametrize("function,N,dtype,backend", [
    ("lstm", 4, "bfloat16", "hip_fused"), ("lstm", 3, "float32", "hip_fused"), ("gru", 5, "bfloat16", "hip_fused"),
    ("slstm", 2, "bfloat16", "hip_fused"), ("elman", 7, "float16", "hip_fused"), ("lstm", 3, "bfloat16", "hip"),
])
def test_head_dim_16_runs_as_paired_heads(gpu, function, N, dtype, backend):
    """D = 16 (in the reference's benchmark sweep) is half a bf16 MFMA k-step: flashrnn() runs two heads
    as one head of 32 units with a block-diagonal R; outputs and all gradients, dR included, must match
    the oracle, which computes the heads separately."""
    print(f"case paired heads {function} N{N} {dtype} {backend}", flush=True)
    check_case(gpu, function, 6, 7, N, 16, dtype, backend, seed=23, init="randn")


@pytest.mark.parametrize("function,B,T,N,D,dtype", FUSED_SMALL)
@pytest.mark.parametrize("init", ["zeros", "randn"])
def test_fused_matches_oracle(gpu, function, B, T, N, D, dtype, init):
    print(f"case fused {function} B{B} T{T} N{N} D{D} {dtype} init={init}", flush=True)
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=7, init=init)


# The library picks 4-, 8- or 16-row batch tiles from the batch size and the device's compute
# units; FRNN_TILE_ROWS forces one so that every ownership mode is covered on any device.
TILINGS = [
    ("lstm", 9, 6, 2, 256, "bfloat16"),      # ragged in every tiling, 4 workgroups per head
    ("lstm", 21, 5, 1, 64, "float32"),
    ("gru", 20, 7, 2, 128, "bfloat16"),
    ("slstm", 6, 8, 2, 192, "bfloat16"),
    ("elman", 18, 5, 1, 1024, "bfloat16"),
    ("elman", 3, 6, 2, 32, "float32"),
    ("lstm", 37, 5, 1, 1024, "bfloat16"),    # wave pairs, at every tile height they are compiled for (reverse: up to 8 rows)
    ("slstm", 21, 4, 1, 1024, "float16"),
]


@pytest.mark.parametrize("function,B,T,N,D,dtype", TILINGS)
@pytest.mark.parametrize("tile_rows", [4, 8, 16])
def test_fused_every_batch_tiling(gpu, monkeypatch, tile_rows, function, B, T, N, D, dtype):
    print(f"case tiling rows={tile_rows} {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    monkeypatch.setenv("FRNN_TILE_ROWS", str(tile_rows))
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=13, init="randn")


# Head dims whose table holds two tilings: small calls run on the one with more workgroups per head (the cases
# above), calls that fill the device on the default one, which FRNN_FUSED_VARIANT=1 (no such entry: the table's
# default, and no switching) selects here at a small size; both with every batch tile height they are compiled for.
TWO_TILINGS = [
    ("gru", 14, 5, 2, 192, "bfloat16"), ("lstm", 10, 5, 2, 160, "bfloat16"), ("lstm", 9, 6, 3, 64, "float32"),
    ("gru", 11, 5, 2, 64, "float32"), ("slstm", 7, 5, 2, 64, "float32"), ("elman", 8, 5, 1, 96, "float32"),
    ("slstm", 9, 6, 2, 160, "bfloat16"), ("slstm", 6, 5, 3, 128, "bfloat16"),
    ("lstm", 6, 5, 1, 320, "float32"),       # backward: 20 workgroups of one wave / 5 of 4 waves
]


@pytest.mark.parametrize("function,B,T,N,D,dtype", TWO_TILINGS)
@pytest.mark.parametrize("tile_rows", [4, 8, 16])
@pytest.mark.parametrize("default_tiling", [True, False])
def test_both_tilings_of_head_dims_with_a_small_batch_one(gpu, monkeypatch, default_tiling, tile_rows, function, B, T, N, D, dtype):
    print(f"case two tilings default={default_tiling} rows={tile_rows} {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    monkeypatch.setenv("FRNN_TILE_ROWS", str(tile_rows))
    if default_tiling:
        monkeypatch.setenv("FRNN_FUSED_VARIANT", "1")
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=17, init="randn")


def test_fused_more_groups_than_one_launch_holds(gpu):
    """Workgroups that wait for each other must be co-resident, so a call with more (head, batch tile)
    groups than compute units / workgroups-per-head is split into several launches over the groups:
    5 heads x 13 batch tiles x 4 workgroups = 260 > 256 compute units."""
    print("case chunked launches", flush=True)
    check_case(gpu, "lstm", 208, 3, 5, 256, "bfloat16", "hip_fused", seed=19, init="randn")
    check_case(gpu, "elman", 130, 3, 2, 1024, "bfloat16", "hip_fused", seed=19, init="randn")  # 2 x 9 x 8 at 16 rows


HALF = [
    # function, B, T, N, D, backend
    ("lstm", 8, 16, 3, 256, "hip_fused"),      # 4 workgroups per head
    ("lstm", 20, 6, 2, 128, "hip_fused"),
    ("gru", 7, 9, 2, 192, "hip_fused"),
    ("slstm", 5, 8, 2, 64, "hip_fused"),
    ("elman", 18, 6, 1, 1024, "hip_fused"),
    ("lstm", 6, 5, 2, 96, "hip"),
    ("gru", 17, 4, 1, 64, "hip"),
    ("slstm", 4, 6, 1, 192, "hip"),
    ("elman", 9, 7, 2, 320, "hip"),
]


@pytest.mark.parametrize("function,B,T,N,D,backend", HALF)
def test_float16_matches_oracle(gpu, function, B, T, N, D, backend):
    """fp16 storage, fp32 accumulation and gate math (the reference's third dtype, flashrnn.py:73-78)."""
    print(f"case fp16 {backend} {function} B{B} T{T} N{N} D{D}", flush=True)
    check_case(gpu, function, B, T, N, D, "float16", backend, seed=23, init="randn")


ALT_SMALL = [
    ("lstm", 4, 8, 1, 64, "float32"),
    ("lstm", 3, 5, 2, 32, "bfloat16"),
    ("lstm", 20, 4, 2, 128, "bfloat16"),
    ("gru", 5, 9, 2, 64, "bfloat16"),
    ("gru", 17, 3, 1, 96, "float32"),
    ("slstm", 8, 6, 2, 64, "bfloat16"),
    ("slstm", 3, 4, 1, 192, "float32"),
    ("elman", 32, 8, 1, 1024, "bfloat16"),
    ("elman", 2, 5, 2, 32, "float32"),
]


@pytest.mark.parametrize("function,B,T,N,D,dtype", ALT_SMALL)
def test_alternating_matches_oracle(gpu, function, B, T, N, D, dtype):
    print(f"case alt {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    check_case(gpu, function, B, T, N, D, dtype, "hip", seed=11, init="randn")


def test_forward_only_no_grad(gpu):
    """Inference call: no cache is written, backward is refused."""
    print("case forward only", flush=True)
    check_case(gpu, "lstm", 6, 9, 2, 64, "bfloat16", "hip_fused", backward=False)
    check_case(gpu, "gru", 6, 9, 2, 64, "bfloat16", "hip", backward=False)


# ---- the benchmark configurations --------------------------------------------------------------
def test_config1_lstm_fp32_forward(gpu):
    print("case C1", flush=True)
    check_case(gpu, "lstm", 4, 256, 1, 64, "float32", "hip_fused", seed=1001, init="zeros", backward=False)
    check_case(gpu, "lstm", 4, 256, 1, 64, "float32", "hip", seed=1001, init="zeros", backward=False)


# Absolute max-abs bounds on the weight gradients of the full-size configurations: twice the larger of the two backends'
# measured errors (dR, db are sums over B*T tokens of bf16-stored factors; the general bound is relative to max|ref|).
# Measured (hip_fused / hip): C2 dR 0.179 / 0.167 (max |ref| 56), db 0.50 / 0.62 (224); C3 dR 0.35 / 0.36 (96), db 0.67 / 0.90
# (408); C4 dR 0.095 / 0.096 (32.5), db 0.71 / 0.70 (254); C5 dR 2.27 / 2.18 (534), db 2.38 / 1.88 (587).
SUM_BOUNDS = {"C2": {"dR": 0.36, "db": 1.24}, "C3": {"dR": 0.72, "db": 1.8}, "C4": {"dR": 0.19, "db": 1.42}, "C5": {"dR": 4.5, "db": 4.8}}


# Full size, both backends; besides the fp32 oracle every bf16 configuration is also held against the
# oracle run in torch.bfloat16 (the reference's vanilla backend in bf16): the HIP path must be closer.
@pytest.mark.parametrize("backend", ["hip_fused", "hip"])
def test_config2_lstm_bf16_full_size(gpu, backend):
    print(f"case C2 full {backend}", flush=True)
    check_case(gpu, "lstm", 8, 1024, 3, 256, "bfloat16", backend, seed=1002, init="randn", vs_bf16_vanilla=True,
               sum_bounds=SUM_BOUNDS["C2"])


@pytest.mark.parametrize("backend", ["hip_fused", "hip"])
def test_config3_gru_bf16_full_size(gpu, backend):
    print(f"case C3 full {backend}", flush=True)
    check_case(gpu, "gru", 16, 2048, 4, 128, "bfloat16", backend, seed=1003, init="zeros", vs_bf16_vanilla=True,
               sum_bounds=SUM_BOUNDS["C3"])


@pytest.mark.parametrize("backend", ["hip_fused", "hip"])
def test_config4_slstm_bf16_full_size(gpu, backend):
    print(f"case C4 full {backend}", flush=True)
    check_case(gpu, "slstm", 16, 4096, 4, 192, "bfloat16", backend, seed=1004, init="zeros",
               forget_bias_linspace=True, grad_on="h", vs_bf16_vanilla=True, sum_bounds=SUM_BOUNDS["C4"])


@pytest.mark.parametrize("backend", ["hip", "hip_fused"])
def test_config5_elman_full_size(gpu, backend):
    print(f"case C5 full {backend}", flush=True)
    check_case(gpu, "elman", 32, 1024, 1, 1024, "bfloat16", backend, seed=1005, init="zeros", vs_bf16_vanilla=True,
               sum_bounds=SUM_BOUNDS["C5"])


@pytest.mark.parametrize("N,D", [(24, 32), (12, 64), (6, 128), (3, 256), (1, 512)])
def test_head_dim_sweep_points_full_length(gpu, N, D):
    """The fused-path head-dim sweep of the fifth configuration (B = 16, T = 1024) at its real length."""
    print(f"case sweep N{N} D{D}", flush=True)
    check_case(gpu, "lstm", 16, 1024, N, D, "bfloat16", "hip_fused", seed=1006, init="zeros", vs_bf16_vanilla=True)


def test_slstm_mixed_fresh_and_running_elements(gpu):
    """Initial n zero for some elements and not for others: the kernels take the first-step branch m' = i per
    element, like the reference's native kernels (slstm_fused_pointwise.cuh:54-62); vanilla/slstm.py:21 would
    take it for none of them.  The HIP path must match the per-element oracle and differ from the whole-tensor
    one at the fresh elements."""
    import torch
    from flashrnn_amd import flashrnn
    from oracle import flashrnn_oracle, make_inputs
    from parity import assert_close

    print("case slstm mixed n0", flush=True)
    B, T, N, D = 6, 5, 2, 64
    for backend in ("hip_fused", "hip"):
        inp = make_inputs("slstm", B, T, N, D, 71, init="randn")
        s0 = inp["states"]
        s0[:, ::2, :, :, ::3] = 0.0              # every third unit of every other batch row starts fresh
        inp["Wx"][::2, 0, 0, :, ::3] = -4.0      # and has an input gate well below log sigmoid(f) + m
        dev = [inp[k].to(gpu) for k in ("Wx", "R", "b")]
        out, _ = flashrnn(*dev, s0.to(gpu), function="slstm", backend=backend, dtype="float32")
        per, _ = flashrnn_oracle(inp["Wx"].double(), inp["R"].double(), inp["b"].double(), s0.double(), "slstm",
                                 slstm_per_element_first_step=True)
        whole, _ = flashrnn_oracle(inp["Wx"].double(), inp["R"].double(), inp["b"].double(), s0.double(), "slstm")
        got = out.float().cpu()
        for k in range(4):
            assert_close(f"{backend} state {k}", got[k], per[k], "float32", "state")
        assert float((got[0].double() - whole[0]).abs().max()) > 1e-2


@pytest.mark.parametrize("function,B,T,N,D,dtype", [
    ("lstm", 336, 24, 12, 64, "bfloat16"), ("slstm", 300, 16, 12, 64, "bfloat16"), ("lstm", 340, 16, 24, 32, "bfloat16"),
    ("gru", 336, 24, 12, 64, "float16"), ("lstm", 160, 16, 12, 64, "float32"),
    # 8 compute waves and the producer wave, which also stores here
    ("lstm", 300, 12, 6, 128, "bfloat16"), ("gru", 290, 10, 6, 128, "float16"), ("lstm", 270, 8, 6, 128, "float16"),
    ("lstm", 330, 10, 8, 96, "bfloat16")])
def test_small_heads_at_large_batches(gpu, function, B, T, N, D, dtype):
    """Heads of one workgroup keep 4-row tiles up to many workgroups per compute unit (16 of up to 4 waves, 8 of up to 6,
    4 of up to 8 in the 16-bit types): here 450 to 2040 workgroups in one launch, with the producer wave and, up to 6
    waves, its stores in both passes."""
    print(f"case large batch {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    check_case(gpu, function, B, T, N, D, dtype, "hip_fused", seed=5, init="randn")
