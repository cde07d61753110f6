"""Parity of the clip / cut options (FlashRNNConfig.forward_clipval, gradient_recurrent_clipval,
gradient_recurrent_cut) through the *_opt entry points of the C ABI, both backends."""
import pytest
import torch

from parity import check_case

pytestmark = pytest.mark.gpu

# clip values small enough to be active on the seeded inputs (h reaches ~1, carried cotangents ~5)
OPTIONS = [
    dict(gradient_recurrent_clipval=0.5),
    dict(gradient_recurrent_cut=True),
    dict(forward_clipval=0.4),
    dict(forward_clipval=0.4, gradient_recurrent_clipval=0.5),
    dict(gradient_recurrent_clipval=0.5, gradient_recurrent_cut=True),
]
CASES = [
    # function, B, T, N, D, dtype, backend
    ("lstm", 5, 9, 2, 64, "float32", "hip_fused"),
    ("lstm", 8, 12, 3, 256, "bfloat16", "hip_fused"),    # 4 workgroups per head
    ("gru", 6, 8, 2, 128, "bfloat16", "hip_fused"),
    ("gru", 4, 7, 1, 256, "float32", "hip_fused"),
    ("slstm", 7, 10, 2, 192, "bfloat16", "hip_fused"),
    ("elman", 9, 8, 1, 512, "bfloat16", "hip_fused"),   # under forward_clipval: gate cache with the unclamped h
    ("elman", 5, 7, 2, 64, "float32", "hip_fused"),
    ("lstm", 5, 6, 1, 448, "float32", "hip_fused"),      # workgroups of two wave pairs
    ("slstm", 6, 5, 1, 1024, "bfloat16", "hip_fused"),   # the same in the 16-bit kernels
    ("gru", 5, 5, 1, 1024, "float32", "hip_fused"),      # four waves per tile, groups that span the device
    ("lstm", 5, 6, 2, 64, "bfloat16", "hip"),
    ("gru", 3, 7, 2, 96, "float32", "hip"),
    ("slstm", 4, 6, 1, 64, "float32", "hip"),
    ("elman", 6, 5, 2, 32, "float32", "hip"),
]


@pytest.mark.parametrize("function,B,T,N,D,dtype,backend", CASES)
@pytest.mark.parametrize("options", OPTIONS, ids=lambda o: "+".join(sorted(o)))
def test_options_match_oracle(gpu, options, function, B, T, N, D, dtype, backend):
    print(f"case options {options} {backend} {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    check_case(gpu, function, B, T, N, D, dtype, backend, seed=17, init="randn", options=options)


def test_options_off_are_bit_identical_to_plain_entry_points(gpu):
    """opt with all fields zero takes the same code path as the plain entry points."""
    from flashrnn_amd import FlashRNNConfig, flashrnn
    from oracle import make_inputs

    inp = make_inputs("lstm", 8, 32, 3, 256, 3, init="randn", round_to=torch.bfloat16)
    args = [inp[k].to(gpu, torch.bfloat16).requires_grad_(True) for k in ("Wx", "R", "b", "states")]
    ds = inp["dstates"].to(gpu, torch.bfloat16)
    outs = []
    for clip in (None, 1e30):  # a clamp that never bites must not change a bit either
        cfg = FlashRNNConfig(backend="hip_fused", function="lstm", dtype="bfloat16", head_dim=256, num_heads=3,
                             gradient_recurrent_clipval=clip, forward_clipval=clip)
        out, _ = flashrnn(*args, config=cfg)
        outs.append((out, torch.autograd.grad(out, args, grad_outputs=ds)))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0])
    for a, c in zip(outs[0][1], outs[1][1]):
        assert torch.equal(a, c)
