"""flashrnn_step / frnn_fused_step / frnn_alt_step: one time step with carried state (the reference's step
kernels, flashrnn.py:957-985).  With the fp32 carry a chain of steps must give the bits of one call over the
whole sequence; without it each step restarts from the rounded states, which still has to match the oracle run
step by step on rounded states."""
import pytest
import torch

from oracle import FUNCTIONS, make_inputs

pytestmark = pytest.mark.gpu

KDT = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
CASES = [
    # function, B, N, D, dtype, backend
    ("lstm", 8, 3, 256, "bfloat16", "hip_fused"),     # 4 workgroups per head
    ("lstm", 5, 2, 64, "float32", "hip_fused"),
    ("gru", 16, 4, 128, "bfloat16", "hip_fused"),
    ("gru", 3, 1, 256, "float16", "hip_fused"),
    ("slstm", 16, 4, 192, "bfloat16", "hip_fused"),
    ("elman", 32, 1, 1024, "bfloat16", "hip_fused"),
    ("lstm", 1, 12, 64, "bfloat16", "hip_fused"),
    ("slstm", 6, 1, 448, "float32", "hip_fused"),    # fp32 from D = 384: pairs of waves, each with half of k
    ("gru", 5, 1, 1024, "float32", "hip_fused"),     # fp32 D = 1024: four waves per tile, a quarter of k each
    ("lstm", 8, 3, 256, "bfloat16", "hip"),
    ("gru", 5, 2, 96, "float32", "hip"),
    ("slstm", 4, 2, 64, "bfloat16", "hip"),
    ("elman", 9, 1, 512, "bfloat16", "hip"),
]


def _device_inputs(gpu, function, B, T, N, D, dtype, seed):
    kdt = KDT[dtype]
    inp = make_inputs(function, B, T, N, D, seed, init="randn", round_to=kdt if kdt != torch.float32 else None)
    return {k: v.to(gpu, kdt).contiguous() for k, v in inp.items()}


@pytest.mark.parametrize("function,B,N,D,dtype,backend", CASES)
def test_64_steps_with_carry_equal_one_call_bit_for_bit(gpu, function, B, N, D, dtype, backend):
    from flashrnn_amd import flashrnn, flashrnn_step, make_carry

    T = 64
    print(f"case steps {backend} {function} B{B} N{N} D{D} {dtype}", flush=True)
    x = _device_inputs(gpu, function, B, T, N, D, dtype, seed=61)
    with torch.no_grad():
        ref, _ = flashrnn(x["Wx"], x["R"], x["b"], x["states"], function=function, backend=backend, dtype=dtype)
    states, carry = x["states"], make_carry(x["states"])
    outs = []
    for t in range(T):
        states = flashrnn_step(x["Wx"][:, t:t + 1].contiguous(), x["R"], x["b"], states, function=function,
                               backend=backend, dtype=dtype, carry=carry)
        outs.append(states)
    got = torch.cat(outs, dim=2)
    torch.cuda.synchronize()
    assert torch.equal(got, ref), f"max diff {(got.float() - ref.float()).abs().max().item():.3e}"


@pytest.mark.parametrize("function,dtype,backend", [("lstm", "bfloat16", "hip_fused"), ("gru", "bfloat16", "hip"),
                                                    ("slstm", "float32", "hip_fused")])
def test_steps_without_carry_match_the_oracle_on_rounded_states(gpu, function, dtype, backend):
    """No carry: every step starts from the stored (rounded) states, as the reference's step kernel does."""
    from flashrnn_amd import flashrnn_step
    from oracle import flashrnn_oracle
    from parity import assert_close

    B, T, N, D = 6, 12, 2, 64
    print(f"case steps no carry {backend} {function} {dtype}", flush=True)
    kdt = KDT[dtype]
    inp = make_inputs(function, B, T, N, D, 62, init="randn", round_to=kdt if kdt != torch.float32 else None)
    x = {k: v.to(gpu, kdt).contiguous() for k, v in inp.items()}
    odt = torch.float64 if dtype == "float32" else torch.float32
    S = FUNCTIONS[function][4]
    states, ref_states = x["states"], inp["states"].to(odt)
    for t in range(T):
        states = flashrnn_step(x["Wx"][:, t:t + 1].contiguous(), x["R"], x["b"], states, function=function,
                               backend=backend, dtype=dtype)
        with torch.no_grad():
            ref, _ = flashrnn_oracle(inp["Wx"][:, t:t + 1].to(odt), inp["R"].to(odt), inp["b"].to(odt), ref_states,
                                     function, slstm_per_element_first_step=True)
        got = states.float().cpu()
        for k in range(S):
            assert_close(f"step {t} state {k}", got[k], ref[k], dtype, "h" if k == 0 else "state")
        ref_states = got.to(odt) if dtype != "float32" else ref   # the oracle follows the rounded states


def test_step_can_be_captured_and_replayed(gpu):
    """A step launches one kernel and allocates nothing besides its output: capture it once, replay it per token."""
    from flashrnn_amd import flashrnn, flashrnn_step, make_carry

    function, B, T, N, D, dtype = "lstm", 8, 24, 3, 256, "bfloat16"
    print("case step graph", flush=True)
    x = _device_inputs(gpu, function, B, T, N, D, dtype, seed=63)
    with torch.no_grad():
        ref, _ = flashrnn(x["Wx"], x["R"], x["b"], x["states"], function=function, backend="hip_fused", dtype=dtype)
    wx_t = torch.empty_like(x["Wx"][:, :1])
    s_in = x["states"].clone()
    carry = make_carry(x["states"])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up outside capture (module load, symbol lookup)
        wx_t.copy_(x["Wx"][:, :1])
        flashrnn_step(wx_t, x["R"], x["b"], s_in, function=function, dtype=dtype, carry=carry.clone())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        s_out = flashrnn_step(wx_t, x["R"], x["b"], s_in, function=function, dtype=dtype, carry=carry)
    outs = []
    for t in range(T):
        wx_t.copy_(x["Wx"][:, t:t + 1])
        g.replay()
        s_in.copy_(s_out)
        outs.append(s_out.clone())
    torch.cuda.synchronize()
    assert torch.equal(torch.cat(outs, dim=2), ref)
