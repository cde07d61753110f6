"""The resident decode kernel (FlashRNNDecoder / flashrnn_decode / frnn_fused_decode_*): R stays in registers across
tokens, Wx arrives through a mailbox.  A chain of tokens must give the bits of one flashrnn() call over the sequence
(the reference's step path, flashrnn.py:957-985, is a sequence call on a sequence of one)."""
import pytest
import torch

from oracle import make_inputs

pytestmark = pytest.mark.gpu

KDT = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
IDLE = 1 << 21  # probes (~0.4 us each) after which a resident kernel of these tests ends by itself


def _device_inputs(gpu, function, B, T, N, D, dtype, seed):
    kdt = KDT[dtype]
    inp = make_inputs(function, B, T, N, D, seed, init="randn", round_to=kdt if kdt != torch.float32 else None)
    return {k: v.to(gpu, kdt).contiguous() for k, v in inp.items()}


CASES = [(f, B, N, D, "bfloat16") for f in ("lstm", "slstm", "gru", "elman") for (B, N, D) in ((8, 2, 64), (3, 2, 192), (8, 3, 256))]
CASES += [("lstm", 5, 2, 64, "float32"), ("gru", 4, 1, 256, "float16"), ("slstm", 4, 1, 128, "float32"),
          ("elman", 6, 1, 512, "bfloat16"), ("lstm", 1, 12, 32, "bfloat16"),
          ("lstm", 5, 1, 448, "float32"), ("gru", 4, 1, 512, "float32"),  # (fp32 from D = 384: waves in pairs, each with half of k)
          ("lstm", 6, 1, 1024, "float32"),  # (64 workgroups per head, spread over the device)
          ("lstm", 3, 1, 1024, "bfloat16")]                               # (the same in the 16-bit kernels at D = 1024)


@pytest.mark.parametrize("function,B,N,D,dtype", CASES)
def test_64_tokens_through_the_resident_kernel_equal_one_call_bit_for_bit(gpu, function, B, N, D, dtype):
    from flashrnn_amd import flashrnn, flashrnn_decode

    T = 64
    print(f"case decode {function} B{B} N{N} D{D} {dtype}", flush=True)
    x = _device_inputs(gpu, function, B, T, N, D, dtype, seed=71)
    with torch.no_grad():
        ref, _ = flashrnn(x["Wx"], x["R"], x["b"], x["states"], function=function, backend="hip_fused", dtype=dtype)
    got, last = flashrnn_decode(x["Wx"], x["R"], x["b"], x["states"], function=function, dtype=dtype, idle_polls=IDLE)
    torch.cuda.current_stream().synchronize()
    assert torch.equal(got, ref), f"max diff {(got.float() - ref.float()).abs().max().item():.3e}"
    assert torch.equal(last, ref[:, :, -1:])


def test_chunks_of_tokens_and_a_resumed_session_give_the_same_bits(gpu):
    """4 tokens per post; and a session that is closed after 24 tokens and continued by a new one from its states and
    fp32 carry."""
    from flashrnn_amd import FlashRNNDecoder, flashrnn, flashrnn_decode

    function, B, N, D, dtype, T = "slstm", 6, 2, 192, "bfloat16", 48
    print("case decode chunks / resume", flush=True)
    x = _device_inputs(gpu, function, B, T, N, D, dtype, seed=72)
    with torch.no_grad():
        ref, _ = flashrnn(x["Wx"], x["R"], x["b"], x["states"], function=function, backend="hip_fused", dtype=dtype)
    got, _ = flashrnn_decode(x["Wx"], x["R"], x["b"], x["states"], function=function, dtype=dtype, chunk=4, idle_polls=IDLE)
    assert torch.equal(got, ref)
    outs = []
    with FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, dtype=dtype, idle_polls=IDLE) as dec:
        for t in range(24):
            outs.append(dec.step(x["Wx"][:, t:t + 1].contiguous()))
    states, carry = dec.states.contiguous(), dec.carry
    with FlashRNNDecoder(x["R"], x["b"], states, function=function, dtype=dtype, carry=carry, idle_polls=IDLE) as dec2:
        for t in range(24, T):
            outs.append(dec2.step(x["Wx"][:, t:t + 1].contiguous()))
    torch.cuda.current_stream().synchronize()
    assert torch.equal(torch.cat(outs, dim=2), ref)


def test_a_session_ends_by_itself_when_idle_and_after_max_tokens(gpu):
    from flashrnn_amd import FlashRNNDecoder

    function, B, N, D, dtype = "lstm", 8, 3, 256, "bfloat16"
    print("case decode idle / max_tokens", flush=True)
    x = _device_inputs(gpu, function, B, 8, N, D, dtype, seed=73)
    dec = FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, dtype=dtype, idle_polls=4096)
    dec.kernel_stream.synchronize()            # nobody posts: the kernel gives up after 4096 probes and ends normally
    c = dec.control()
    assert c["ended"] == "idle bound reached" and c["tokens_served"] == 0 and not c["wait_expired"]
    assert torch.equal(dec.carry, x["states"][:, :, 0].float())   # the state it was given comes back untouched
    dec.close()
    dec = FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, dtype=dtype, idle_polls=IDLE, max_tokens=5)
    for t in range(5):
        out = dec.step(x["Wx"][:, t:t + 1].contiguous())
    dec.kernel_stream.synchronize()
    c = dec.control()
    assert c["ended"] == "max_tokens served" and c["tokens_served"] == 5 and c["tokens_posted"] == 5
    assert torch.isfinite(out.float()).all()
    dec.close()


def test_every_wait_gives_up_when_forced_from_the_host_and_every_kernel_ends_normally(gpu, monkeypatch):
    """FRNN_SPIN_LIMIT=-2: the resident kernel gives up its first wait at once, the collecting kernel too; nothing
    hangs, the results are NaN, close() reports it, and the next session is clean."""
    from flashrnn_amd import FlashRNNDecoder, flashrnn

    print("case decode forced give-up", flush=True)
    for function, B, N, D in (("lstm", 8, 3, 256), ("gru", 4, 2, 64)):
        x = _device_inputs(gpu, function, B, 4, N, D, "bfloat16", seed=74)
        monkeypatch.setenv("FRNN_SPIN_LIMIT", "-2")
        dec = FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, idle_polls=IDLE)
        out = dec.step(x["Wx"][:, 0:1].contiguous())
        dec.kernel_stream.synchronize()
        torch.cuda.current_stream().synchronize()
        assert torch.isnan(out.float()).all()
        with pytest.raises(RuntimeError, match="bounded wait"):
            dec.close()
        monkeypatch.delenv("FRNN_SPIN_LIMIT")
        with torch.no_grad():
            ref, _ = flashrnn(x["Wx"], x["R"], x["b"], x["states"], function=function, backend="hip_fused")
        with FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, idle_polls=IDLE) as dec:
            got = dec.step(x["Wx"].contiguous())
        torch.cuda.current_stream().synchronize()
        assert torch.equal(got, ref)


def test_a_captured_step_replays_token_after_token(gpu):
    """The step launch takes its token numbers from the mailbox, so one captured launch serves every token."""
    from flashrnn_amd import FlashRNNDecoder, flashrnn

    function, B, N, D, dtype, T = "lstm", 8, 3, 256, "bfloat16", 24
    print("case decode graph replay", flush=True)
    x = _device_inputs(gpu, function, B, T, N, D, dtype, seed=75)
    with torch.no_grad():
        ref, _ = flashrnn(x["Wx"], x["R"], x["b"], x["states"], function=function, backend="hip_fused", dtype=dtype)
    wx_in = torch.empty_like(x["Wx"][:, 0:1].contiguous())
    out = torch.empty((2, B, 1, N, D), dtype=torch.bfloat16, device=gpu)
    side = torch.cuda.Stream()
    outs = []
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # (capture needs a stream other than the default one; the session belongs to it)
        dec = FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, dtype=dtype, idle_polls=IDLE)
        wx_in.copy_(x["Wx"][:, 0:1])
        dec.step(wx_in, out=out)                       # token 0, eagerly (also warms up the launch path)
        outs.append(out.clone())
        # (not `with torch.cuda.graph(g)`: that context manager synchronises the whole device first, which waits for
        # the resident kernel to idle out)
        g = torch.cuda.CUDAGraph()
        g.capture_begin()
        dec.step(wx_in, out=out)
        g.capture_end()
        for t in range(1, T):
            wx_in.copy_(x["Wx"][:, t:t + 1])
            g.replay()
            outs.append(out.clone())
        dec.close()
    side.synchronize()
    assert torch.equal(torch.cat(outs, dim=2), ref)


def test_decode_arguments_are_checked_on_the_host(gpu):
    from flashrnn_amd import FlashRNNDecoder

    x = _device_inputs(gpu, "lstm", 4, 2, 2, 64, "bfloat16", seed=76)
    with pytest.raises(RuntimeError, match="slots"):
        FlashRNNDecoder(x["R"], x["b"], x["states"], slots=3)
    with pytest.raises(TypeError):
        FlashRNNDecoder(x["R"].float(), x["b"], x["states"])
    big = _device_inputs(gpu, "lstm", 4, 1, 2, 64, "bfloat16", seed=76)
    with pytest.raises(ValueError, match="fit"):       # 600 heads x 4-row tiles: more workgroups than stay resident at once
        s = torch.zeros(2, 4, 1, 1200, 64, dtype=torch.bfloat16, device=gpu)
        FlashRNNDecoder(torch.zeros(4, 1200, 64, 64, dtype=torch.bfloat16, device=gpu),
                        torch.zeros(4, 1200, 64, dtype=torch.bfloat16, device=gpu), s)
    with FlashRNNDecoder(x["R"], x["b"], x["states"], idle_polls=IDLE) as dec:
        with pytest.raises(RuntimeError, match="count"):
            dec.step(torch.zeros(4, 5, 4, 2, 64, dtype=torch.bfloat16, device=gpu))   # 5 tokens into 4 slots
