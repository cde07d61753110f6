"""Size-independent properties of the HIP path at the full benchmark sizes (no oracle needed):
chunked sequences, batch padding, agreement of the two backends, determinism."""
import pytest
import torch

from oracle import FUNCTIONS, make_inputs

pytestmark = pytest.mark.gpu


def _run(gpu, function, inp, backend, dtype="bfloat16", states=None, sl=slice(None)):
    from flashrnn_amd import flashrnn

    kdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    s0 = inp["states"] if states is None else states
    return flashrnn(inp["Wx"][:, sl].to(gpu, kdt), inp["R"].to(gpu, kdt), inp["b"].to(gpu, kdt), s0.to(gpu, kdt),
                    function=function, backend=backend, dtype=dtype)


FULL = [
    ("lstm", 8, 1024, 3, 256, 1002, "randn", False),
    ("gru", 16, 2048, 4, 128, 1003, "zeros", False),
    ("slstm", 16, 4096, 4, 192, 1004, "zeros", True),
    ("elman", 32, 1024, 1, 1024, 1005, "zeros", False),
]


@pytest.mark.parametrize("function,B,T,N,D,seed,init,fb", FULL)
def test_chunked_sequence_equals_one_pass(gpu, function, B, T, N, D, seed, init, fb):
    """run(T) == run(T1) then run(T2) from the carried last state, bit for bit: every step reads
    only the stored state of the step before."""
    print(f"case chunk {function} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs(function, B, T, N, D, seed, init=init, round_to=torch.bfloat16, forget_bias_linspace=fb)
    backend = "hip" if D == 1024 else "hip_fused"
    full, last = _run(gpu, function, inp, backend)
    T1 = T // 2 + 3
    a, la = _run(gpu, function, inp, backend, sl=slice(0, T1))
    if function in ("lstm", "slstm", "gru", "elman"):
        c, lc = _run(gpu, function, inp, backend, states=la, sl=slice(T1, T))
    torch.cuda.synchronize()
    assert torch.equal(a, full[:, :, :T1])
    # the carried state is rounded to the storage type; states kept in fp32 registers inside one
    # pass (c, n, m) therefore differ in the last bits after the cut, h by what that propagates
    ref = full[:, :, T1:].float()
    err = (c.float() - ref).abs()
    assert float(err[0].max()) <= 2e-2, float(err[0].max())  # h
    assert not bool((err > 4e-2 * torch.clamp(ref.abs(), min=1.0)).any()), float(err.max())
    assert torch.equal(lc, c[:, :, -1:])


@pytest.mark.parametrize("function,B,T,N,D,seed,init,fb", FULL[:3] + [("lstm", 16, 512, 1, 768, 1006, "zeros", False)])
def test_fused_and_alternating_agree(gpu, function, B, T, N, D, seed, init, fb):
    print(f"case fused-vs-alt {function} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs(function, B, T, N, D, seed, init=init, round_to=torch.bfloat16, forget_bias_linspace=fb)
    f, _ = _run(gpu, function, inp, "hip_fused")
    a, _ = _run(gpu, function, inp, "hip")
    torch.cuda.synchronize()
    assert torch.isfinite(f.float()).all() and torch.isfinite(a.float()).all()
    S = FUNCTIONS[function][4]
    for k in range(S):
        ref = a[k].float()
        err = (f[k].float() - ref).abs()
        # two bf16 trajectories of the same recurrence: each is within the parity tolerance of the oracle
        assert not bool((err > 4e-2 * torch.clamp(ref.abs(), min=1.0)).any()), (k, float(err.max()))


@pytest.mark.parametrize("tile_rows", [4, 8, 16])
def test_batch_rows_are_independent_of_padding(gpu, monkeypatch, tile_rows):
    """Rows of a run equal the same rows of a run with more rows: padded rows of the MFMA tile never
    reach valid rows.  Bit for bit within one batch tiling (forced here); between tilings the
    compiler schedules the same fp32 math differently, so those agree to rounding only."""
    print(f"case padding rows={tile_rows}", flush=True)
    function, T, N, D = "lstm", 33, 2, 256
    inp = make_inputs(function, 21, T, N, D, 5, init="randn", round_to=torch.bfloat16)

    def run(B):
        sub = {k: (v[:B] if k == "Wx" else v[:, :B] if k in ("states", "dstates") else v) for k, v in inp.items()}
        return _run(gpu, function, sub, "hip_fused")[0]

    monkeypatch.setenv("FRNN_TILE_ROWS", str(tile_rows))
    outs = {B: run(B) for B in (3, 5, 8, 16, 21)}
    monkeypatch.setenv("FRNN_TILE_ROWS", str(16 if tile_rows == 4 else 4))
    other = run(21)
    torch.cuda.synchronize()
    for B in (3, 5, 8, 16):
        assert torch.equal(outs[B], outs[21][:, :B]), B
    assert float((outs[21].float() - other.float()).abs().max()) <= 2e-2


def test_padded_rows_do_not_reach_weight_gradients(gpu):
    from flashrnn_amd import flashrnn

    print("case padding grads", flush=True)
    function, T, N, D = "gru", 12, 2, 128
    inp = make_inputs(function, 16, T, N, D, 9, init="randn", round_to=torch.bfloat16)

    def grads(B, zero_tail):
        Wx = inp["Wx"][:B].to(gpu).requires_grad_(True)
        R = inp["R"].to(gpu).requires_grad_(True)
        b = inp["b"].to(gpu).requires_grad_(True)
        s0 = inp["states"][:, :B].to(gpu).requires_grad_(True)
        ds = inp["dstates"][:, :B].clone()
        if zero_tail:
            ds[:, 5:] = 0
        out, _ = flashrnn(Wx, R, b, s0, function=function, backend="hip_fused", dtype="bfloat16")
        return torch.autograd.grad(out, [R, b], grad_outputs=ds.to(gpu).to(out.dtype))

    g5 = grads(5, False)
    g16 = grads(16, True)  # rows 5..15 present but with zero cotangent: must contribute nothing
    torch.cuda.synchronize()
    for a, c in zip(g5, g16):
        assert float((a - c).abs().max()) <= 1e-3 * max(1.0, float(a.abs().max()))


def test_repeated_calls_are_deterministic(gpu):
    print("case determinism", flush=True)
    inp = make_inputs("lstm", 8, 256, 3, 256, 3, init="randn", round_to=torch.bfloat16)
    a = _run(gpu, "lstm", inp, "hip_fused")[0]
    for _ in range(3):
        c = _run(gpu, "lstm", inp, "hip_fused")[0]
        assert torch.equal(a, c)


def test_sequence_longer_than_the_tag_period(gpu):
    """T = 66000 steps: the step tags of the workgroup exchange (16 bits forward, 8 bits backward)
    wrap around; the fused kernels must still agree with the alternating backend, which has no
    exchange, in every state and in dWx."""
    from flashrnn_amd import flashrnn

    function, B, T, N, D = "lstm", 2, 66000, 1, 256
    print(f"case tag-wrap {function} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs(function, B, T, N, D, 77, init="zeros", round_to=torch.bfloat16)
    g = torch.Generator(device="cpu").manual_seed(78)
    dst = (torch.randn((2, B, T, N, D), generator=g) * 0.1).to(gpu, torch.bfloat16)
    out = {}
    for backend in ("hip_fused", "hip"):
        Wx = inp["Wx"].to(gpu, torch.bfloat16).requires_grad_(True)
        st, _ = flashrnn(Wx, inp["R"].to(gpu, torch.bfloat16), inp["b"].to(gpu, torch.bfloat16), None,
                         function=function, backend=backend, dtype="bfloat16")
        (dWx,) = torch.autograd.grad(st, [Wx], grad_outputs=dst)
        out[backend] = (st.detach().float(), dWx.float())
    torch.cuda.synchronize()
    for k, name in enumerate(("states", "dWx")):
        f, a = out["hip_fused"][k], out["hip"][k]
        assert torch.isfinite(f).all() and torch.isfinite(a).all(), name
        err = (f - a).abs()
        # two bf16 trajectories of the same recurrence, as in test_fused_and_alternating_agree
        assert not bool((err > 4e-2 * torch.clamp(a.abs(), min=1.0)).any()), (name, float(err.max()))
        # and the last steps (forward) / first steps (backward) are as close as the others: no drift after the wrap
        tail = err[:, :, -256:] if name == "states" else err[:, :256]
        assert float(tail.max()) <= 4e-2 * max(1.0, float(a.abs().max())), (name, float(tail.max()))


@pytest.mark.parametrize("function,B,T,N,D", [("lstm", 16, 512, 1, 768), ("slstm", 8, 256, 1, 768), ("gru", 8, 256, 1, 1024), ("lstm", 8, 256, 1, 1024),
                                              ("lstm", 8, 512, 3, 256)])
def test_fused_and_alternating_gradients_agree(gpu, function, B, T, N, D):
    """Backward of long sequences on the largest tilings (12 and 16 workgroups per head, part of the
    transposed R in LDS): dWx and dR of the two backends agree as two bf16 trajectories do."""
    from flashrnn_amd import flashrnn

    print(f"case fused-vs-alt gradients {function} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs(function, B, T, N, D, 31, init="zeros", round_to=torch.bfloat16)
    S = FUNCTIONS[function][4]
    g = torch.Generator(device="cpu").manual_seed(32)
    dst = (torch.randn((S, B, T, N, D), generator=g) * 0.1).to(gpu, torch.bfloat16)
    out = {}
    for backend in ("hip_fused", "hip"):
        Wx = inp["Wx"].to(gpu, torch.bfloat16).requires_grad_(True)
        R = inp["R"].to(gpu, torch.bfloat16).requires_grad_(True)
        st, _ = flashrnn(Wx, R, inp["b"].to(gpu, torch.bfloat16), None, function=function, backend=backend, dtype="bfloat16")
        out[backend] = [x.float() for x in torch.autograd.grad(st, [Wx, R], grad_outputs=dst)]
    torch.cuda.synchronize()
    for k, name in enumerate(("dWx", "dR")):
        f, a = out["hip_fused"][k], out["hip"][k]
        assert torch.isfinite(f).all() and torch.isfinite(a).all(), name
        err = (f - a).abs()
        scale = float(a.abs().max())
        # dWx: per element as in test_fused_and_alternating_agree; dR: a sum over B*T tokens, bf16-rounded on return
        tol = 4e-2 * torch.clamp(a.abs(), min=1.0) if name == "dWx" else torch.full_like(a, max(4e-2, 2e-2 * scale))
        assert not bool((err > tol).any()), (name, float(err.max()), scale)


def test_layout_options_equal_the_default_layouts(gpu):
    """A call that declares other public layouts (time-major input, head-major R and bias, time-major
    output) returns the default call's result in the declared output layout, gradients included."""
    from flashrnn_amd import FlashRNNConfig, flashrnn

    print("case layouts", flush=True)
    B, T, N, D = 5, 7, 2, 64
    inp = make_inputs("lstm", B, T, N, D, 77, init="randn", round_to=torch.bfloat16)
    leaves = [inp[k].to(gpu, torch.bfloat16).requires_grad_(True) for k in ("Wx", "R", "b", "states")]
    ds = inp["dstates"].to(gpu, torch.bfloat16)
    out, last = flashrnn(*leaves, function="lstm", backend="hip_fused")
    g = torch.autograd.grad(out, leaves, grad_outputs=ds)
    cfg = FlashRNNConfig(function="lstm", backend="hip_fused", head_dim=D, num_heads=N, batch_size=B,
                         input_shape="TBGHD", recurrent_shape="HPGD", bias_shape="HDG", output_shape="STBHD")
    Wx2 = leaves[0].detach().permute(1, 0, 2, 3, 4).contiguous().requires_grad_(True)     # T B G H D
    R2 = leaves[1].detach().permute(1, 3, 0, 2).contiguous().requires_grad_(True)         # H P G D
    b2 = leaves[2].detach().permute(1, 2, 0).contiguous().requires_grad_(True)            # H D G
    s2 = leaves[3].detach().permute(0, 2, 1, 3, 4).contiguous().requires_grad_(True)      # S T B H D
    out2, last2 = flashrnn(Wx2, R2, b2, s2, config=cfg)
    g2 = torch.autograd.grad(out2, [Wx2, R2, b2, s2], grad_outputs=ds.permute(0, 2, 1, 3, 4))
    torch.cuda.synchronize()
    assert out2.shape == (2, T, B, N, D) and last2.shape == (2, 1, B, N, D)
    assert torch.equal(out2.permute(0, 2, 1, 3, 4), out) and torch.equal(last2.permute(0, 2, 1, 3, 4), last)
    assert torch.equal(g2[0].permute(1, 0, 2, 3, 4), g[0])
    assert torch.equal(g2[1].permute(2, 0, 3, 1), g[1])
    assert torch.equal(g2[2].permute(2, 0, 1), g[2])
    assert torch.equal(g2[3].permute(0, 2, 1, 3, 4), g[3])
    # default initial state from initial_val
    cfg0 = FlashRNNConfig(function="lstm", backend="hip_fused", head_dim=D, num_heads=N, batch_size=B, initial_val=0.25)
    a, _ = flashrnn(leaves[0].detach(), leaves[1].detach(), leaves[2].detach(), None, config=cfg0)
    s_const = torch.full((2, B, 1, N, D), 0.25, device=gpu, dtype=torch.bfloat16)
    c, _ = flashrnn(leaves[0].detach(), leaves[1].detach(), leaves[2].detach(), s_const, function="lstm", backend="hip_fused")
    torch.cuda.synchronize()
    assert torch.equal(a, c)


@pytest.mark.parametrize("function,B,T,N,D", [("lstm", 8, 24, 3, 256), ("gru", 16, 8, 1, 768)])
def test_cooperative_launch_gives_the_same_result(gpu, function, B, T, N, D, monkeypatch):
    """FRNN_COOPERATIVE=1 launches the kernels whose workgroups wait for each other as cooperative
    kernels (one at a time per device, for callers that overlap fused calls on several streams):
    same bits as the plain launch."""
    print(f"case cooperative {function} B{B} T{T} N{N} D{D}", flush=True)
    inp = make_inputs(function, B, T, N, D, 31, init="randn", round_to=torch.bfloat16)

    def run():
        from flashrnn_amd import flashrnn

        leaves = [inp[k].to(gpu, torch.bfloat16).requires_grad_(True) for k in ("Wx", "R", "b", "states")]
        out, _ = flashrnn(*leaves, function=function, backend="hip_fused")
        g = torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"].to(gpu, torch.bfloat16))
        torch.cuda.synchronize()
        return (out,) + g

    plain = run()
    monkeypatch.setenv("FRNN_COOPERATIVE", "1")
    coop = run()
    for a, b in zip(plain, coop):
        assert torch.equal(a, b)


@pytest.mark.parametrize("function,B,T,N,D,dtype", [
    ("lstm", 8, 24, 3, 256, torch.bfloat16), ("elman", 9, 20, 1, 1024, torch.bfloat16), ("gru", 5, 9, 1, 256, torch.float32),
])
def test_agent_scope_exchange_stores_give_the_same_result(gpu, function, B, T, N, D, dtype, monkeypatch):
    """The workgroups of a head exchange h (forward) and partial sums (backward) through tagged words.  When a
    group's workgroups share an XCD (checked by the kernels at launch) the stores stay in that XCD's L2; otherwise,
    or with FRNN_AGENT_STORES=1, they are written through to memory.  Both paths carry the same words: same bits."""
    print(f"case agent stores {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    inp = make_inputs(function, B, T, N, D, 33, init="randn", round_to=dtype)

    def run():
        from flashrnn_amd import flashrnn

        leaves = [inp[k].to(gpu, dtype).requires_grad_(True) for k in ("Wx", "R", "b", "states")]
        out, _ = flashrnn(*leaves, function=function, backend="hip_fused", dtype={torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype])
        g = torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"].to(gpu, dtype))
        torch.cuda.synchronize()
        return (out,) + g

    near = run()
    monkeypatch.setenv("FRNN_AGENT_STORES", "1")
    far = run()
    for a, b in zip(near, far):
        assert torch.equal(a, b)


@pytest.mark.parametrize("function,B,N,D,note", [
    ("lstm", 80, 1, 768, "12 workgroups per head: an XCD of 32 compute units holds 2 groups, a launch 16; 20 groups"),
    ("slstm", 100, 4, 192, "3 workgroups per head forward: 10 groups per XCD, 80 per launch; 100 groups"),
    ("lstm", 70, 1, 320, "5 workgroups per head: 6 groups per XCD, 48 per launch; 18 groups at 4 rows"),
])
def test_launches_sized_by_the_room_of_an_xcd(gpu, monkeypatch, function, B, N, D, note):
    """The workgroups of a group share one XCD, so a launch holds 8 * floor(32 / workgroups per head) groups;
    calls with more groups run as several launches.  4-row tiles are forced to get many groups from a small
    batch."""
    from parity import check_case

    print(f"case xcd room {function} B{B} N{N} D{D}: {note}", flush=True)
    monkeypatch.setenv("FRNN_TILE_ROWS", "4")
    check_case(gpu, function, B, 3, N, D, "bfloat16", "hip_fused", seed=27, init="randn")


@pytest.mark.parametrize("copies", [False, True])
@pytest.mark.parametrize("function,options", [("lstm", None), ("gru", None), ("slstm", None), ("elman", None),
                                              ("lstm", {"recompute_gates": True})])
def test_batch_ranges_for_tensors_beyond_32_bit_offsets(gpu, monkeypatch, function, options, copies):
    """flashrnn() splits a fused problem whose tensors would reach 2 GiB into calls over batch ranges (the kernels use
    32-bit byte offsets); dR and db are summed over the ranges.  The ranges use the full state tensors in place
    (frnn_options.batch_stride), or contiguous copies of their slices where the planes lie too far apart (forced here
    with FRNN_RANGES_COPY).  FRNN_TEST_MAX_BATCH makes the wrapper believe that a call takes at most 17 rows, so that
    a small problem splits into ranges of 16, 16 and 8 rows; the real limit is crossed by
    test_a_problem_whose_tensors_pass_2_gib_at_its_real_size."""
    import importlib

    from parity import check_case

    mod = importlib.import_module("flashrnn_amd.flashrnn")  # (the package attribute of that name is the function)
    print(f"case batch ranges {function} {options} copies={copies}", flush=True)
    B, T, N, D = 40, 6, 2, 64
    monkeypatch.setenv("FRNN_TEST_MAX_BATCH", "17")
    if copies:
        monkeypatch.setenv("FRNN_RANGES_COPY", "1")
    calls = []
    real = mod._run_forward
    monkeypatch.setattr(mod, "_run_forward", lambda *a, **k: (calls.append((a[0].shape[0], k.get("batch_stride", 0))), real(*a, **k))[1])
    check_case(gpu, function, B, T, N, D, "bfloat16", "hip_fused", seed=28, init="randn", options=options)
    assert calls == [(16, 0 if copies else B), (16, 0 if copies else B), (8, 0 if copies else B)], calls


@pytest.mark.parametrize("backend", ["hip_fused", "hip"])
def test_slstm_backward_through_the_carried_state_of_two_calls(gpu, backend):
    """Truncated sequences: the second call starts from the last states of the first and autograd carries its
    ds0 (cotangents on h, c and n; 0 on the stabiliser m) back into the first call.  In fp32 the result must
    equal the oracle over the whole sequence (stabiliser held constant, as the native adjoint holds it)."""
    from flashrnn_amd import flashrnn
    from oracle import flashrnn_oracle_backward
    from parity import assert_close

    print(f"case slstm two chunks {backend}", flush=True)
    B, T, N, D, T1 = 5, 12, 2, 64, 7
    inp = make_inputs("slstm", B, T, N, D, 29, init="randn", grad_on="all")
    inp["dstates"][3] = 0
    leaves = [inp[k].to(gpu).requires_grad_(True) for k in ("Wx", "R", "b", "states")]
    Wx, R, b, s0 = leaves
    o1, last1 = flashrnn(Wx[:, :T1], R, b, s0, function="slstm", backend=backend, dtype="float32")
    o2, _ = flashrnn(Wx[:, T1:], R, b, last1, function="slstm", backend=backend, dtype="float32")
    out = torch.cat([o1, o2], dim=2)
    grads = torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"].to(gpu))
    torch.cuda.synchronize()
    ref_out, ref_g = flashrnn_oracle_backward(*[inp[k].double() for k in ("Wx", "R", "b", "states")], "slstm",
                                              inp["dstates"].double(), slstm_per_element_first_step=True,
                                              slstm_detach_m=True)
    for k in range(4):
        assert_close(f"state {k}", out[k].detach().cpu(), ref_out[k], "float32", "state")
    for name, g, r in zip(("dWx", "dR", "db", "ds0"), grads, ref_g):
        assert_close(name, g.cpu(), r, "float32", "token")


@pytest.mark.parametrize("function,B,T,N,D,dtype", [
    ("lstm", 9, 11, 3, 64, "bfloat16"), ("lstm", 6, 7, 5, 32, "bfloat16"), ("lstm", 5, 6, 2, 128, "bfloat16"),
    ("slstm", 7, 9, 2, 64, "bfloat16"), ("slstm", 4, 5, 3, 32, "float16"), ("gru", 10, 8, 2, 64, "bfloat16"),
    ("gru", 3, 6, 4, 32, "bfloat16"), ("gru", 6, 5, 1, 96, "float16"), ("lstm", 4, 1, 2, 64, "bfloat16"),
    ("gru", 7, 6, 2, 128, "bfloat16"), ("lstm", 6, 5, 1, 128, "float16")])
def test_producer_wave_stores_give_the_same_bits(gpu, monkeypatch, function, B, T, N, D, dtype):
    """The instantiations whose producer wave stores the outputs (forward: states and gate cache; backward: dWx), which
    the host picks for launches that fill the device, only move data differently: every output and gradient must come
    out bit for bit as with the compute lanes' own stores."""
    from flashrnn_amd import flashrnn

    print(f"case producer stores {function} B{B} T{T} N{N} D{D} {dtype}", flush=True)
    kdt = {"bfloat16": torch.bfloat16, "float16": torch.float16}[dtype]
    inp = make_inputs(function, B, T, N, D, 41, init="randn", round_to=kdt)
    res = {}
    for flag in ("0", "1"):
        monkeypatch.setenv("FRNN_PRODUCER_STORES", flag)
        leaves = [inp[k].to(gpu, kdt).requires_grad_() for k in ("Wx", "R", "b", "states")]
        out, last = flashrnn(*leaves, function=function, backend="hip_fused", dtype=dtype)
        grads = torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"].to(gpu, kdt))
        with torch.no_grad():  # the inference forward (no gate cache) as well
            out2, _ = flashrnn(*[x.detach() for x in leaves], function=function, backend="hip_fused", dtype=dtype)
        torch.cuda.synchronize()
        res[flag] = [out.detach(), out2] + [g.detach() for g in grads]
    for a, b in zip(res["0"], res["1"]):
        assert torch.equal(a, b), f"max diff {(a.float() - b.float()).abs().max().item():.3e}"


def test_a_problem_whose_tensors_pass_2_gib_at_its_real_size(gpu):
    """LSTM bf16 B = 400, T = 1024, N = 12, D = 64: Wx, dWx and the gate cache are 2.5 GB each, beyond the 32-bit offsets
    of the fused kernels, so flashrnn() runs the call as batch ranges.  Batch rows are independent: 16 rows (the first 8
    and the last 8, i.e. both ends of the range split) go through the oracle; dR and db, which sum over all rows, are
    compared with the alternating backend's on the whole problem (64-bit addressing, one call)."""
    from flashrnn_amd import flashrnn
    from oracle import flashrnn_oracle_backward
    from parity import assert_close

    function, B, T, N, D = "lstm", 400, 1024, 12, 64
    print(f"case beyond 2 GiB {function} B{B} T{T} N{N} D{D}", flush=True)
    g = torch.Generator(device=gpu).manual_seed(77)
    rnd = lambda *shape, scale=1.0: (torch.randn(*shape, generator=g, device=gpu, dtype=torch.float32) * scale).to(torch.bfloat16)
    Wx = torch.empty((B, T, 4, N, D), dtype=torch.bfloat16, device=gpu)
    for b0 in range(0, B, 50):  # (drawn in fp32 in slices: the whole tensor in fp32 would be 5 GB more)
        Wx[b0:b0 + 50] = rnd(50, T, 4, N, D)
    assert Wx.numel() * 2 >= 2 ** 31
    R, b, s0 = rnd(4, N, D, D, scale=D ** -0.5), rnd(4, N, D, scale=0.1), rnd(2, B, 1, N, D)
    ds = torch.empty((2, B, T, N, D), dtype=torch.bfloat16, device=gpu)
    for b0 in range(0, B, 50):
        ds[:, b0:b0 + 50] = rnd(2, 50, T, N, D)
    res = {}
    for backend in ("hip_fused", "hip"):
        leaves = [x.clone().requires_grad_() for x in (Wx, R, b, s0)]
        out, last = flashrnn(*leaves, function=function, backend=backend)
        grads = torch.autograd.grad(out, leaves, grad_outputs=ds)
        torch.cuda.synchronize()
        res[backend] = (out.detach(), [x.detach() for x in grads])
        del leaves, out, grads
    rows = list(range(8)) + list(range(B - 8, B))
    ref_out, ref_g = flashrnn_oracle_backward(Wx[rows].float().cpu(), R.float().cpu(), b.float().cpu(), s0[:, rows].float().cpu(),
                                              function, ds[:, rows].float().cpu())
    out, grads = res["hip_fused"]
    got = out[:, rows].float().cpu()
    assert_close("h", got[0], ref_out[0], "bfloat16", "h")
    assert_close("c", got[1], ref_out[1], "bfloat16", "state")
    assert_close("dWx", grads[0][rows].float().cpu(), ref_g[0], "bfloat16", "token")
    assert_close("ds0", grads[3][:, rows].float().cpu(), ref_g[3], "bfloat16", "token")
    # the weight gradients of the two backends: each is within 3e-3 .. 4e-3 of max|ref| of the exact sum
    for name, i in (("dR", 1), ("db", 2)):
        a, c = grads[i].float(), res["hip"][1][i].float()
        e, m = float((a - c).abs().max()), float(c.abs().max())
        print(f"  {name}: fused (batch ranges) vs alternating: max abs diff {e:.3e}, max |ref| {m:.1f}", flush=True)
        assert e <= 1e-2 * m, f"{name}: {e:.3e} > 1e-2 * {m:.1f}"
    assert torch.equal(res["hip_fused"][0][:, rows], res["hip"][0][:, rows]) or \
        float((res["hip_fused"][0][:, rows].float() - res["hip"][0][:, rows].float()).abs().max()) <= 2e-2
