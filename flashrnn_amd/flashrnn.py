"""Functional API and autograd shim.

Mirrors the reference's operator interface (flashrnn/flashrnn/flashrnn.py):
  * ``flashrnn(Wx, R, b, states=None, function=, config=, backend=, dtype=)``   :1114-1135
  * ``FlashRNNConfig`` and ``rnn_function_registry``                           :49-71, :124-337
  * the autograd.Function shims ``FlashRNNFunctionFused`` / ``FlashRNNFunction`` :679-889
with backends ``hip_fused`` (for the reference's ``cuda_fused``) and ``hip`` (for ``cuda``).

What the shim does NOT do, because the kernels make it unnecessary: permute inputs to internal
layouts (:1130-1133), make them contiguous copies (:1053), pad the batch (:699-717), transpose R
for the backward pass (:746) or slice dWx (:789-796).
"""
from __future__ import annotations

import atexit
import functools
import os
from dataclasses import dataclass
from typing import Optional, Sequence, Union

import torch

from . import _lib

# function -> (num_gates_r, num_gates_w, num_gates_i, num_gates_t, num_states); flashrnn.py:49-71
rnn_function_registry = {
    "slstm": {"gates_states": (4, 4, 4, 4, 4), "constants": {}, "simple_agg": True},
    "lstm": {"gates_states": (4, 4, 4, 4, 2), "constants": {}, "simple_agg": True},
    "gru": {"gates_states": (3, 3, 4, 4, 1), "constants": {}, "simple_agg": False},
    "elman": {"gates_states": (1, 1, 1, 1, 1), "constants": {}, "simple_agg": True},
}

DTYPE_DICT = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}
BACKENDS = ("hip_fused", "hip")


@dataclass
class FlashRNNConfig:
    """The fields of the reference's FlashRNNConfig (flashrnn.py:124-231) that describe the
    problem; tiling, internal layouts and per-tensor dtypes have no counterpart here."""

    backend: str = "hip_fused"
    function: str = "lstm"
    dtype: str = "bfloat16"
    head_dim: int = -1
    num_heads: int = -1
    hidden_dim: int = -1
    batch_size: int = 8
    # truncated backpropagation: no gradient through R h (flashrnn.py:132, backward_cut)
    gradient_recurrent_cut: bool = False
    # clamp of the cotangent carried into h_t from step t+1 (flashrnn.py:134)
    gradient_recurrent_clipval: Optional[float] = None
    # clamp of every new h, invisible to the backward pass (flashrnn.py:136); unlike the reference,
    # which wires gradient_recurrent_clipval into both clamps (:361-382), it acts on its own
    forward_clipval: Optional[float] = None
    num_states: int = 0
    num_gates_r: int = 0
    num_gates_w: int = 0
    num_gates_i: int = 0
    num_gates_t: int = 0
    simple_agg: bool = True
    # layouts of the tensors the caller hands over and gets back (flashrnn.py:163-173; B batch, T time,
    # G gate, H head, D unit, P previous unit, S state).  The kernels read the defaults as they are;
    # any other layout is permuted on the way in and out (the reference permutes every layout to an
    # internal one, flashrnn.py:892-924)
    input_shape: str = "BTGHD"
    output_shape: str = "SBTHD"
    recurrent_shape: str = "GHDP"
    bias_shape: str = "GHD"
    # value of the default initial state, one number or one per state (flashrnn.py:204, :946-953)
    initial_val: Union[float, Sequence[float]] = 0.0
    # hip_fused only, no counterpart in the reference (which always stores the activated gates of every step,
    # fused/flashrnn.cc:97-112): the training forward writes no gate cache and the backward pass rebuilds the
    # gates from Wx, b and R h_(t-1).  Halves what a training forward writes and the activation memory it
    # leaves behind; ValueError where no such kernel exists (see frnn_fused_recompute_supported)
    recompute_gates: bool = False
    # per-tensor types of the reference (flashrnn.py:190-197: biases, recurrent matrix, inputs, gates,
    # states, internal accumulation).  The kernels take every tensor in the one storage type `dtype`,
    # accumulate in fp32 and compute the gates in fp32, so each may only be None or `dtype`
    # (dtype_acc and dtype_a also "float32", which is what happens)
    dtype_acc: Optional[str] = "float32"
    dtype_b: Optional[str] = None
    dtype_r: Optional[str] = None
    dtype_w: Optional[str] = None
    dtype_g: Optional[str] = None
    dtype_s: Optional[str] = None
    dtype_a: Optional[str] = None
    # True: inputs of any floating type are cast to `dtype` on the way in (the reference's
    # custom_fwd(cast_inputs=...), flashrnn.py:690-695); False: they must arrive in `dtype`
    enable_automatic_mixed_precision: bool = True

    def __post_init__(self):
        if self.function not in rnn_function_registry:
            raise ValueError(f"RNN function {self.function} not in registry")
        if self.backend not in BACKENDS:
            raise ValueError(
                f"Unknown backend {self.backend}: this package provides {BACKENDS}; the pure-PyTorch "
                "'vanilla' loop is the test oracle and is not part of the package")
        if self.dtype not in DTYPE_DICT:
            raise ValueError(f"dtype {self.dtype} not supported (bfloat16, float16, float32)")
        for name, canon in (("input_shape", "BTGHD"), ("output_shape", "SBTHD"), ("recurrent_shape", "GHDP"),
                            ("bias_shape", "GHD")):
            if sorted(getattr(self, name)) != sorted(canon):
                raise ValueError(f"{name} must be a permutation of {canon}, got {getattr(self, name)}")
        for name in ("dtype_b", "dtype_r", "dtype_w", "dtype_g", "dtype_s"):
            v = getattr(self, name)
            if v is None:
                setattr(self, name, self.dtype)
            elif v != self.dtype:
                raise ValueError(f"{name}={v}: the HIP kernels take every tensor in the one storage type "
                                 f"dtype={self.dtype} (accumulation and gate math are fp32 whatever it is)")
        for name in ("dtype_acc", "dtype_a"):
            v = getattr(self, name)
            if v is None:
                setattr(self, name, "float32")
            elif v not in ("float32", self.dtype):
                raise ValueError(f"{name}={v}: accumulation and gate math are fp32")
        for name in ("gradient_recurrent_clipval", "forward_clipval"):
            v = getattr(self, name)
            if v is not None and not v > 0:
                raise ValueError(f"{name} must be positive or None, got {v}")
        (self.num_gates_r, self.num_gates_w, self.num_gates_i, self.num_gates_t,
         self.num_states) = rnn_function_registry[self.function]["gates_states"]
        self.simple_agg = rnn_function_registry[self.function]["simple_agg"]
        if self.num_heads <= 0 and self.head_dim <= 0:
            self.num_heads = 1
        if self.num_heads <= 0:
            self.num_heads = self.hidden_dim // self.head_dim
        elif self.head_dim <= 0:
            self.head_dim = self.hidden_dim // self.num_heads
        if self.hidden_dim <= 0:
            self.hidden_dim = self.num_heads * self.head_dim


def _raw_stream(device: torch.device) -> int:
    """The current stream of `device` as the integer handle that the C ABI takes."""
    get = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # (no Stream object is built: several microseconds per call)
    if get is not None:
        return get(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """`with torch.cuda.device(d)` that does nothing when d is already the current device (the usual case)."""

    def __init__(self, device: torch.device):
        self._ctx = None
        if device.index is not None and device.index != torch.cuda.current_device():
            self._ctx = torch.cuda.device(device)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            self._ctx.__exit__(*exc)
        return False


def _entry(backend: str, name: str):
    prefix = "frnn_fused_" if backend == "hip_fused" else "frnn_alt_"
    return getattr(_lib.load_library(), prefix + name)


def _options(cfg: "FlashRNNConfig", batch_stride: int = 0):
    import ctypes

    return ctypes.byref(_lib.Options(float(cfg.forward_clipval or 0.0), float(cfg.gradient_recurrent_clipval or 0.0),
                                     int(bool(cfg.gradient_recurrent_cut)),
                                     int(bool(cfg.recompute_gates) and cfg.backend == "hip_fused"), int(batch_stride)))


def _workspace_bytes(cfg: "FlashRNNConfig", f_id, d_id, B, T, N, D, backward: int) -> int:
    if cfg.backend == "hip_fused":
        return _lib.load_library().frnn_fused_workspace_bytes_opt(f_id, d_id, B, T, N, D, backward, _options(cfg))
    return _lib.load_library().frnn_alt_workspace_bytes(f_id, d_id, B, T, N, D, backward)


def _raise(code: int, what: str):
    msg = f"{what}: {_lib.last_error()} (code {code})"
    if code == _lib.E_UNSUPPORTED:
        raise ValueError(msg)  # the reference raises ValueError when no tiling exists
    raise RuntimeError(msg)


class _StatusLog:
    """Status words of the fused calls, checked without a device-wide synchronisation.

    A fused kernel whose bounded wait between workgroups ran out fills its outputs with NaN and sets the
    status word at the head of its workspace.  Every fused call copies that word to pinned host memory
    behind the kernels (4 bytes, asynchronous) and records an event; the entries whose event has
    completed are read at the start of every later call (forward or backward, any stream), and a non-zero
    one raises RuntimeError there.  ``check_status()`` waits for the entries still pending (their events
    only) and does the same.  Entries made under stream capture are not logged: a replay repeats the
    kernels, not this bookkeeping.  The pinned words and events of entries that have been read are used again
    (except the most recent entry of each kind, which ``last()`` may still be asked for)."""

    def __init__(self):
        import collections
        import threading

        self._lock = threading.Lock()
        self._pending = collections.deque()
        self._last = {}
        self._free = []

    def log(self, kind: str, ws: torch.Tensor, what: str):
        if torch.cuda.is_current_stream_capturing():
            return
        with self._lock:
            host, ev = self._free.pop() if self._free else (None, None)
        if host is None:
            host, ev = torch.empty(1, dtype=torch.int32, pin_memory=True), torch.cuda.Event()
        host.copy_(ws[:4].view(torch.int32), non_blocking=True)
        ev.record()
        entry = (kind, what, host, ev)
        with self._lock:
            self._pending.append(entry)
            self._last[kind] = entry

    def note_ok(self, kind: str):
        """A call that cannot fail this way (heads of one workgroup: nothing waits): nothing to fetch."""
        with self._lock:
            self._last[kind] = None

    def poll(self, wait: bool = False):
        if torch.cuda.is_current_stream_capturing():
            return  # (querying an event is not allowed while this thread captures)
        failed = []
        with self._lock:
            keep = []
            while self._pending:
                entry = self._pending.popleft()
                kind, what, host, ev = entry
                if wait:
                    ev.synchronize()
                if ev.query():
                    if int(host[0]) != 0:
                        failed.append(f"{kind} of {what}")
                    if self._last.get(kind) is not entry and len(self._free) < 64:
                        self._free.append((host, ev))
                else:
                    keep.append(entry)
            self._pending.extend(keep)
        if failed:
            raise RuntimeError(
                "flashrnn_amd: a bounded wait between the workgroups of a head ran out in an earlier fused call ("
                + "; ".join(failed) + "): its outputs are NaN.  The workgroups of a head must all be resident; "
                "another process's kernels on the same device can prevent that")

    def last(self, kind: str) -> int:
        with self._lock:
            entry = self._last.get(kind)
        if entry is None:
            return 0
        entry[3].synchronize()
        return int(entry[2][0])

    def drain(self) -> list:
        """Waits for every pending entry, then lets go of all events and pinned words (while the HIP runtime is
        still up).  Returns the descriptions of the calls whose status word was set."""
        with self._lock:
            pending, self._pending = list(self._pending), type(self._pending)()
            self._last, self._free = {}, []
        failed = []
        for kind, what, host, ev in pending:
            ev.synchronize()
            if int(host[0]) != 0:
                failed.append(f"{kind} of {what}")
        return failed


_status = _StatusLog()
# devices on which a backward pass of this package ran: their autograd worker threads are what _teardown orders
_backward_devices = set()
_used_devices = set()  # every device a call of this package launched kernels on


def _teardown() -> None:
    """Runs once, from atexit, before the interpreter starts to finalise.  Never raises.

    Why it exists.  A process that ended within milliseconds of a backward pass died now and then with
    "terminate called without an active exception" (exit status 134) after all its work was done.  torch >= 2.10
    releases the Python wrapper of a tensor on whatever thread drops the last other C++ reference to it
    (c10::intrusive_ptr: decref_pyobject() noexcept on the 2 -> 1 transition), and that needs the interpreter
    lock.  CPython 3.10 ends any thread that is waiting for the lock when finalisation begins with
    pthread_exit(); the forced unwinding then meets the noexcept frame and C++ answers with std::terminate().
    The one foreign thread that handles this package's tensors is the autograd engine's worker thread of the
    device: after ``torch.autograd.grad`` / ``backward`` has returned to the caller it may still have the tail
    of its loop iteration to run (it wakes the caller first and lets go of the finished graph task, whose
    result holds the gradient tensors, afterwards), and on a busy machine that tail can be preempted for
    milliseconds.

    What it does.  (1) waits for the device work of every device this package used; (2) drains the status
    log: events and pinned words are released now, by this thread; (3) sends one trivial backward pass through
    the worker thread of every device a backward pass of this package ran on.  The worker takes tasks one at
    a time, so when that pass has come back the worker has finished every iteration before it, all its
    references to this package's tensors are gone, and what the trivial pass itself leaves behind holds no
    Python-wrapped tensor (it accumulates into .grad, nothing is captured)."""
    try:
        if not torch.cuda.is_available() or not torch.cuda.is_initialized():
            return
        for dec in list(_open_decoders):  # (a resident kernel that nobody stops holds the device until it idles out)
            dec.close(check=False)
        devices = sorted(_backward_devices)
        _backward_devices.clear()
        for index in sorted(_used_devices):
            torch.cuda.synchronize(index)
        failed = _status.drain()
        if failed:
            import sys

            print("flashrnn_amd: a bounded wait between workgroups ran out in: " + "; ".join(failed)
                  + " (outputs of those calls were NaN)", file=sys.stderr)
        for index in devices:
            with torch.enable_grad():
                x = torch.zeros(1, device=torch.device("cuda", index), requires_grad=True)
                (x * 1.0).backward(torch.zeros_like(x))
            del x
    except Exception:  # (at exit there is nobody left to tell)
        pass


# (registered when the package is imported, i.e. after torch: exit functions run last-in first-out, so this one runs
# while everything torch registered for exit is still in place)
atexit.register(_teardown)


def check_status() -> None:
    """Waits for the fused calls made so far (their events, not the device) and raises RuntimeError if one of
    them reported that a bounded wait between workgroups ran out."""
    _status.poll(wait=True)


def last_status(kind: str = "forward") -> int:
    """Status word of the most recent fused call of this kind (waits for that call): 0 ok, 1 = a bounded
    wait between workgroups ran out and the outputs were filled with NaN.  Does not raise."""
    return _status.last(kind)


def fused_plan(function: str, dtype: str, B: int, N: int, D: int, backward: bool = False):
    """(waves per workgroup, unit tiles per wave, workgroups per head, workgroups doing work)."""
    import ctypes

    out = [ctypes.c_int() for _ in range(4)]
    rc = _lib.load_library().frnn_fused_plan(_lib.FUNCTION_IDS[function], _lib.DTYPE_IDS[dtype], B, N, D,
                                            int(backward), *[ctypes.byref(o) for o in out])
    if rc != 0:
        _raise(rc, "fused_plan")
    return tuple(o.value for o in out)


@functools.lru_cache(maxsize=None)
def _heads_wait_cached(function: str, dtype: str, B: int, N: int, D: int, backward: bool, variant) -> bool:
    return fused_plan(function, dtype, B, N, D, backward)[2] > 1


def _heads_wait(cfg: FlashRNNConfig, B: int, N: int, D: int, backward: bool) -> bool:
    """Whether the heads of this fused call run as several workgroups that wait for each other: only then can the
    status word of the call become non-zero, and only then is it fetched (a copy on the stream per call).  The
    recompute-mode reverse kernels have tilings of their own, so their calls always fetch it."""
    if cfg.recompute_gates and backward:
        return True
    return _heads_wait_cached(cfg.function, cfg.dtype, B, N, D, backward, os.environ.get("FRNN_FUSED_VARIANT"))


def _cast_inputs(Wx, R, b, s0, cfg: FlashRNNConfig):
    """The inputs in the kernel type and the kernels' layouts, as the reference's custom_fwd(cast_inputs=...) does
    (flashrnn.py:690-695); s0 comes back as [S,B,N,D]."""
    kdt = DTYPE_DICT[cfg.dtype]
    if not cfg.enable_automatic_mixed_precision:
        for name, x in (("Wx", Wx), ("R", R), ("b", b), ("states", s0)):
            if x.dtype != kdt:
                raise TypeError(f"{name} is {x.dtype}, the kernel type is {kdt} and "
                                "enable_automatic_mixed_precision is off")
    S, B = cfg.num_states, Wx.shape[0]
    N, D = Wx.shape[3], Wx.shape[4]
    return (Wx.detach().to(kdt).contiguous(), R.detach().to(kdt).contiguous(), b.detach().to(kdt).contiguous(),
            s0.detach().to(kdt).reshape(S, B, N, D).contiguous())


def _run_forward(Wx_k, R_k, b_k, s0_k, cfg: FlashRNNConfig, training: bool, out=None, batch_stride: int = 0):
    """One forward call of the library on kernel-typed, contiguous tensors: (states [S,B,T,N,D], gate cache).
    out / batch_stride: the call covers a range of rows of a larger batch; s0_k and out are then the slices
    [:, b0:b1] of the full tensors [S, batch_stride, ...], used in place (see frnn_options.batch_stride)."""
    kdt = DTYPE_DICT[cfg.dtype]
    f_id, d_id = _lib.FUNCTION_IDS[cfg.function], _lib.DTYPE_IDS[cfg.dtype]
    B, T, Gw, N, D = Wx_k.shape
    S = cfg.num_states
    _used_devices.add(Wx_k.device.index if Wx_k.device.index is not None else torch.cuda.current_device())
    with _on_device(Wx_k.device):
        rc = _entry(cfg.backend, "supported")(f_id, d_id, B, N, D)
        if rc == 0 and cfg.recompute_gates:
            if cfg.backend != "hip_fused":
                raise ValueError("recompute_gates is an option of the hip_fused backend")
            rc = _lib.load_library().frnn_fused_recompute_supported(f_id, d_id, B, N, D)
        if rc != 0:
            _raise(rc, f"{cfg.backend} backend")
        states = out if out is not None else torch.empty((S, B, T, N, D), dtype=kdt, device=Wx_k.device)
        cache_bytes = _entry(cfg.backend, "cache_bytes_opt")(f_id, d_id, B, T, N, D, _options(cfg)) if training else 0
        cache = torch.empty(max(cache_bytes, 16), dtype=torch.uint8, device=Wx_k.device)
        ws_bytes = _workspace_bytes(cfg, f_id, d_id, B, T, N, D, 0)
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=Wx_k.device)
        stream = _raw_stream(Wx_k.device)
        rc = _entry(cfg.backend, "forward_opt")(
            f_id, d_id, int(training), B, T, N, D, Wx_k.data_ptr(), R_k.data_ptr(), b_k.data_ptr(),
            s0_k.data_ptr(), states.data_ptr(), cache.data_ptr() if training else None,
            ws.data_ptr(), ws.numel(), stream, _options(cfg, batch_stride))
        if rc != 0:
            _raise(rc, f"{cfg.backend} forward")
        if cfg.backend == "hip_fused":
            if _heads_wait(cfg, B, N, D, False):
                _status.log("forward", ws, f"{cfg.function} B{B} T{T} N{N} D{D}")
            else:
                _status.note_ok("forward")
    return states, cache


def _run_backward(cfg: FlashRNNConfig, R_k, b_k, s0_k, states, cache, Wx_k, ds, dWx, ds0=None, batch_stride: int = 0):
    """One backward call of the library; ds [S,B,T,N,D] contiguous in the kernel type, dWx [B,T,G_w,N,D] is written.
    Returns (dR, db, ds0 [S,B,N,D]); dR and db are fp32.  ds0 / batch_stride: as in _run_forward, the state-shaped
    tensors (s0_k, states, ds, ds0) are slices [:, b0:b1] of full tensors of batch_stride rows, used in place."""
    kdt = DTYPE_DICT[cfg.dtype]
    f_id, d_id = _lib.FUNCTION_IDS[cfg.function], _lib.DTYPE_IDS[cfg.dtype]
    S, B, T, N, D = states.shape
    Gr, Gt = cfg.num_gates_r, cfg.num_gates_t
    dev = states.device
    with _on_device(dev):
        if ds0 is None:
            ds0 = torch.empty((S, B, N, D), dtype=kdt, device=dev)
        dR = torch.empty((Gr, N, D, D), dtype=torch.float32, device=dev)
        db = torch.empty((Gt, N, D), dtype=torch.float32, device=dev)
        ws_bytes = _workspace_bytes(cfg, f_id, d_id, B, T, N, D, 1)
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
        stream = _raw_stream(dev)
        if cfg.recompute_gates:
            rc = _lib.load_library().frnn_fused_backward_recompute(
                f_id, d_id, B, T, N, D, Wx_k.data_ptr(), R_k.data_ptr(), b_k.data_ptr(), s0_k.data_ptr(),
                states.data_ptr(), ds.data_ptr(), dWx.data_ptr(), ds0.data_ptr(), dR.data_ptr(), db.data_ptr(),
                ws.data_ptr(), ws.numel(), stream, _options(cfg, batch_stride))
        else:
            rc = _entry(cfg.backend, "backward_opt")(
                f_id, d_id, B, T, N, D, R_k.data_ptr(), b_k.data_ptr(), s0_k.data_ptr(), states.data_ptr(),
                cache.data_ptr(), ds.data_ptr(), dWx.data_ptr(), ds0.data_ptr(), dR.data_ptr(), db.data_ptr(),
                ws.data_ptr(), ws.numel(), stream, _options(cfg, batch_stride))
        if rc != 0:
            _raise(rc, f"{cfg.backend} backward")
        if cfg.backend == "hip_fused":
            if _heads_wait(cfg, B, N, D, True):
                _status.log("backward", ws, f"{cfg.function} B{B} T{T} N{N} D{D}")
            else:
                _status.note_ok("backward")
    return dR, db, ds0


class _FlashRNNFunction(torch.autograd.Function):
    """forward(Wx [B,T,G_w,N,D], R [G_r,N,D,D], b [G_t,N,D], s0 [S,B,1,N,D]) -> states [S,B,T,N,D]."""

    @staticmethod
    def forward(ctx, Wx, R, b, s0, cfg: FlashRNNConfig, training: bool):
        if not Wx.is_cuda:
            raise RuntimeError("flashrnn_amd runs on a GPU only (got a CPU tensor); there is no CPU fallback")
        _status.poll()
        Wx_k, R_k, b_k, s0_k = _cast_inputs(Wx, R, b, s0, cfg)
        states, cache = _run_forward(Wx_k, R_k, b_k, s0_k, cfg, training)
        ctx.cfg, ctx.training = cfg, training
        # (recompute mode reads Wx again in the backward pass; it is the caller's tensor unless it was cast)
        ctx.save_for_backward(R_k, b_k, s0_k, states, cache, Wx_k if cfg.recompute_gates else cache)
        return states

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dstates):
        if not ctx.training:
            raise RuntimeError("FlashRNN backward can only be called in training mode")
        cfg = ctx.cfg
        R_k, b_k, s0_k, states, cache, Wx_k = ctx.saved_tensors
        S, B, T, N, D = states.shape
        _backward_devices.add(states.device.index if states.device.index is not None else torch.cuda.current_device())
        _status.poll()
        ds = dstates.to(states.dtype).contiguous()
        with _on_device(states.device):
            dWx = torch.empty((B, T, cfg.num_gates_w, N, D), dtype=states.dtype, device=states.device)
        dR, db, ds0 = _run_backward(cfg, R_k, b_k, s0_k, states, cache, Wx_k, ds, dWx)
        # dR / db stay fp32: autograd casts them to the dtype of the leaf they belong to, so fp32
        # master weights receive unrounded gradients
        return dWx, dR, db, ds0.reshape(S, B, 1, N, D), None, None


class _FlashRNNRangesFunction(torch.autograd.Function):
    """The same over ranges of `rows` batch rows, one library call each (see _apply_in_batch_ranges).  A range of Wx
    and of dWx is contiguous (the batch is their leading axis), so the calls read and write the full tensors in
    place.  The state-shaped tensors [S,B,...] have the batch as their second axis: with `inplace` the calls name the
    full tensors' plane stride (frnn_options.batch_stride) and use their slices as they are, nothing is copied and
    the states are held once; where even that does not fit 32-bit offsets (the planes of the later states lie too far
    apart: sLSTM at very large batches) each range gets contiguous copies of its slices."""

    @staticmethod
    def forward(ctx, Wx, R, b, s0, cfg: FlashRNNConfig, training: bool, rows: int, inplace: bool):
        if not Wx.is_cuda:
            raise RuntimeError("flashrnn_amd runs on a GPU only (got a CPU tensor); there is no CPU fallback")
        _status.poll()
        Wx_k, R_k, b_k, s0_k = _cast_inputs(Wx, R, b, s0, cfg)
        B, T, _, N, D = Wx_k.shape
        S = cfg.num_states
        with _on_device(Wx_k.device):
            states = torch.empty((S, B, T, N, D), dtype=Wx_k.dtype, device=Wx_k.device)
        saved = []
        for b0 in range(0, B, rows):
            b1 = min(B, b0 + rows)
            if inplace:
                _, cache_r = _run_forward(Wx_k[b0:b1], R_k, b_k, s0_k[:, b0:b1], cfg, training, out=states[:, b0:b1],
                                          batch_stride=B)
                saved.append(cache_r)
            else:
                s0_r = s0_k[:, b0:b1].contiguous()
                states_r, cache_r = _run_forward(Wx_k[b0:b1], R_k, b_k, s0_r, cfg, training)
                states[:, b0:b1].copy_(states_r)
                saved += [s0_r, states_r, cache_r]
        ctx.cfg, ctx.training, ctx.rows, ctx.inplace, ctx.batch = cfg, training, rows, inplace, B
        if inplace:
            saved = [s0_k, states] + saved
        ctx.save_for_backward(R_k, b_k, Wx_k if cfg.recompute_gates else R_k, *saved)
        return states

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dstates):
        if not ctx.training:
            raise RuntimeError("FlashRNN backward can only be called in training mode")
        cfg, rows, B = ctx.cfg, ctx.rows, ctx.batch
        R_k, b_k, Wx_k, *saved = ctx.saved_tensors
        S, _, T, N, D = dstates.shape
        kdt = DTYPE_DICT[cfg.dtype]
        _backward_devices.add(dstates.device.index if dstates.device.index is not None else torch.cuda.current_device())
        _status.poll()
        ds = dstates.to(kdt)
        if ctx.inplace:
            ds = ds.contiguous()
            s0_k, states, *caches = saved
        with _on_device(dstates.device):
            dWx = torch.empty((B, T, cfg.num_gates_w, N, D), dtype=kdt, device=dstates.device)
            ds0 = torch.empty((S, B, N, D), dtype=kdt, device=dstates.device)
        dR = db = None
        for i, b0 in enumerate(range(0, B, rows)):
            b1 = min(B, b0 + rows)
            wx_r = Wx_k[b0:b1] if cfg.recompute_gates else Wx_k
            if ctx.inplace:
                dR_r, db_r, _ = _run_backward(cfg, R_k, b_k, s0_k[:, b0:b1], states[:, b0:b1], caches[i], wx_r,
                                              ds[:, b0:b1], dWx[b0:b1], ds0=ds0[:, b0:b1], batch_stride=B)
            else:
                s0_r, states_r, cache_r = saved[3 * i:3 * i + 3]
                dR_r, db_r, ds0_r = _run_backward(cfg, R_k, b_k, s0_r, states_r, cache_r, wx_r,
                                                  ds[:, b0:b1].contiguous(), dWx[b0:b1])
                ds0[:, b0:b1].copy_(ds0_r)
            dR = dR_r if dR is None else dR.add_(dR_r)
            db = db_r if db is None else db.add_(db_r)
        return dWx, dR, db, ds0.reshape(S, B, 1, N, D), None, None, None, None


def _get_config(Wx, R, b, function, backend, dtype) -> FlashRNNConfig:
    return FlashRNNConfig(head_dim=Wx.shape[4], num_heads=Wx.shape[3], batch_size=Wx.shape[0],
                          function=function, backend=backend,
                          dtype=dtype if dtype is not None else "bfloat16")


def permute_to(input_shape: str, output_shape: str):
    """Axis permutation that takes a tensor laid out as `input_shape` to `output_shape`, None if they
    are equal (flashrnn.py:100-110): permute_to("ABC", "BAC") == (1, 0, 2)."""
    if input_shape == output_shape:
        return None
    return tuple(input_shape.index(x) for x in output_shape)


def _permuted(x: torch.Tensor, have: str, want: str) -> torch.Tensor:
    p = permute_to(have, want)
    return x if p is None else x.permute(p)


def _zero_state(config: FlashRNNConfig, Wx: torch.Tensor) -> torch.Tensor:
    """Default initial state [S,B,1,N,D] for a Wx in the kernels' layout [B,T,G,N,D]: `initial_val`
    everywhere, or one value per state (flashrnn.py:927-954)."""
    B, _, _, N, D = Wx.shape
    state = torch.zeros((config.num_states, B, 1, N, D), dtype=Wx.dtype, device=Wx.device)
    if isinstance(config.initial_val, (int, float)):
        if config.initial_val != 0.0:
            state += float(config.initial_val)
    else:
        for i in range(config.num_states):
            state[i] += float(config.initial_val[i])
    return state


def flashrnn(
    Wx: torch.Tensor,  # [B, T, G_w, N, D]
    R: torch.Tensor,  # [G_r, N, D, D]   (gate, head, output unit, previous unit)
    b: torch.Tensor,  # [G_t, N, D]
    states: Optional[torch.Tensor] = None,  # [S, B, 1, N, D]
    function: str = "lstm",
    config: Optional[FlashRNNConfig] = None,
    backend: str = "hip_fused",
    dtype: str = "bfloat16",
):
    """Same call as the reference's ``flashrnn`` (flashrnn.py:1114-1135).

    Returns ``(all_states [S,B,T,N,D], last_states [S,B,1,N,D])`` in the kernel dtype ``dtype``
    (shapes as named by ``config.input_shape`` / ``output_shape`` / ``recurrent_shape`` / ``bias_shape``
    when a config with other layouts is given).
    Differentiable w.r.t. Wx, R, b and states.  Raises ValueError if the chosen backend has no
    kernel for the head dimension (as the reference does when no tiling exists)."""
    if config is None:
        config = _get_config(Wx, R, b, function, backend, dtype)
    # to the layouts the kernels read (views; nothing is copied for the default layouts)
    Wx = _permuted(Wx, config.input_shape, "BTGHD")
    R = _permuted(R, config.recurrent_shape, "GHDP")
    b = _permuted(b, config.bias_shape, "GHD")
    if states is not None:
        states = _permuted(states, config.output_shape, "SBTHD")
    Gr, Gw, _, Gt, S = rnn_function_registry[config.function]["gates_states"]
    if Wx.dim() != 5 or Wx.shape[2] != Gw:
        raise ValueError(f"Wx must be [B,T,{Gw},N,D], got {tuple(Wx.shape)}")
    B, T, _, N, D = Wx.shape
    if tuple(R.shape) != (Gr, N, D, D):
        raise ValueError(f"R must be [{Gr},{N},{D},{D}], got {tuple(R.shape)}")
    if tuple(b.shape) != (Gt, N, D):
        raise ValueError(f"b must be [{Gt},{N},{D}], got {tuple(b.shape)}")
    if states is None:
        states = _zero_state(config, Wx)
    if tuple(states.shape) != (S, B, 1, N, D):
        raise ValueError(f"states must be [{S},{B},1,{N},{D}], got {tuple(states.shape)}")
    training = torch.is_grad_enabled() and any(x.requires_grad for x in (Wx, R, b, states))
    if D == 16:
        out = _paired_heads(Wx, R, b, states, config, training)
    else:
        out = _apply_in_batch_ranges(Wx, R, b, states, config, training)
    return _permuted(out, "SBTHD", config.output_shape), _permuted(out[:, :, -1:], "SBTHD", config.output_shape)


def _apply_in_batch_ranges(Wx, R, b, states, config, training):
    """Batch rows are independent, so a fused problem one of whose tensors (Wx, the states or the gate cache)
    would reach 2 GiB (32-bit offsets inside the fused kernels) runs as several library calls over ranges of the batch
    (_FlashRNNRangesFunction), dR and db summed over the ranges.  How many rows a call can take is the library's
    answer (frnn_fused_max_batch), for calls that use the full tensors in place and for calls on copies."""
    B, T, Gw, N, D = Wx.shape
    if config.backend != "hip_fused":
        return _FlashRNNFunction.apply(Wx, R, b, states, config, training)
    f_id, d_id = _lib.FUNCTION_IDS[config.function], _lib.DTYPE_IDS[config.dtype]
    max_batch = lambda stride: _lib.load_library().frnn_fused_max_batch(f_id, d_id, T, N, D, stride, int(training), _options(config))
    limit = os.environ.get("FRNN_TEST_MAX_BATCH")  # (tests: pretend that a call takes no more rows than this)
    rows = max_batch(0) if limit is None else min(max_batch(0), int(limit))
    if rows >= B:
        return _FlashRNNFunction.apply(Wx, R, b, states, config, training)
    rows_in_place = max_batch(B) if limit is None else min(max_batch(B), int(limit))
    inplace = rows_in_place >= min(16, rows) and os.environ.get("FRNN_RANGES_COPY") != "1"
    if inplace:
        rows = rows_in_place
    if rows < 1:
        raise ValueError("flashrnn_amd: one batch row of this problem already reaches 2 GiB per tensor; use backend='hip'")
    rows = max(16, rows // 16 * 16) if rows >= 16 else rows  # whole batch tiles
    if rows >= 16:  # ranges of about the same size, still whole tiles
        n_ranges = -(-B // rows)
        rows = min(rows, -(-B // (16 * n_ranges)) * 16)
    return _FlashRNNRangesFunction.apply(Wx, R, b, states, config, training, rows, inplace)


def flashrnn_step(
    Wx: torch.Tensor,  # [B, 1, G_w, N, D]
    R: torch.Tensor,  # [G_r, N, D, D]
    b: torch.Tensor,  # [G_t, N, D]
    states: torch.Tensor,  # [S, B, 1, N, D]
    function: str = "lstm",
    config: Optional[FlashRNNConfig] = None,
    backend: str = "hip_fused",
    dtype: str = "bfloat16",
    carry: Optional[torch.Tensor] = None,  # [S, B, N, D] float32, updated in place
) -> torch.Tensor:
    """One time step with carried state, for inference / decoding (the reference's step kernels,
    flashrnn.py:957-985): returns the new states [S,B,1,N,D].  One kernel launch, no workspace, nothing cleared;
    not differentiable.  Tensors must already be in the kernel dtype and the default layouts (nothing is cast
    or copied on this path).

    ``carry`` (``make_carry(states)`` before the first step, then the same tensor every step) holds the unrounded
    state: with it a chain of steps yields bit for bit what one ``flashrnn()`` call over the sequence does, which
    keeps the state in fp32 registers between time steps; without it every step starts from the rounded
    ``states``."""
    if config is None:
        config = _get_config(Wx, R, b, function, backend, dtype)
    kdt = DTYPE_DICT[config.dtype]
    Gr, Gw, _, Gt, S = rnn_function_registry[config.function]["gates_states"]
    if Wx.dim() != 5 or Wx.shape[1] != 1 or Wx.shape[2] != Gw:
        raise ValueError(f"Wx must be [B,1,{Gw},N,D], got {tuple(Wx.shape)}")
    B, _, _, N, D = Wx.shape
    if tuple(R.shape) != (Gr, N, D, D) or tuple(b.shape) != (Gt, N, D) or tuple(states.shape) != (S, B, 1, N, D):
        raise ValueError(f"R, b, states must be [{Gr},{N},{D},{D}], [{Gt},{N},{D}], [{S},{B},1,{N},{D}]; got "
                         f"{tuple(R.shape)}, {tuple(b.shape)}, {tuple(states.shape)}")
    for name, x in (("Wx", Wx), ("R", R), ("b", b), ("states", states)):
        if not x.is_cuda:
            raise RuntimeError("flashrnn_amd runs on a GPU only (got a CPU tensor); there is no CPU fallback")
        if x.dtype != kdt or not x.is_contiguous():
            raise TypeError(f"{name} must be a contiguous {kdt} tensor (the step path casts and copies nothing)")
    if carry is not None and (carry.dtype != torch.float32 or tuple(carry.shape) != (S, B, N, D)
                              or not carry.is_contiguous() or carry.device != Wx.device):
        raise TypeError(f"carry must be a contiguous float32 tensor [{S},{B},{N},{D}] on the device of Wx")
    f_id, d_id = _lib.FUNCTION_IDS[config.function], _lib.DTYPE_IDS[config.dtype]
    with _on_device(Wx.device):
        out = torch.empty((S, B, 1, N, D), dtype=kdt, device=Wx.device)
        rc = _entry(config.backend, "step")(
            f_id, d_id, B, N, D, Wx.data_ptr(), R.data_ptr(), b.data_ptr(), states.data_ptr(), out.data_ptr(),
            carry.data_ptr() if carry is not None else None, _raw_stream(Wx.device), _options(config))
        if rc != 0:
            _raise(rc, f"{config.backend} step")
    return out


def make_carry(states: torch.Tensor) -> torch.Tensor:
    """The fp32 carry of ``flashrnn_step`` for a chain that starts at ``states`` [S,B,1,N,D]."""
    return states[:, :, 0].to(torch.float32).contiguous()

class FlashRNNDecoder:
    """A decode session: the fused forward kernel of the head dimension stays on the device, R in its registers and the
    state in fp32 registers, and serves one token after the other (the reference decodes with one launch per token that
    reloads R, flashrnn.py:957-985).  A chain of tokens gives bit for bit what ``flashrnn()`` gives over the sequence.

        dec = FlashRNNDecoder(R, b, states, function="lstm")       # launches the resident kernel on a stream of its own
        for t in ...:  new_states = dec.step(Wx_t)                 # [B,C,G_w,N,D] -> [S,B,C,N,D], C <= dec.slots tokens
        dec.close()                                                # stops the kernel; dec.states / dec.carry hold the end

    ``step`` is one small launch on the current stream that posts the tokens into the session's mailbox and collects
    the new states; it allocates its output only (pass ``out=`` to allocate nothing) and can be captured into a HIP
    graph.  While the session is open: its workgroups keep their compute units, so do not call
    ``torch.cuda.synchronize()`` (it would wait until the kernel has idled out; synchronise streams or events
    instead), and run every ``step`` on one stream, not on ``dec.kernel_stream``.  Every wait is bounded: the kernel
    ends by itself after ``idle_polls`` probes without a token (about 0.4 us each) or ``max_tokens`` tokens; the
    session can then be continued with a new ``FlashRNNDecoder(..., states=dec.states, carry=dec.carry)``.  Tensors
    must be in the kernel dtype and the default layouts (nothing is cast or copied on this path); not differentiable."""

    def __init__(self, R, b, states, function: str = "lstm", dtype: str = "bfloat16", config: Optional[FlashRNNConfig] = None,
                 carry: Optional[torch.Tensor] = None, slots: int = 4, max_tokens: int = 1 << 30, idle_polls: int = 1 << 22,
                 kernel_stream: Optional["torch.cuda.Stream"] = None):
        Gr, Gw, _, Gt, S = rnn_function_registry[function]["gates_states"]
        if states.dim() != 5 or states.shape[0] != S or states.shape[2] != 1:
            raise ValueError(f"states must be [{S},B,1,N,D], got {tuple(states.shape)}")
        _, B, _, N, D = states.shape
        if config is None:
            config = FlashRNNConfig(head_dim=D, num_heads=N, batch_size=B, function=function, backend="hip_fused", dtype=dtype)
        if config.backend != "hip_fused":
            raise ValueError("the resident decode kernel is the hip_fused backend's")
        kdt = DTYPE_DICT[config.dtype]
        if tuple(R.shape) != (Gr, N, D, D) or tuple(b.shape) != (Gt, N, D):
            raise ValueError(f"R, b must be [{Gr},{N},{D},{D}], [{Gt},{N},{D}]; got {tuple(R.shape)}, {tuple(b.shape)}")
        for name, x in (("R", R), ("b", b), ("states", states)):
            if not x.is_cuda:
                raise RuntimeError("flashrnn_amd runs on a GPU only (got a CPU tensor); there is no CPU fallback")
            if x.dtype != kdt or not x.is_contiguous():
                raise TypeError(f"{name} must be a contiguous {kdt} tensor (the decode path casts and copies nothing)")
        self.config, self.function, self.kdt = config, function, kdt
        self.B, self.N, self.D, self.S, self.Gw, self.slots = B, N, D, S, Gw, slots
        self.device = states.device
        self._ids = (_lib.FUNCTION_IDS[function], _lib.DTYPE_IDS[config.dtype], B, N, D)
        lib = _lib.load_library()
        with _on_device(self.device):
            rc = lib.frnn_fused_decode_mailbox_layout(*self._ids, slots, None, None, None, None)
            if rc != 0:
                _raise(rc, "decode session")
            nbytes = lib.frnn_fused_decode_mailbox_bytes(*self._ids, slots)
            self.mailbox = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
            self.carry = carry if carry is not None else make_carry(states)
            if (self.carry.dtype != torch.float32 or tuple(self.carry.shape) != (S, B, N, D)
                    or not self.carry.is_contiguous() or self.carry.device != self.device):
                raise TypeError(f"carry must be a contiguous float32 tensor [{S},{B},{N},{D}] on the device of the states")
            self.states = states  # the states behind the last collected token, [S,B,1,N,D]
            self._keep = (R, b, states)  # the kernel reads them when it starts
            self.kernel_stream = kernel_stream if kernel_stream is not None else _kernel_stream_for(self.device)
            _used_devices.add(self.device.index if self.device.index is not None else torch.cuda.current_device())
            rc = lib.frnn_fused_decode_open(*self._ids, R.data_ptr(), b.data_ptr(), states.data_ptr(), self.carry.data_ptr(),
                                            self.mailbox.data_ptr(), nbytes, slots, int(max_tokens), int(idle_polls),
                                            _raw_stream(self.device), self.kernel_stream.cuda_stream, _options(config))
            if rc != 0:
                _raise(rc, "decode session")
        self.open = True
        _open_decoders.add(self)

    def step(self, Wx: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Wx [B,C,G_w,N,D] (C <= slots tokens) -> their new states [S,B,C,N,D]."""
        if not self.open:
            raise RuntimeError("the decode session is closed")
        if Wx.dim() != 5 or (Wx.shape[0], Wx.shape[2], Wx.shape[3], Wx.shape[4]) != (self.B, self.Gw, self.N, self.D):
            raise ValueError(f"Wx must be [{self.B},C,{self.Gw},{self.N},{self.D}], got {tuple(Wx.shape)}")
        C = Wx.shape[1]
        if Wx.dtype != self.kdt or not Wx.is_contiguous() or Wx.device != self.device:
            raise TypeError(f"Wx must be a contiguous {self.kdt} tensor on {self.device}")
        with _on_device(self.device):
            if out is None:
                out = torch.empty((self.S, self.B, C, self.N, self.D), dtype=self.kdt, device=self.device)
            elif tuple(out.shape) != (self.S, self.B, C, self.N, self.D) or out.dtype != self.kdt or not out.is_contiguous():
                raise TypeError(f"out must be a contiguous {self.kdt} tensor [{self.S},{self.B},{C},{self.N},{self.D}]")
            rc = _lib.load_library().frnn_fused_decode_step(*self._ids, C, Wx.data_ptr(), out.data_ptr(), self.mailbox.data_ptr(),
                                                            self.mailbox.numel(), self.slots, _raw_stream(self.device))
            if rc != 0:
                _raise(rc, "decode step")
        self.states = out[:, :, -1:]
        return out

    def control(self) -> dict:
        """The session's control block (synchronises the current stream): status, end reason, tokens served."""
        c = self.mailbox[:64 * 4].view(torch.int32).cpu()
        reasons = {0: "running", 1: "a wait between workgroups ran out", 2: "idle bound reached", 3: "stopped", 4: "max_tokens served"}
        return {"wait_expired": int(c[0]) != 0, "ended": reasons.get(int(c[2]), str(int(c[2]))), "tokens_served": int(c[3]),
                "collect_gave_up": int(c[4]) != 0, "tokens_posted": int(c[9])}

    def close(self, check: bool = True) -> None:
        """Sets the stop word and orders the current stream behind the end of the resident kernel.  check: read the
        control block (a synchronisation of the current stream) and raise RuntimeError if a wait ran out."""
        if not self.open:
            return
        self.open = False
        _open_decoders.discard(self)
        with _on_device(self.device):
            rc = _lib.load_library().frnn_fused_decode_close(self.mailbox.data_ptr(), _raw_stream(self.device),
                                                             self.kernel_stream.cuda_stream)
            if rc != 0:
                _raise(rc, "decode close")
        self._keep = None
        if check:
            c = self.control()
            if c["wait_expired"] or c["collect_gave_up"]:
                raise RuntimeError(f"flashrnn_amd decode session: a bounded wait ran out ({c}); states collected after that are NaN")

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close(check=exc[0] is None)
        return False


_open_decoders = set()
_kernel_streams = {}


def _kernel_stream_for(device: torch.device):
    """A stream on which a resident kernel can run while the current stream of `device` keeps launching: the runtime
    maps streams onto a few hardware queues, and two streams of one queue run one after the other, so candidates are
    tried (frnn_streams_overlap measures it) and the first that works is kept for this pair."""
    cur = _raw_stream(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), cur)
    known = _kernel_streams.setdefault(key, [])
    busy = {d.kernel_stream.cuda_stream for d in _open_decoders}  # (a stream serves one resident kernel at a time)
    for cand in known:
        if cand.cuda_stream not in busy:
            return cand
    lib = _lib.load_library()
    for _ in range(24):
        cand = torch.cuda.Stream(device=device)
        if cand.cuda_stream in busy or any(cand.cuda_stream == k.cuda_stream for k in known):
            continue
        rc = lib.frnn_streams_overlap(cur, cand.cuda_stream)
        if rc < 0:
            _raise(rc, "stream probe")
        if rc == 1:
            known.append(cand)
            return cand
    raise RuntimeError("flashrnn_amd: found no free stream whose kernels run beside those of the current stream "
                       "(every candidate shares its hardware queue or serves another open session)")


def flashrnn_decode(Wx, R, b, states=None, function: str = "lstm", dtype: str = "bfloat16", chunk: int = 1,
                    idle_polls: int = 1 << 22):
    """``flashrnn()`` for inference, token by token through one decode session (``chunk`` tokens per post): returns
    ``(all_states [S,B,T,N,D], last_states [S,B,1,N,D])``, bit for bit what ``flashrnn(..., backend="hip_fused")``
    returns.  Meant for tests and for callers that have the whole Wx; a serving loop uses FlashRNNDecoder itself."""
    B, T, Gw, N, D = Wx.shape
    if states is None:
        cfg = FlashRNNConfig(head_dim=D, num_heads=N, batch_size=B, function=function, backend="hip_fused", dtype=dtype)
        states = _zero_state(cfg, Wx)
    S = states.shape[0]
    out = torch.empty((S, B, T, N, D), dtype=Wx.dtype, device=Wx.device)
    with FlashRNNDecoder(R, b, states, function=function, dtype=dtype, slots=max(2, 1 << (chunk - 1).bit_length()),
                         idle_polls=idle_polls) as dec:
        for t0 in range(0, T, chunk):
            t1 = min(T, t0 + chunk)
            out[:, :, t0:t1] = dec.step(Wx[:, t0:t1].contiguous())
    return out, out[:, :, -1:]



def _paired_heads(Wx, R, b, states, config, training):
    """Head dimension 16 (half a bf16 MFMA k-step; the reference's benchmark sweep has it): two heads
    run as one head of 32 units whose recurrent matrix is block diagonal, so a unit still sees only the
    h of its own head.  Wx, b and the states are views (adjacent heads are adjacent in memory); only
    the small R is rebuilt, with differentiable ops, so its gradient arrives by autograd."""
    B, T, Gw, N, D = Wx.shape
    if N % 2:  # one all-zero head completes the last pair; its outputs are dropped
        pad = lambda x: torch.nn.functional.pad(x, (0, 0, 0, 1))
        Wx, b, states = pad(Wx), pad(b), pad(states)
        R = torch.nn.functional.pad(R, (0, 0, 0, 0, 0, 1))
    M = (N + 1) // 2
    Gr = R.shape[0]
    Rp = R.reshape(Gr, M, 2, 16, 16)
    R2 = torch.cat([torch.cat([Rp[:, :, 0], torch.zeros_like(Rp[:, :, 0])], -1),
                    torch.cat([torch.zeros_like(Rp[:, :, 1]), Rp[:, :, 1]], -1)], -2)
    cfg2 = FlashRNNConfig(**{**{k: getattr(config, k) for k in ("function", "backend", "dtype", "forward_clipval",
                                                                "gradient_recurrent_clipval", "gradient_recurrent_cut", "recompute_gates")},
                             "head_dim": 32, "num_heads": M, "batch_size": B})
    out = _FlashRNNFunction.apply(Wx.reshape(B, T, Gw, M, 32), R2, b.reshape(b.shape[0], M, 32),
                                  states.reshape(states.shape[0], B, 1, M, 32), cfg2, training)
    return out.reshape(out.shape[0], B, T, 2 * M, 16)[:, :, :, :N]
