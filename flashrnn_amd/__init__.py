"""flashrnn_amd: MI355X (gfx950) recurrent hot path of FlashRNN behind the reference's
functional API ``flashrnn(Wx, R, b, states, function=..., backend=...)``.

Backends: ``hip_fused`` (persistent fused kernels) and ``hip`` (alternating per-step kernels).
There is no CPU path: calls fail loudly without the HIP library or a GPU.
"""
from .flashrnn import (  # noqa: F401
    FlashRNNConfig,
    FlashRNNDecoder,
    check_status,
    flashrnn,
    flashrnn_decode,
    flashrnn_step,
    fused_plan,
    last_status,
    make_carry,
    rnn_function_registry,
)
from ._lib import build_library, library_path, load_library  # noqa: F401

__all__ = ["flashrnn", "flashrnn_step", "flashrnn_decode", "FlashRNNDecoder", "make_carry", "FlashRNNConfig", "rnn_function_registry", "fused_plan",
           "last_status", "check_status",
           "load_library", "library_path", "build_library"]
