"""MI355X-native DFlash speculative-decoding step.

Host-side mirror of the reference engine's interfaces for this path, over the C ABI
of ``libdflash_hip.so`` (hand-written HIP for gfx950, declared in
``include/dflash_hip.h``).  Device memory and streams come from PyTorch-ROCm; every
array argument that reaches the library is a device tensor.

There is no CPU fallback: if the HIP library is missing or no GPU is present, the
calls raise.
"""
from __future__ import annotations

from . import synth  # noqa: F401
from .binding import (  # noqa: F401
    DFlashError,
    LIB_PATH,
    STATUS,
    TYPE_F16,
    TYPE_F32,
    TYPE_Q4_K,
    TYPE_Q4_K_TILED,
    TYPE_Q6_K_TILED,
    TYPE_Q6_K,
    TYPE_Q8_0,
    TYPE_RANGE_CHECKED,
    QT_RANGE_CHECKED,
    XF_NONE,
    XF_Q4K,
    XF_Q6K,
    AcceptDecision,
    CARRY_BONUS,
    CARRY_CORRECTION,
    CARRY_NONE,
    Context,
    RNG_PHILOX,
    RNG_XOSHIRO,
    STOP_EOS,
    STOP_NONE,
    STOP_TOKEN_LIMIT,
    Sampler,
    declared_symbols,
    lib,
)
from .model import (  # noqa: F401,E402
    DraftConfig,
    DraftHead,
    DraftSession,
    ModelConfig,
    Session,
    AdaptiveStateC,
    SpeculativeDecoder,
    adaptive_lib,
    TargetModel,
    accept_greedy,
    synth_draft_weights,
    synth_draft_weights_device,
    synth_target_weights_device,
    synth_target_weights,
    synth_target_weights_blocks,
)
from . import gguf  # noqa: F401,E402
from .gguf import GgufFile, open_dflash_drafter, open_target, write_gguf  # noqa: F401,E402
