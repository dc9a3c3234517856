"""MI355X (gfx950) implementation of the fused training-step kernels: causal flash attention,
the fp8 fused MLP, the RMSNorm / residual blocks and the LM-head + cross-entropy loss, as
hand-written HIP behind a C-ABI library (include/tfb_kernels.h), with a Python host layer that
keeps the call signatures of the reference's training loop."""
from . import _lib  # noqa: F401

__all__ = ["_lib", "ops"]
