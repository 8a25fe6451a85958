"""RNN-T loss and gradient for compact-layout inputs on AMD MI355X (gfx950).

`transducer_loss` keeps the entry point of CompactWarpRNNTLoss (cwarp_rnnt/__init__.py:32-73);
the work is done by hand-written HIP kernels behind the C ABI of include/cwarp_rnnt_hip.h.
"""
from .loss import (ForwardState, joint_forward, lattice_state, pack_padded, rnnt_backward,  # noqa: F401
                   rnnt_forward, rnnt_loss, transducer_loss)
from .joiner import CompactJoiner, compact_join, fused_joiner_loss, fused_joint_loss  # noqa: F401

__version__ = "0.1.0"
__all__ = ["transducer_loss", "rnnt_loss", "pack_padded", "lattice_state", "rnnt_forward", "rnnt_backward",
           "ForwardState", "joint_forward", "compact_join", "fused_joint_loss", "fused_joiner_loss", "CompactJoiner", "__version__"]
