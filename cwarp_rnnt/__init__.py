"""Drop-in name of the reference package: `import cwarp_rnnt; cwarp_rnnt.transducer_loss(...)`
(cwarp_rnnt/__init__.py:32 of CompactWarpRNNTLoss) resolves to the MI355X implementation."""
from compactwarprnntloss_amd import __version__, transducer_loss  # noqa: F401

__all__ = ["transducer_loss", "__version__"]
