"""MI355X-native kernels for the ReBeL search hot path of P2 (phulin/poker2):
7-card hand ranker, river showdown with blocker correction, unblocked mass and
the fused DCFR iteration, behind the reference's Python function names."""
from ._lib import P2HipError, hip_is_available, library_path  # noqa: F401

__all__ = ["P2HipError", "hip_is_available", "library_path"]
