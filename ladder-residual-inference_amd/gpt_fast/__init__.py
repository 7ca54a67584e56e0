"""Ladder-Residual inference, MI355X-native: the reference's gpt_fast package surface
(gpt_fast/__init__.py:1-5) on hand-written gfx950 kernels."""
from .gpt_dense_TP import GPTDense
from .gpt_desync_TP import GPTDesync
from .gpt_ladder_TP import GPTLadder
from .gpt_parallel_TP import GPTParallel
from .tp import maybe_init_dist, set_virtual_tp

__all__ = ["GPTDense", "GPTDesync", "GPTLadder", "GPTParallel", "maybe_init_dist", "set_virtual_tp"]
