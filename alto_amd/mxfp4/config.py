"""Recipe-level configuration of the low-precision training ops (alto/kernels/dispatch/config.py:10-51)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

import torch


@dataclass(unsafe_hash=True, kw_only=True, slots=True)
class TrainingOpConfig:
    precision: Literal["mxfp4"] = "mxfp4"
    use_2dblock_x: bool = False
    use_2dblock_w: bool = True
    use_hadamard: bool = True
    use_sr_grad: bool = True
    use_dge: bool = False
    clip_mode: Literal["none", "static", "dynamic"] = "none"
    two_level_scaling: Literal["none", "tensorwise", "blockwise"] = "none"
    use_uos: bool = False

    def __post_init__(self):
        if self.precision != "mxfp4":
            raise ValueError(f"this build implements precision='mxfp4' only, got {self.precision!r}")
        if self.clip_mode not in ("none", "static", "dynamic"):
            raise ValueError(f"Invalid clip mode: {self.clip_mode}")


torch.serialization.add_safe_globals([TrainingOpConfig])   # dispatch/config.py:57
