"""Plain data carriers shared by the model and the generators
(reference ``megakernels/model_types.py:20-60``, batch-1 decode subset)."""

from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import Tensor

KV_Cache = tuple[Tensor, Tensor]
DeviceType = torch.device | str


@dataclass
class BatchState:
    """Inputs / outputs of one model call.  Only the fields the batch-1 decode
    path touches are kept."""

    input_ids: Tensor
    position_ids: Tensor | None = None
    seq_len: int | None = None
    output_ids: Tensor | None = None
    hidden_states: Tensor | None = None
    position_embeddings: tuple[Tensor, Tensor] | None = None

    def __post_init__(self):
        if self.seq_len is None:
            self.seq_len = self.input_ids.shape[-1]


@dataclass
class ExtraModelConfig:
    """Flags that are not part of the architecture description."""

    interleave_rope: bool = False
    max_len_override: int | None = None
    max_batch_size: int = 1
    rope_scaling: dict | None = None
