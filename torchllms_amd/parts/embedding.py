"""Token embedding and output head."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamSpec


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Embedding):
    """``h = weight[token]`` (reference: torchllms/models/networks.py:793,1017, which has no scale
    factor).  ``stream_dtype`` "float32": the rows open a 32-bit residual stream whatever the model's
    dtype, as ``float(weight[token]) * scale``."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, stream_dtype: Optional[str] = None):
        if stream_dtype not in (None, "float32"):
            raise ValueError(f"embedding: stream_dtype {stream_dtype!r} (None: the model's dtype, or \"float32\")")
        if stream_dtype is None and float(scale) != 1.0:
            raise ValueError("embedding: a scale factor needs the 32-bit residual stream (stream_dtype=\"float32\")")
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)
        self.stream_dtype = stream_dtype
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        if self.stream_dtype == "float32":
            return ops.embed_scaled(tokens, self.weight, self.scale)
        return ops.embed(tokens, self.weight)


@HEADS.register("lm_head")
class LMHead(Head):
    """``logits = x W^T`` with W [vocab, hidden], no bias; with ``tied`` W is the embedding
    matrix (reference: torchllms/models/networks.py:804-809,1047).  Logits are returned in 32-bit.
    ``softcap`` c > 0: the logits become ``c * tanh(logits / c)``."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool, softcap: float = 0.0):
        if softcap < 0:
            raise ValueError(f"lm_head: softcap {softcap!r} must not be negative")
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied
        self.softcap = float(softcap)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.tied:
            return {}
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        if not self.tied:
            self.weight = tensors["weight"].contiguous()

    def tie(self, embedding: TokenEmbedding) -> None:
        self.weight = embedding.weight

    def linear_weights(self):
        return [(self.weight, "plain", torch.float32)]

    def ignorable_params(self):
        # checkpoints of tied models sometimes carry the output matrix all the same
        return ["weight"] if self.tied else []

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(x, self.weight, out_dtype=torch.float32)
        if self.softcap > 0:
            if not logits.is_contiguous():
                logits = logits.contiguous()
            ops.softcap_(logits, self.softcap)
        return logits
