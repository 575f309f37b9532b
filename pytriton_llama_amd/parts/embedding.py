"""Token embedding and the output head."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    """h[t] = E[ids[t]], no scaling (lite_llama/models/llama.py:179,201). With
    ``float32_stream`` the result is E[ids[t]] * scale in float32 whatever the engine's dtype:
    the start of a residual stream that blocks keep in float32. ``norm``: an RMS norm part (a
    weight and an eps; its tensor is named ``norm_name`` behind the table's name) applied to the
    embedding before anything reads it; the stream then starts from the normed rows."""
    kernel_libraries = ("embedding",)

    def __init__(self, vocab_size: int, hidden_size: int, weight_name: str = "weight",
                 scale: float = 1.0, float32_stream: bool = False, copies: int = 1,
                 norm: Optional[Part] = None, norm_name: str = ".norm"):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.scale, self.float32_stream = float(scale), bool(float32_stream)
        self.copies = int(copies)           # > 1: a row holds the result that many times (a model
                                            # with several residual streams a token)
        if self.copies != 1 and not self.float32_stream:
            raise ValueError("several copies of the embedding are written into a float32 stream")
        if self.float32_stream:
            self.kernel_libraries = ("stream",)
        if self.scale != 1.0 and not self.float32_stream:
            raise ValueError("a scaled embedding is computed into a float32 stream")
        if norm is not None and (not self.float32_stream or self.copies != 1
                                 or not (hasattr(norm, "weight") and hasattr(norm, "eps"))):
            raise ValueError("a norm behind the embedding is an RMS norm (a weight and an eps) and writes "
                             "one float32 stream")
        self.norm, self.norm_name = norm, weight_name + norm_name
        self.weight_name = weight_name
        self.weight: Optional[torch.Tensor] = None

    def param_sources(self) -> List[ParamSource]:
        out = [ParamSource(self.weight_name, (self.vocab_size, self.hidden_size))]
        if self.norm is not None:
            out += [ParamSource(self.norm_name, s.shape, s.kind, s.init) for s in self.norm.param_sources()]
        return out

    def load(self, tensors, dtype, device) -> None:
        self.weight = place(tensors[self.weight_name], "matrix", dtype, device)
        if self.norm is not None:
            (src,) = self.norm.param_sources()
            self.norm.load({src.name: tensors[self.norm_name]}, dtype, device)

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        if self.norm is not None:           # lookup, statistics and weight in one pass over the row
            return ops.embedding_rmsnorm(self.weight, token_ids, self.norm.weight, self.norm.eps, self.scale)
        if self.float32_stream:
            return ops.embedding_scaled(self.weight, token_ids, self.scale, self.copies)
        return ops.embedding(self.weight, token_ids)


@register_part("head", "linear_head")
class LinearHead(Part):
    """logits = x W^T in float32 for the wanted rows only
    (lite_llama/models/llama.py:183,221 computes every row in half precision).
    ``tied_to``: an embedding part whose table is the matrix; then the head has
    no tensor of its own."""
    kernel_libraries = LINEAR_LIBRARIES

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: Optional[TokenEmbedding] = None,
                 weight_name: str = "weight"):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to
        self.weight_name = weight_name
        self._weight: Optional[torch.Tensor] = None
        self.blocked: Optional[torch.Tensor] = None              # decode copy (make_decode_copies)

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def param_sources(self) -> List[ParamSource]:
        if self.tied_to is not None:
            return []
        return [ParamSource(self.weight_name, (self.vocab_size, self.hidden_size))]

    def load(self, tensors, dtype, device) -> None:
        if self.tied_to is None:
            self._weight = place(tensors[self.weight_name], "matrix", dtype, device)

    def make_decode_copies(self) -> int:
        self.blocked = decode_copy(self.weight)
        return 0 if self.blocked is None else self.blocked.numel() * self.blocked.element_size()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, out_dtype=torch.float32, blocked=self.blocked)
