"""Interfaces of the parts a layer is put together from.

A part gets its sizes and constants through its ``PartSpec``; it never sees a
model configuration or knows which model it is in.  A part says which tensors
it wants (``param_specs``), takes them (``bind``) and runs on the tokens of
one step (``forward``).  What a mixer keeps between steps it declares as a
``CacheNeed``; the cache manager groups layers by need.
"""

from __future__ import annotations

import dataclasses
from typing import TYPE_CHECKING, Optional, Sequence

import torch

if TYPE_CHECKING:  # pragma: no cover
    from ..engine.batch import StepBatch


# --------------------------------------------------------------------------
# Parameters
# --------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class ParamSpec:
    """One tensor a part reads from the checkpoint.

    ``init`` tells the random-weights mode how to fill it: ``("normal", std)``
    for floating tensors, ``("randint", lo, hi)`` for integer tables."""

    name: str
    shape: tuple[int, ...]
    init: tuple = ("normal", 0.02)
    integer: bool = False


class Part:
    """Base of every part.

    ``capturable`` says whether the part's ``forward`` may be recorded into a
    HIP graph and replayed: it must launch the same kernels with the same
    grids and addresses whatever the data, never wait for the device and never
    read a result on the host.  A part that does any of that sets it to False,
    and steps of a model that holds such a part are never taken from a graph."""

    capturable: bool = True
    # Whether the part lays bf16 matrices out in tiles for the few-row product (``linear.decode_weight``): the
    # engine's setting, which the model writes into every part it holds before it binds them.
    tiled_weights: bool = True

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return []

    def bind(self, tensors: dict[str, torch.Tensor], prefix: str, device: torch.device, dtype: torch.dtype) -> None:
        """Take the tensors named by ``param_specs(prefix)``.  ``dtype`` is the
        dtype of activations; a part may fuse or re-lay tensors here."""


# --------------------------------------------------------------------------
# What a mixer keeps between steps
# --------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class KVNeed:
    """Keys and values of earlier tokens, in pages.

    ``window`` is None when every earlier token stays visible, else the
    number of most recent positions (the current one included) a token can
    see.  Layers with the same ``window`` share a page group and block table;
    head counts and sizes may differ between them."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class StateNeed:
    """A state of fixed size for every live request (one slot each)."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


CacheNeed = "KVNeed | StateNeed | None"


@dataclasses.dataclass
class KVCacheView:
    """What an attention-like mixer gets for its layer: the key pages
    ``[num_pages, num_kv_heads, page_size, head_dim]``, the value pages
    ``[num_pages, num_kv_heads, page_size / 16, head_dim, 16]`` (transposed
    inside groups of 16 slots: ``csrc/kv_layout.h``) and the name of the group
    whose block table addresses them.
    ``writes`` is False for a layer that reads another layer's cache."""

    k_pages: torch.Tensor
    v_pages: torch.Tensor
    group: str
    page_size: int
    writes: bool = True

    def reader(self) -> "KVCacheView":
        return dataclasses.replace(self, writes=False)


@dataclasses.dataclass
class StateView:
    """What a mixer with fixed-size state gets: ``[num_slots, *shape]``; the
    step batch tells the slot of each request.  A request's slot is zeroed
    when it is handed out."""

    slots: torch.Tensor
    writes: bool = True

    def reader(self) -> "StateView":
        return dataclasses.replace(self, writes=False)


# --------------------------------------------------------------------------
# Parts
# --------------------------------------------------------------------------
class Norm(Part):
    """y = norm(x) over the last dimension."""

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError

    def forward_rows(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """norm(x[rows]) for an int32 index tensor."""
        return self.forward(x.index_select(0, rows.long()))

    def add_into(
        self,
        branch: torch.Tensor,
        residual: torch.Tensor,
        then: "Optional[Norm]" = None,
        then_out: Optional[torch.Tensor] = None,
    ) -> Optional[torch.Tensor]:
        """residual += norm(branch), in place; when ``then`` is given also
        return then(residual).  The default runs the pieces one by one; a norm
        with a fused kernel overrides it."""
        from ..kernels import ops

        normed = self.forward(ops.as_tensor(branch))
        residual.add_(normed)
        return then.forward(residual, out=then_out) if then is not None else None


class PositionEncoding(Part):
    """How a mixer marks positions.  ``rotary_dim`` is the number of rotated
    dimensions of a head and ``tables(step)`` the 32-bit cosines and sines of
    the step's tokens, ``([tokens, rotary_dim / 2], the same)``, or None when
    nothing is rotated: what the fused query/key kernel needs.  Layers that
    rotate alike share one pair of tables per step (``step.shared``)."""

    rotary_dim: int = 0

    def inv_freq(self, device: torch.device) -> Optional[torch.Tensor]:
        return None

    def tables(self, step: "StepBatch") -> Optional[tuple[torch.Tensor, torch.Tensor]]:
        return None


class Embedding(Part):
    """What enters the first layer: ``forward`` fills ``out[tokens, hidden]``
    from the step (its token ids, and its positions if the part adds learned
    ones)."""

    def forward(self, step: "StepBatch", out: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Logits from the normed rows: ``forward(x[rows, hidden])`` returns 32-bit
    ``[rows, vocab]``.  A head is built with the model's embedding in hand
    (``embedding=``), so that it can share its table."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the tokens of a request.  ``forward`` returns
    ``[tokens, hidden]``: a tensor, or ``ops.SlicedSums`` when its last product
    was left unreduced for the norm that follows (``ops.as_tensor`` reduces)."""

    def cache_need(self):
        return None

    def forward(self, x: torch.Tensor, step: "StepBatch", cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """Works on every token alone."""

    def forward(self, x: torch.Tensor, step: "StepBatch") -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """The arrangement of norm, mixer, feed-forward and the residual sum in
    one layer.  ``forward`` updates the residual stream ``x`` in place.

    ``entry_norm`` is the norm the block applies to the residual stream first,
    or None.  ``forward`` may be given that norm's output (``entered``) when
    the block before has computed it, and may be asked to return
    ``then(x)`` for the block after; a block that does not fuse returns None
    and the caller applies the norm itself."""

    mixer: Mixer
    feed_forward: FeedForward

    def parts(self) -> Sequence[Part]:
        """Every part the block holds (the model asks each whether it can be
        recorded into a graph)."""
        return (self.mixer, self.feed_forward)

    @property
    def capturable(self) -> bool:
        return all(part.capturable for part in self.parts())

    def entry_norm(self) -> Optional[Norm]:
        return None

    def forward(self, x: torch.Tensor, step: "StepBatch", cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        raise NotImplementedError
