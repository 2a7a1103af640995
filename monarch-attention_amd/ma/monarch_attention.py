"""Operator API of MonarchAttention - the drop-in boundary.

Mirrors the reference's ``ma/monarch_attention.py`` name for name
(``MonarchAttentionFn`` ``:11-13``, ``_IMPLEMENTATIONS`` / ``register_impl``
``:15-19``, ``PadType`` ``:32-34``, ``MonarchAttention`` ``:37-66``) so model
code written against it runs unchanged.  The implementation registered here is
``"hip"``: hand-written gfx950 kernels behind a C ABI (see ``ma_hip.py``).
There is no CPU or eager-PyTorch implementation in this package and therefore
no silent fallback: constructing the module with an unknown ``impl`` raises
the reference's ``ValueError`` and calling ``"hip"`` without the built library
or on CPU tensors raises as well.  Other implementations (for instance the
reference's own ``"torch"``) can be added with ``register_impl``.
"""
from __future__ import annotations

from collections.abc import Callable
from enum import Enum

import torch
import torch.nn as nn

from .ma_hip import monarch_attention_hip, monarch_matrix_hip

Tensor = torch.Tensor

# fn(q, k, v, attn_mask, T, B, pre_pad) -> out
MonarchAttentionFn = Callable[[Tensor, Tensor, Tensor, "Tensor | None", int, int, bool], Tensor]

_IMPLEMENTATIONS: dict[str, MonarchAttentionFn] = {}


def register_impl(name: str, fn: MonarchAttentionFn) -> None:
    """Make ``fn`` selectable as ``MonarchAttention(..., impl=name)``."""
    _IMPLEMENTATIONS[name] = fn


register_impl("hip", monarch_attention_hip)


class PadType(str, Enum):
    """Where the zero padding up to a multiple of the block size goes.

    String-valued like the reference's ``StrEnum`` (which needs Python 3.11):
    ``PadType.pre == "pre"`` and ``str(PadType.pre) == "pre"`` both hold.
    """
    pre = "pre"
    post = "post"

    def __str__(self) -> str:
        return self.value

    __format__ = str.__format__


class MonarchAttention(nn.Module):
    """Monarch-structured attention ``A = P^T L P R`` fitted by ``num_steps``
    rounds of alternating maximisation, applied to ``value``.

    ``block_size`` is the block size ``b`` (``m = ceil(N / b)`` blocks),
    ``pad_type`` a ``PadType`` or its string.  The module has no parameters and
    keeps no state between calls.
    """

    def __init__(self, block_size, num_steps, pad_type, impl="hip"):
        super().__init__()
        self.block_size = block_size
        self.num_steps = num_steps
        self.pad_type = pad_type

        if impl not in _IMPLEMENTATIONS:
            known = ", ".join(sorted(_IMPLEMENTATIONS))
            raise ValueError(f"Unknown impl {impl!r}. Available: {known}")
        self._impl_fn = _IMPLEMENTATIONS[impl]

    def forward(self, query, key, value, attention_mask=None):
        """``query, key (E,H,N,D)``, ``value (E,H,N,Dv)``, optional
        ``attention_mask (E,N)`` (truthy = keep) -> ``(E,H,N,Dv)``."""
        pre_pad = self.pad_type == PadType.pre
        return self._impl_fn(query, key, value, attention_mask, self.num_steps, self.block_size, pre_pad)

    def get_matrix(self, query, key, attention_mask=None):
        """Dense ``(E,H,N,N)`` fp32 attention matrix: the forward pass applied to
        an fp32 identity (reference ``:61-66``).  The ``"hip"`` implementation
        writes the matrix directly (no identity, no ``(E,H,Np,N)`` intermediate)
        and takes the identity route only for sequences its matrix kernel does
        not hold on chip; other implementations always take that route."""
        E, H, N, _ = query.shape
        if self._impl_fn is monarch_attention_hip:
            pre_pad = self.pad_type == PadType.pre
            try:
                return monarch_matrix_hip(query, key, attention_mask, self.num_steps, self.block_size, pre_pad)
            except NotImplementedError:
                pass
        eye = torch.eye(N, device=query.device).expand(E, H, N, N)
        return self.forward(query, key, eye, attention_mask)

    def extra_repr(self) -> str:
        return f"block_size={self.block_size}, num_steps={self.num_steps}, pad_type={str(self.pad_type)!r}"
