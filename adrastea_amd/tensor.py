"""Stride algebra of the reference's tensors (adrastea_models/src/tensor.rs:25-150) and a
view type over device memory.  Strides are in elements; dims are outermost first."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence, Tuple


@dataclass(frozen=True)
class TensorLayout:
    dims: Tuple[int, ...]
    strides: Tuple[int, ...]

    def __post_init__(self):
        # tensor.rs:32-39
        if len(self.dims) != len(self.strides) or len(self.dims) == 0:
            raise ValueError("dims and strides must be non-empty and of equal length")
        if any(d == 0 for d in self.dims) or any(s == 0 for s in self.strides):
            raise ValueError("zero-sized dims or zero strides are not representable")
        object.__setattr__(self, "dims", tuple(int(d) for d in self.dims))
        object.__setattr__(self, "strides", tuple(int(s) for s in self.strides))

    @staticmethod
    def row_major(dims: Sequence[int]) -> "TensorLayout":  # tensor.rs:41-50
        strides, s = [], 1
        for d in reversed(dims):
            strides.append(s)
            s *= d
        return TensorLayout(tuple(dims), tuple(reversed(strides)))

    @staticmethod
    def column_major(dims: Sequence[int]) -> "TensorLayout":  # tensor.rs:52-60
        rm = TensorLayout.row_major(dims)
        st = list(rm.strides)
        st[-2], st[-1] = st[-1], st[-2]
        return TensorLayout(rm.dims, tuple(st))

    def largest_address(self) -> int:  # tensor.rs:62-68
        return sum((d - 1) * s for d, s in zip(self.dims, self.strides))

    def permute(self, order: Sequence[int]) -> "TensorLayout":  # tensor.rs:70-79
        if len(order) != len(self.dims):
            raise ValueError("permute needs one index per dimension")
        return TensorLayout(tuple(self.dims[i] for i in order),
                            tuple(self.strides[i] for i in order))

    def shape_cast(self, dims: Sequence[int]) -> "TensorLayout":  # tensor.rs:82-105
        """Reinterprets the VOLUME with fresh contiguous strides: like the reference it ignores
        any permutation or gaps of the current layout ("poor man's .view()")."""
        vol = 1
        for d in self.dims:
            vol *= d
        if sum(1 for d in dims if d < 0) > 1:
            raise ValueError("at most one inferred dimension")
        known = 1
        for d in dims:
            if d >= 0:
                known *= d
        out = [d if d >= 0 else vol // known for d in dims]
        prod = 1
        for d in out:
            prod *= d
        if prod != vol:
            raise ValueError("shape_cast must preserve the volume")
        return TensorLayout.row_major(out)

    def size(self, dim: int) -> int:  # tensor.rs:107-113
        return self.dims[dim]

    def stride(self, dim: int) -> int:  # tensor.rs:115-121
        return self.strides[dim]

    def skip(self, sizes: Sequence[int]) -> Tuple[int, "TensorLayout"]:  # tensor.rs:123-136
        offset, nd = 0, []
        for d, s, sz in zip(self.dims, self.strides, sizes):
            sz = d if sz == -1 else sz
            if not 0 <= sz <= d:
                raise ValueError("skip size out of range")
            offset += s * sz
            nd.append(d - sz)
        return offset, TensorLayout(tuple(nd), self.strides[:len(nd)])

    def take(self, sizes: Sequence[int]) -> "TensorLayout":  # tensor.rs:138-149
        nd = []
        for d, sz in zip(self.dims, sizes):
            sz = d if sz == -1 else sz
            if not 0 <= sz <= d:
                raise ValueError("take size out of range")
            nd.append(sz)
        return TensorLayout(tuple(nd), self.strides[:len(nd)])


class TensorView:
    """A layout over device memory.  ``storage`` is any object with ``data_ptr()`` and
    ``element_size()`` (a torch tensor: PyTorch is used for device memory only)."""

    def __init__(self, storage, layout: TensorLayout, offset: int = 0):
        self.storage, self.layout, self.offset = storage, layout, int(offset)

    @staticmethod
    def of(t) -> "TensorView":
        """View of a torch tensor with its own sizes and strides."""
        return TensorView(t, TensorLayout(tuple(t.shape), tuple(t.stride())), 0)

    def data_ptr(self) -> int:
        return self.storage.data_ptr() + self.offset * self.storage.element_size()

    def size(self, dim: int) -> int:
        return self.layout.size(dim)

    def stride(self, dim: int) -> int:
        return self.layout.stride(dim)

    def permute(self, order) -> "TensorView":
        return TensorView(self.storage, self.layout.permute(order), self.offset)

    def shape_cast(self, dims) -> "TensorView":
        return TensorView(self.storage, self.layout.shape_cast(dims), self.offset)

    def skip(self, sizes) -> "TensorView":
        off, lay = self.layout.skip(sizes)
        return TensorView(self.storage, lay, self.offset + off)

    def take(self, sizes) -> "TensorView":
        return TensorView(self.storage, self.layout.take(sizes), self.offset)
