"""Symbolic shape placeholders used when an op is registered.

Mirrors the interface of dlblas/symbolic_var.py:134-177 of the reference: ``SymVar`` is a named dimension
(equal and hashed by name) and ``Tensor`` is a shape/dtype/device description, never real storage.
"""
import torch


class SymVar:
    """A named, unknown dimension.  Two SymVars are the same dimension iff their names are equal."""

    __slots__ = ('name', )

    def __init__(self, name):
        assert isinstance(name, str)
        self.name = name

    def __eq__(self, other) -> bool:
        return isinstance(other, SymVar) and other.name == self.name

    def __hash__(self) -> int:
        return hash(self.name)

    def __repr__(self) -> str:
        return f'SymVar({self.name!r})'


class Tensor:
    """Registration-time description of a tensor argument: symbolic shape, device prefix, dtype."""

    def __init__(self, shape, *, device: str, dtype: torch.dtype):
        for dim in shape:
            assert isinstance(dim, SymVar), f'expect a SymVar, but got {dim}'
        self._shape = tuple(shape)
        self._device = device
        self._dtype = dtype

    shape = property(lambda self: self._shape)
    device = property(lambda self: self._device)
    dtype = property(lambda self: self._dtype)

    def __repr__(self) -> str:
        return f'Tensor({self._shape}, device={self._device!r}, dtype={self._dtype})'
