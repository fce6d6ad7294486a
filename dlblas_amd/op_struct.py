"""Op descriptors and the argument matcher of the registry.

Observable behaviour follows dlblas/op_struct.py of the reference:
  * ``OpParams`` equality looks only at the arity and the per-argument kind tags (:20-27), so implementations
    for several dtypes can share one op name;
  * ``parse_args`` tags registration arguments (:47-71): ``Tensor`` -> 'tensor', str -> 'str', int and
    ``torch.SymInt`` -> 'int', ``torch.SymFloat`` / ``torch.SymBool`` -> the class itself;
  * ``match`` (:74-131) checks arity, python kinds, tensor dtype equality, device prefix, and that dimensions
    registered under the same ``SymVar`` carry equal sizes (:134-161); a ``None`` argument skips every check.
"""
from dataclasses import dataclass
from typing import Any, Callable, Sequence

import torch

from .symbolic_var import Tensor

_KIND_TENSOR, _KIND_STR, _KIND_INT = 'tensor', 'str', 'int'


@dataclass(frozen=True, eq=False)
class OpParams:
    n_args: int
    args_types: list
    args: tuple

    def __eq__(self, other: object) -> bool:
        assert isinstance(other, OpParams)
        if self.n_args != other.n_args or len(self.args_types) != len(other.args_types):
            return False
        return all(self.args_types[i] == other.args_types[i] for i in range(self.n_args))

    def __hash__(self) -> int:
        return hash((self.n_args, tuple(str(t) for t in self.args_types)))


@dataclass
class OpImpl:
    params: OpParams
    file_path: str
    src: Any
    spaces: Any
    call: Callable
    bench_fn: Callable
    kernel: Callable

    def __call__(self, *args: Any, **kwargs: Any) -> Any:
        return self.call(*args, **kwargs)

    def bench(self, *args: Any, **kwargs: Any) -> Any:
        """Milliseconds per call as measured by the implementation's own bench function (lower is better)."""
        return self.bench_fn(*args, **kwargs)


def _kind_of(position: int, arg: Any):
    if isinstance(arg, Tensor):
        return _KIND_TENSOR
    if isinstance(arg, str):
        return _KIND_STR
    if isinstance(arg, int) or arg is torch.SymInt:
        return _KIND_INT
    if arg is torch.SymFloat or arg is torch.SymBool:
        return arg
    raise TypeError(f'arg {position} has unsupported type {type(arg)}')


def parse_args(args: Sequence) -> OpParams:
    kinds = [_kind_of(i, arg) for i, arg in enumerate(args)]
    return OpParams(n_args=len(args), args_types=kinds, args=tuple(args))


_PY_KIND = {_KIND_TENSOR: torch.Tensor, _KIND_STR: str, _KIND_INT: int, torch.SymFloat: float, torch.SymBool: bool}


def match(user_args, op_params: OpParams) -> bool:
    if not isinstance(user_args, tuple):
        raise TypeError(f'user_args must be a tuple, but got {type(user_args)}')
    if not isinstance(op_params, OpParams):
        raise TypeError(f'op_params must be an OpParams, but got {type(op_params)}')
    if len(user_args) != op_params.n_args:
        return False

    concrete, symbolic = [], []
    for kind, spec, arg in zip(op_params.args_types, op_params.args, user_args):
        if arg is None:
            continue
        if not isinstance(arg, _PY_KIND[kind]):
            return False
        if isinstance(arg, torch.Tensor):
            if arg.dtype != spec.dtype:
                return False
            if not str(arg.device).startswith(spec.device):
                return False
            symbolic.append(spec.shape)
            concrete.append(arg.shape)
    return not violate_symbolic_constraints(concrete, symbolic)


def violate_symbolic_constraints(concrete_shapes, sym_shapes) -> bool:
    """True when one symbol is bound to two different sizes, or a shape has fewer dims than registered."""
    bound = {}
    for shape, syms in zip(concrete_shapes, sym_shapes):
        for axis, sym in enumerate(syms):
            if axis >= len(shape):
                return True
            size = shape[axis]
            if bound.setdefault(sym, size) != size:
                return True
    return False
