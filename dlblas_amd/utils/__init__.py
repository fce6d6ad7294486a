"""Registry exports under the names of dlblas/utils/__init__.py:2-23 of the reference."""
from ..autotune.configs import AutotuneConfig
from ..autotune.space import ChoiceSpace, DictSpace, DiscreteSpace, FixedSpace, PowerOfTwoSpace, RangeSapce
from ..op_registry import op_registry
from ..op_struct import OpImpl, OpParams
from ..symbolic_var import SymVar, Tensor

register_dlblas_op = op_registry.register


def get_list_op_names():
    return op_registry.get_list_op_names()


def get_args_from_op_name(name: str):
    return op_registry.get_args_from_op_name(name)


def get_op(name: str, args, configs=None, cache_key=None):
    """Select (and cache) the implementation of ``name`` that fits ``args``; returns an ``OpImpl``."""
    return op_registry.get_op(name, args, configs, cache_key)
