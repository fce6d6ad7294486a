"""Name -> implementations registry with benchmark-based selection and caching.

Same surface and control flow as dlblas/op_registry.py:18-136 of the reference:
``register(name, spaces, args, call, bench_fn, kernel)``; ``get_op(name, args, configs=None, cache_key=None)``
looks the cache up first, otherwise filters implementations with ``match``, runs ``bench`` of EVERY candidate
(also when there is only one, :130-135), caches and returns the fastest.  Errors: ``NameError`` for an unknown
op (:74-75), ``LookupError`` when nothing matches (:102), ``AssertionError`` when a name is re-registered with a
different parameter signature (:57-60).

One conscious change: registering the same (name, call) pair again is a no-op.  The reference executes each
kernel file twice under two module names and appends duplicates (its own FIXME at :56).
"""
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

from .autotune.configs import AutotuneConfig
from .cache import Cache
from .op_struct import OpImpl, match, parse_args
from .utils.logger import get_logger

logger = get_logger(__name__)


@dataclass
class OpRegistry:
    ops: Dict[str, List[OpImpl]] = field(default_factory=dict)
    cache: Cache = field(default_factory=Cache)

    def register(self, name, spaces, args, call, bench_fn, kernel):
        params = parse_args(args)
        here = os.path.dirname(os.path.realpath(__file__))
        kernel_file = os.path.join(here, 'kernels', call.__module__.rsplit('.', 1)[-1] + '.py')
        impl = OpImpl(params, kernel_file, None, spaces, call, bench_fn, kernel)
        impls = self.ops.setdefault(name, [])
        if impls:
            assert impls[0].params == params, \
                f'Multiple implementations of a kernel:{name} must have the same parameters.'
            for known in impls:
                if known.call is call and _same_specs(known.params.args, params.args):
                    return
        impls.append(impl)

    def get_op_count(self, name):
        return len(self.ops[name])

    def get_list_op_names(self):
        return list(self.ops.keys())

    def get_args_from_op_name(self, op_name: str):
        return [impl.params for impl in self.ops[op_name]]

    def get_op(self, op_name: str, args: tuple, configs=None, cache_key=None) -> OpImpl:
        if op_name not in self.ops:
            raise NameError(f'op {op_name} not found')
        cached = self.look_up_cache(op_name, args, cache_key)
        if cached is not None:
            logger.debug(f'cache hit for op {op_name}')
            return cached
        if configs is None:
            configs = AutotuneConfig()
        else:
            assert isinstance(configs, AutotuneConfig)
        return self._tunning(op_name, args, configs, cache_key)

    def look_up_cache(self, op_name: str, args: tuple, cache_key) -> Optional[OpImpl]:
        cached = self.cache.get(op_name, args, cache_key)
        if cached is not None:
            assert isinstance(cached, OpImpl)
        return cached

    def _tunning(self, op_name: str, args: tuple, configs=None, cache_key=None):
        candidates = self._get_candidates(op_name, args)
        if not candidates:
            raise LookupError(f'no candidates for op {op_name} with args')
        best_idx, _ = self._selection(args, candidates, configs)
        best = candidates[best_idx]
        self.cache.put(best, op_name, args, cache_key, impl_index=self.ops[op_name].index(best))
        return best

    def _get_candidates(self, op_name: str, args: tuple):
        return [impl for impl in self.ops[op_name] if match(args, impl.params)]

    def _selection(self, args, candidates, configs):
        best_idx, best_perf = -1, None
        for i, impl in enumerate(candidates):
            perf = impl.bench(*args)
            if best_perf is None or perf < best_perf:
                best_idx, best_perf = i, perf
        return best_idx, best_perf


def _same_specs(a, b) -> bool:
    if len(a) != len(b):
        return False
    for x, y in zip(a, b):
        x_t, y_t = hasattr(x, 'dtype'), hasattr(y, 'dtype')
        if x_t != y_t:
            return False
        if x_t:
            if (x.dtype, x.device, x.shape) != (y.dtype, y.device, y.shape):
                return False
        elif x != y:
            return False
    return True


op_registry = OpRegistry()
