"""In-process selection cache of the registry.

Key format follows dlblas/cache.py:63-75 of the reference: ``<op>-<i>:<dtype>_<d0>x<d1>...`` for tensor
arguments and ``<op>-<i>:<str(arg)>`` for the rest; an explicit ``cache_key`` replaces the generated one
(dlblas/op_registry.py:73,92-96).  Two deliberate differences from the reference:
  * the dtype table knows the float8 types (the reference's raises LookupError for them, cache.py:23-39),
    so ``get_op('fp8_gemm', ...)`` can build a key;
  * ``to_file`` / ``from_file`` use one file name (the reference writes ``.pkl`` and reads ``.pickle``,
    cache.py:130-138) and store only keys -> (op name, implementation index), never code objects.
"""
import json
from typing import Optional

import torch

from .op_struct import OpImpl

_DTYPE_TAGS = {
    torch.float32: 'f32',
    torch.float16: 'f16',
    torch.bfloat16: 'bf16',
    torch.int64: 'i64',
    torch.int32: 'i32',
    torch.int8: 'i8',
    torch.bool: 'bool',
    torch.float8_e4m3fn: 'f8e4m3',
    torch.float8_e5m2: 'f8e5m2',
    torch.uint8: 'u8',
}


def convert_dtype(t: torch.Tensor) -> str:
    try:
        return _DTYPE_TAGS[t.dtype]
    except KeyError:
        raise LookupError(f'unsupported dtype {t.dtype}') from None


def convert_shapes(t: torch.Tensor) -> str:
    return 'x'.join(str(s) for s in t.shape)


def convert_device(t: torch.Tensor) -> str:
    if t.device.type in ('cuda', 'cpu'):
        return t.device.type
    raise LookupError(f'unsupported device {t.device}')


class Cache:

    def __init__(self):
        self._cache = {}
        self._origin = {}  # key -> (op name, index among that op's implementations), for persistence

    def gen_key(self, op_name, args) -> str:
        parts = [op_name]
        for i, arg in enumerate(args):
            if isinstance(arg, torch.Tensor):
                parts.append(f'{i}:{convert_dtype(arg)}_{convert_shapes(arg)}')
            else:
                parts.append(f'{i}:{arg}')
        return '-'.join(parts)

    def _key(self, op_name, args, cache_key):
        return self.gen_key(op_name, args) if cache_key is None else cache_key

    def put(self, op: OpImpl, op_name, args, cache_key, impl_index: Optional[int] = None):
        key = self._key(op_name, args, cache_key)
        self._cache[key] = op
        if impl_index is not None:
            self._origin[key] = (op_name, impl_index)

    def get(self, op_name, args, cache_key) -> Optional[OpImpl]:
        return self._cache.get(self._key(op_name, args, cache_key))

    def __len__(self):
        return len(self._cache)

    def to_file(self, fname):
        with open(f'{fname}.json', 'w') as handle:
            json.dump({k: list(v) for k, v in self._origin.items()}, handle, indent=1, sort_keys=True)

    def from_file(self, fname, ops=None):
        """Reload selections saved by ``to_file``; ``ops`` maps op name -> list of registered OpImpl."""
        with open(f'{fname}.json') as handle:
            data = json.load(handle)
        for key, (op_name, index) in data.items():
            self._origin[key] = (op_name, index)
            if ops is not None and op_name in ops and 0 <= index < len(ops[op_name]):
                self._cache[key] = ops[op_name][index]
