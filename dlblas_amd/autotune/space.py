"""Search-space value types accepted by ``register_dlblas_op(spaces=...)``.

The reference's tuner (dlblas/autotune/*) rewrites Triton launch sites and is bypassed by its own
registry (dlblas/op_registry.py:131-132); a hand-written HIP kernel has nothing for it to rewrite.  Only the
container types survive here so registrations written against the reference keep importing
(dlblas/autotune/space.py:34-178).
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List


def next_power_of_2(n: int) -> int:
    """Smallest power of two >= n (n >= 1)."""
    return 1 if n <= 1 else 1 << (int(n) - 1).bit_length()


@dataclass
class FixedSpace:
    value: Any

    def sample(self):
        return self.value


@dataclass
class DiscreteSpace:
    choices: List[Any]

    def sample(self):
        return self.choices[0]


@dataclass
class RangeSapce:  # spelling kept from the reference's public name
    start: int
    end: int

    def sample(self):
        return self.start


@dataclass
class PowerOfTwoSpace:
    start: int
    end: int

    def sample(self):
        return next_power_of_2(self.start)


@dataclass
class ChoiceSpace:
    """A flat list of complete configurations."""
    choices: List[Any] = field(default_factory=list)

    def __len__(self):
        return len(self.choices)

    def __getitem__(self, i):
        return self.choices[i]


@dataclass
class DictSpace:
    """One sub-space per named parameter."""
    params: Dict[str, Any] = field(default_factory=dict)

    def sample(self):
        return {k: (v.sample() if hasattr(v, 'sample') else v) for k, v in self.params.items()}
