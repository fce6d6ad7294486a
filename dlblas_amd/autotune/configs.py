"""Tuner settings object accepted by ``get_op(configs=...)`` (dlblas/autotune/configs.py:6-12)."""
from dataclasses import dataclass


@dataclass
class AutotuneConfig:
    total_iteration: int = 5
    tunner: str = 'enumeration'
