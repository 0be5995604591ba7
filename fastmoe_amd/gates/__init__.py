r"""Gates of the single-GPU MoE layer (fmoe/gates/__init__.py of the reference
lists more policies; the ones here are those that touch the native capacity
ops or define the default behaviour)."""
from .base_gate import BaseGate
from .naive_gate import NaiveGate
from .gshard_gate import GShardGate
from .switch_gate import SwitchGate
from .utils import limit_by_capacity

__all__ = ["BaseGate", "NaiveGate", "GShardGate", "SwitchGate", "limit_by_capacity"]
