"""tandem_amd: tandem's data-parallel reduction path on one AMD MI355X.

A drop-in for the reference's `Group` plug-in point (`Group(backend="hip")`),
its DDP / ZeRO / FSDP wrappers and ShardedAdamW, driving hand-written HIP
kernels through the C ABI in include/tandem_hip.h. There is no CPU path.
"""

from .comm import CommError, Group, Work, launch
from .local import LocalWorld
from .optim import ShardedAdamW

__all__ = ["CommError", "Group", "Work", "launch", "LocalWorld", "ShardedAdamW"]
