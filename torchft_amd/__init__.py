"""torchft_amd: the replica-synchronisation hot path of torchft, native to MI355X.

Public names follow the reference package (``torchft``): ``Manager``,
``LocalSGD`` / ``DiLoCo`` (in ``torchft_amd.local_sgd``), ``DistributedDataParallel``,
``OptimizerWrapper``, ``CheckpointTransport`` / ``CheckpointServer`` and the
process-group plugins.  The arithmetic runs in HIP kernels behind the C ABI
declared in ``include/torchft_amd.h``; there is no CPU fallback.
"""

from .checkpointing import CheckpointServer, CheckpointTransport
from .ddp import DistributedDataParallel, GradBucketAverager, PureDistributedDataParallel
from .local_cluster import InProcessLighthouse, ProcessGroupThreads, ThreadWorld
from .local_sgd import DiLoCo, LocalSGD
from .manager import (
    Manager,
    ManagerClientAdapter,
    QuorumClient,
    QuorumResult,
    StaticQuorum,
    WorldSizeMode,
)
from .optim import OptimizerWrapper as Optimizer
from .optim import OptimizerWrapper
from .process_group import (
    ProcessGroup,
    ProcessGroupDummy,
    ProcessGroupLocalReplicas,
)

__all__ = (
    "CheckpointServer",
    "CheckpointTransport",
    "DiLoCo",
    "DistributedDataParallel",
    "GradBucketAverager",
    "InProcessLighthouse",
    "LocalSGD",
    "Manager",
    "ManagerClientAdapter",
    "Optimizer",
    "OptimizerWrapper",
    "ProcessGroup",
    "ProcessGroupDummy",
    "ProcessGroupLocalReplicas",
    "ProcessGroupThreads",
    "PureDistributedDataParallel",
    "QuorumClient",
    "QuorumResult",
    "StaticQuorum",
    "ThreadWorld",
    "WorldSizeMode",
)
