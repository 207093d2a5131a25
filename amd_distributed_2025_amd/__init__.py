"""MI355X-native MoE dispatch/combine (one rank's share of the all2all task)."""
from .task import MoEConfig, RankTestData, TestSpec, generate_input, generate_world, WORKLOADS  # noqa: F401
from .all2all import HIPAllToAll, LocalExchange, LocalWorld, run_lockstep  # noqa: F401
from .submission import custom_kernel, custom_kernel_job, set_peer_inputs  # noqa: F401

__all__ = [
    "MoEConfig", "RankTestData", "TestSpec", "generate_input", "generate_world", "WORKLOADS",
    "HIPAllToAll", "LocalExchange", "LocalWorld", "run_lockstep", "custom_kernel", "custom_kernel_job",
    "set_peer_inputs",
]
