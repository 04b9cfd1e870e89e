from .collective_runtime_estimation import (  # noqa: F401
    XGMITopoConfig,
    collective_comm_cost,
    configure,
    detect_mesh_topo_config,
    estimate_strategy_comms_cost,
    get_mesh_topo_config,
    get_nccl_topo_config,
    mi300x_topo_config,
    mi355x_topo,
    mi355x_topo_config,
    redistribute_cost,
    reset_comms_cost_cache,
    set_mesh_topo_config,
    set_nccl_topo_config,
)
from .compute_estimation import (  # noqa: F401
    DeviceLimit,
    compute_memory_cost,
    compute_read_write_time,
    einsum_flop,
    estimate_strategy_runtime_cost,
    reset_compute_cost_cache,
)
from .nccl_cost_model import (  # noqa: F401
    GpuArch,
    MeshDimTopo,
    NCCLTopoConfig,
    a100_topo_config,
    derive_mesh_dim_topo,
    detect_nccl_topo_config,
    gb200_topo_config,
    h100_topo_config,
)
