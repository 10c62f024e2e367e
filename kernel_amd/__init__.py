"""MI355X-native MoE all-to-all dispatch/combine (one GPU, emulated destination ranks)."""
from .contract import (  # noqa: F401
    COMBINE_F32,
    COMBINE_STRICT,
    META_DIM,
    STUB_EXPERT_FRACTION,
    STUB_OWNER_RANK,
    MoEConfig,
    RankData,
    TestSpec,
    Workload,
    generate_input,
    generate_workload,
    generate_world,
)
