"""MI355X-native FastTree decode attention: host planner + HIP kernels behind a C ABI.

Public surface (same names and argument meaning as the reference's
kernel_bench/fasttree.py): ``FastTreeParams``, ``fasttree_preparation``,
``fasttree_decode``.
"""

from .kv_tree import (  # noqa: F401
    KVTreeNode, retrive_from_file, generate_tree, generate_irregular_tree, save_tree,
    nodes_from_rows, assign_requests, kv_prefix_sums,
)
from .planner import (  # noqa: F401
    FastTreeParams, FastTreePlan, PlanBuffers, fasttree_plan, fasttree_preparation, _tree_heuristic,
)
from .launch_schedule import LaunchPhases, LaunchSchedule, block_programs  # noqa: F401

__all__ = [
    "KVTreeNode", "retrive_from_file", "generate_tree", "generate_irregular_tree", "save_tree",
    "nodes_from_rows", "assign_requests", "kv_prefix_sums",
    "FastTreeParams", "FastTreePlan", "PlanBuffers", "fasttree_plan", "fasttree_preparation",
    "LaunchPhases", "LaunchSchedule", "block_programs",
    "fasttree_decode",
]


def __getattr__(name):
    # The decode entry point loads the HIP library; keep planner-only users free of it.
    if name == "fasttree_decode":
        import importlib
        return importlib.import_module(__name__ + ".decode").fasttree_decode
    raise AttributeError(name)
