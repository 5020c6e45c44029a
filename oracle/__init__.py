"""CPU oracle of the hierarchical sparse attention forward path.

TEST INFRASTRUCTURE ONLY.  Nothing under the shipped package imports this; it is
used by tests/, by the smoke check and by the benchmark's CPU-baseline leg.
"""
from .hsa_oracle import (  # noqa: F401
    attention_dense,
    attention_ref,
    build_parent_nodes_ref,
    build_tree_ref,
    cross_update_y_ref,
    slot_multiplicity,
    span_input_y_ref,
    topology_scalar,
    topology_tables,
    update_x_from_y_ref,
)
from .lm_ref import lm_forward_ref  # noqa: F401
from .bruteforce import BruteForce, build_bruteforce  # noqa: F401
