from .functional import (  # noqa: F401
    attention_forward,
    build_parent_nodes,
    build_parents_forward,
    build_parents_strided,
    build_tree,
    hierarchical_attention,
)
from .topology import build_tree_topology, generate_span_input_Y  # noqa: F401
