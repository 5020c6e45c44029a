"""MI355X-native forward path of hierarchical sparse attention.

Exports the reference library's public names (hierarchical_attention/__init__.py:3-18).
"""
__version__ = "0.1.0"

from ._lib import HsaError  # noqa: F401,E402
from .modules import HierarchicalAttention  # noqa: F401,E402
from .ops import (  # noqa: F401,E402
    attention_forward,
    build_parent_nodes,
    build_tree,
    build_tree_topology,
    generate_span_input_Y,
    hierarchical_attention,
)

from .transformer import TransformerLM  # noqa: F401,E402

__all__ = [
    "TransformerLM",
    "HierarchicalAttention",
    "build_tree_topology",
    "generate_span_input_Y",
    "build_parent_nodes",
    "hierarchical_attention",
    "build_tree",
    "attention_forward",
    "HsaError",
    "__version__",
]
