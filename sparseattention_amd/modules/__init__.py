from .attention import HierarchicalAttention  # noqa: F401
