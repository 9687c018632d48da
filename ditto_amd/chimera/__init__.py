"""Layer-to-scheduler binding and graph-level fusion (reference: python/ditto/chimera)."""
from .graph_fusion import graph_fusion
from .task_binding import task_binding
