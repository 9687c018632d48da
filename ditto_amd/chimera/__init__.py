"""Layer-to-scheduler binding and graph-level fusion (reference: python/ditto/chimera)."""
from .graph_fusion import fuse_activation, graph_fusion, is_act_layer, is_elem_layer
from .task_binding import task_binding
