from .graph_engine import Graph, GraphEngine, create_cuda_graph_engine, create_graph_engine, create_hip_graph_engine
