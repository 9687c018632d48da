"""Graph engine: runs a sequence of built chain layers over device buffers.

Counterpart of src/runtime/graph_runtime.cc:14-260 (``GraphEngine``: init / set_inputs /
set_weight / compile / run / timeit / get_outputs) and python/ditto/runtime/graph_engine.py
(``create_graph_engine``, ``create_cuda_graph_engine``).  Buffers are torch tensors on a HIP
device; every layer's function is called as ``f(*inputs, *weights, *outputs)``
(``Layer.schedule_tensors`` order, graph_runtime.cc:170-196).  The graph-replay engine records
the whole sequence once into a HIP graph and replays it, the counterpart of the reference's
CUDA-graph engine.
"""
import time

import torch

TORCH_DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32,
                "int8": torch.int8, "int32": torch.int32}


class Graph:
    """An ordered list of layers and the tensors that connect them.

    ``edges[(consumer index, input index)] = (producer index, output index)``; layer inputs
    without an edge are the graph inputs, in layer order (the reference derives the same
    information from its ``LayerTensor`` wiring, auto_compute/graph.py:136-203).
    ``outputs`` lists ``(layer index, output index)`` pairs; default: the last layer's outputs."""

    def __init__(self, layers, edges=None, outputs=None):
        self.layers = list(layers)
        self.edges = dict(edges or {})
        for (ci, ii), (pi, oi) in self.edges.items():
            if not (0 <= pi < ci < len(self.layers)):
                raise ValueError("edge (%d,%d)<-(%d,%d): producers must precede consumers" % (ci, ii, pi, oi))
            src = self.layers[pi].ops[oi].output(0)
            dst = self.layers[ci].inputs[ii]
            if tuple(src.shape) != tuple(dst.shape) or src.dtype != dst.dtype:
                raise ValueError("edge (%d,%d)<-(%d,%d): %s %s does not match %s %s"
                                 % (ci, ii, pi, oi, src.shape, src.dtype, dst.shape, dst.dtype))
        self.graph_inputs = [(li, ii) for li, l in enumerate(self.layers) for ii in range(len(l.inputs))
                             if (li, ii) not in self.edges]
        last = len(self.layers) - 1
        self.graph_outputs = list(outputs) if outputs is not None else [(last, i) for i in range(len(self.layers[last].ops))]

    def get_all_layers(self):
        return self.layers


class GraphEngine:
    def __init__(self, graph, built_mods, dev="cuda:0", prepare_weights=True):
        self.graph = graph
        # conv chain layers with weights: repack the weights once per compile (set_weight compiles
        # again) instead of on every run.  Weights changed in place afterwards are noticed through their
        # version counters: the bound function repacks them at its next call, the graph-replay engine
        # records its graph again
        self.prepare_weights = prepare_weights
        self.built_mods = built_mods  # {layer fingerprint: callable f(*inputs, *weights, *outputs)}
        self.dev = torch.device(dev)
        self._init = False
        self._to_exe = []

    # -- buffers ---------------------------------------------------------------------------
    def _random(self, t):
        """Uniform(-10, 10) like the reference's runtime.ndarray.random fill (graph_runtime.cc:76-77)."""
        dt = TORCH_DTYPES[t.dtype]
        if dt in (torch.int8, torch.int32):
            return torch.randint(-10, 11, tuple(t.shape), dtype=dt, device=self.dev)
        return (torch.rand(tuple(t.shape), device=self.dev) * 20.0 - 10.0).to(dt)

    def init(self):
        self.input_buffer, self.weight_buffer, self.output_buffer = {}, {}, {}
        for li, layer in enumerate(self.graph.layers):
            self.output_buffer[li] = [self._random(op.output(0)) for op in layer.ops]
            self.weight_buffer[li] = [self._random(w) for w in layer.weights]
            ins = []
            for ii, t in enumerate(layer.inputs):
                if (li, ii) in self.graph.edges:
                    pi, oi = self.graph.edges[(li, ii)]
                    ins.append(self.output_buffer[pi][oi])
                else:
                    ins.append(self._random(t))
            self.input_buffer[li] = ins
        self._init = True

    def set_inputs(self, inputs):
        if len(inputs) != len(self.graph.graph_inputs):
            raise ValueError("expected %d graph inputs, got %d" % (len(self.graph.graph_inputs), len(inputs)))
        if not self._init:
            self.init()
        for (li, ii), data in zip(self.graph.graph_inputs, inputs):
            want = self.graph.layers[li].inputs[ii]
            if tuple(data.shape) != tuple(want.shape):
                raise ValueError("input for %s has shape %s, expected %s" % (want.name, tuple(data.shape), want.shape))
            self.input_buffer[li][ii] = data
        self._to_exe = []  # bound arguments changed: compile again

    def set_weight(self, layer, tensor, data):
        if not self._init:
            self.init()
        li = next(i for i, l in enumerate(self.graph.layers) if l is layer)
        wi = next(i for i, w in enumerate(layer.weights) if w is tensor)
        self.weight_buffer[li][wi] = data
        self._to_exe = []

    # -- execution -------------------------------------------------------------------------
    def compile(self):
        if not self._init:
            self.init()
        self._to_exe = []
        for li, layer in enumerate(self.graph.layers):
            key = layer.fingerprint
            if key not in self.built_mods:
                raise KeyError("no built function for layer %s" % layer.name)
            func = self.built_mods[key]
            if (self.prepare_weights and len(layer.weights) == 2 and len(layer.inputs) == 1
                    and getattr(getattr(func, "sch", None), "kind", None) == "conv_chain"):
                # fixed weights: repack them once, here, into a workspace this layer owns
                func = func.specialize(*self.weight_buffer[li])
            args = [*self.input_buffer[li], *self.weight_buffer[li], *self.output_buffer[li]]
            self._to_exe.append((func, args))
        self._weight_versions = self._versions()

    def _versions(self):
        return [w._version for li in sorted(self.weight_buffer) for w in self.weight_buffer[li]]

    def run(self):
        if not self._to_exe:
            self.compile()
        for func, args in self._to_exe:
            func(*args)

    def timeit(self, number):
        """Mean milliseconds per run over ``number`` runs after one warm-up (graph_runtime.cc:215-229)."""
        self.run()
        torch.cuda.synchronize(self.dev)
        beg = time.perf_counter()
        for _ in range(number):
            self.run()
        torch.cuda.synchronize(self.dev)
        return (time.perf_counter() - beg) * 1e3 / number

    def get_outputs(self):
        return [self.output_buffer[li][oi] for li, oi in self.graph.graph_outputs]


class HipGraphEngine(GraphEngine):
    """Records the layer sequence into a HIP graph at compile time and replays it on run."""

    def compile(self):
        super().compile()
        self._graph = None
        GraphEngine.run(self)  # warm-up outside the capture (first-call set-up, cached workspaces)
        torch.cuda.synchronize(self.dev)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            GraphEngine.run(self)
        self._graph = g

    def run(self):
        # (a recorded graph holds the repacked weights of compile time: weights updated in place since then
        # need the repacking, and with it the recording, done again)
        if not self._to_exe or getattr(self, "_graph", None) is None or self._versions() != self._weight_versions:
            self.compile()
        self._graph.replay()


def create_graph_engine(graph, built_mods, dev="cuda:0"):
    return GraphEngine(graph, built_mods, dev)


def create_hip_graph_engine(graph, built_mods, dev="cuda:0"):
    return HipGraphEngine(graph, built_mods, dev)


create_cuda_graph_engine = create_hip_graph_engine  # the reference's name for the graph-replay engine
