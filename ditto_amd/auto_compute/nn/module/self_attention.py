"""Multi-head attention over the fused BMM -> softmax -> BMM chain.

Counterpart of python/ditto/auto_compute/nn/module/self_attention.py:15-82.  The reference
splits the packed ``[batch, M, 3 * hidden]`` projection into query / key / value, then
reshapes and transposes each into ``[batch * heads, M, d]`` (key into ``[batch * heads, d, M]``)
before the chain and merges the heads back afterwards (:47-57, :71-73) -- five layout ops that
each copy the tensor.  Here those ops are *views*: the chain kernel walks the two batch levels
(batch, head) by stride, reads query / key / value where the projection left them and writes
every head straight into its columns of the ``[batch, M, hidden]`` output.
"""
import torch

from .... import chain, te
from ...graph import Layer

MUTI_HEAD_ATTENTION_LAYER = "multi_head_attention_mma_layer"  # the reference's dispatch key (:7)
SELF_ATTENTION_MODULE_REG = set([MUTI_HEAD_ATTENTION_LAYER])


def is_self_attention_layer(layer):
    return layer.name in SELF_ATTENTION_MODULE_REG


class MultiHeadAttentionMMA:
    """MultiHead Attention with MMA fusion (same constructor arguments as the reference, plus
    ``scale``: the reference applies none, i.e. 1.0; pass ``None`` for 1/sqrt(head_dim))."""

    name = MUTI_HEAD_ATTENTION_LAYER

    def __init__(self, num_heads, hidden_size, in_dtype="float32", acc_dtype="float32", mma_MI=16, mma_NI=16,
                 mma_KI=16, scale=1.0):
        assert hidden_size % num_heads == 0
        self.num_heads = num_heads
        self.hidden_size = hidden_size
        self.model_k = hidden_size // num_heads
        self.in_dtype = in_dtype
        self.acc_dtype = acc_dtype
        self.MI, self.NI, self.KI = mma_MI, mma_NI, mma_KI
        self.scale = float(scale) if scale is not None else self.model_k ** -0.5

    def head_views(self, query_key_value):
        """query [batch, heads, M, d], key [batch, heads, d, M], value [batch, heads, M, d] as
        views of the packed projection (what :47-57 materialise with reshape + transpose)."""
        batch, M, Kx3 = query_key_value.shape
        if Kx3 != 3 * self.hidden_size:
            raise RuntimeError("Can't prove the self attention inputs conform to the hidden size.")
        query, key, value = query_key_value.split(self.hidden_size, dim=-1)
        shape = (batch, M, self.num_heads, self.model_k)
        return (query.view(shape).permute(0, 2, 1, 3), key.view(shape).permute(0, 2, 3, 1),
                value.view(shape).permute(0, 2, 1, 3))

    def layer(self, batch, M):
        """The attention block as a ``Layer`` named ``multi_head_attention_mma_layer`` (the name
        ``is_self_attention_layer`` / ``chimera.task_binding`` dispatch on, :7-12): one input, the
        packed ``[batch, M, 3 * hidden]`` projection, one output ``[batch, M, hidden]``.  The head
        split / merge of :47-57, :71-73 is part of the op (``kind = "mha"``) rather than separate
        layout ops, because the kernel does it by addressing."""
        qkv = te.placeholder([batch, M, 3 * self.hidden_size], name="query_key_value", dtype=self.in_dtype)
        out = te.compute(
            [batch, M, self.hidden_size], "multi_head_attention", self.in_dtype, "mha",
            lambda b, m, c: [(qkv, [b, m, c])], axis_names=["b", "m", "c"],
            attrs={"num_heads": self.num_heads, "head_dim": self.model_k, "scale": self.scale,
                   "acc_dtype": self.acc_dtype, "mma": (self.MI, self.NI, self.KI)},
        )
        return Layer(self.name, [out.op], [qkv], [], [], [])

    def __call__(self, query_key_value, out=None):
        return self.forward(query_key_value, out)

    def forward(self, query_key_value, out=None, tile_variant=0):
        """query_key_value: [batch, M, 3 * hidden] (query | key | value along the last axis).
        Returns [batch, M, hidden]; ``out`` may be given (destination passing)."""
        q, k, v = self.head_views(query_key_value)
        batch, M = query_key_value.shape[0], query_key_value.shape[1]
        if out is None:
            out = torch.empty(batch, M, self.hidden_size, dtype=query_key_value.dtype, device=query_key_value.device)
        o = out.view(batch, M, self.num_heads, self.model_k).permute(0, 2, 1, 3)
        chain.run_bmm_chain(q, k, v, o, "softmax", self.scale, tile_variant=tile_variant)
        return out

    __call__ = forward
