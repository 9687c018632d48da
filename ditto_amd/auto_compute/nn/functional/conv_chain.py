"""Builders of the conv -> conv chains on plain NCHW tensors.

Op names and the 14-number shape convention ``(N, C0, P0, Q0, C1, R1, S1, C2, R2, S2, padding1,
padding2, stride1, stride2)`` follow ``conv_relu_conv`` of
python_test/auto_tensorize/test_hyper_fusion.py:51-192 (pad1, conv1, relu, pad2, conv2);
``Conv3x3Conv1x1`` has the argument list of benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:77-172
but takes / returns plain NCHW tensors rather than the reference's pre-padded 16-channel
packed layouts.
"""
from .... import te


def conv_chain(N, C0, P0, Q0, C1, R1, S1, C2, R2, S2, padding1=0, padding2=0, stride1=1, stride2=1,
               in_dtype="float16", acc_dtype="float32", relu=False, relu_out=False, groups1=1):
    """conv(R1xS1) -> cast | relu -> conv(R2xS2); returns ``([Img, Weight1, Weight2], [Conv2])``.
    ``groups1 = C0`` makes the first convolution depthwise (C1 / C0 outputs per input channel)."""
    assert groups1 in (1, C0) and C1 % groups1 == 0, "groups1 must be 1 or C0, and divide C1"
    P1 = (P0 + 2 * padding1 - R1) // stride1 + 1
    Q1 = (Q0 + 2 * padding1 - S1) // stride1 + 1
    P2 = (P1 + 2 * padding2 - R2) // stride2 + 1
    Q2 = (Q1 + 2 * padding2 - S2) // stride2 + 1
    assert P1 > 0 and Q1 > 0 and P2 > 0 and Q2 > 0, "empty convolution output"
    Img = te.placeholder([N, C0, P0, Q0], dtype=in_dtype, name="Img")
    Weight1 = te.placeholder([C1, C0 // groups1, R1, S1], dtype=in_dtype, name="Weight1")
    Weight2 = te.placeholder([C2, C1, R2, S2], dtype=in_dtype, name="Weight2")
    Pad1 = te.compute(
        [N, C0, P0 + 2 * padding1, Q0 + 2 * padding1], "pad1", in_dtype, "pad",
        lambda n, c, p, q: [(Img, [n, c, p, q])], axis_names=["n", "c", "p", "q"],
        attrs={"padding": padding1, "pad_value": 0},
    )
    r1 = te.reduce_axis((0, R1), "rr1")
    s1 = te.reduce_axis((0, S1), "rs1")
    c1 = te.reduce_axis((0, C0 // groups1), "rc1")
    Conv1 = te.compute(
        [N, C1, P1, Q1], "conv1", acc_dtype, "contract",
        lambda n, k, p, q: [(Pad1, [n, c1, p, r1, q, s1]), (Weight1, [k, c1, r1, s1])],
        axis_names=["n", "k", "p", "q"], reduce_axes=[c1, r1, s1],
        attrs={"conv": True, "stride": stride1, "padding": padding1, "R": R1, "S": S1, "groups": groups1},
        # nine taps do not make a substantial reduction on their own; the tag marks the op as a
        # contraction the way the reference's pattern check honours tags (pattern.cc:13-100)
        tag="PATTERN_CUBIC" if groups1 > 1 else "",
    )
    inter = te.compute(
        [N, C1, P1, Q1], "relu" if relu else "cast", in_dtype, "relu" if relu else "cast",
        lambda n, c, p, q: [(Conv1, [n, c, p, q])], axis_names=["n", "c", "p", "q"],
    )
    Pad2 = te.compute(
        [N, C1, P1 + 2 * padding2, Q1 + 2 * padding2], "pad2", in_dtype, "pad",
        lambda n, c, p, q: [(inter, [n, c, p, q])], axis_names=["n", "c", "p", "q"],
        attrs={"padding": padding2, "pad_value": 0},
    )
    r2 = te.reduce_axis((0, R2), "rr2")
    s2 = te.reduce_axis((0, S2), "rs2")
    c2 = te.reduce_axis((0, C1), "rc2")
    Conv2_acc = te.compute(
        [N, C2, P2, Q2], "conv2_fact", acc_dtype, "contract",
        lambda n, k, p, q: [(Pad2, [n, c2, p, r2, q, s2]), (Weight2, [k, c2, r2, s2])],
        axis_names=["n", "k", "p", "q"], reduce_axes=[c2, r2, s2],
        attrs={"conv": True, "stride": stride2, "padding": padding2, "R": R2, "S": S2},
    )
    Conv2 = te.compute(
        [N, C2, P2, Q2], "conv2", in_dtype, "relu_cast" if relu_out else "unpack_cast",
        lambda n, c, p, q: [(Conv2_acc, [n, c, p, q])], axis_names=["n", "c", "p", "q"],
    )
    return [Img, Weight1, Weight2], [Conv2]


def conv_relu_conv(N, C0, P0, Q0, C1, R1, S1, C2, R2, S2, padding1=0, padding2=0, stride1=1, stride2=1,
                   in_dtype="float16", acc_dtype="float32"):
    """The reference's test chain: ReLU between the convolutions (test_hyper_fusion.py:51-192)."""
    return conv_chain(N, C0, P0, Q0, C1, R1, S1, C2, R2, S2, padding1, padding2, stride1, stride2, in_dtype,
                      acc_dtype, relu=True)


def Conv3x3Conv1x1(batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1,
                   in_dtype="float16", acc_dtype="float32"):
    """conv3x3 (pad 1) -> cast -> conv1x1; argument list of conv3x3_conv1x1_cuda.py:77-88."""
    assert stride2 == 1
    return conv_chain(batch, in_channel, H, W, out_channel1, 3, 3, out_channel2, 1, 1, 1, 0, stride1, stride2,
                      in_dtype, acc_dtype)


def Conv1x1Conv1x1(batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1,
                   in_dtype="float16", acc_dtype="float32", relu=False):
    """conv1x1 -> cast | relu -> conv1x1; argument list of benchmark/chimera/cuda/conv1x1_conv1x1_cuda.py:77-88
    (``relu=True``: conv1x1_relu_conv1x1.py, the ReLU on the first accumulator, :146-153 of its 3x3 sibling)."""
    assert stride2 == 1
    return conv_chain(batch, in_channel, H, W, out_channel1, 1, 1, out_channel2, 1, 1, 0, 0, stride1, stride2,
                      in_dtype, acc_dtype, relu=relu)


def Conv3x3ReluConv1x1(batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1,
                       in_dtype="float16", acc_dtype="float32"):
    """conv3x3 (pad 1) -> relu -> conv1x1 (benchmark/chimera/cuda/conv3x3_relu_conv1x1.py:77-172)."""
    assert stride2 == 1
    return conv_chain(batch, in_channel, H, W, out_channel1, 3, 3, out_channel2, 1, 1, 1, 0, stride1, stride2,
                      in_dtype, acc_dtype, relu=True)


def Conv1x1ReluConv3x3(batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1,
                       in_dtype="float16", acc_dtype="float32"):
    """conv1x1 -> relu -> conv3x3 (pad 1) (benchmark/chimera/cuda/conv1x1_relu_conv3x3_cuda.py:77-200)."""
    assert stride2 == 1
    return conv_chain(batch, in_channel, H, W, out_channel1, 1, 1, out_channel2, 3, 3, 0, 1, stride1, stride2,
                      in_dtype, acc_dtype, relu=True)


def Conv1x1Conv3x3(batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1,
                   in_dtype="float16", acc_dtype="float32"):
    """conv1x1 -> cast -> conv3x3 (pad 1, zero padding of the intermediate); argument list of
    benchmark/chimera/cuda/conv1x1_conv3x3_cuda.py:77-88."""
    assert stride2 == 1
    return conv_chain(batch, in_channel, H, W, out_channel1, 1, 1, out_channel2, 3, 3, 0, 1, stride1, stride2,
                      in_dtype, acc_dtype)


def Depthwise3x3Conv1x1(batch, in_channel, H, W, out_channel, factor=16, stride1=1, stride2=1,
                        in_dtype="float16", acc_dtype="float32"):
    """depthwise conv3x3 (pad 1, ``factor`` outputs per input channel) -> cast -> conv1x1; argument
    list of benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py:77-88.  Weights are
    plain ``[in_channel * factor, 1, 3, 3]`` and ``[out_channel, in_channel * factor, 1, 1]``: the
    reference pads the nine taps to a 16-deep tensor-core step, the gfx950 kernel runs them on the
    vector ALU and needs no padding."""
    assert stride2 == 1
    return conv_chain(batch, in_channel, H, W, in_channel * factor, 3, 3, out_channel, 1, 1, 1, 0, stride1,
                      stride2, in_dtype, acc_dtype, groups1=in_channel)
