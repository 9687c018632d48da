"""Shared pieces of the chain drivers.

Protocol of the reference drivers (benchmark/chimera/cuda/bmm_bmm_cuda.py:152-270, 328-397):
one chain per shape row is described, scheduled and built; with ``--only_once`` it is called a
single time untimed (for profilers) and the cost is -1; otherwise the mean time per call is taken
with ``time_evaluator(min_repeat_ms=600)`` and printed in **milliseconds**; a failing
build / run yields the sentinel cost 1e10 instead of an exception (:45-66).
"""
import argparse

import ditto_amd as ditto
from ditto_amd import auto_compute as ac
from ditto_amd import auto_tensorize as at
from ditto_amd import hardware as hw

SENTINEL_COST = 1e10

# sm flag of the reference -> hardware table key; "gfx950" is this build's device
DEVICES = {"70": "gpu.cuda.V100", "80": "gpu.cuda.A100", "86": "gpu.cuda.RTX3090", "gfx950": "gpu.hip.MI355X"}


def ceil(x, y):
    return (x + y - 1) // y


def uround(x, y):
    return int(ceil(x, y) * y)


# (batch, M, N, K, L): bmm_bmm_cuda.py:304-321 / bmm_softmax_bmm_cuda.py:289-303
BMM_SHAPES = [
    (8, 512, 512 // 8, 512 // 8, 512),  # Bert-Small
    (12, 512, 768 // 12, 768 // 12, 512),  # Bert-Base
    (16, 512, 1024 // 16, 1024 // 16, 512),  # Bert-Large
    (12, 256, 768 // 12, 768 // 12, 256),  # ViT-Base/14
    (16, 256, 1024 // 16, 1024 // 16, 256),  # ViT-Large/14
    (16, 256, 1280 // 16, 1280 // 16, 256),  # ViT-Huge/14
    (12, uround(196, 16), 768 // 12, 768 // 12, uround(196, 16)),  # ViT-Base/16
    (16, uround(196, 16), 1024 // 16, 1024 // 16, uround(196, 16)),  # ViT-Large/16
    (16, uround(196, 16), 1280 // 16, 1280 // 16, uround(196, 16)),  # ViT-Huge/16
    (1, 512, uround(49, 16), uround(49, 16), 256),  # Mixer-Small/32-S
    (1, 768, uround(49, 16), uround(49, 16), 384),  # Mixer-Base/32-S
    (1, 1024, uround(49, 16), uround(49, 16), 512),  # Mixer-Large/32-S
]

# (C, H, W, K1, K2, stride1, stride2): conv3x3_conv1x1_cuda.py:331-337
CONV3X3_CONV1X1_SHAPES = [
    (64, 112, 112, 192, 128, 2, 1),  # Yolo
    (32, 147, 147, 64, 80, 2, 1),  # Inception-V3
    (64, 56, 56, 128, 64, 1, 1),  # Darknet-19
    (128, 28, 28, 256, 128, 1, 1),  # Darknet-19
    (16, 227, 227, 64, 16, 4, 1),  # Squeezenet-V1.1
]
# (C, H, W, K1, K2, stride1, stride2): conv1x1_conv3x3_cuda.py:348-350
CONV1X1_CONV3X3_SHAPES = [
    (64, 56, 56, 64, 64, 1, 1),  # ResNet-50
]
# (C, H, W, K1, K2, stride1, stride2): conv1x1_conv1x1_cuda.py:315-318 (and conv1x1_relu_conv1x1.py:326-329)
CONV1X1_CONV1X1_SHAPES = [
    (64, 56, 56, 64, 64, 1, 1),  # modified ResNet-50
    (256, 56, 56, 256, 64, 1, 1),  # modified ResNet-50
]
# (C, H, W, K, stride1, stride2): depthwise3x3_conv1x1_small_channel_cuda.py:340-346
DEPTHWISE3X3_CONV1X1_SHAPES = [
    (32, 112, 112, 64, 1, 1),  # mobilenet-v1
    (32, 56, 56, 64, 1, 1),
    (64, 112, 112, 64, 1, 1),
    (16, 224, 224, 32, 2, 1),
]


def cal_ai(B, M, N, K, L):
    """Arithmetic intensity of the two GEMMs as the reference prints it (bmm_bmm_cuda.py:324-325)."""
    return (M * L / (M + L)), (M * N / (M + N))


def describe_bmm_chain(ins, outs, in_dtype, acc_dtype, sm):
    """Steps 2-8 of the reference driver: fusion choice, intrinsic match, layer, hyper-fusion
    state, hardware table, tensorize parameters, tensorize."""
    A, B, C = ins[:3]  # (a requantised int8 chain may carry a fourth input, the scale vector)
    (F,) = outs
    E_frag = F.op.input_tensors[0]
    mid, C_ext = E_frag.op.input_tensors
    D_frag = mid.op.input_tensors[0]
    b, m, n, mi, ni = E_frag.op.axis
    rlo, rli = E_frag.op.reduce_axis
    fuse_choice = at.fusion_choice(D_frag.op, E_frag.op, [b, m, n, rlo, mi, ni, rli], 3)
    first_packed = at.cuda_wmma(M=16, N=16, K=16, in_dtype=in_dtype, out_dtype=acc_dtype, scope="shared")
    first_match_info = at.match_info(at.intrinsic_match(D_frag, first_packed, ["InnerMost", "SameRange"])[0],
                                     first_packed)
    second_packed = at.cuda_wmma(M=16, N=16, K=16, in_dtype=in_dtype, out_dtype=acc_dtype, scope="global")
    second_match_info = at.match_info(at.intrinsic_match(E_frag, second_packed, ["InnerMost", "SameRange"])[0],
                                      second_packed)
    layer = ac.layer([F.op], inputs=list(ins))
    state = at.tensorize_hyper_fusion_state(layer, fuse_choice,
                                            {D_frag.op: first_match_info, E_frag.op: second_match_info})
    device = hw.query_hw_param(DEVICES[sm])
    N = int(C.shape[2])
    if N > 64:  # the reference's two parameter sets (bmm_bmm_cuda.py:222-243)
        param = at.cuda_tensorize_param(warp_size=32, ty_size=4, tz_size=2, input_vector_len=4, serial_y=2,
                                        serial_z=1, block_rx=8, warp_rx=4, block_ry=1, warp_ry=4, unroll_steps=512)
    else:
        param = at.cuda_tensorize_param(warp_size=32, ty_size=2, tz_size=2, input_vector_len=8, serial_y=2,
                                        serial_z=1, block_rx=8, warp_rx=8, block_ry=4, warp_ry=4, unroll_steps=64)
    sch = at.tensorize_cuda(layer, state, device, param)
    return layer, sch


def describe_layer(layer, sm="gfx950", tile_variant=0):
    """Any chain layer (GEMM or conv chain, e.g. one ``chimera.graph_fusion`` produced) -> its schedule, by the
    flow of python_test/auto_tensorize/test_hyper_fusion.py:833-880: serial fusion state, validate, intrinsic
    match, ``register_tensorize_axes``, ``build_fusion_choice``, hyper-fusion state, tensorize."""
    sfs = at.build_serial_fusion_state(layer)
    ok, why = at.validate(sfs)
    if not ok:
        raise ValueError(why)
    op1, op2 = sfs.first_op, sfs.second_op
    in_dtype, acc_dtype = layer.inputs[0].dtype, op1.output(0).dtype
    if op1.attrs.get("conv"):
        mfma = at.hip_mfma(32, 32, 32 if in_dtype == "int8" else 16, in_dtype, acc_dtype)
        # pixel x output channel x input channel
        infos = {op: at.match_info([op.axis[3], op.axis[1], op.reduce_axis[0]], mfma) for op in (op1, op2)}
    else:
        infos = {}
        for op, scope in ((op1, "shared"), (op2, "global")):
            packed = at.cuda_wmma(M=16, N=16, K=16, in_dtype=in_dtype, out_dtype=acc_dtype, scope=scope)
            infos[op] = at.match_info(at.intrinsic_match(op.output(0), packed, ["InnerMost", "SameRange"])[0], packed)
    sfs.register_tensorize_axes([iv for mi in infos.values() for iv in mi.axis])
    device = hw.query_hw_param(DEVICES[sm])
    fuse_choice = at.build_fusion_choice(sfs, hw_param=device, dtype=acc_dtype, simple_mode=-1)
    state = at.tensorize_hyper_fusion_state(layer, fuse_choice, infos)
    return at.tensorize_hip(layer, state, device, at.cuda_tensorize_param(), tile_variant=tile_variant)


def random_args(layer, in_dtype, n_inputs, scale=1.0, device="cuda:0"):
    """uniform(-1, 1) tensors for every schedule tensor, as the reference drivers create them."""
    import torch

    dts = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32, "float64": torch.float64,
           "int8": torch.int8, "int32": torch.int32}
    args = []
    for i, t in enumerate(layer.schedule_tensors):
        dt = dts[t.dtype]
        if dt == torch.int8:  # uniform integers in [-127, 127]
            args.append(torch.randint(-127, 128, tuple(t.shape), dtype=torch.int8, device=device))
            continue
        if dt == torch.int32:
            args.append(torch.zeros(tuple(t.shape), dtype=torch.int32, device=device))
            continue
        x = (torch.rand(*t.shape, device=device) * 2 - 1)
        if i < n_inputs:
            x = x * scale
        args.append(x.to(dt))
    return args


def evaluate(sch, layer, args, only_once):
    """Build and run; cost in ms, -1 for ``--only_once``, 1e10 if anything fails."""
    import torch

    try:
        func = ditto.build(sch, layer.schedule_tensors, "hip")
        if only_once:
            func(*args)
            torch.cuda.synchronize()
            return -1
        evaluator = func.time_evaluator(func.entry_name, None, min_repeat_ms=600)
        return evaluator(*args).mean * 1e3
    except Exception as error:  # the reference swallows build / run failures the same way
        print("chain failed:", type(error).__name__, error)
        return SENTINEL_COST


def base_parser(example, n_shapes, with_ai=True):
    parser = argparse.ArgumentParser(prog="base_maker", description="template maker", epilog=example,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--only_once", action="store_true")
    parser.add_argument("--in_dtype", type=str, choices=["float16", "bfloat16", "float64", "int8"],
                        default="float16")
    parser.add_argument("--acc_dtype", type=str, choices=["float16", "float32", "float64", "int32"],
                        default="float32")
    parser.add_argument("--begin", type=int, choices=list(range(n_shapes)), default=0)
    parser.add_argument("--num", type=int, choices=list(range(1, n_shapes + 1)), default=n_shapes)
    parser.add_argument("--sm", type=str, choices=sorted(DEVICES), default="gfx950")
    if with_ai:
        parser.add_argument("--ai", action="store_true")
    return parser


# (sm, in_dtype, acc_dtype) combinations with a kernel on this device
# (the int8 / int32 row is the reference's ("80", "int8", "int32"), bmm_bmm_cuda.py:273-288; GEMM chain only)
# (float16 / float16, the reference's ("80" | "86", "float16", "float16") rows: the kernels accumulate in the MFMA's
# fp32 accumulator whatever is asked for, the precision of that row and more)
# (float64 / float64: the plain-FMA kernel on doubles, head dimensions up to 128)
SUPPORTED_DTYPES = {("gfx950", "float16", "float32"), ("gfx950", "float16", "float16"), ("gfx950", "bfloat16", "float32"),
                    ("gfx950", "float64", "float64"), ("gfx950", "int8", "int32")}
# the requantisation scale the int8 driver rows use for the middle result (2^-10 for every column)
INT8_REQUANT_SCALE = 2.0 ** -10


def check_dtypes(args, int8_ok=False):
    ok = (args.sm, args.in_dtype, args.acc_dtype) in SUPPORTED_DTYPES and (int8_ok or args.in_dtype != "int8")
    if not ok:
        print(f"Data type not supported: sm_{args.sm}, in_dtype={args.in_dtype}, out_dtype={args.acc_dtype}.")
    return ok


def conv_cal_ai(batch, C, H, W, K1, K2, stride1, stride2):
    """Arithmetic intensity of the two convolutions as the reference's conv drivers print it (--ai)."""
    return (batch * (H // stride1) * (W // stride1) * K1 / (batch * (H // stride1) * (W // stride1) + K1),
            batch * (H // stride1 // stride2) * (W // stride1 // stride2) * K2
            / (batch * (H // stride1 // stride2) * (W // stride1 // stride2) + K2))


def conv_chain_main(builder, batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1,
                    in_dtype="float16", acc_dtype="float32", sm="gfx950", only_once=False):
    """``main`` of a conv -> conv driver: describe the chain the way the reference's drivers do (serial fusion state,
    the [b, no, p, mo] fusion of the second convolution, one matrix intrinsic per convolution, the tensorize
    parameters of conv3x3_conv1x1_cuda.py:266-278), build it and measure; failures give the sentinel cost."""
    from ditto_amd import auto_compute as ac
    from ditto_amd import auto_tensorize as at
    from ditto_amd import hardware as hw

    try:
        ins, outs = builder(batch, in_channel, H, W, out_channel1, out_channel2, stride1, stride2, in_dtype, acc_dtype)
        layer = ac.layer([outs[0].op], inputs=[ins[0]], weights=ins[1:])
        sfs = at.build_serial_fusion_state(layer)
        ok, why = at.validate(sfs)
        if not ok:
            raise ValueError(why)
        conv1, conv2 = sfs.first_op, sfs.second_op
        n, k, p, q = conv2.axis
        fuse_choice = at.fusion_choice(conv1, conv2, [n, p, q, k] + list(conv2.reduce_axis), 2)
        mfma = at.hip_mfma(32, 32, 16, in_dtype, acc_dtype)
        state = at.tensorize_hyper_fusion_state(layer, fuse_choice, {
            conv1: at.match_info([conv1.axis[3], conv1.axis[1], conv1.reduce_axis[0]], mfma),
            conv2: at.match_info([conv2.axis[3], conv2.axis[1], conv2.reduce_axis[0]], mfma)})
        param = at.cuda_tensorize_param(warp_size=32, ty_size=2, tz_size=2, input_vector_len=8, serial_y=2,
                                        serial_z=2, block_rx=1, warp_rx=2, block_ry=1, warp_ry=2, unroll_steps=64)
        sch = at.tensorize_cuda(layer, state, hw.query_hw_param(DEVICES[sm]), param)
    except Exception as error:
        print("chain failed:", type(error).__name__, error)
        return SENTINEL_COST
    args = random_args(layer, in_dtype, 1)
    args[1] = args[1] * 0.05
    args[2] = args[2] * 0.05
    return evaluate(sch, layer, args, only_once)


def conv_chain_cli(main, shapes, example_text):
    """The command line the reference's conv drivers share: --batch, --begin / --num over the shape table, --ai,
    the CSV with one cost (ms) per row."""
    parser = base_parser(example_text, len(shapes))
    parser.add_argument("--batch", type=int, default=1)
    args = parser.parse_args()
    if args.ai:
        for ss in shapes[args.begin: args.begin + args.num]:
            print(ss, *conv_cal_ai(args.batch, *ss))
    elif check_dtypes(args):
        costs = []
        for ss in shapes[args.begin: args.begin + args.num]:
            C, H, W, K1, K2, stride1, stride2 = ss
            costs.append((ss, main(args.batch, C, H, W, K1, K2, stride1, stride2, args.in_dtype, args.acc_dtype,
                                   args.sm, args.only_once)))
        print("batch,C,H,W,K1,K2,stride1,stride2,in_dtype,acc_dtype,sm,cost")
        for cc in costs:
            print(f"{args.batch}," + ",".join(map(str, cc[0])) + f",{args.in_dtype},{args.acc_dtype},{args.sm},{cc[1]}")
        for cc in costs:
            print(cc[1])
