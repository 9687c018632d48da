"""depthwise conv3x3 -> conv1x1 chain driver (reference:
benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py).  Takes plain NCHW tensors and
unpadded 3x3 filters where the reference's driver takes its packed, pre-padded layout."""
from ditto_amd import auto_compute as ac
from ditto_amd import auto_tensorize as at
from ditto_amd import hardware as hw

from . import common

example_text = """
 example:
    python -m ditto_amd.drivers.depthwise3x3_conv1x1 --in_dtype float16 --acc_dtype float32 --begin 0 --num 1
"""
shapes = common.DEPTHWISE3X3_CONV1X1_SHAPES


def cal_ai(batch, C, H, W, K, stride1, stride2, factor):
    pix1 = batch * (H // stride1) * (W // stride1)
    pix2 = batch * (H // stride1 // stride2) * (W // stride1 // stride2)
    return pix1 * factor / (pix1 + factor), pix2 * K / (pix2 + K)


def main(batch, in_channel, H, W, out_channel, factor=16, stride1=1, stride2=1, in_dtype="float16",
         acc_dtype="float32", sm="gfx950", only_once=False):
    try:
        ins, outs = ac.nn.functional.Depthwise3x3Conv1x1(batch, in_channel, H, W, out_channel, factor, stride1,
                                                         stride2, in_dtype, acc_dtype)
        layer = ac.layer([outs[0].op], inputs=[ins[0]], weights=ins[1:])
        sfs = at.build_serial_fusion_state(layer)
        ok, why = at.validate(sfs)
        if not ok:
            raise ValueError(why)
        conv1, conv2 = sfs.first_op, sfs.second_op
        n, k, p, q = conv2.axis
        # the reference fuses [b, m, n, ric] of the second contraction
        # (depthwise3x3_conv1x1_small_channel_cuda.py:207)
        fuse_choice = at.fusion_choice(conv1, conv2, [n, p, q, k] + list(conv2.reduce_axis), 4)
        mfma = at.hip_mfma(32, 32, 16, in_dtype, acc_dtype)
        state = at.tensorize_hyper_fusion_state(layer, fuse_choice, {
            conv1: at.match_info([conv1.axis[3], conv1.axis[1], conv1.reduce_axis[1]], mfma),
            conv2: at.match_info([conv2.axis[3], conv2.axis[1], conv2.reduce_axis[0]], mfma)})
        param = at.cuda_tensorize_param(warp_size=32, ty_size=2, tz_size=2, input_vector_len=8, serial_y=2,
                                        serial_z=2, block_rx=1, warp_rx=2, block_ry=1, warp_ry=2, unroll_steps=64)
        sch = at.tensorize_cuda(layer, state, hw.query_hw_param(common.DEVICES[sm]), param)
    except Exception as error:
        print("chain failed:", type(error).__name__, error)
        return common.SENTINEL_COST
    args = common.random_args(layer, in_dtype, 1)
    args[1] = args[1] * 0.3
    args[2] = args[2] * 0.05
    return common.evaluate(sch, layer, args, only_once)


if __name__ == "__main__":
    parser = common.base_parser(example_text, len(shapes))
    parser.add_argument("--batch", type=int, default=1)
    parser.add_argument("--factor", type=int, default=16)
    args = parser.parse_args()
    if args.ai:
        for ss in shapes[args.begin: args.begin + args.num]:
            print(ss, *cal_ai(args.batch, *ss, args.factor))
    elif common.check_dtypes(args):
        costs = []
        for ss in shapes[args.begin: args.begin + args.num]:
            C, H, W, K, stride1, stride2 = ss
            costs.append((ss, main(args.batch, C, H, W, K, args.factor, stride1, stride2, args.in_dtype,
                                   args.acc_dtype, args.sm, args.only_once)))
        print("batch,C,H,W,K,stride1,stride2,factor,in_dtype,acc_dtype,sm,cost")
        for cc in costs:
            print(f"{args.batch}," + ",".join(map(str, cc[0])) +
                  f",{args.factor},{args.in_dtype},{args.acc_dtype},{args.sm},{cc[1]}")
        for cc in costs:
            print(cc[1])
