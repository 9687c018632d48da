"""GEMM -> GEMM chain driver (reference: benchmark/chimera/cuda/bmm_bmm_cuda.py)."""
from ditto_amd import auto_compute as ac

from . import common

example_text = """
 example:
    python -m ditto_amd.drivers.bmm_bmm --in_dtype float16 --acc_dtype float32 --begin 0 --num 1
"""
shapes = common.BMM_SHAPES


def main(batch=12, M=512, N=64, K=64, L=512, in_dtype="float16", acc_dtype="float32", sm="gfx950",
         only_once=False, requant=False):
    # int8 / int32: the reference's chain as it stands (the middle result and F wrap with astype("int8"),
    # bmm_bmm_cuda.py:116, :147), or with ``requant`` the middle result requantised (scale 2^-10, round to nearest
    # even, saturate) and F left in int32
    requant = common.INT8_REQUANT_SCALE if in_dtype == "int8" and requant else None
    ins, outs = ac.nn.functional.BatchGemmGemm(batch=batch, M=M, N=N, K=K, L=L, in_dtype=in_dtype,
                                               acc_dtype=acc_dtype, requant_scale=requant)
    try:
        layer, sch = common.describe_bmm_chain(ins, outs, in_dtype, acc_dtype, sm)
    except Exception as error:
        print("chain failed:", type(error).__name__, error)
        return common.SENTINEL_COST
    args = common.random_args(layer, in_dtype, 3, scale=0.25)
    return common.evaluate(sch, layer, args, only_once)


if __name__ == "__main__":
    parser = common.base_parser(example_text, len(shapes))
    parser.add_argument("--requant", action="store_true",
                        help="int8: requantise the middle result instead of the reference's wrapping cast")
    args = parser.parse_args()
    if args.ai:
        for ss in shapes[args.begin: args.begin + args.num]:
            print(ss, *common.cal_ai(*ss))
    elif common.check_dtypes(args, int8_ok=True):
        costs = []
        for ss in shapes[args.begin: args.begin + args.num]:
            B, M, N, K, L = ss
            costs.append((ss, main(B, M, N, K, L, args.in_dtype, args.acc_dtype, args.sm, args.only_once, args.requant)))
        print("B,M,N,K,L,in_dtype,acc_dtype,sm,cost")
        for cc in costs:
            print(f"{cc[0][0]},{cc[0][1]},{cc[0][2]},{cc[0][3]},{cc[0][4]},{args.in_dtype},{args.acc_dtype},"
                  f"{args.sm},{cc[1]}")
        for cc in costs:
            print(cc[1])
