"""conv3x3 -> conv1x1 chain driver (reference: benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py).
Takes plain NCHW tensors where the reference's driver takes its packed, pre-padded layout."""
from ditto_amd import auto_compute as ac

from . import common

example_text = """
 example:
    python -m ditto_amd.drivers.conv3x3_conv1x1 --in_dtype float16 --acc_dtype float32 --begin 0 --num 1
"""
shapes = common.CONV3X3_CONV1X1_SHAPES
cal_ai = common.conv_cal_ai


def main(batch, in_channel, H, W, out_channel1, out_channel2, stride1=1, stride2=1, in_dtype="float16",
         acc_dtype="float32", sm="gfx950", only_once=False):
    return common.conv_chain_main(ac.nn.functional.Conv3x3Conv1x1, batch, in_channel, H, W, out_channel1, out_channel2,
                                  stride1, stride2, in_dtype, acc_dtype, sm, only_once)


if __name__ == "__main__":
    common.conv_chain_cli(main, shapes, example_text)
