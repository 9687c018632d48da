"""The per-chain drivers keep the reference's flags, shape tables, CSV header and cost unit
(benchmark/chimera/cuda/bmm_bmm_cuda.py:304-397, conv3x3_conv1x1_cuda.py:331-337)."""
import subprocess
import sys

import pytest

from ditto_amd.drivers import (bmm_bmm, bmm_softmax_bmm, common, conv1x1_conv1x1, conv1x1_conv3x3,
                               conv1x1_relu_conv1x1, conv1x1_relu_conv3x3, conv3x3_conv1x1, conv3x3_relu_conv1x1,
                               depthwise3x3_conv1x1)


def test_shape_tables_match_reference():
    assert len(common.BMM_SHAPES) == 12
    assert common.BMM_SHAPES[1] == (12, 512, 64, 64, 512)      # Bert-Base
    assert common.BMM_SHAPES[6] == (12, 208, 64, 64, 208)      # ViT-Base/16: uround(196, 16)
    assert common.BMM_SHAPES[9] == (1, 512, 64, 64, 256)       # Mixer-Small/32-S: uround(49, 16)
    assert common.CONV3X3_CONV1X1_SHAPES[2] == (64, 56, 56, 128, 64, 1, 1)
    assert common.DEPTHWISE3X3_CONV1X1_SHAPES[3] == (16, 224, 224, 32, 2, 1)
    assert conv1x1_conv1x1.shapes == conv1x1_relu_conv1x1.shapes == [(64, 56, 56, 64, 64, 1, 1), (256, 56, 56, 256, 64, 1, 1)]
    assert conv3x3_relu_conv1x1.shapes is common.CONV3X3_CONV1X1_SHAPES
    assert conv1x1_relu_conv3x3.shapes == [(64, 56, 56, 64, 64, 1, 1)]
    assert common.cal_ai(12, 512, 64, 64, 512) == (256.0, 512 * 64 / 576)


def test_cli_ai_and_unsupported_dtype():
    out = subprocess.run([sys.executable, "-m", "ditto_amd.drivers.bmm_bmm", "--ai", "--begin", "1", "--num", "1"],
                         capture_output=True, text=True, check=True).stdout
    assert out.strip() == "(12, 512, 64, 64, 512) 256.0 56.888888888888886"
    out = subprocess.run([sys.executable, "-m", "ditto_amd.drivers.bmm_softmax_bmm", "--in_dtype", "float64",
                          "--acc_dtype", "float32", "--num", "1"], capture_output=True, text=True, check=True).stdout
    assert "Data type not supported" in out and "cost" not in out


def test_descriptor_failure_gives_sentinel_cost():
    # N not a multiple of 16: the builder's assert is turned into the sentinel cost, not an exception
    # (the reference swallows failures of its measurement worker the same way, bmm_bmm_cuda.py:58-64)
    assert conv3x3_conv1x1.main(1, 16, 8, 8, 12, 16) == common.SENTINEL_COST


@pytest.mark.gpu
def test_drivers_run_one_row_each(capsys):
    assert bmm_bmm.main(*common.BMM_SHAPES[9], only_once=True) == -1
    cost = bmm_softmax_bmm.main(*common.BMM_SHAPES[3])
    assert 0 < cost < 5.0  # milliseconds
    C, H, W, K1, K2, s1, s2 = common.CONV3X3_CONV1X1_SHAPES[2]
    cost = conv3x3_conv1x1.main(1, C, H, W, K1, K2, s1, s2)
    assert 0 < cost < 5.0
    C, H, W, K1, K2, s1, s2 = common.CONV1X1_CONV3X3_SHAPES[0]
    cost = conv1x1_conv3x3.main(1, C, H, W, K1, K2, s1, s2)
    assert 0 < cost < 5.0
    # the sibling drivers of the conv chains (ReLU between the convolutions; conv1x1 -> conv1x1)
    for drv in (conv1x1_conv1x1, conv1x1_relu_conv1x1, conv3x3_relu_conv1x1, conv1x1_relu_conv3x3):
        C, H, W, K1, K2, s1, s2 = drv.shapes[-1 if drv is conv1x1_relu_conv3x3 else 0]
        if drv is conv3x3_relu_conv1x1:
            C, H, W, K1, K2, s1, s2 = drv.shapes[2]
        cost = drv.main(1, C, H, W, K1, K2, s1, s2)
        assert 0 < cost < 5.0, drv.__name__
    for C, H, W, K, s1, s2 in common.DEPTHWISE3X3_CONV1X1_SHAPES:
        cost = depthwise3x3_conv1x1.main(1, C, H, W, K, 16, s1, s2)
        assert 0 < cost < 5.0


@pytest.mark.gpu
def test_int8_driver_row():
    # the ("80", "int8", "int32") combination of bmm_bmm_cuda.py:273-288 (GEMM chain only)
    cost = bmm_bmm.main(*common.BMM_SHAPES[1], in_dtype="int8", acc_dtype="int32")  # the reference's wrapping chain
    assert 0 < cost < 5.0
    cost = bmm_bmm.main(*common.BMM_SHAPES[1], in_dtype="int8", acc_dtype="int32", requant=True)
    assert 0 < cost < 5.0
    out = subprocess.run([sys.executable, "-m", "ditto_amd.drivers.bmm_bmm", "--in_dtype", "int8", "--acc_dtype",
                          "int32", "--begin", "9", "--num", "1", "--only_once"], capture_output=True, text=True,
                         check=True).stdout.strip().splitlines()
    assert out[-2] == "1,512,64,64,256,int8,int32,gfx950,-1"
    out = subprocess.run([sys.executable, "-m", "ditto_amd.drivers.bmm_softmax_bmm", "--in_dtype", "int8",
                          "--acc_dtype", "int32", "--num", "1"], capture_output=True, text=True, check=True).stdout
    assert "Data type not supported" in out  # no int8 softmax chain


@pytest.mark.gpu
def test_cli_csv_format():
    out = subprocess.run([sys.executable, "-m", "ditto_amd.drivers.bmm_softmax_bmm", "--begin", "3", "--num", "1",
                          "--only_once"], capture_output=True, text=True, check=True).stdout.strip().splitlines()
    assert out[-2] == "B,M,N,K,L,in_dtype,acc_dtype,sm,cost"
    assert out[-1] == "12,256,64,64,256,float16,float32,gfx950,-1"
