"""The C-ABI library loads and exports every symbol the header declares; descriptor
validation and tile choice work without a GPU (no compute is launched here)."""
import ctypes
import os
import re

import pytest

from ditto_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ditto_chain.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ditto_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = declared_functions()
    assert "ditto_bmm_chain_run" in names and "ditto_conv_chain_run" in names
    assert len(names) >= 8


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), "libditto_chain.so does not export %s" % name
    bound = {n for n, _, _ in _lib.EXPORTS}
    assert bound == set(declared_functions()), "ctypes binding and header disagree"
    assert lib.ditto_chain_abi_version() == _lib.ABI_VERSION


def test_struct_layout_matches_header():
    # field order / count of the ctypes mirrors against the header text
    text = open(HEADER).read()
    for struct, cls in (("ditto_bmm_chain_desc", _lib.BmmChainDesc), ("ditto_conv_chain_desc", _lib.ConvChainDesc),
                        ("ditto_tile_param", _lib.TileParam)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (struct, struct), text, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            names = decl.split(None, 1)[1]
            fields += [n.strip() for n in names.split(",")]
        assert fields == [n for n, _ in cls._fields_], struct


def _desc(**kw):
    d = _lib.BmmChainDesc()
    d.abi_version = _lib.ABI_VERSION
    d.in_dtype, d.acc_dtype, d.out_dtype = _lib.F16, _lib.F32, _lib.F16
    d.inter_op, d.b_layout = _lib.INTER_SOFTMAX, _lib.B_LK
    d.batch, d.M, d.N, d.K, d.L = 96, 512, 64, 64, 512
    d.a_batch_stride, d.a_row_stride = 512 * 64, 64
    d.b_batch_stride, d.b_row_stride = 512 * 64, 64
    d.c_batch_stride, d.c_row_stride = 512 * 64, 64
    d.f_batch_stride, d.f_row_stride = 512 * 64, 64
    d.softmax_scale = 0.125
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_select_tile_and_validation_without_gpu():
    lib = _lib.load()
    tile = _lib.TileParam()
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(_desc()), ctypes.byref(tile)) == _lib.OK
    # 96 heads of 512 rows, head size 64, keys stored [L][K]: 64-row workgroups, three per compute unit
    assert (tile.variant, tile.block_threads, tile.block_m, tile.head_pad) == (644, 256, 64, 64)
    assert tile.grid_x == (512 // tile.block_m) * 96 and 3 * tile.lds_bytes <= 160 * 1024
    long_keys = _desc(L=2048, b_batch_stride=2048 * 64, c_batch_stride=2048 * 64)
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(long_keys), ctypes.byref(tile)) == _lib.OK and tile.variant == 645
    # every fp variant can be forced through the descriptor; ids come back in tile.variant
    for q, threads, bm in ((1, 256, 128), (2, 256, 256), (8, 512, 256), (9, 512, 256), (6, 512, 256), (7, 512, 384),
                           (4, 256, 64), (5, 256, 64)):
        assert lib.ditto_bmm_chain_select_tile(ctypes.byref(_desc(tile_variant=640 + q)), ctypes.byref(tile)) == _lib.OK
        assert (tile.variant, tile.block_threads, tile.block_m) == (640 + q, threads, bm)
        assert tile.lds_bytes <= 160 * 1024
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(_desc(tile_variant=1288)), ctypes.byref(tile)) == _lib.EINVAL
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(_desc(tile_variant=643)), ctypes.byref(tile)) == _lib.EINVAL
    # every kernel reads B in either layout
    for v in (646, 647, 644, 645):
        kl = _desc(tile_variant=v, b_layout=_lib.B_KL, b_row_stride=512)
        assert lib.ditto_bmm_chain_select_tile(ctypes.byref(kl), ctypes.byref(tile)) == _lib.OK and tile.variant == v
    # the 64-row kernels serve head sizes up to 64
    wide = _desc(tile_variant=1284, N=128, K=128, a_row_stride=128, b_row_stride=128, c_row_stride=128, f_row_stride=128,
                 a_batch_stride=512 * 128, b_batch_stride=512 * 128, c_batch_stride=512 * 128, f_batch_stride=512 * 128)
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(wide), ctypes.byref(tile)) == _lib.EINVAL
    # the library's own choice: two 256-row workgroups per CU and B stored [L][K] -> that kernel, with eight of a
    # head's row blocks 384 rows tall and four 256 (4096 rows on four compute units: 2 x 384 + 256 each)
    big = _desc(in_dtype=_lib.BF16, out_dtype=_lib.BF16, batch=64, M=4096, L=4096, N=128, K=128, a_row_stride=128,
                b_row_stride=128, c_row_stride=128, f_row_stride=128, a_batch_stride=4096 * 128,
                b_batch_stride=4096 * 128, c_batch_stride=4096 * 128, f_batch_stride=4096 * 128)
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(big), ctypes.byref(tile)) == _lib.OK and tile.variant == 1287
    assert (tile.block_m, tile.grid_x) == (384, 64 * 12)
    big.b_layout, big.b_row_stride = _lib.B_KL, 4096   # keys stored [K][L]: the same kernel (transposing reads)
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(big), ctypes.byref(tile)) == _lib.OK and tile.variant == 1287
    big.inter_op = _lib.INTER_CAST                    # without the softmax: four waves, 256-row workgroups
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(big), ctypes.byref(tile)) == _lib.OK and tile.variant == 1282
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(_desc(relu_out=2)), ctypes.byref(tile)) == _lib.EINVAL
    # the long-sequence configuration picks the 128-wide head tile
    big = _desc(in_dtype=_lib.BF16, out_dtype=_lib.BF16, batch=64, M=4096, L=4096, K=128, N=128,
                a_row_stride=128, b_row_stride=128, c_row_stride=128, f_row_stride=128,
                a_batch_stride=4096 * 128, b_batch_stride=4096 * 128, c_batch_stride=4096 * 128,
                f_batch_stride=4096 * 128)
    assert lib.ditto_bmm_chain_select_tile(ctypes.byref(big), ctypes.byref(tile)) == _lib.OK
    assert tile.head_pad == 128 and tile.lds_bytes <= 160 * 1024

    def rc_msg(d):
        rc = lib.ditto_bmm_chain_select_tile(ctypes.byref(d), ctypes.byref(tile))
        return rc, _lib.last_error()

    assert rc_msg(_desc(abi_version=99))[0] == _lib.EINVAL
    rc, msg = rc_msg(_desc(K=60))
    assert rc == _lib.EINVAL and "multiples of 8" in msg
    assert rc_msg(_desc(M=0))[0] == _lib.EINVAL
    assert rc_msg(_desc(softmax_scale=0.0))[0] == _lib.EINVAL
    assert rc_msg(_desc(a_row_stride=32))[0] == _lib.EINVAL
    assert rc_msg(_desc(K=512, a_row_stride=512, b_row_stride=512))[0] == _lib.EUNSUPPORTED
    with pytest.raises(ValueError):
        _lib.check(rc_msg(_desc(N=12))[0])
    with pytest.raises(NotImplementedError):
        _lib.check(rc_msg(_desc(K=512, a_row_stride=512, b_row_stride=512))[0])


def _conv_desc(**kw):
    d = dict(abi_version=_lib.ABI_VERSION, in_dtype=_lib.F16, acc_dtype=_lib.F32, out_dtype=_lib.F16, inter_op=_lib.INTER_CAST,
             relu_out=0, N=32, C0=64, H=56, W=56, C1=64, R1=3, S1=3, pad1=1, stride1=1, C2=256, R2=1, S2=1, pad2=0,
             stride2=1, groups1=1)
    d.update(kw)
    return _lib.ConvChainDesc(**d)


def test_conv_tile_choice_without_gpu():
    lib = _lib.load()
    tile = _lib.TileParam()
    # the workload shape runs on the row pipeline: bands of 7 output rows, one workgroup per CU, seven waves
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc()), ctypes.byref(tile)) == _lib.OK
    assert (tile.variant, tile.grid_x, tile.grid_y, tile.block_threads) == (3707, 256, 7, 512)
    assert tile.lds_bytes <= 160 * 1024
    rows_ws = lib.ditto_conv_chain_workspace_bytes(ctypes.byref(_conv_desc()))
    # W1 as MFMA fragments takes 9 * 64 * 64 * 2 bytes; the query covers the general kernel too, which a call
    # with less aligned pointers falls back to
    assert rows_ws == max(9 * 64 * 64 * 2, 2 * 9 * 64 * 40 * 2)
    # fp32 output, wider rows or more channels stay on the general kernel, and so does everything with tile_variant 3000
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(out_dtype=_lib.F32)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant == 3022
    # ... and narrow outputs with enough images to fill the CUs with the general kernel's tiles (measured slower there)
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C2=128)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant == 3022
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C2=128, N=8)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant // 100 == 37
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C0=32, C1=32)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant // 100 == 30
    for forced in (3000, 3022):  # the family, or the exact kernel
        general = _conv_desc(tile_variant=forced)
        assert lib.ditto_conv_chain_select_tile(ctypes.byref(general), ctypes.byref(tile)) == _lib.OK
        assert tile.variant == 3022 and tile.grid_x == 32 * 14 and tile.lds_bytes <= 80 * 1024  # two workgroups per CU
        default_ws = lib.ditto_conv_chain_workspace_bytes(ctypes.byref(general))
        assert default_ws == 2 * 9 * 64 * 40 * 2  # two chunks of 32 input channels, [tap][c1][32 + 8]
    # the row pipeline by family and by exact id; an id the planner does not arrive at is refused, and so are
    # families that cannot run the chain and ids that name nothing
    for forced in (3700, 3707):
        assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(tile_variant=forced)), ctypes.byref(tile)) == _lib.OK
        assert tile.variant == 3707
    assert lib.ditto_conv_chain_workspace_bytes(ctypes.byref(_conv_desc(tile_variant=3707))) == 9 * 64 * 64 * 2
    # (narrow outputs, where the library's own choice is the general kernel: the pipeline can still be asked for)
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C2=128, tile_variant=3700)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant == 3707
    for bad in (3705, 3800, 3600, 3500, 4000, 4024, 1286, 17, -1):
        assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(tile_variant=bad)), ctypes.byref(tile)) == _lib.EINVAL, bad
        assert lib.ditto_conv_chain_workspace_bytes(ctypes.byref(_conv_desc(tile_variant=bad))) == 0
    # the persistent 3x3 -> 1x1 kernel is switched off: asking for it is refused, not silently ignored
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(tile_variant=3900)), ctypes.byref(tile)) == _lib.EUNSUPPORTED
    assert b"switched off" in lib.ditto_last_error()
    assert lib.ditto_conv_chain_workspace_bytes(ctypes.byref(_conv_desc(tile_variant=3900))) == 0
    # depthwise first convolution: persistent kernel with the matrix-core depthwise stage; at multiplier 1 the
    # row-streaming kernel (bands of 14 rows: one workgroup per CU, nine waves) for up to 32 -> 64 channels and
    # the persistent kernel with the vector-ALU stage beyond
    dw = dict(C0=32, H=112, W=112, C2=64, groups1=32)
    # (sixteen outputs per input channel: the row-streaming kernel for that factor, bands of 14 rows too, nine waves)
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C1=512, **dw)), ctypes.byref(tile)) == _lib.OK
    assert (tile.variant, tile.grid_x, tile.grid_y, tile.block_threads) == (4025, 256, 14, 576)
    assert tile.lds_bytes <= 160 * 1024
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C1=512, tile_variant=4000, **dw)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant == 4022 and tile.grid_x == 256
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C1=512, tile_variant=4024, **dw)), ctypes.byref(tile)) == _lib.EINVAL
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C1=32, **dw)), ctypes.byref(tile)) == _lib.OK
    assert (tile.variant, tile.grid_x, tile.grid_y, tile.block_threads) == (4024, 256, 14, 832)
    assert tile.lds_bytes <= 160 * 1024
    for forced in (4000, 4023):
        assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C1=32, tile_variant=forced, **dw)), ctypes.byref(tile)) == _lib.OK
        assert tile.variant == 4023
    dw = dict(C0=64, H=56, W=56, C2=128, groups1=64)
    assert lib.ditto_conv_chain_select_tile(ctypes.byref(_conv_desc(C1=64, **dw)), ctypes.byref(tile)) == _lib.OK
    assert tile.variant == 4043


def test_run_rejects_bad_arguments_before_touching_the_device():
    lib = _lib.load()
    # null pointers are refused by validation, no launch happens
    rc = lib.ditto_bmm_chain_run(ctypes.byref(_desc(K=60)), None, None, None, None, None, None, 0, None)
    assert rc == _lib.EINVAL


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.ChainLibraryError, match="no CPU or PyTorch fallback"):
        _lib.load()
