"""C-ABI checks that need no GPU: the library loads, exports every symbol the header declares,
and the descriptor validation / shape deduction / chooser surface behave like the reference's
host-side checks (dnn/src/common/conv_bias.cpp:8-133, dnn/src/common/convolution.cpp:633-1049)."""
import ctypes as C
import os
import re

import pytest

from megengine_amd import _abi, lib, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_header_symbols():
    L = lib.lib()
    assert L.mi355_abi_version() == _abi.ABI_VERSION
    hdr = open(os.path.join(ROOT, "include", "mi355_convbias.h")).read()
    declared = set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(L, name), "library does not export %s" % name
    assert declared == set(lib.EXPORTS)


def test_struct_layout_matches_header():
    # sizes fixed by the C header (checked against a C compiler in test_host_cpp)
    assert C.sizeof(_abi.ConvDesc) == 4 * 24 + 8 * 3
    assert C.sizeof(_abi.Algo) == 16
    assert C.sizeof(_abi.RelayoutDesc) == 4 * 2 + 28 + 4 * 5


def test_status_strings():
    L = lib.lib()
    for st in range(8):
        assert L.mi355_status_string(st)
    assert L.mi355_status_string(99) == b"unknown status"


def test_algorithm_table():
    names = lib.algo_names()
    assert names == ["MI355_DIRECT_DOT4", "MI355_IGEMM_MFMA_I8", "MI355_DEPTHWISE_DOT4", "MI355_C4_MFMA_I8",
                     "MI355_NCHW_RELAYOUT_MFMA_I8"]
    assert lib.lib().mi355_convbias_algo_name(17) is None
    assert len(lib.tile_names()) >= 3


@pytest.mark.parametrize("fmt,n,ic,ih,iw,oc,f,kw,want", [
    ("NCHW4", 16, 64, 56, 56, 64, 3, dict(pad=1), (16, 16, 56, 56, 4)),
    ("NCHW32", 64, 256, 56, 56, 64, 1, {}, (64, 2, 56, 56, 32)),
    ("NCHW4", 64, 4, 224, 224, 64, 7, dict(pad=3, stride=2), (64, 16, 112, 112, 4)),
    ("NCHW32", 128, 512, 32, 32, 1024, 3, dict(pad=1, stride=2), (128, 32, 16, 16, 32)),
    ("NCHW", 2, 3, 9, 9, 5, 3, dict(dilate=2), (2, 5, 5, 5)),
    ("NCHW4_NCHW32", 1, 8, 6, 6, 32, 3, dict(pad=1), (1, 1, 6, 6, 32)),
])
def test_deduce_layout(fmt, n, ic, ih, iw, oc, f, kw, want):
    d = _abi.make_conv_desc(fmt, n, ic, ih, iw, oc, f, **kw)
    assert ops.conv_bias_deduce_layout(d) == want


def _status(d):
    oh, ow = C.c_uint32(), C.c_uint32()
    return lib.lib().mi355_convbias_deduce_out(C.byref(d), C.byref(oh), C.byref(ow))


def test_validation_errors():
    # group conv channel mismatch (convolution.cpp:803-808)
    assert _status(_abi.make_conv_desc("NCHW4", 1, 10, 8, 8, 8, 3)) == _abi.ERR_SHAPE
    # oc % 4 (convolution.cpp:811)
    assert _status(_abi.make_conv_desc("NCHW4", 1, 8, 8, 8, 6, 3)) == _abi.ERR_SHAPE
    assert _status(_abi.make_conv_desc("NCHW32", 1, 32, 8, 8, 48, 3)) == _abi.ERR_SHAPE
    # NCHWx dilation must be 1 (convolution.cpp:411-414)
    assert _status(_abi.make_conv_desc("NCHW4", 1, 8, 8, 8, 8, 3, dilate=2)) == _abi.ERR_SHAPE
    # quantized SIGMOID (naive/conv_bias/opr_impl.cpp:79-88)
    assert _status(_abi.make_conv_desc("NCHW4", 1, 8, 8, 8, 8, 3, nonline="SIGMOID")) == _abi.ERR_UNSUPPORTED
    # z with the 4<->32 formats (conv_bias.cpp:127-129)
    assert _status(_abi.make_conv_desc("NCHW4_NCHW32", 1, 8, 8, 8, 32, 3, has_z=True)) == _abi.ERR_SHAPE
    # unknown format
    d = _abi.make_conv_desc("NCHW4", 1, 8, 8, 8, 8, 3)
    d.format = 1  # NHWC
    assert _status(d) == _abi.ERR_UNSUPPORTED
    # filter larger than padded input
    assert _status(_abi.make_conv_desc("NCHW4", 1, 8, 2, 2, 8, 5)) == _abi.ERR_SHAPE
    # dense with group
    d = _abi.make_conv_desc("NCHW4", 1, 8, 8, 8, 8, 3)
    d.group = 2
    assert _status(d) == _abi.ERR_SHAPE
    assert b"group" in lib.lib().mi355_last_error()
    # batch stride smaller than an image
    assert _status(_abi.make_conv_desc("NCHW4", 2, 8, 8, 8, 8, 3, pad=1, src_stride_n=16)) == _abi.ERR_SHAPE
    with pytest.raises(lib.Mi355Error):
        ops.conv_bias_deduce_layout(_abi.make_conv_desc("NCHW4", 1, 10, 8, 8, 8, 3))


def test_query_chooser_and_workspace():
    igemm = lib.algo_names().index("MI355_IGEMM_MFMA_I8")
    dw = lib.algo_names().index("MI355_DEPTHWISE_DOT4")
    a, ws = ops.conv_bias_query(_abi.make_conv_desc("NCHW32", 64, 256, 56, 56, 64, 1, scale_bias=2e-4, scale_dst=0.05))
    assert (a.id, ws) == (igemm, 0)
    a, _ = ops.conv_bias_query(_abi.make_conv_desc("NCHW4", 1, 32, 8, 8, 32, 3, pad=1, group=32))
    assert a.id == dw
    # scales outside the fast epilogue's envelope: 32-packed inputs run the MFMA kernel with its general epilogue
    # (a second-generation tile), 4-packed inputs the generic kernel
    d = _abi.make_conv_desc("NCHW32", 1, 32, 8, 8, 32, 3, pad=1, scale_dst=1e-30)
    a, _ = ops.conv_bias_query(d)
    assert a.id == igemm and lib.tile_names()[a.tile_cfg].startswith("v2_")
    d = _abi.make_conv_desc("NCHW4", 1, 32, 8, 8, 32, 3, pad=1, scale_dst=1e-30)
    a, _ = ops.conv_bias_query(d)
    assert a.id == 0
    with pytest.raises(lib.Mi355Error) as e:
        ops.conv_bias_query(d, igemm)
    assert e.value.status == _abi.ERR_ALGO
    with pytest.raises(lib.Mi355Error):
        ops.conv_bias_query(d, 42)
    # asking for the depthwise kernel on a dense conv
    assert lib.lib().mi355_convbias_algo_usable(C.byref(_abi.make_conv_desc("NCHW4", 1, 8, 8, 8, 8, 3)), dw) == _abi.ERR_ALGO


def test_relayout_deduce():
    assert ops.relayout_deduce_layout(ops.relayout_desc(_abi.RL_NCHW_NCHW4, (1, 6, 1, 2), group=2)) == (1, 2, 1, 2, 4)
    assert ops.relayout_deduce_layout(ops.relayout_desc(_abi.RL_NCHW4_NCHW, (1, 2, 1, 2, 4), oc=7)) == (1, 7, 1, 2)
    assert ops.relayout_deduce_layout(ops.relayout_desc(_abi.RL_NCHW_NCHW4_WEIGHT, (2, 2, 1, 2, 2))) == (2, 4, 1, 2, 2, 4)
    assert ops.relayout_deduce_layout(ops.relayout_desc(_abi.RL_NCHW_NCHW32, (2, 40, 3, 3))) == (2, 2, 3, 3, 32)
    assert ops.relayout_deduce_layout(ops.relayout_desc(_abi.RL_NCHW_NCHW4_IC_SMALL, (2, 3, 8, 8))) == (2, 1, 8, 8, 4)
    with pytest.raises(lib.Mi355Error):
        ops.relayout_deduce_layout(ops.relayout_desc(_abi.RL_NCHW_NCHW4_IC_SMALL, (2, 5, 8, 8)))
    with pytest.raises(lib.Mi355Error):
        ops.relayout_deduce_layout(ops.relayout_desc(99, (2, 5, 8, 8)))


def test_exec_rejects_host_tensors():
    import torch
    d = _abi.make_conv_desc("NCHW4", 1, 8, 4, 4, 8, 1)
    x = torch.zeros(1, 2, 4, 4, 4, dtype=torch.int8)
    with pytest.raises(RuntimeError):
        ops.conv_bias_exec(d, x, x, None, None)


def test_stream_probe_argument_checks():
    L = lib.lib()
    assert L.mi355_stream_probe(None, None, 16, None, 0) == _abi.ERR_BAD_ARG       # bytes to read but no buffer
    assert L.mi355_stream_probe(None, None, 0, None, 16) == _abi.ERR_BAD_ARG
    assert L.mi355_stream_probe(None, 4096, 24, 8192, 16) == _abi.ERR_BAD_ARG      # not a multiple of 16
    assert L.mi355_stream_probe(None, 4100, 16, 8192, 16) == _abi.ERR_BAD_ARG      # misaligned
    assert L.mi355_stream_probe(None, None, 0, None, 0) == 0                       # nothing to do
    assert L.mi355_stream_probe(None, 4096, 64, 8192, 0) == _abi.ERR_BAD_ARG       # reads that reach no store


def test_tile_usable_names_the_kernel_that_runs():
    """Every tile is an algorithm of its own (cf. the per-tile algorithm packs of dnn/src/cuda/conv_bias/algo.cpp:216-253):
    a tile is usable only when exec would run that very kernel, and what the heuristic hands out is always usable."""
    names = lib.tile_names()
    igemm = lib.algo_names().index("MI355_IGEMM_MFMA_I8")

    def usable(d):
        return {names[t] for t in range(len(names)) if lib.tile_usable(d, t)}

    d4 = _abi.make_conv_desc("NCHW4", 2, 64, 14, 14, 64, 3, pad=1, scale_bias=2e-4, scale_dst=0.05)
    u = usable(d4)
    assert "128x128x64" in u and not any(n.startswith(("v2_", "dma")) or n == "pw4_stream" for n in u), u
    d32 = _abi.make_conv_desc("NCHW32", 2, 64, 14, 14, 64, 3, pad=1, has_z=True, scale_bias=2e-4, scale_z=0.05, scale_dst=0.05)
    u = usable(d32)
    assert {"128x128x64", "dma128x128x64", "v2_128x128x64r4", "v2_256x256x64r3w8"} <= u and not any(n.startswith("dma4_") for n in u), u
    # 4-packed pointwise: the 4-packed LDS-direct tiles, and the streaming kernel only where it applies
    dpw = _abi.make_conv_desc("NCHW4", 2, 16, 14, 14, 96, 1, scale_bias=2e-4, scale_dst=0.05)
    assert {"dma4_128x128x64", "pw4_stream"} <= usable(dpw)
    dpw2 = _abi.make_conv_desc("NCHW4", 2, 256, 14, 14, 96, 1, scale_bias=2e-4, scale_dst=0.05)
    u = usable(dpw2)
    assert "dma4_128x128x64" in u and "pw4_stream" not in u
    # the general epilogue (here: a dst scale outside the fast forms) is instantiated on two second-generation tiles
    dg = _abi.make_conv_desc("NCHW32", 1, 64, 8, 8, 64, 3, pad=1, scale_dst=1e-30)
    assert usable(dg) == {"v2_128x128x64r4", "v2_64x128x128r3"}
    dgrp = _abi.make_conv_desc("NCHW32", 1, 128, 8, 8, 128, 3, pad=1, group=2, scale_bias=2e-4, scale_dst=0.05)
    u = usable(dgrp)
    assert u and all(n.startswith("v2_") for n in u), u
    # not an MFMA problem at all
    ddw = _abi.make_conv_desc("NCHW4", 1, 32, 8, 8, 32, 3, pad=1, group=32)
    assert lib.lib().mi355_igemm_tile_usable(C.byref(ddw), 0) == _abi.ERR_ALGO
    assert lib.lib().mi355_igemm_tile_usable(C.byref(d32), len(names)) == _abi.ERR_ALGO
    for d in (d4, d32, dpw, dpw2, dg, dgrp):
        for req in (_abi.ALGO_HEURISTIC, _abi.ALGO_HEURISTIC_PREPROCESS, igemm):
            a, _ = ops.conv_bias_query(d, req)
            if a.id == igemm:
                assert lib.tile_usable(d, a.tile_cfg), (names[a.tile_cfg], req)


def test_plain_nchw_reports_a_workspace():
    """Format::NCHW runs relayout -> NCHW32 MFMA kernel -> relayout through the caller's workspace: query reports its
    size (get_workspace_in_bytes, dnn/include/megdnn/oprs/nn.h:419-422), the packed-format algorithms report 0."""
    names = lib.algo_names()
    nchw = names.index("MI355_NCHW_RELAYOUT_MFMA_I8")
    up = lambda x: (x + 255) // 256 * 256
    d = _abi.make_conv_desc("NCHW", 4, 24, 28, 28, 40, 3, pad=1, nonline="RELU", has_z=True, scale_bias=2e-4, scale_z=0.05,
                            scale_dst=0.05)
    a, ws = ops.conv_bias_query(d)
    assert a.id == nchw
    # src and filter with 24 -> 32 channels, dst and z with 40 -> 64 channels, the padded bias
    assert ws == up(4 * 32 * 28 * 28) + up(64 * 32 * 9) + 2 * up(4 * 64 * 28 * 28) + up(64 * 4)
    assert ops.conv_bias_query(d, 0)[1] == 0
    # whole blocks on both sides, no residual: three tensors
    d = _abi.make_conv_desc("NCHW", 4, 64, 14, 14, 128, 1, scale_bias=2e-4, scale_dst=0.05)
    a, ws = ops.conv_bias_query(d)
    assert a.id == nchw and ws == up(4 * 64 * 196) + up(128 * 64) + up(4 * 128 * 196)
    # small problems, dilation, flipped filters, groups that split a channel block, QuantizedS32 dst: the generic kernel
    for kw in (dict(n=1, ic=8, hw=8, oc=8), dict(dilate=2), dict(mode=_abi.MODE_CONVOLUTION), dict(group=2, ic=32, oc=32),
               dict(dst_dtype=_abi.DT_QS32)):
        kw = dict(kw)
        n, ic, hw, oc = kw.pop("n", 4), kw.pop("ic", 24), kw.pop("hw", 28), kw.pop("oc", 40)
        d = _abi.make_conv_desc("NCHW", n, ic, hw, hw, oc, 3, pad=1, scale_bias=2e-4, scale_dst=0.05, **kw)
        a, ws = ops.conv_bias_query(d)
        assert (a.id, ws) == (0, 0), kw
    # groups of whole 32-channel blocks stay on the MFMA path
    d = _abi.make_conv_desc("NCHW", 2, 64, 14, 14, 128, 3, pad=1, group=2, scale_bias=2e-4, scale_dst=0.05)
    assert ops.conv_bias_query(d)[0].id == nchw
    assert lib.lib().mi355_convbias_algo_usable(C.byref(_abi.make_conv_desc("NCHW32", 2, 64, 14, 14, 128, 1)), nchw) == _abi.ERR_ALGO
