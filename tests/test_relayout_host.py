"""The layout-conversion kernels stepped through on the CPU: the body that the
GPU kernels run (rocmlir_amd/csrc/relayout_body.h) is compiled for the host
(tests/relayout_host.cpp) and run over the conversion kernels of real plans,
every block and thread, with source and destination placed against guard pages.
The result must equal the conversion's definition (element (i0..i4) moves from
src[sum i*src_stride] to dst[sum i*dst_stride], zero beyond the source's
extent), and no access may leave the tensors."""
import ctypes as C
import os
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PARAMS = 312  # sizeof(RockRelayoutParams): strides 80, sizes 40, src_fast dst_fast mode tile_d 16, divisors 40, resolved tiling 136


@pytest.fixture(scope="session")
def host_body(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("relayout_host") / "relayout_host.so")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-I", os.path.join(ROOT, "rocmlir_amd", "csrc"),
                           "-o", out, os.path.join(ROOT, "tests", "relayout_host.cpp")])
    lib = C.CDLL(out)
    lib.relayout_host_run.restype = C.c_int
    lib.relayout_host_run.argtypes = [C.c_char_p, C.c_int, C.c_uint, C.c_void_p, C.c_size_t, C.c_size_t,
                                      C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int]
    return lib


def conv(t, il, fl, n, c, h, w, k, y, x, stride=1, pad=0, g=1, op="conv", extra=""):
    ho = (h + 2 * pad - y) // stride + 1
    wo = (w + 2 * pad - x) // stride + 1
    ot = {"i8": "i32"}.get(t, t)
    return ("--operation %s --arch gfx950 --in_type %s --fil_type %s --out_type %s --fil_layout %s --in_layout %s "
            "--out_layout %s --batchsize %d --groupsize %d --in_channels %d --out_channels %d --in_h %d --in_w %d "
            "--out_h %d --out_w %d --fil_h %d --fil_w %d --dilation_h 1 --dilation_w 1 --conv_stride_h %d "
            "--conv_stride_w %d --padding_h %d --padding_w %d %s" % (
                op, t, t, ot, fl, il, il.replace("c", "k").replace("C", "K"), n, g, c * g, k * g, h, w, ho, wo, y, x,
                stride, stride, pad, pad, extra))


PROBLEMS = [
    # NCHW tensors with rows that start on every alignment: 7x7, 14x14, 15x15 images of 16-bit, 8-bit, 32-bit elements
    conv("fp16", "ngchw", "gkcyx", 2, 96, 7, 7, 64, 3, 3, pad=1),
    conv("fp16", "ngchw", "gkcyx", 3, 40, 14, 14, 32, 3, 3, pad=1),
    conv("fp16", "ngchw", "gkcyx", 2, 72, 15, 15, 32, 3, 3),
    conv("i8", "ngchw", "gkcyx", 2, 96, 7, 7, 64, 3, 3, pad=1),
    conv("i8", "ngchw", "gkcyx", 2, 48, 15, 13, 32, 3, 3),
    conv("f32", "ngchw", "gkcyx", 2, 36, 7, 7, 32, 3, 3, pad=1),
    conv("f32", "ngchw", "gkcyx", 1, 40, 13, 9, 32, 5, 5, pad=2),
    conv("bf16", "ngchw", "gkcyx", 2, 64, 16, 16, 64, 3, 3, pad=1),
    # groups, long rows, a 5x5 filter (25-element runs) and a 7x7 (49)
    conv("fp16", "ngchw", "gkcyx", 1, 24, 30, 30, 32, 5, 5, g=2),
    conv("fp16", "ngchw", "gkcyx", 1, 32, 20, 20, 32, 7, 7, pad=3),
    # a strided 1x1 filter: every other pixel of every other row is copied
    conv("fp16", "ngchw", "gkcyx", 2, 64, 14, 14, 128, 1, 1, stride=2),
    conv("i8", "ngchw", "gkcyx", 2, 64, 10, 10, 128, 1, 1, stride=2),
    conv("f32", "ngchw", "gkcyx", 2, 32, 9, 9, 64, 1, 1, stride=2),
    # ... of rows that start on 16-byte boundaries: aligned vectors, every other element kept
    conv("fp16", "ngchw", "gkcyx", 2, 64, 16, 24, 128, 1, 1, stride=2),
    conv("i8", "ngchw", "gkcyx", 2, 64, 32, 32, 128, 1, 1, stride=2),
    conv("f32", "ngchw", "gkcyx", 2, 40, 8, 8, 64, 1, 1, stride=2),
    # three channels padded to one 16-byte chunk per pixel, NCHW and NHWC
    conv("fp16", "ngchw", "gkcyx", 2, 3, 30, 30, 64, 7, 7, stride=2, extra="--tap_rows false"),
    conv("i8", "ngchw", "gkcyx", 2, 3, 30, 30, 64, 7, 7, stride=2, extra="--tap_rows false"),
    conv("fp16", "nhwgc", "gkyxc", 2, 3, 30, 30, 64, 7, 7, stride=2, extra="--tap_rows false"),
    # ... and into rows of taps: 3 -> 4 channels of 16 bits (two pixels a chunk), 3 -> 8 of 8 bits, the filter
    # rows padded to whole chunks
    conv("fp16", "ngchw", "gkcyx", 2, 3, 30, 30, 64, 7, 7, stride=2),
    conv("i8", "ngchw", "gkcyx", 2, 3, 30, 30, 64, 7, 7, stride=2),
    conv("i8", "nhwgc", "gkyxc", 2, 3, 30, 30, 64, 7, 7, stride=2),
    conv("f32", "ngchw", "gkcyx", 2, 3, 18, 18, 64, 3, 3),
    conv("fp16", "nhwgc", "gkyxc", 2, 3, 30, 30, 64, 7, 7, stride=2),
    # channel counts that are not whole chunks
    conv("fp16", "ngchw", "gkcyx", 2, 20, 9, 9, 24, 3, 3),
    conv("fp16", "nhwgc", "gkyxc", 2, 12, 9, 9, 24, 3, 3),
    # backward data: flipped filters, one phase per stride offset
    conv("fp16", "ngchw", "gkcyx", 2, 32, 12, 12, 32, 3, 3, stride=2, pad=1, op="conv_bwd_data"),
    conv("fp16", "nhwgc", "gkyxc", 2, 128, 14, 14, 128, 3, 3, pad=1, op="conv_bwd_data"),
    conv("fp16", "nhwgc", "gkyxc", 2, 64, 12, 12, 64, 3, 3, stride=2, pad=1, op="conv_bwd_data"),
    # backward weight through channels-last copies, and the filter gradient written back as gkcyx
    conv("fp16", "ngchw", "gkcyx", 4, 32, 10, 10, 32, 3, 3, pad=1, op="conv_bwd_weight"),
    conv("f32", "ngchw", "gkcyx", 4, 16, 8, 8, 32, 3, 3, pad=1, op="conv_bwd_weight"),
    # filter gradient over a few channels: 3 -> 4 channels of 16 bits, two pixels a chunk (NHWC and NCHW sources);
    # 2 and 1 channels; 32-bit elements
    conv("fp16", "nhwgc", "gkyxc", 2, 3, 20, 20, 16, 7, 7, stride=2, op="conv_bwd_weight"),
    conv("fp16", "ngchw", "gkcyx", 2, 3, 20, 20, 16, 7, 7, stride=2, op="conv_bwd_weight"),
    conv("bf16", "nhwgc", "gkyxc", 2, 2, 9, 16, 8, 3, 5, stride=4, op="conv_bwd_weight"),
    conv("fp16", "ngchw", "gkcyx", 1, 1, 10, 24, 8, 3, 3, stride=8, op="conv_bwd_weight"),
    conv("f32", "ngchw", "gkcyx", 2, 2, 9, 16, 8, 3, 5, stride=4, op="conv_bwd_weight"),
    # the window-resident kernel's fragment-major filter
    conv("fp16", "nhwgc", "gkyxc", 8, 128, 28, 28, 128, 3, 3, pad=1, extra="--perf_config v2:224,128,8,224,32,8,1,1,1"),
    # ragged GEMM operands copied into padded rows (two conversions in one launch)
    "-operation gemm -arch gfx950 -t f16 -g 2 -m 70 -n 45 -k 97",
    "-operation gemm -arch gfx950 -t i8 -out_datatype i32 -g 1 -m 33 -n 50 -k 75 -transA true",
    "-operation gemm -arch gfx950 -t f32 -g 1 -m 30 -n 41 -k 37 -transB true",
    # input gradients with their phases merged: filter slices, the phases put together (4-byte words), to NCHW
    conv("fp16", "nhwgc", "gkyxc", 2, 3, 20, 16, 8, 7, 7, stride=2, op="conv_bwd_data"),
    conv("fp16", "ngchw", "gkcyx", 2, 3, 16, 16, 8, 7, 7, stride=2, pad=3, op="conv_bwd_data"),
    conv("f32", "nhwgc", "gkyxc", 1, 2, 12, 18, 8, 5, 5, stride=3, pad=2, op="conv_bwd_data"),
    conv("bf16", "ngchw", "gkcyx", 2, 1, 16, 16, 5, 4, 4, stride=2, pad=1, op="conv_bwd_data"),
]


def _conversions(rock, options):
    """(element size, grid, RockRelayoutParams bytes) of every conversion in the problem's plan."""
    first = rock.RockKernel(options)
    out = []
    for kid in range(first.kernel_count):
        k = first if kid == 0 else rock.RockKernel("%s --kernel_id %d" % (options, kid))
        name = k.kernel_name
        if not name.startswith("rock_relayout"):
            continue
        es = int(name[-1])
        grid = k.execution_dims()[0] // 256
        raw = k.params()
        if "pair" in name:
            first_blocks = struct.unpack_from("<i", raw, 2 * PARAMS)[0]
            out.append((es, first_blocks, raw[:PARAMS]))
            out.append((es, grid - first_blocks, raw[PARAMS:2 * PARAMS]))
        else:
            out.append((es, grid, raw[:PARAMS]))
    return out


def _definition(params, es, rng):
    """Random source of exactly the extent the conversion reads, the destination it must produce
    (untouched elements keep their sentinel), and the byte offsets of the kernel's two pointers."""
    ss = np.array(struct.unpack_from("<5q", params, 0))
    ds = np.array(struct.unpack_from("<5q", params, 40))
    size = struct.unpack_from("<5i", params, 80)
    src_size = np.array(struct.unpack_from("<5i", params, 100))
    idx = np.indices(size).reshape(5, -1)
    inside = np.all(idx < src_size[:, None], axis=0)
    so = (idx * ss[:, None]).sum(0)
    do = (idx * ds[:, None]).sum(0)
    assert do.min() == 0 and len(np.unique(do)) == do.size
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[es]
    lo, hi = so[inside].min(), so[inside].max()
    src = rng.integers(1, np.iinfo(dt).max, size=hi - lo + 1, dtype=dt)
    dst = np.full(do.max() + 1, 0xEE, dt)
    want = dst.copy()
    vals = np.zeros(do.size, dt)
    vals[inside] = src[so[inside] - lo]
    want[do] = vals
    return src, -int(lo) * es, dst, want


@pytest.mark.parametrize("options", PROBLEMS)
def test_conversion_kernels_on_the_host(rock, host_body, options):
    rng = np.random.default_rng(len(options))
    convs = _conversions(rock, options)
    assert convs, "the plan holds no conversion kernel"
    for es, grid, params in convs:
        src, src_off, dst, want = _definition(params, es, rng)
        for shift, front in ((0, 0), (es, 1), (16 - es, 0), (8, 1)):
            got = dst.copy()
            rc = host_body.relayout_host_run(params, es, grid, src.ctypes.data, src.nbytes, src_off, got.ctypes.data,
                                             got.nbytes, 0, shift, front)
            assert rc == 0
            mode, tile_d = struct.unpack_from("<2i", params, 128)
            assert np.array_equal(got, want), (mode, tile_d, shift)


def test_modes_chosen(rock):
    """Which kernel body the plans pick: one chunk per pixel copies, tiles reshape to short dimensions."""
    def params_of(options, kid):
        raw = rock.RockKernel("%s --kernel_id %d" % (options, kid)).params()
        return struct.unpack_from("<5i", raw, 80), struct.unpack_from("<4i", raw, 120)
    # 3 channels -> 8: RELAYOUT_COPY for the NCHW image as well (source contiguous along the folded pixels)
    size, (sf, df, mode, _) = params_of(conv("fp16", "ngchw", "gkcyx", 2, 3, 30, 30, 64, 7, 7, stride=2,
                                             extra="--tap_rows false"), 1)
    assert size[-2:] == (900, 8) and (sf, df, mode) == (3, 4, 1)
    # a 3x3 filter gkcyx -> gkyxc: runs of 9 along the source, tiles of 256 channels x 16 taps
    size, (sf, df, mode, td) = params_of(conv("fp16", "ngchw", "gkcyx", 2, 256, 14, 14, 256, 3, 3, pad=1), 0)
    assert size[-2:] == (9, 256) and (mode, td) == (2, 256)
    # 14 x 14 images of 256 channels: 64 x 64 tiles
    size, (sf, df, mode, td) = params_of(conv("fp16", "ngchw", "gkcyx", 2, 256, 14, 14, 256, 3, 3, pad=1), 1)
    assert size[-2:] == (196, 256) and (mode, td) == (2, 64)
    # 3 -> 4 channels of 16 bits: two pixels a chunk
    size, (sf, df, mode, ppc) = params_of(conv("fp16", "ngchw", "gkcyx", 2, 3, 20, 20, 16, 7, 7, stride=2,
                                               op="conv_bwd_weight"), 0)
    assert size[-2:] == (400, 4) and (mode, ppc) == (1, 2)
    # every other pixel of every other row: vector tiles with element-wise reads (the 1x1 filter needs no kernel)
    size, (sf, df, mode, td) = params_of(conv("fp16", "ngchw", "gkcyx", 2, 64, 14, 14, 128, 1, 1, stride=2), 0)
    assert size[-2:] == (7, 64) and (mode, td) == (2, 256)


def test_plan_time_divisors(rock):
    """n / d == (n * mul) >> shift for every divisor a plan stores, over the dividends the kernels form."""
    rng = np.random.default_rng(5)
    seen = set()
    for options in PROBLEMS:
        for es, grid, params in _conversions(rock, options):
            size = struct.unpack_from("<5i", params, 80)
            for i in range(5):
                mul, shift = struct.unpack_from("<2I", params, 136 + 8 * i)
                assert 31 <= shift <= 62 and mul >= 1 << 31
                seen.add((mul, shift))
    assert len(seen) > 10
    for mul, shift in seen:
        d = -(-(1 << shift) // mul)  # the divisor: mul = ceil(2^shift / d) determines it for shift = 31 + ceil(log2 d)
        assert mul == -(-(1 << shift) // d)
        n = np.concatenate([np.arange(0, 4 * d + 2), rng.integers(0, 2 ** 31, 4096), [2 ** 31 - 1, 2 ** 31 - d, d * (2 ** 31 // d) - 1]])
        n = n[(n >= 0) & (n < 2 ** 31)]
        assert all((int(v) * mul) >> shift == int(v) // d for v in n)
