"""Host-side check of the window-resident convolution's plan, without a GPU:
the conversion kernel in front of it is replayed in numpy from its parameter
block and must produce the fragment-major filter the contraction kernel
streams,
  F'[g][32-channel block][K-step of 128 bytes][chunk 0..7][channel 0..31][16 bytes],
every group padded with zero rows to whole 128-channel tiles; the contraction
kernel's tile geometry must keep its LDS window within the 80 KiB a block has."""
import struct

import numpy as np
import pytest

from tests.test_conv3d_plan import _pointer_map, _replay_relayout

ASK = " --perf_config v2:224,128,8,224,32,8,1,1,1"


def _options(t, n, g, c, k, hi, wi, y, x, pad):
    return ("--operation conv --arch gfx950 -t %s --fil_layout gkyxc --in_layout nhwgc --out_layout nhwgk --batchsize %d"
            " --groupsize %d --in_channels %d --out_channels %d --in_h %d --in_w %d --fil_h %d --fil_w %d"
            " --padding_h %d --padding_w %d" % (t, n, g, g * c, g * k, hi, wi, y, x, pad[0], pad[1]))


@pytest.mark.parametrize("t,es", [("f16", 2), ("f32", 4), ("i8", 1)])
@pytest.mark.parametrize("shape", [(3, 1, 128, 128, 28, 28, 3, 3, (1, 1)), (2, 2, 128, 96, 12, 20, 3, 5, (1, 2)),
                                   (5, 1, 256, 160, 9, 7, 3, 3, (1, 1))])
def test_filter_is_repacked_fragment_major(rock, shape, t, es):
    n, g, pixel_bytes, k, hi, wi, y, x, pad = shape
    c = pixel_bytes // es
    opts = _options(t, n, g, c, k, hi, wi, y, x, pad) + ASK
    first, second = rock.RockKernel(opts), rock.RockKernel(opts + " --kernel_id 1")
    assert (first.kernel_name, second.kernel_name) == ("rock_relayout_b%d" % es, "rock_conv_%s_direct224" % t)
    assert first.kernel_count == second.kernel_count == 2 and first.caller_pointers == second.caller_pointers == 5
    K = y * x * c
    tiles_n = -(-k // 128)
    rows_p = tiles_n * 128
    assert first.workspace_bytes == second.workspace_bytes >= g * rows_p * K * es
    fil = np.arange(1, g * k * K + 1, dtype=np.float32)
    ws = np.full(first.workspace_bytes // es, np.nan, np.float32)
    (s_src, s_off), (d_src, d_off) = _pointer_map(rock, first)
    assert (s_src, s_off, d_src, d_off) == (0, 0, 4, 0)
    _replay_relayout(first.params(), fil, 0, ws, 0)
    e = 16 // es                                     # elements per 16-byte chunk
    nk = K * es // 128
    want = np.zeros((g, rows_p, K), np.float32)
    want[:, :k] = fil.reshape(g, k, K)
    want = want.reshape(g, rows_p // 32, 32, nk, 8, e).transpose(0, 1, 3, 4, 2, 5)   # g blk kt chunk row e
    assert np.array_equal(ws[:want.size], want.ravel())
    # the contraction kernel reads the repacked filter from the workspace and the other tensors where they lie
    assert [src for src, _ in _pointer_map(rock, second)] == [4, 1, 2, 3, -1]


@pytest.mark.parametrize("shape", [(256, 128, 28, 28, 3), (64, 64, 56, 56, 3), (32, 256, 14, 14, 3), (8, 128, 28, 28, 5),
                                   (3, 128, 6, 50, 3), (7, 64, 10, 12, 3)])
def test_window_fits_its_share_of_lds(rock, shape):
    n, c, hi, wi, y = shape
    pad = y // 2
    opts = _options("f16", n, 1, c, 128, hi, wi, y, y, (pad, pad)) + ASK + " --kernel_id 1"
    try:
        k = rock.RockKernel(opts)
    except rock.RockError:
        pytest.skip("plan has one kernel: the request fell back")
    if "direct224" not in k.kernel_name:
        return
    params = k.params()
    hi_, wi_, y_, x_, ho, wo = struct.unpack_from("<6i", params, 136)
    rows = struct.unpack_from("<i", params, 216)[0]
    assert 1 <= rows <= ho and rows * wo <= 224
    pitch = -(-((wi + 2 * pad) * c * 2) // 1024) * 1024
    window_rows = rows + y - 1 + (y - 1 if ho % rows else 0)     # tiles that straddle two images hold the padding rows between them
    assert window_rows * pitch <= 80 * 1024


@pytest.mark.parametrize("fil_layout", ["gkyxc", "gkcyx"])
def test_backward_data_filter_is_flipped_and_repacked_in_one_kernel(rock, fil_layout):
    """Unit-stride input gradient of the 3x3 ResNet layer: a stride-1 convolution
    of dY with the flipped, k <-> c swapped filter, on the window-resident
    kernel; ONE conversion kernel writes that filter fragment-major."""
    n, c, k, hw, y = 256, 128, 128, 28, 3
    opts = ("--operation conv_bwd_data --arch gfx950 -t f16 --fil_layout %s --in_layout nhwgc --out_layout nhwgk"
            " --batchsize %d --groupsize 1 --in_channels %d --out_channels %d --in_h %d --in_w %d --fil_h %d --fil_w %d"
            " --padding_h 1 --padding_w 1" % (fil_layout, n, c, k, hw, hw, y, y))
    first, second = rock.RockKernel(opts), rock.RockKernel(opts + " --kernel_id 1")
    assert (first.kernel_count, first.kernel_name, second.kernel_name) == (2, "rock_relayout_b2",
                                                                          "rock_conv_f16_direct224")
    K = y * y * k
    assert first.workspace_bytes == c * K * 2
    W = np.arange(1, k * c * y * y + 1, dtype=np.float32).reshape(k, c, y, y)          # canonical k c y x
    fil = np.ascontiguousarray(W.transpose(0, 2, 3, 1) if fil_layout == "gkyxc" else W).ravel()
    ws = np.full(first.workspace_bytes // 2, np.nan, np.float32)
    (s_src, s_off), (d_src, d_off) = _pointer_map(rock, first)
    assert (s_src, d_src, d_off) == (0, 4, 0)
    _replay_relayout(first.params(), fil, s_off // 2, ws, 0)
    virt = W[:, :, ::-1, ::-1].transpose(1, 2, 3, 0).reshape(c, K)                    # rows c, reduction (t_h, t_w, k)
    want = virt.reshape(c // 32, 32, K // 64, 8, 8).transpose(0, 2, 3, 1, 4)           # blk kt chunk row e
    assert np.array_equal(ws, want.ravel())
    assert [src for src, _ in _pointer_map(rock, second)] == [4, 2, 1, -1, -1]
    # off the table's choice the phase keeps the implicit-GEMM kernel and its K-contiguous filter copy
    plain = rock.RockKernel(opts + " --window_resident false --kernel_id 1")
    assert plain.kernel_name == "rock_conv_f16_128x128_fast" and plain.kernel_count == 2
