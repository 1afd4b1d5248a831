"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every symbol the header declares, follows the Miir call protocol and error
behaviour (rocmlir-lib.cpp:117-316, rocmlir-lib-test.cpp:31-96), and renders
perf-config / problem-key strings in the reference's grammar."""
import ctypes as C
import os
import re
import struct

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CONV_RESNET = (
    "--operation conv --arch amdgcn-amd-amdhsa:gfx950 --num_cu 256 --in_type fp16 --fil_type fp16 "
    "--out_type fp16 --fil_layout GNYXC --in_layout NHWGC --out_layout NHWGC --batchsize 256 "
    "--groupsize 1 --in_channels 128 --out_channels 128 --in_h 28 --in_w 28 --out_h 28 --out_w 28 "
    "--fil_h 3 --fil_w 3 --dilation_h 1 --dilation_w 1 --conv_stride_h 1 --conv_stride_w 1 "
    "--padding_h 1 --padding_w 1")
# the same problem on the implicit-GEMM kernel alone (the table's own plan puts a filter conversion in front of
# the window-resident kernel)
CONV_IMPLICIT = CONV_RESNET + " --perf_config v2:128,128,8,64,16,8,1,1,1"


def test_every_declared_symbol_is_exported(rock):
    header = open(os.path.join(ROOT, "include", "rocmlir_amd.h")).read()
    names = re.findall(r"ROCMLIR_AMD_API\s+[\w\s\*]+?\b(\w+)\s*\(", header)
    assert len(names) >= 18
    lib = C.CDLL(rock.library_path())
    for n in names:
        assert hasattr(lib, n), n


def test_miir_protocol_conv(rock):
    lib = rock.load_library()
    h = lib.miirCreateHandle(CONV_IMPLICIT.encode())
    assert h
    assert lib.miirGetKernelCount(h) == 1
    assert lib.miirGetWorkspaceSize(h) == 0
    g, l = C.c_size_t(), C.c_size_t()
    # launch dims and the binary need the lowering calls first
    assert lib.miirGetExecutionDims(h, C.byref(g), C.byref(l)) == 2  # MIIR_INVALID_MODULE
    n = C.c_size_t(0)
    assert lib.miirBufferGet(h, None, C.byref(n)) == 2
    assert lib.miirLowerTuningParams(h) == 0
    assert lib.miirGetExecutionDims(h, C.byref(g), C.byref(l)) == 0
    assert l.value in (256, 512) and g.value % l.value == 0
    assert lib.miirLowerBin(h) == 0
    assert lib.miirBufferGet(h, None, C.byref(n)) == 0 and n.value > 1000
    buf = C.create_string_buffer(n.value)
    small = C.c_size_t(10)
    assert lib.miirBufferGet(h, buf, C.byref(small)) == 1  # MIIR_INVALID_PARAM: too small
    assert lib.miirBufferGet(h, buf, C.byref(n)) == 0
    assert buf.raw[:4] == b"\x7fELF"  # mlir/test/mlir-rock-lib/populate_fw.mlir checks "ELF"
    # one kernel per code object, as the reference hands them out (rocmlir-lib.cpp:292-316):
    # the image holds the selected kernel alone and stays small
    from rocmlir_amd._elf import kernel_symbols
    name_len = C.c_size_t(0)
    assert lib.rockamdGetKernelName(h, None, C.byref(name_len)) == 0
    name = C.create_string_buffer(name_len.value)
    assert lib.rockamdGetKernelName(h, name, C.byref(name_len)) == 0
    assert kernel_symbols(buf.raw[:n.value]) == [name.value.decode()]
    assert n.value <= 512 * 1024
    assert lib.miirDestroyHandle(h) == 0


@pytest.mark.parametrize("options", [
    "-operation gemm -arch gfx950 -t i8 -out_datatype f16 -g 1 -m 4096 -n 4096 -k 4096 -transB true -scale 0.01",
    "-operation gemm -arch gfx950 -t fp8 -g 1 -m 8192 -n 8192 -k 8192 -transB true -residual add -activation gelu",
    "-operation gemm -arch gfx950 -t f16 -g 1 -m 512 -n 512 -k 512",
    "-operation gemm -arch gfx950 -t f32 -g 1 -m 512 -n 512 -k 512 -transB true",
    "-operation gemm -arch gfx950 -t bf16 -g 1 -m 70 -n 45 -k 97 -layout_conversion false",
    "-operation attention -arch gfx950 -t f16 -g 128 -seq_len_q 2048 -seq_len_k 2048 -head_dim_qk 128 "
    "-head_dim_v 128 -transK true",
    "-operation attention -arch gfx950 -t bf16 -g 2 -seq_len_q 64 -seq_len_k 64 -head_dim_qk 64 -head_dim_v 64",
    CONV_RESNET.replace("NHWGC", "NGCHW").replace("GNYXC", "GNCHW"),                    # relayout kernel first
    CONV_RESNET.replace("--operation conv", "--operation conv_bwd_weight"),               # filter gradient as one GEMM
    CONV_RESNET.replace("--operation conv", "--operation conv_bwd_weight") + " --kernel_id 1",
    CONV_RESNET.replace("--operation conv", "--operation conv_bwd_weight") + " --bwd_weight_gemm false --kernel_id 2",
])
def test_every_handle_gets_its_kernel_alone(rock, options):
    """miirBufferGet: a gfx950 ELF whose only kernel is the one the handle names, at most 512 KiB."""
    from rocmlir_amd._elf import kernel_symbols
    k = rock.RockKernel(options)
    blob = k.code_object()
    assert kernel_symbols(blob) == [k.kernel_name]
    assert len(blob) <= 512 * 1024


def test_null_handle_behaviour(rock):
    lib = rock.load_library()
    assert lib.miirGetKernelCount(None) == -1
    assert lib.miirLowerBin(None) == 1
    assert lib.miirLowerTuningParams(None) == 1
    assert lib.miirDestroyHandle(None) == 1
    n = C.c_size_t(0)
    assert lib.miirBufferGet(None, None, C.byref(n)) == 1


@pytest.mark.parametrize("bad", [
    "",                                                        # nothing
    "--operation conv --arch gfx950",                          # missing tensor keys
    CONV_RESNET.replace("--out_h 28", "--out_h 27"),           # inconsistent output size
    CONV_RESNET.replace("--conv_stride_h 1", "--conv_stride_h 0"),
    CONV_RESNET.replace("--padding_h 1", "--padding_h -1"),
    CONV_RESNET.replace("--in_layout NHWGC", "--in_layout NHWC3"),
    CONV_RESNET.replace("gfx950", "gfx906"),                   # no kernels for other chips
    CONV_RESNET.replace("--operation conv", "--operation conv_bwd_data").replace("fp16", "i8"),  # float gradients only
    CONV_RESNET.replace("--operation conv", "--operation conv_bwd_weight") + " --kernel_id 4",
    CONV_RESNET.replace("--fil_type fp16", "--fil_type fp32"),
    "--operation gemm --arch gfx950 -t f32 -m 4 -n 4",         # k missing
    "--operation gemm --arch gfx950 -t f32 -m 4 -n 4 -k 0",
    "--operation gemm --arch gfx950 -t f16 -out_datatype i32 -m 4 -n 4 -k 4",  # float in, int out
    "--operation gemm --arch gfx950 -t f16_i8 -m 4 -n 4 -k 4",
    "--operation attention --arch gfx950 -t f16 -g 1 -seq_len_q 8 -seq_len_k 8 -head_dim_qk 8",
    "--operation attention --arch gfx950 -t fp8 -g 1 -seq_len_q 8 -seq_len_k 8 -head_dim_qk 64 -head_dim_v 8",
    "--operation attention --arch gfx950 -t f16 -g 1 -seq_len_q 8 -seq_len_k 8 -head_dim_qk 256 -head_dim_v 8 "
    "--kernel_id 3",
    "--operation transpose --arch gfx950",
    CONV_IMPLICIT + " --kernel_id 1",
    CONV_RESNET + " --kernel_id 2",
    "-operation gemm -arch gfx950 -t f16 -g 1 -m 64 -n 64 -k 64 -store-method atomic_max",   # would change the result: refused, not ignored
    "-operation gemm -arch gfx950 -t fp8 -g 1 -m 64 -n 64 -k 64 -force-f8-types fnuz",
])
def test_bad_problems_give_null(rock, bad):
    lib = rock.load_library()
    assert not lib.miirCreateHandle(bad.encode())
    assert lib.rockamdGetLastError() != b""
    with pytest.raises(rock.RockError):
        rock.RockKernel(bad)


def test_baseline_configs_select_kernels(rock):
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f32 -g 1 -m 512 -n 512 -k 512 -transB true")
    # 64 output tiles of 64x64 would leave 3/4 of the CUs idle: K is split over waves
    assert k.kernel_name == "rock_gemm_f32_32x32_splitk"
    assert (k.block_size, k.grid_size) == (256, 256)
    assert k.perf_config == "v2:32,32,4,32,32,4,4,1,1"
    k = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -out_datatype f16 -g 1 -m 4096 -n 4096 "
                        "-k 4096 -transB true -scale 0.01")
    assert k.kernel_name == "rock_gemm_i8_256x256_fast"
    assert (k.block_size, k.grid_size) == (512, 256)
    assert k.execution_dims() == (512 * 256, 512)
    assert k.perf_config == "v2:256,256,8,128,16,16,1,1,1"
    # the 3x3 ResNet layer: the filter repacked for the window-resident kernel, then that kernel, two blocks per CU
    k = rock.RockKernel(CONV_RESNET)
    assert (k.kernel_name, k.kernel_count, k.workspace_bytes, k.caller_pointers) == ("rock_relayout_b2", 2, 128 * 1152 * 2, 5)
    k = rock.RockKernel(CONV_RESNET + " --kernel_id 1")
    assert (k.kernel_name, k.block_size, k.grid_size) == ("rock_conv_f16_direct224", 256, 1024)
    assert rock.RockKernel(CONV_IMPLICIT).kernel_name == "rock_conv_f16_128x128_fast"
    k = rock.RockKernel(CONV_RESNET + " --window_resident false")
    assert (k.kernel_name, k.kernel_count, k.workspace_bytes) == ("rock_conv_f16_128x128_fast", 1, 0)
    # a 64-channel layer would leave half of the window-resident kernel's waves idle: the table keeps it off
    k = rock.RockKernel(CONV_RESNET.replace("--out_channels 128", "--out_channels 64"))
    assert k.kernel_count == 1 and "direct224" not in k.kernel_name
    k = rock.RockKernel("-operation gemm -arch gfx950 -t fp8 -g 1 -m 8192 -n 8192 -k 8192 -transB true")
    assert k.kernel_name == "rock_gemm_fp8_256x256_fast" and k.grid_size == 1024
    k = rock.RockKernel("-operation attention -arch gfx950 -t f16 -g 128 -seq_len_q 2048 -seq_len_k 2048 "
                        "-head_dim_qk 128 -head_dim_v 128 -transK true -scale 0.08838834764831845")
    assert k.kernel_name == "rock_attention_f16_d128x128_fast"
    assert (k.block_size, k.grid_size, k.num_pointers, k.caller_pointers) == (256, 128 * 16, 8, 5)


def test_generic_kernels_for_unaligned_or_transposed(rock):
    odd_k = "-operation gemm -arch gfx950 -t f16 -g 3 -m 1024 -k 769 -n 1024 -transB true"
    k = rock.RockKernel(odd_k + " -layout_conversion false")
    assert k.kernel_name == "rock_gemm_f16_64x64_generic"          # odd K: no 16-byte chunks
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 64 -k 64 -n 60 -layout_conversion false")
    assert k.kernel_name == "rock_gemm_f16_64x64_generic"          # B is [K,N] with rows of 120 bytes
    # by default such operands are first copied into whole, zero-padded chunks (PrGemm.toml's
    # -k 769: the reference pads inside its kernel, GridwiseGemmParams.cpp:91-103) and the
    # vector kernel reads the copies: one launch copying both operands + the GEMM for the odd K,
    # a copy of B + the GEMM for N = 60
    plan = [rock.RockKernel("%s -kernel_id %d" % (odd_k, i)) for i in range(2)]
    assert plan[0].kernel_name == "rock_relayout_pair_b2" and plan[0].num_pointers == 4
    assert plan[1].kernel_name.startswith("rock_gemm_f16_") and plan[1].kernel_name.endswith("_fast")
    assert plan[0].kernel_count == 2 and plan[0].workspace_bytes == 2 * 3 * 1024 * 776 * 2
    assert plan[1].caller_pointers == 5 and plan[1].problem_key.endswith("-g 3 -m 1024 -n 1024 -k 769")
    n60 = [rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 64 -k 64 -n 60 -kernel_id %d" % i)
           for i in range(2)]
    assert n60[0].kernel_name == "rock_relayout_b2" and n60[1].kernel_name.endswith("_fast")
    assert n60[1].kernel_count == 2
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 64 -k 64 -n 64 -transA false -transB true")
    assert k.kernel_name.endswith("_fast")
    # K-major operands of whole 16-byte chunks take the transposing-read kernels
    for flags, suffix in (("", "_fast_nn"), ("-transA true", "_fast_tn"), ("-transA true -transB true", "_fast_tt")):
        k = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -g 1 -m 4096 -k 4096 -n 4096 " + flags)
        assert k.kernel_name == "rock_gemm_i8_256x256" + suffix
    nchw = CONV_RESNET.replace("NHWGC", "NGCHW").replace("GNYXC", "GNCHW")
    assert rock.RockKernel(nchw + " --layout_conversion false").kernel_name == "rock_conv_f16_64x64_generic"
    odd = CONV_RESNET.replace("--in_channels 128", "--in_channels 100")
    assert rock.RockKernel(odd + " --layout_conversion false").kernel_name == "rock_conv_f16_64x64_generic"


def test_pointwise_nchw_convolution_is_a_k_major_gemm(rock):
    """1x1, stride 1, no padding, one group, NCHW: filter[k,c] x image[c,h*w]
    batched over n on the transposing-read GEMM kernel, one kernel, no workspace."""
    pw = ("--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout GNCYX "
          "--in_layout NGCHW --out_layout NGCHW --batchsize 256 --groupsize 1 --in_channels 256 --out_channels 64 "
          "--in_h 56 --in_w 56 --fil_h 1 --fil_w 1 --dilation_h 1 --dilation_w 1 --conv_stride_h 1 "
          "--conv_stride_w 1 --padding_h 0 --padding_w 0")
    k = rock.RockKernel(pw)
    assert k.kernel_name.startswith("rock_gemm_f16_") and k.kernel_name.endswith("_fast_nn")
    assert (k.kernel_count, k.workspace_bytes, k.num_pointers, k.caller_pointers) == (1, 0, 5, 4)
    assert "convfp16" in k.problem_key and " -y 1 -x 1 " in k.problem_key
    # anything the GEMM form cannot express converts the image instead; the 1x1 filter, whose gkcyx form is
    # the channels-last one as it lies, is read in place
    for change in (("--conv_stride_h 1", "--conv_stride_h 2"), ("--padding_w 0", "--padding_w 1"),
                   ("--in_h 56 --in_w 56", "--in_h 7 --in_w 7"), ("--out_layout NGCHW", "--out_layout NHWGC")):
        k = rock.RockKernel(pw.replace(*change))
        assert k.kernel_count == 2, change
    assert rock.RockKernel(pw + " --bias true").kernel_count == 2
    assert rock.RockKernel(pw + " --pointwise_as_gemm false").kernel_count == 2
    from tests.test_conv3d_plan import _pointer_map
    conv = rock.RockKernel(pw + " --pointwise_as_gemm false --kernel_id 1")
    assert conv.kernel_name.startswith("rock_conv_f16_") and _pointer_map(rock, conv)[0] == (0, 0)


def test_layout_conversion_pads_channel_runs_to_whole_chunks(rock):
    """Channel runs that are not a multiple of 16 bytes (3-channel images, 100
    channels of f16) are zero-padded by the conversion kernels, so the vector
    contraction kernel runs with the padded count; the problem key keeps the
    caller's."""
    first = ("--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout GNYXC "
             "--in_layout NHWGC --out_layout NHWGK --batchsize 4 --groupsize 1 --in_channels 3 --out_channels 64 "
             "--in_h 230 --in_w 230 --fil_h 7 --fil_w 7 --dilation_h 1 --dilation_w 1 --conv_stride_h 2 "
             "--conv_stride_w 2 --padding_h 0 --padding_w 0")
    # (this layer has no padding along w and an even stride: by itself it takes the rows-of-taps plan,
    # tests/test_conv_narrow_channels_plan.py; the switch keeps it on the plan for any narrow layer)
    assert rock.RockKernel(first + " --kernel_id 2").kernel_name == "rock_conv_f16_64x64_fast_runs"
    first += " --tap_rows false"
    ks = [rock.RockKernel(first + " --kernel_id %d" % i) for i in range(3)]
    assert [k.kernel_name for k in ks[:2]] == ["rock_relayout_b2", "rock_relayout_b2"]
    assert ks[2].kernel_name.startswith("rock_conv_f16_") and ks[2].kernel_name.endswith("_fast")
    fil_bytes, in_bytes = 64 * 7 * 7 * 8 * 2, 4 * 230 * 230 * 8 * 2   # 3 -> 8 channels
    for k in ks:
        assert k.kernel_count == 3 and k.workspace_bytes == fil_bytes + in_bytes
    # n, h and w fold into one dimension; one thread per 16-byte chunk, 256 chunks a block
    assert ks[1].grid_size == -(-4 * 230 * 230 // 256)
    assert " -c 3 " in ks[2].problem_key
    # NCHW with the same channels: h and w fold; again one thread per pixel (one 16-byte chunk), 256 pixels a block
    k = rock.RockKernel(first.replace("NHWGC", "NGCHW") + " --kernel_id 1")
    assert k.kernel_name == "rock_relayout_b2" and k.grid_size == -(-4 * 230 * 230 // 256)
    # 128 channels: 64 x 64 tiles of 16-bit elements over (channel, folded pixel)
    nchw = CONV_RESNET.replace("NHWGC", "NGCHW").replace("GNYXC", "GNCHW")
    k = rock.RockKernel(nchw + " --kernel_id 1")
    assert k.grid_size == -(-28 * 28 // 64) * (128 // 64) * 256
    # int8: 16 channels a chunk
    k8 = rock.RockKernel(first.replace("fp16 --fil_type fp16 --out_type fp16", "i8 --fil_type i8 --out_type i32"))
    assert k8.workspace_bytes == 64 * 7 * 7 * 16 + (4 * 230 * 230 * 16 + 255) // 256 * 256


def test_layout_conversion_plan_follows_the_multi_kernel_protocol(rock):
    """NCHW tensors (the reference's default layouts): one conversion kernel
    per tensor, then the vector contraction kernel, behind miirGetKernelCount /
    --kernel_id / miirGetWorkspaceSize (rocmlir-lib.cpp:150-199)."""
    lib = rock.load_library()
    nchw = CONV_RESNET.replace("NHWGC", "NGCHW").replace("GNYXC", "GNCHW")
    ks = [rock.RockKernel(nchw + " --kernel_id %d" % i) for i in range(3)]
    assert [k.kernel_name for k in ks] == ["rock_relayout_b2", "rock_relayout_b2", "rock_conv_f16_128x128_fast"]
    fil_bytes, in_bytes = 128 * 128 * 9 * 2, 256 * 128 * 28 * 28 * 2
    for k in ks:
        assert k.kernel_count == 3 and k.caller_pointers == 5
        assert k.workspace_bytes == lib.miirGetWorkspaceSize(k._h) == fil_bytes + in_bytes
    maps = []
    for k in ks:
        ncall, nk = C.c_int(), C.c_int()
        src, off = (C.c_int32 * 8)(), (C.c_int64 * 8)()
        assert lib.rockamdGetPointerMap(k._h, C.byref(ncall), C.byref(nk), src, off) == 0
        assert ncall.value == 5 and nk.value == k.num_pointers
        maps.append([(src[i], off[i]) for i in range(nk.value)])
    # the contraction kernel's fifth pointer is the residual tensor: none here (-1 = pass NULL)
    assert maps == [[(0, 0), (4, 0)], [(1, 0), (4, fil_bytes)],
                    [(4, 0), (4, fil_bytes), (2, 0), (3, 0), (-1, 0)]]
    # with a residual the caller's list grows to six and the workspace moves to its end
    ks = [rock.RockKernel(nchw + " --residual add --kernel_id %d" % i) for i in range(3)]
    maps = []
    for k in ks:
        ncall, nk = C.c_int(), C.c_int()
        src, off = (C.c_int32 * 8)(), (C.c_int64 * 8)()
        assert lib.rockamdGetPointerMap(k._h, C.byref(ncall), C.byref(nk), src, off) == 0
        assert ncall.value == 6
        maps.append([(src[i], off[i]) for i in range(nk.value)])
    assert maps == [[(0, 0), (5, 0)], [(1, 0), (5, fil_bytes)],
                    [(5, 0), (5, fil_bytes), (2, 0), (3, 0), (4, 0)]]
    with pytest.raises(rock.RockError, match="kernel_id out of range"):
        rock.RockKernel(nchw + " --kernel_id 3")
    # only the input needs converting when the filter is already channel-contiguous
    mixed = CONV_RESNET.replace("--in_layout NHWGC", "--in_layout NGCHW")
    ks = [rock.RockKernel(mixed + " --kernel_id %d" % i) for i in range(2)]
    assert [k.kernel_name for k in ks] == ["rock_relayout_b2", "rock_conv_f16_128x128_fast"]
    assert ks[0].workspace_bytes == in_bytes
    # single-kernel problems: identity map, no workspace
    k = rock.RockKernel(CONV_IMPLICIT)
    assert (k.kernel_count, k.workspace_bytes, k.caller_pointers) == (1, 0, 4)
    # a conversion kernel has no epilogue scalars to set
    assert lib.rockamdSetScale(rock.RockKernel(nchw)._h, C.c_float(2.0)) != 0


def test_argument_info_describes_the_caller_list(rock):
    """Element type and dimensions per pointer, as mlirGetKernelInfo reports
    them per kernel argument (MIGraphX.cpp:54-90)."""
    k = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -out_datatype f16 -g 2 -m 64 -n 48 -k 32 -transB true "
                        "-scale 0.01 -residual add")
    assert k.arguments() == [(3, [2, 64, 32]), (3, [2, 48, 32]), (1, [2, 64, 48]), (0, [48]), (1, [2, 64, 48])]
    k = rock.RockKernel(CONV_IMPLICIT)
    assert k.arguments() == [(1, [1, 128, 3, 3, 128]), (1, [256, 28, 28, 1, 128]), (1, [256, 28, 28, 1, 128]),
                             (0, [128])]
    assert rock.RockKernel(CONV_RESNET).arguments() == k.arguments() + [(-1, [128 * 1152 * 2])]
    nchw = CONV_RESNET.replace("NHWGC", "NGCHW").replace("GNYXC", "GNCHW")
    args = rock.RockKernel(nchw + " --kernel_id 1").arguments()     # every kernel of a plan: the same list
    assert args[1] == (1, [256, 1, 128, 28, 28]) and args[4] == (-1, [rock.RockKernel(nchw).workspace_bytes])
    k = rock.RockKernel("-operation attention -arch gfx950 -t f16 -g 4 -seq_len_q 256 -seq_len_k 77 -head_dim_qk 64 "
                        "-head_dim_v 32 -transK true -with-attn-scale true")
    assert k.arguments() == [(1, [4, 256, 64]), (1, [4, 77, 64]), (1, [4, 77, 32]), (1, [4, 256, 77]),
                             (1, [4, 256, 77]), (1, [4, 256, 32])]
    lib = rock.load_library()
    assert lib.rockamdGetArgumentInfo(k._h, 6, None, None, None) != 0


def test_attention_pre_softmax_tensors(rock):
    """-with-attn-scale / -with-attn-bias (rocmlir-gen.cpp:2185-2196): the
    caller list is Q, K, V, [scale tensor], bias slot, O."""
    base = ("-operation attention -arch gfx950 -t f16 -g 4 -seq_len_q 256 -seq_len_k 256 -head_dim_qk 64 "
            "-head_dim_v 64 -transK true")
    assert rock.RockKernel(base).kernel_name == "rock_attention_f16_d64x64_fast"
    k = rock.RockKernel(base + " -with-attn-bias true")
    assert (k.kernel_name, k.caller_pointers) == ("rock_attention_f16_d64x64_fast_bias", 5)
    k = rock.RockKernel(base + " -with-attn-scale true")
    assert (k.kernel_name, k.caller_pointers, k.num_pointers) == ("rock_attention_f16_d64x64_fast_bias", 6, 8)


def test_attention_as_three_kernels(rock):
    """Head dimensions above 128 and f32 (attention-configs' sdxl vae lines):
    GEMM, row softmax in place over an f32 score workspace, GEMM."""
    vae = ("-operation attention -arch gfx950 -t %s -g 1 -seq_len_q 16384 -seq_len_k 16384 -head_dim_qk 512 "
           "-head_dim_v 512 -transK true")
    whole = " -score_workspace_limit %d" % (1 << 40)      # the whole score matrix in one piece
    for t in ("f16", "f32"):
        ks = [rock.RockKernel(vae % t + whole + " -kernel_id %d" % i) for i in range(3)]
        assert ks[0].kernel_name.startswith("rock_gemm_%s_" % t) and ks[0].kernel_name.endswith("_fast")
        assert ks[1].kernel_name == "rock_softmax_rows" and ks[1].grid_size == 16384
        assert ks[2].kernel_name.startswith("rock_gemm_%s_" % t) and ks[2].kernel_name.endswith("_fast_nn")
        assert all(k.kernel_count == 3 and k.workspace_bytes == 16384 * 16384 * 4 and k.caller_pointers == 6
                   for k in ks)
        # by default in chunks of at most 32 MiB of scores: 512 query rows x 16384 keys, 32 chunks of four kernels
        # (the second GEMM's 512 x 512 result in 8 shares of the keys, f32 partial sums behind the scores)
        ks = [rock.RockKernel(vae % t + " -kernel_id %d" % i) for i in (0, 1, 2, 3, 125, 126, 127)]
        assert all(k.kernel_count == 128 and k.workspace_bytes == (32 << 20) + 8 * 512 * 512 * 4 and
                   k.caller_pointers == 6 for k in ks)
        assert ks[1].kernel_name == "rock_softmax_rows" and ks[1].grid_size == 512
        assert ks[2].kernel_name.startswith("rock_gemm_%s_" % t) and struct.unpack_from("<4i", ks[2].params(), 72) == (8, 512, 512, 2048)   # G M N K
        assert ks[3].kernel_name == "rock_reduce_splits" and ks[6].kernel_name == "rock_reduce_splits"
        assert ks[4].kernel_name == "rock_softmax_rows" and ks[5].kernel_name == ks[2].kernel_name
        with pytest.raises(rock.RockError):
            rock.RockKernel(vae % t + " -kernel_id 128")
        three = [rock.RockKernel(vae % t + " -split_k false -kernel_id %d" % i) for i in (0, 95)]
        assert all(k.kernel_count == 96 and k.workspace_bytes == 32 << 20 for k in three)
    # many small groups: whole groups per chunk (8 x 2048 x 2048 f32 scores = 128 MiB -> 2 groups a chunk)
    k = rock.RockKernel("-operation attention -arch gfx950 -t f32 -g 7 -seq_len_q 2048 -seq_len_k 2048 "
                        "-head_dim_qk 64 -head_dim_v 64 -transK true -kernel_id 9")
    assert k.kernel_count == 12 and k.workspace_bytes == 32 << 20 and k.grid_size > 0
    # int8 first GEMM: one fused kernel where the layout allows it (its score tile is dequantised in
    # registers); "-fused false", K stored [G, d, seq_k] or a head dimension above 128 give the three
    # kernels: int8 contraction into f32 scores, f16 from there on
    i8 = ("-operation attention -arch gfx950 -t i8 -g 2 -seq_len_q 128 -seq_len_k 128 -head_dim_qk 64 "
          "-head_dim_v 64 -transK true -zero_point 3 -scale 0.001")
    fused = rock.RockKernel(i8)
    assert fused.kernel_name == "rock_attention_i8_d64x64_fast" and fused.kernel_count == 1
    assert fused.workspace_bytes == 0 and fused.caller_pointers == 5
    with pytest.raises(rock.RockError):
        rock.RockKernel(i8 + " -kernel_id 1")
    # K stored [G, d, seq_k]: a copy to [G, seq_k, d] in front of the fused kernel
    copied = i8.replace("-transK true", "-transK false")
    plan = [rock.RockKernel(copied + " -kernel_id %d" % i) for i in range(2)]
    assert [k.kernel_name for k in plan] == ["rock_relayout_b1", "rock_attention_i8_d64x64_fast"]
    assert all(k.kernel_count == 2 and k.workspace_bytes == 2 * 128 * 64 and k.caller_pointers == 6 for k in plan)
    for three in (i8 + " -fused false", copied + " -layout_conversion false",
                  i8.replace("-head_dim_qk 64", "-head_dim_qk 256")):
        q8 = [rock.RockKernel(three + " -kernel_id %d" % i) for i in range(3)]
        assert q8[0].kernel_name.startswith("rock_gemm_i8_") and q8[2].kernel_name.startswith("rock_gemm_f16_")
        assert q8[1].kernel_name == "rock_softmax_rows" and q8[0].kernel_count == 3
    lib = rock.load_library()
    k = rock.RockKernel((vae % "f16").replace("-g 1 ", "-g 4 ") + whole)
    assert k.workspace_bytes == 4 * 16384 * 16384 * 4 and lib.miirGetWorkspaceSize(k._h) == -1   # beyond an int


def test_backward_convolution_plans(rock):
    """conv_bwd_data / conv_bwd_weight behind the multi-kernel protocol
    (rocmlir-lib.cpp:150-199): kernel lists, workspace, problem keys with the
    reference's direction codes (RockTuningImpl.cpp:759-772)."""
    bwd_data = CONV_RESNET.replace("--operation conv", "--operation conv_bwd_data")
    # (this unit-stride layer fills the window-resident kernel's tiles: the table takes it, "--window_resident false"
    # keeps the implicit-GEMM kernel; either way one filter conversion and one contraction)
    for switch, name in (("", "rock_conv_f16_direct224"), (" --window_resident false", "rock_conv_f16_128x128_fast")):
        ks = [rock.RockKernel(bwd_data + switch + " --kernel_id %d" % i) for i in range(2)]
        assert [k.kernel_name for k in ks] == ["rock_relayout_b2", name]
        assert all(k.kernel_count == 2 and k.workspace_bytes == 128 * 128 * 9 * 2 and k.caller_pointers == 5 for k in ks)
        assert "convfp16 -F 2 " in ks[1].problem_key
    # stride 2: one sub-filter conversion and one convolution per phase of the input grid
    s2 = bwd_data.replace("--conv_stride_h 1 --conv_stride_w 1", "--conv_stride_h 2 --conv_stride_w 2") \
                 .replace("--out_h 28 --out_w 28", "--out_h 14 --out_w 14")
    k = rock.RockKernel(s2)
    assert k.kernel_count == 8
    # 1x1 filter, stride 2: three phases get no tap and are cleared by the zero-fill kernel
    s3 = s2.replace("--fil_h 3 --fil_w 3", "--fil_h 1 --fil_w 1").replace("--padding_h 1 --padding_w 1",
                                                                          "--padding_h 0 --padding_w 0")
    names = [rock.RockKernel(s3 + " --kernel_id %d" % i).kernel_name for i in range(rock.RockKernel(s3).kernel_count)]
    assert names == ["rock_fill_zero", "rock_relayout_b2", "rock_conv_f16_128x128_fast"]
    # tensors as they lie: one element-wise kernel per phase, no workspace pointer
    k = rock.RockKernel(s2 + " --layout_conversion false")
    assert (k.kernel_count, k.workspace_bytes, k.caller_pointers) == (4, 0, 4)
    assert k.kernel_name == "rock_conv_f16_64x64_generic"
    # channels-last, one group: one K-major GEMM over the tensors as they lie (the second operand is the
    # im2col matrix, gathered by the kernel) into f32 partial sums per pixel split, and their reduction
    bwd_w = CONV_RESNET.replace("--operation conv", "--operation conv_bwd_weight")
    ks = [rock.RockKernel(bwd_w + " --kernel_id %d" % i) for i in range(2)]
    assert [k.kernel_name for k in ks] == ["rock_conv_bwd_weight_f16_128x128", "rock_reduce_splits"]
    splits = ks[0].grid_size // 9                      # 128 x 1152 gradient: nine 128 x 128 tiles per split
    assert ks[0].grid_size == 9 * splits and (256 * 28 * 28) % splits == 0 and splits >= 32
    assert all(k.kernel_count == 2 and k.caller_pointers == 5 and k.workspace_bytes == splits * 128 * 1152 * 4
               for k in ks)
    assert "convfp16 -F 4 " in ks[0].problem_key
    # the plan it replaces, still there for the other layouts: two copies, a forward kernel, the reduction
    old = bwd_w + " --bwd_weight_gemm false"
    names = [rock.RockKernel(old + " --kernel_id %d" % i).kernel_name for i in range(4)]
    assert names[:2] == ["rock_relayout_b2", "rock_relayout_b2"] and names[3] == "rock_reduce_splits"
    assert names[2].startswith("rock_conv_f16_") and names[2].endswith("_fast")
    assert "convfp16 -F 4 " in rock.RockKernel(old + " --kernel_id 2").problem_key
    # any other gradient layout comes out of the reduction kernel; tensors that are not channels-last are
    # first copied into that form
    kcyx = bwd_w.replace("GNYXC", "GNCHW")
    assert [rock.RockKernel(kcyx + " --kernel_id %d" % i).kernel_name for i in range(2)] == \
        ["rock_conv_bwd_weight_f16_128x128", "rock_reduce_splits"]
    nchw = kcyx.replace("NHWGC", "NGCHW")
    assert [rock.RockKernel(nchw + " --kernel_id %d" % i).kernel_name for i in range(4)] == \
        ["rock_relayout_b2", "rock_relayout_b2", "rock_conv_bwd_weight_f16_128x128", "rock_reduce_splits"]
    k = rock.RockKernel(old + " --layout_conversion false")
    assert (k.kernel_count, k.workspace_bytes, k.kernel_name) == (1, 0, "rock_conv_f16_64x64_generic")


def test_elementwise_epilogue_options(rock):
    """The element-wise tail MIGraphX fuses behind a contraction
    (MIGraphXToTosa.cpp:1009-1016, 1089-1100, 1283-1295): activation names,
    clip bounds, a residual tensor as a fifth pointer."""
    base = "-operation gemm -arch gfx950 -t f16 -g 1 -m 256 -n 256 -k 256 -transB true"
    k = rock.RockKernel(base)
    assert (k.num_pointers, k.caller_pointers) == (5, 4)
    # relu and clip are a clamp in the plain kernel; the transcendental ones and a
    # residual take the kernel's rolled-epilogue twin ("_e")
    for act in ("relu", "none", "clip -clip_min 0 -clip_max 6"):
        assert rock.RockKernel(base + " -activation " + act).kernel_name == k.kernel_name
    for act in ("sigmoid", "tanh", "erf", "gelu", "exp"):
        assert rock.RockKernel(base + " -activation " + act).kernel_name == k.kernel_name + "_e"
    assert rock.RockKernel(base + " -residual add").kernel_name == k.kernel_name + "_e"
    assert rock.RockKernel(base + " -activation clip -clip_min 0 -clip_max 6").caller_pointers == 4
    # the element-wise kernels handle every epilogue themselves
    odd = base.replace("-k 256", "-k 255") + " -layout_conversion false"
    assert rock.RockKernel(odd + " -activation erf").kernel_name == rock.RockKernel(odd).kernel_name
    assert rock.RockKernel(odd).kernel_name.endswith("_generic")
    for bad in (" -activation swish", " -activation clip", " -activation clip -clip_min 2 -clip_max 1",
                " -residual sub"):
        with pytest.raises(rock.RockError):
            rock.RockKernel(base + bad)
    for op in ("add", "mul"):
        assert rock.RockKernel(base + " -residual " + op).caller_pointers == 5
    # integer results stay integer: no float activation, but an integer residual is fine
    i8 = "-operation gemm -arch gfx950 -t i8 -g 1 -m 256 -n 256 -k 256 -transB true"
    with pytest.raises(rock.RockError):
        rock.RockKernel(i8 + " -activation tanh")
    assert rock.RockKernel(i8 + " -residual add").caller_pointers == 5
    assert rock.RockKernel(i8 + " -out_datatype f16 -scale 0.01 -activation tanh").caller_pointers == 4


def test_perf_config_override_and_fallback(rock):
    base = "-operation gemm -arch gfx950 -t i8 -g 1 -m 4096 -n 4096 -k 4096 -transB true"
    assert rock.RockKernel(base + " -perf_config v2:128,128,8,64,16,16,1,1,1").kernel_name == \
        "rock_gemm_i8_128x128_fast"
    # a config naming no available tile falls back to the table
    assert rock.RockKernel(base + " -perf_config v2:48,48,8,16,16,16,1,1,1").kernel_name == \
        "rock_gemm_i8_256x256_fast"
    # the split-K tile can be asked for by name as well
    assert rock.RockKernel(base + " -perf_config v2:32,32,4,32,32,16,4,1,1").kernel_name == \
        "rock_gemm_i8_32x32_splitk"


def test_problem_keys_follow_reference_format(rock):
    # mlir/test/rocmlir-gen/problem-key.mlir CHECK_2 / CHECK_4 (numCU in the key)
    k = rock.RockKernel("--arch gfx950 --num_cu 304 --operation attention -seq_len_q 256 -seq_len_k 512 "
                        "-head_dim_qk 64 -head_dim_v 32 -t f16 -g 4")
    arch, ncu, prob = k.problem_key.split("\t")
    assert (arch, ncu) == ("gfx950", "304")
    assert prob == ("-t f16 -transQ false -transK false -transV false -transO false -g 4 "
                    "-seq_len_q 256 -seq_len_k 512 -head_dim_qk 64 -head_dim_v 32")
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 1024 -n 512 -k 769 -transB true")
    assert k.problem_key.split("\t")[2] == \
        "-t f16 -out_datatype f16 -transA false -transB true -g 1 -m 1024 -n 512 -k 769"
    k = rock.RockKernel(CONV_RESNET + " --kernel_id 1")
    assert rock.RockKernel(CONV_IMPLICIT).problem_key == k.problem_key
    assert k.problem_key.split("\t")[2] == (
        "convfp16 -F 1 -f GN01C -I N01GC -O N01GC -n 256 -c 128 -H 28 -W 28 -k 128 -y 3 -x 3 "
        "-p 1 -q 1 -u 1 -v 1 -l 1 -j 1 -g 1")


def test_param_block_and_setters(rock):
    k = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -out_datatype f16 -g 1 -m 64 -n 64 -k 64 "
                        "-transB true -scale 0.5 -zero_point 3")
    import struct
    blob = k.params()
    # strides, sizes / tiling, epilogue scalars, per-channel vector flags + padding + four pointer fields
    assert len(blob) == k.params_size == 9 * 8 + 8 * 4 + 10 * 4 + 2 * 4 + 4 * 8
    assert struct.unpack_from("i", blob, 72 + 32 + 40) == (0,) and not any(blob[72 + 32 + 48:])   # no vectors
    G, M, N, K = struct.unpack_from("4i", blob, 72)
    assert (G, M, N, K) == (1, 64, 64, 64)
    scale, inv_q, zp = struct.unpack_from("ffi", blob, 72 + 32)
    assert (scale, inv_q, zp) == (0.5, 1.0, 3)
    k.set_scale(0.25)
    k.set_zero_point(-2)
    scale, inv_q, zp = struct.unpack_from("ffi", k.params(), 72 + 32)
    assert (scale, zp) == (0.25, -2)


def test_tuning_space_lists_the_kernels_a_problem_can_run_on(rock):
    """mlirRockTuningSpaceCreate / GetNumParams / ParamGet / ToString
    (mlir-c/Dialect/Rock.h:39-84): entry 0 is the table's choice, every entry
    selects a different kernel, and strings follow the v2 grammar."""
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 4096 -n 4096 -k 4096 -transB true")
    space = k.tuning_space()
    assert space[0] == k.perf_config
    # RocmlirTuningParamSetKind (RockEnums.h:19-23): quick is a prefix of full, exhaustive holds full
    quick, exhaustive = k.tuning_space("quick"), k.tuning_space("exhaustive")
    assert quick == space[:3]
    assert exhaustive[:len(space)] == space
    names = []
    for perf in space:
        assert re.fullmatch(r"v2:\d+(,\d+){8}", perf)
        k.set_perf_config(perf)
        assert k.perf_config == perf
        names.append(k.kernel_name)
    assert len(set(names)) == len(names) == 5  # four tiles and the K-split kernel
    # a convolution the window-resident kernel can run offers it
    assert "v2:224,128,8,224,32,8,1,1,1" in rock.RockKernel(CONV_RESNET).tuning_space()
    # exhaustive: every tile once more as the twin with the rolled epilogue (forceUnroll 0)
    assert len(exhaustive) == len(space) + 4 and "v2:256,256,8,128,16,8,1,0,1" in exhaustive
    k.set_perf_config("v2:256,256,8,128,16,8,1,0,1")
    assert k.kernel_name == "rock_gemm_f16_256x256_fast_e" and k.perf_config == "v2:256,256,8,128,16,8,1,0,1"
    # attention: the three kernels a plain problem can run on, in "attn:v1:" strings that
    # are accepted back (RockAttrDefs.td:241-329, parser RockDialect.cpp:2122-2170); a head
    # dimension of 64 can also run on the 128 instantiation
    att = rock.RockKernel("--arch gfx950 --operation attention -seq_len_q 256 -seq_len_k 512 "
                          "-head_dim_qk 128 -head_dim_v 128 -t f16 -g 4 -transK true")
    sp = att.tuning_space()
    assert sp[0] == att.perf_config == "attn:v1:64,128,128,8,32,32,8,1" and len(sp) == 3
    kernels = []
    for perf in sp:
        assert re.fullmatch(r"attn:v1:\d+(,\d+){7}", perf)
        att.set_perf_config(perf)
        assert att.perf_config == perf
        kernels.append(att.kernel_name)
    assert kernels == ["rock_attention_f16_d128x128_fast", "rock_attention_f16_d128x128_fast_bias",
                       "rock_attention_f16_d128x128_generic"]
    att64 = rock.RockKernel("--arch gfx950 --operation attention -seq_len_q 256 -seq_len_k 512 "
                            "-head_dim_qk 64 -head_dim_v 64 -t f16 -g 4 -transK true")
    assert len(att64.tuning_space()) == 6
    att64.set_perf_config("attn:v1:64,128,128,8,32,32,8,1")
    assert att64.kernel_name == "rock_attention_f16_d128x128_fast"
    # with a bias the pipelined kernel is not on offer, and asking for it falls back
    attb = rock.RockKernel("--arch gfx950 --operation attention -seq_len_q 256 -seq_len_k 512 "
                           "-head_dim_qk 128 -head_dim_v 128 -t f16 -g 4 -transK true -with-attn-bias true")
    assert len(attb.tuning_space()) == 2
    attb.set_perf_config("attn:v1:64,128,128,8,32,32,8,1")
    assert attb.kernel_name == "rock_attention_f16_d128x128_fast_bias"
    # K-major operands have the three square tiles; unaligned ones only the generic kernel
    nn = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 256 -n 256 -k 256")
    assert len(nn.tuning_space()) == 3
    gen = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 256 -n 250 -k 256 -layout_conversion false")
    assert gen.tuning_space() == [gen.perf_config]
    # ... unless they are copied into padded ones first: the GEMM handle of that plan has the K-contiguous tiles
    padded = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 256 -n 250 -k 256 -kernel_id 1")
    assert padded.kernel_count == 2 and len(padded.tuning_space()) >= 4
    # raw entry points: bad position, short buffer
    lib = rock.load_library()
    sp = lib.rockamdTuningSpaceCreate(k._h, 1)
    assert lib.rockamdTuningGetNumParams(sp) == 5
    assert lib.rockamdTuningParamToString(sp, 99, None, 0) == C.c_size_t(-1).value
    # a short buffer gets what fits, terminated; the full length comes back
    buf = C.create_string_buffer(b"\xff" * 8, 8)
    n = lib.rockamdTuningParamToString(sp, 0, buf, 4)
    assert n == len(space[0]) and buf.raw[:3] == space[0][:3].encode() and buf.raw[3] == 0
    assert buf.raw[4:] == b"\xff" * 4
    lib.rockamdTuningSpaceDestroy(sp)
    assert lib.rockamdTuningSpaceCreate(None, 0) is None
    assert lib.rockamdTuningSpaceCreate(k._h, 7) is None
    for getter in (lib.rockamdGetPerfConfig, lib.rockamdGetProblemKey):
        buf = C.create_string_buffer(b"\xff" * 8, 8)
        n = getter(k._h, buf, 5)
        assert n > 5 and buf.raw[4] == 0 and buf.raw[5:] == b"\xff" * 3


def test_set_perf_config_keeps_epilogue_scalars_and_launch_geometry(rock):
    import struct
    k = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -out_datatype f16 -g 1 -m 1024 -n 1024 -k 1024 "
                        "-transB true -scale 0.5")
    k.set_scale(0.125)
    k.set_perf_config("v2:64,64,8,32,16,16,1,1,1")
    assert k.kernel_name == "rock_gemm_i8_64x64_fast"
    assert (k.block_size, k.grid_size) == (256, 16 * 16)
    assert k.execution_dims() == (256 * 256, 256)
    assert struct.unpack_from("f", k.params(), 72 + 32)[0] == 0.125
    assert len(k.code_object()) > 1000


def test_tuning_table_keeps_the_best_entry(rock, tmp_path):
    """mlirRockTuningUpdateTable / SetFromTable (Rock.h:94-117)."""
    from rocmlir_amd import tuning
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 4096 -n 4096 -k 4096 -transB true")
    other = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 512 -n 4096 -k 4096 -transB true")
    t = tuning.TuningTable()
    assert not t.apply(k)
    assert t.update(k.problem_key, "v2:64,64,8,32,16,8,1,1,1", 2.0)
    assert t.update(k.problem_key, "v2:128,128,8,64,16,8,1,1,1", 1.0)      # faster: replaces
    assert not t.update(k.problem_key, "v2:64,64,8,32,16,8,1,1,1", 1.5)   # slower: refused
    assert t.apply(k) and k.kernel_name == "rock_gemm_f16_128x128_fast"
    untouched = other.kernel_name
    assert not t.apply(other) and other.kernel_name == untouched
    # the text form is the reference's four-column tuning database
    path = tmp_path / "gfx950.tuning"
    t.save(str(path))
    line = path.read_text().splitlines()
    assert len(line) == 1 and line[0].split("\t") == ["gfx950", "256", k.problem_key.split("\t")[2],
                                                      "v2:128,128,8,64,16,8,1,1,1"]
    again = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 4096 -n 4096 -k 4096 -transB true")
    assert tuning.TuningTable.load(str(path)).apply(again)
    assert again.kernel_name == "rock_gemm_f16_128x128_fast"


def test_split_k_likelihood(rock):
    """mlirIsSplitKFaster (Rock.h:136-142) for this library's K-split kernel:
    ALWAYS exactly where the built-in table picks it."""
    lib = rock.load_library()
    never, maybe, always = 0, 1, 2
    assert lib.rockamdIsSplitKFaster(1, 512, 512, 512, 256, 4) == always
    assert rock.RockKernel("-operation gemm -arch gfx950 -t f32 -g 1 -m 512 -n 512 -k 512 "
                           "-transB true").kernel_name.endswith("_splitk")
    assert lib.rockamdIsSplitKFaster(1, 1024, 1024, 4096, 256, 2) == maybe
    assert lib.rockamdIsSplitKFaster(1, 4096, 4096, 4096, 256, 1) == never
    assert lib.rockamdIsSplitKFaster(1, 64, 64, 64, 256, 2) == never   # K too short to split
    assert lib.rockamdIsSplitKFaster(0, 64, 64, 4096, 256, 2) == never


def test_product_does_not_touch_the_oracle():
    """The shipped package must not import, load or link the CPU oracle."""
    pkg = os.path.join(ROOT, "rocmlir_amd")
    for dirpath, _, files in os.walk(pkg):
        if "_build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".h", ".hip", ".S", ".inc")):
                text = open(os.path.join(dirpath, f)).read()
                assert "rock_oracle" not in text and "oracle/" not in text, f


def test_window_resident_request_with_asymmetric_padding_falls_back(rock):
    """The window-resident kernel sizes its LDS window from the top / left
    padding alone, so a problem whose two sides differ must not get it."""
    asym = (CONV_RESNET.replace("--padding_h 1", "--padding_h_l 0 --padding_h_r 1")
            .replace("--fil_h 3", "--fil_h 2").replace("--out_h 28", "--out_h 28"))
    base = rock.RockKernel(asym)
    asked = rock.RockKernel(asym + " --perf_config v2:224,128,8,224,32,8,1,1,1")
    assert "direct224" not in asked.kernel_name and asked.kernel_name == base.kernel_name
    assert "v2:224,128,8,224,32,8,1,1,1" not in base.tuning_space()
    sym = rock.RockKernel(CONV_RESNET + " --perf_config v2:224,128,8,224,32,8,1,1,1 --kernel_id 1")
    assert sym.kernel_name == "rock_conv_f16_direct224"


def test_reference_style_perf_config_keeps_its_tile(rock):
    """A reference-style string carries MPerWave = 32 and MnPerXdl = 32 in its
    fourth and fifth fields; only the FIRST two fields name the block tile."""
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 4096 -n 4096 -k 4096 -transB true "
                        "-perf_config v2:64,64,8,32,32,8,1,1,1")
    assert k.kernel_name == "rock_gemm_f16_64x64_fast" and k.grid_size == 64 * 64
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 4096 -n 4096 -k 4096 -transB true "
                        "-perf_config v2:32,32,4,32,32,8,4,1,1")
    assert k.kernel_name == "rock_gemm_f16_32x32_splitk"
    conv = rock.RockKernel(CONV_RESNET + " --perf_config v2:128,128,8,224,128,8,1,1,1")
    assert conv.kernel_name == "rock_conv_f16_128x128_fast"


def test_reduction_split_over_blocks_covers_both_storages(rock):
    """A single float GEMM with few output tiles and a long K is cut over
    blocks whichever way its operands are stored."""
    for flags in ("-transB true", ""):
        k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 16384 " + flags)
        assert k.kernel_count == 2 and k.workspace_bytes > 0, flags
        assert k.grid_size >= 128, (flags, k.kernel_name, k.grid_size)
        red = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 16384 %s -kernel_id 1" % flags)
        assert red.kernel_name == "rock_reduce_splits"
    one = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 16384 -transB true -split_k false")
    assert one.kernel_count == 1 and one.kernel_name == "rock_gemm_f16_32x32_splitk"


def test_attention_scale_sign_selects_the_kernel(rock):
    """The plain fused kernel takes the row maximum before scaling, which needs
    a non-negative scale; rockamdSetScale moves the handle when the sign changes."""
    opts = ("-operation attention -arch gfx950 -t f16 -g 2 -seq_len_q 256 -seq_len_k 256 "
            "-head_dim_qk 64 -head_dim_v 64 -transK true -scale 0.125")
    k = rock.RockKernel(opts)
    assert k.kernel_name == "rock_attention_f16_d64x64_fast"
    k.set_scale(-0.125)
    k._refresh()
    assert k.kernel_name == "rock_attention_f16_d64x64_fast_bias"
    k.set_scale(0.5)
    k._refresh()
    assert k.kernel_name == "rock_attention_f16_d64x64_fast"
    b = rock.RockKernel(opts + " -with-attn-bias true")
    b.set_scale(0.5)
    b._refresh()
    assert b.kernel_name == "rock_attention_f16_d64x64_fast_bias"


def test_attention_set_scale_keeps_a_code_object(rock):
    """Head dimension 256 exists only as the scale-first kernel: rockamdSetScale must leave the handle on it
    (kernel name, perf_config with its 256 tile, a code object that still lowers), whatever the sign; and a
    handle put on the scale-first kernel by its perf_config stays there when the scale is set."""
    opts = ("-operation attention -arch gfx950 -t f16 -g 2 -seq_len_q 256 -seq_len_k 256 "
            "-head_dim_qk 256 -head_dim_v 256 -transK true -scale 0.125")
    k = rock.RockKernel(opts)
    assert k.kernel_name == "rock_attention_f16_d256x256_fast_bias"
    size = len(k.code_object())
    for scale in (0.0625, -0.0625, 0.25):
        k.set_scale(scale)
        k._refresh()
        assert k.kernel_name == "rock_attention_f16_d256x256_fast_bias"
        assert k.perf_config.split(":")[2].split(",")[1] == "256"
        assert len(k.code_object()) == size
    chosen = rock.RockKernel(opts.replace("256 -head_dim_v 256", "64 -head_dim_v 64") +
                             " -perf_config attn:v1:64,64,128,8,32,32,8,0")
    assert chosen.kernel_name == "rock_attention_f16_d64x64_fast_bias"
    chosen.set_scale(0.5)
    chosen._refresh()
    assert chosen.kernel_name == "rock_attention_f16_d64x64_fast_bias"


def test_fusibility_and_prefill_queries(rock):
    """mlirIsModuleFusible / mlirGetNumPrefillArgs (mlir-c/Dialect/Rock.h:145-158)."""
    lib = rock.load_library()
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 4096 -transB true "
                        "-bias true -activation relu")
    assert lib.rockamdIsFusible(k._h, b"v2:32,32,4,32,32,8,4,1,1") == 1   # split inside the block: tail stays
    assert lib.rockamdIsFusible(k._h, b"v2:128,128,8,64,16,8,1,1,1") == 1
    assert lib.rockamdIsFusible(None, b"v2:128,128,8,64,16,8,1,1,1") == 0
    assert lib.rockamdIsFusible(k._h, None) == 0
    assert lib.rockamdGetNumPrefillArgs(k._h) == 0
    idx, val = (C.c_size_t * 2)(7, 7), (C.c_float * 2)(7.0, 7.0)
    lib.rockamdGetPrefillArgsInfo(k._h, idx, val, 0)
    assert list(idx) == [7, 7]


def test_operands_beyond_31_bit_offsets_leave_the_vector_kernels(rock):
    """The direct-to-LDS loads address a block's operand rows with 32-bit byte
    offsets below 2^31: 256 rows plus one of about 8 MiB each cannot, and such a
    problem must run on the element-wise kernel instead."""
    ok = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -g 1 -m 256 -n 256 -k 8355840 -transB true")
    assert "_generic" not in ok.kernel_name
    big = rock.RockKernel("-operation gemm -arch gfx950 -t i8 -g 1 -m 256 -n 256 -k 8356096 -transB true")
    assert big.kernel_name == "rock_gemm_i8_64x64_generic"
    km = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 1048576 -n 256 -k 2048 -transA true -transB true")
    assert km.kernel_name == "rock_gemm_f16_64x64_generic"   # K-major A: k * M * 2 bytes passes 2^31


def test_handles_from_eight_threads(rock):
    """The header promises that entry points may be called from several threads
    (one handle per thread): create, query, re-tune and destroy concurrently."""
    import threading
    errors = []

    def work(i):
        try:
            for j in range(40):
                m = 64 * (1 + (i + j) % 9)
                k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m %d -n 256 -k 512 -transB true" % m)
                assert k.grid_size > 0 and k.kernel_name.startswith("rock_gemm_f16_")
                space = k.tuning_space()
                k.set_perf_config(space[-1])
                assert k.perf_config == space[-1]
                bad = rock.load_library().miirCreateHandle(b"--operation gemm --arch gfx950 -t f16 -m 4")
                assert not bad and rock.api.last_error() != ""
                del k
        except Exception as e:  # noqa: BLE001 - collected for the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_tuning_table_shared_by_threads(rock):
    """mlirRockTuningUpdateTable keeps the best entry under a lock
    (RockTuningImpl.cpp:902-931): concurrent updates of one key must end with the minimum."""
    import threading
    from rocmlir_amd.tuning import TuningTable
    lib = rock.load_library()
    table = TuningTable()
    key = b"gfx950\t256\t-t f16 -out_datatype f16 -transA false -transB true -g 1 -m 64 -n 256 -k 512"

    def work(i):
        for j in range(200):
            t = 1.0 + ((i * 200 + j) * 7919 % 1000) / 10.0
            lib.rockamdTuningUpdateTable(table._t, key, b"v2:64,64,8,32,16,8,1,1,1" if t > 1.0 else
                                         b"v2:128,128,8,64,16,8,1,1,1", C.c_float(t))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert lib.rockamdTuningUpdateTable(table._t, key, b"v2:64,64,8,32,16,8,1,1,1", C.c_float(1.0)) == 0
    assert lib.rockamdTuningUpdateTable(table._t, key, b"v2:64,64,8,32,16,8,1,1,1", C.c_float(0.5)) == 1


def test_split_plans_round_trip_through_their_perf_config(rock):
    """A plan whose reduction is split over blocks reports the split in the splitK field of its perf_config
    (RockAttrDefs.td:241-251), and applying that string again leads back to the same plan: same kernels, same
    workspace, for every kernel_id; splitK 1 names the unsplit plan; the tuning space lists both."""
    conv = ("--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout gkyxc "
            "--in_layout nhwgc --out_layout nhwgk --batchsize 2 --groupsize 1 --in_channels 1920 --out_channels 1280 "
            "--in_h 16 --in_w 16 --fil_h 3 --fil_w 3 --dilation_h 1 --dilation_w 1 --conv_stride_h 1 "
            "--conv_stride_w 1 --padding_h 1 --padding_w 1")
    problems = [conv, conv.replace("--operation conv", "--operation conv_bwd_data"),
                "-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 1280 -k 5120",
                "-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 16384 -transB true"]
    for opts in problems:
        flag = "--" if opts.startswith("--") else "-"
        first = rock.RockKernel(opts)
        assert first.kernel_count >= 2 and first.workspace_bytes > 0
        # the contraction kernel of the plan carries the string
        plan = [rock.RockKernel("%s %skernel_id %d" % (opts, flag, i)) for i in range(first.kernel_count)]
        strings = [k.perf_config for k in plan if k.perf_config]
        assert len(strings) == 1
        pc = strings[0]
        assert int(pc.split(":")[1].split(",")[6]) > 1
        for i, k in enumerate(plan):
            again = rock.RockKernel("%s %skernel_id %d %sperf_config %s" % (opts, flag, i, flag, pc))
            assert (again.kernel_name, again.kernel_count, again.workspace_bytes, again.grid_size) == \
                   (k.kernel_name, k.kernel_count, k.workspace_bytes, k.grid_size)
            k.set_perf_config(pc)       # rockamdTuningSetFromStr on a separately held handle
            assert (k.kernel_name, k.kernel_count, k.workspace_bytes) == \
                   (again.kernel_name, again.kernel_count, again.workspace_bytes)
        # splitK = 1: the same tile without the split
        fields = pc.split(":")[1].split(",")
        fields[6] = "4" if fields[:2] == ["32", "32"] else "1"
        single = rock.RockKernel("%s %sperf_config v2:%s" % (opts, flag, ",".join(fields)))
        assert single.kernel_count < first.kernel_count
        space = plan[[bool(k.perf_config) for k in plan].index(True)].tuning_space("full")
        assert space[0] == pc
        assert any(int(t.split(":")[1].split(",")[6]) in (1, 4) and t.split(",")[:2] == pc.split(",")[:2] for t in space[1:])


def test_reference_attention_list_resolves_to_fused_vector_kernels(rock):
    """Every case of mlir/test/e2e/PrAttentionF16.toml:20-67, with -transK true and false (its axis, :10-13), and
    the int8 shape of mixr-attention-first-gemm-i8.mlir:6-10 (K stored [G, d, seq_k]) end on a fused vector
    kernel, conversion kernels around it where a tensor is not laid out for it."""
    cases = ["-seq_len_q 384 -seq_len_k 384 -head_dim_qk 64 -head_dim_v 64",
             "-seq_len_q 64 -seq_len_k 64 -head_dim_qk 64 -head_dim_v 64 -perf_config attn:v1:32,32,64,32,32,32,4,1",
             "-seq_len_q 256 -seq_len_k 256 -head_dim_qk 128 -head_dim_v 128 -perf_config attn:v1:128,128,128,32,64,64,4,1",
             "-seq_len_q 64 -seq_len_k 64 -head_dim_qk 64 -head_dim_v 64",
             "-seq_len_q 64 -seq_len_k 64 -head_dim_qk 64 -head_dim_v 64 -perf_config attn:v1:64,64,256,4,64,64,8,1",
             "-seq_len_q 256 -seq_len_k 256 -head_dim_qk 128 -head_dim_v 128 -perf_config attn:v1:128,128,128,32,128,32,4,1",
             "-seq_len_q 384 -seq_len_k 384 -head_dim_qk 64 -head_dim_v 64 -perf_config attn:v1:32,32,64,8,32,32,8,1",
             "-seq_len_q 384 -seq_len_k 384 -head_dim_qk 64 -head_dim_v 64 -perf_config attn:v1:32,32,64,8,16,16,8,1",
             "-seq_len_q 384 -seq_len_k 384 -head_dim_qk 64 -head_dim_v 64 -with-attn-scale true",
             "-seq_len_q 384 -seq_len_k 384 -head_dim_qk 64 -head_dim_v 64 -with-attn-bias true",
             "-seq_len_q 384 -seq_len_k 384 -head_dim_qk 64 -head_dim_v 64 -with-attn-scale true -with-attn-bias true",
             "-seq_len_q 128 -seq_len_k 27 -head_dim_qk 64 -head_dim_v 32 -with-attn-scale true -with-attn-bias true"]
    problems = ["-operation attention -arch gfx950 -t f16 -g 1 %s -transK %s" % (c, tk) for c in cases
                for tk in ("true", "false")]
    problems.append("-operation attention -arch gfx950 -t i8 -g 1 -seq_len_q 64 -seq_len_k 64 -head_dim_qk 32 "
                    "-head_dim_v 32 -with-attn-bias true")
    for opts in problems:
        first = rock.RockKernel(opts)
        names = [rock.RockKernel("%s -kernel_id %d" % (opts, i)).kernel_name for i in range(first.kernel_count)]
        fused = [n for n in names if n.startswith("rock_attention")]
        assert len(fused) == 1 and "_fast" in fused[0], (opts, names)
        assert all(n.startswith("rock_relayout_b") for n in names if n not in fused), (opts, names)


def test_per_channel_quantisation_vectors_in_the_caller_list(rock):
    """--scale_vector / --zero_point_vector / --quant_scale_vector / --out_zero_point_vector: the kernel with the
    rolled epilogue, the vectors as further caller tensors behind the problem's own and in front of the
    workspace, their addresses written into pointer fields of the parameter block (rockamdGetParamPointers)."""
    lib = rock.load_library()

    def param_ptrs(k):
        n = C.c_int(0)
        off = (C.c_int32 * 4)()
        src = (C.c_int32 * 4)()
        assert lib.rockamdGetParamPointers(k._h, C.byref(n), off, src) == 0
        return [(off[i], src[i]) for i in range(n.value)]

    gemm = "-operation gemm -arch gfx950 -t i8 -g 1 -m 512 -n 384 -k 256 -transB true -out_datatype i8"
    plain = rock.RockKernel(gemm + " -scale 0.01 -quant_scale 0.5")
    assert plain.kernel_name == "rock_gemm_i8_64x64_fast" and plain.caller_pointers == 4 and param_ptrs(plain) == []
    k = rock.RockKernel(gemm + " -scale_vector true -zero_point_vector i8 -quant_scale_vector true -out_zero_point_vector i32")
    assert k.kernel_name == "rock_gemm_i8_64x64_fast_e" and k.caller_pointers == 8
    ptrs = param_ptrs(k)
    assert [s for _, s in ptrs] == [4, 5, 6, 7]
    assert all(0 < o < k.params_size and o % 8 == 0 for o, _ in ptrs) and len({o for o, _ in ptrs}) == 4
    args = k.arguments()
    assert args[4:] == [(0, [384]), (3, [384]), (0, [384]), (6, [384])]   # f32, i8, f32, i32
    # with a residual the vectors follow it; a plan with a workspace keeps it last
    r = rock.RockKernel(gemm + " -residual add -scale_vector true")
    assert r.caller_pointers == 6 and [s for _, s in param_ptrs(r)] == [5]
    nchw = ("--operation conv --arch gfx950 --in_type i8 --fil_type i8 --out_type i8 --fil_layout gkcyx --in_layout ngchw "
            "--out_layout ngkhw --batchsize 1 --groupsize 1 --in_channels 128 --out_channels 128 --in_h 56 --in_w 56 "
            "--fil_h 3 --fil_w 3 --dilation_h 1 --dilation_w 1 --conv_stride_h 2 --conv_stride_w 2 --padding_h 1 "
            "--padding_w 1 --scale_vector true --quant_scale_vector true")
    first = rock.RockKernel(nchw)
    plan = [rock.RockKernel("%s --kernel_id %d" % (nchw, i)) for i in range(first.kernel_count)]
    assert first.kernel_count == 3 and first.workspace_bytes > 0
    assert all(p.caller_pointers == 7 for p in plan)          # filter, input, output, bias, 2 vectors, workspace
    assert [param_ptrs(p) != [] for p in plan] == [False, False, True]
    assert [s for _, s in param_ptrs(plan[2])] == [4, 5] and plan[2].kernel_name.endswith("_e")
    ncall = C.c_int(0)
    nk = C.c_int(0)
    src = (C.c_int32 * 8)()
    off = (C.c_int64 * 8)()
    for p in plan:   # the conversion kernels write into, the contraction reads from, the LAST caller pointer
        assert lib.rockamdGetPointerMap(p._h, C.byref(ncall), C.byref(nk), src, off) == 0
        assert ncall.value == 7 and max(src[i] for i in range(nk.value)) == 6
    assert plan[2].arguments()[-1][0] == -1 and plan[2].arguments()[4] == (0, [128])   # bytes of workspace last
    # what the vectors need: the float step, an integer accumulator for zero points, an int8 result to quantise
    for bad in (gemm.replace("-out_datatype i8", "-out_datatype i32") + " -scale_vector true",
                gemm.replace("-out_datatype i8", "-out_datatype f16") + " -quant_scale_vector true",
                gemm.replace("-t i8", "-t f16") + " -zero_point_vector i32",
                "-operation attention -arch gfx950 -t f16 -g 1 -seq_len_q 64 -seq_len_k 64 -head_dim_qk 64 "
                "-head_dim_v 64 -scale_vector true",
                nchw.replace("--operation conv ", "--operation conv_bwd_data ").replace("i8", "f16")):
        with pytest.raises(rock.RockError):
            rock.RockKernel(bad)


def test_attention_where_mask_in_the_caller_list(rock):
    """-with-attn-mask: the int8 mask and the tensor of replacement scores (migraphx.where in front of the softmax,
    mixr-attn-where.mlir:4-13) follow the bias slot in the caller's list; the plain fused kernel, which scales
    after the row maximum, is never chosen for such a problem."""
    base = "-operation attention -arch gfx950 -t f16 -g 12 -seq_len_q 256 -seq_len_k 256 -transK true "
    k = rock.RockKernel(base + "-head_dim_qk 256 -head_dim_v 256 -with-attn-mask true")
    assert k.kernel_name == "rock_attention_f16_d256x256_fast_bias" and k.kernel_count == 1
    assert k.caller_pointers == 7          # Q, K, V, bias slot, mask, other, O
    args = k.arguments()
    assert [a[0] for a in args] == [1, 1, 1, 1, 3, 1, 1]   # f16 tensors and the int8 mask
    assert args[4][1] == [12, 256, 256] and args[5][1] == [12, 256, 256]
    k = rock.RockKernel(base + "-head_dim_qk 64 -head_dim_v 64 -with-attn-mask true")
    assert k.kernel_name == "rock_attention_f16_d64x64_fast_bias"
    k = rock.RockKernel(base + "-head_dim_qk 64 -head_dim_v 64 -with-attn-mask true -perf_config attn:v1:64,64,128,8,64,32,8,1")
    assert k.kernel_name.endswith("_fast_bias")
    k = rock.RockKernel(base + "-head_dim_qk 64 -head_dim_v 64 -with-attn-scale true -with-attn-mask true")
    assert k.caller_pointers == 8
    # three-kernel form: the row softmax takes them, the workspace still closes the list
    k = rock.RockKernel(base.replace("f16", "f32") + "-head_dim_qk 64 -head_dim_v 64 -with-attn-mask true -kernel_id 1")
    assert k.kernel_name == "rock_softmax_rows" and k.kernel_count == 3 and k.caller_pointers == 8


def test_accumulating_store_is_the_residual_epilogue_on_the_output(rock):
    """-store-method atomic_add (rocmlir-gen.cpp:295-331): the caller's list stays A, B, C, bias; the kernel's
    residual pointer is fed from C; plans with a workspace keep it last."""
    lib = rock.load_library()

    def pointer_map(k):
        nc, nk = C.c_int(0), C.c_int(0)
        src, off = (C.c_int32 * 8)(), (C.c_int64 * 8)()
        assert lib.rockamdGetPointerMap(k._h, C.byref(nc), C.byref(nk), src, off) == 0
        return nc.value, [src[i] for i in range(nk.value)]

    g = "-operation gemm -arch gfx950 -t f16 -g 1 -m 1024 -n 1024 -k 512 -transB true"
    k = rock.RockKernel(g + " -store-method atomic_add")
    assert k.kernel_name == "rock_gemm_f16_64x64_fast_e" and k.kernel_count == 1
    assert pointer_map(k) == (4, [0, 1, 2, 3, 2]) and len(k.arguments()) == 4
    assert rock.RockKernel(g + " -store-method set").kernel_name == "rock_gemm_f16_64x64_fast"
    # few tiles and a long reduction: no split (the sum does not commute with a split's reduction kernel)
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 1280 -k 5120 -store-method atomic_add")
    assert k.kernel_count == 1
    # ragged operands: the copy kernel in front, workspace as the fifth caller pointer
    ragged = "-operation gemm -arch gfx950 -t f16 -g 1 -m 130 -n 60 -k 77 -store-method atomic_add"
    plan = [rock.RockKernel(ragged + " -kernel_id %d" % i) for i in range(2)]
    assert plan[0].kernel_name == "rock_relayout_pair_b2" and pointer_map(plan[0]) == (5, [0, 4, 1, 4])
    assert pointer_map(plan[1]) == (5, [4, 4, 2, 3, 2])
    for bad in (g + " -store-method atomic_add -residual add", g + " -store-method atomic_max",
                "--operation conv --arch gfx950 --in_type fp16 --fil_type fp16 --out_type fp16 --fil_layout gkyxc "
                "--in_layout nhwgc --out_layout nhwgk --batchsize 1 --in_channels 8 --out_channels 8 --in_h 4 "
                "--in_w 4 --fil_h 1 --fil_w 1 --store-method atomic_add"):
        with pytest.raises(rock.RockError):
            rock.RockKernel(bad)


def test_attention_pre_softmax_program(rock):
    """-attn_elementwise: the pre-softmax region of rock.attention as postfix code (RockOps.td:208-254; the trees
    of mixr-attention-padded-scale-bias-exp.mlir and ...-complex-tree-elemwise.mlir).  Such a problem runs as GEMM,
    row softmax, GEMM; the program's tensors stand between V and O in the caller's list and reach the softmax
    kernel through pointer fields of its parameter block."""
    lib = rock.load_library()
    base = "-operation attention -arch gfx950 -t f32 -g 1 -seq_len_q 7 -seq_len_k 7 -head_dim_qk 3 -head_dim_v 3 "
    ks = [rock.RockKernel(base + "-attn_elementwise x,t0,mul,exp,t1,add -kernel_id %d" % i) for i in range(3)]
    assert [k.kernel_name.split("_")[1] for k in ks] == ["gemm", "softmax", "gemm"]
    assert all(k.kernel_count == 3 and k.caller_pointers == 7 for k in ks)      # Q K V t0 t1 O workspace
    assert [a[1] for a in ks[0].arguments()[3:5]] == [[1, 7, 7], [1, 7, 7]]
    n, off, src = C.c_int(0), (C.c_int32 * 8)(), (C.c_int32 * 8)()
    assert lib.rockamdGetParamPointers(ks[1]._h, C.byref(n), off, src) == 0
    assert n.value == 2 and [src[i] for i in range(2)] == [3, 4] and off[1] - off[0] == 8
    assert lib.rockamdGetParamPointers(ks[0]._h, C.byref(n), off, src) == 0 and n.value == 0
    # f16 problems with a program leave the fused kernels; input types as listed, an int8 mask among them
    f16 = base.replace("-t f32", "-t f16").replace("-seq_len_q 7 -seq_len_k 7 -head_dim_qk 3 -head_dim_v 3",
                                                   "-seq_len_q 256 -seq_len_k 256 -head_dim_qk 64 -head_dim_v 64 -transK true")
    k = rock.RockKernel(f16 + "-attn_elementwise t0,x,c:0.125,mul,t1,where -attn_inputs i8,f16")
    assert k.kernel_count == 3 and [a[0] for a in k.arguments()[3:5]] == [3, 1]
    assert rock.RockKernel(f16).kernel_name == "rock_attention_f16_d64x64_fast"
    for bad in ("x,add", "x,x", "x,t9,add", "x,frobnicate", "x,c:abc,mul", "x,t0,t1,t2,t3,add,add,add,add,t4",
                "x,t0,mul -attn_inputs f16,fp8", "x,t0,t1,add,mul -attn_inputs f16", "x,t0,mul -with-attn-bias true",
                "x,t0,mul -scale 0.5"):
        with pytest.raises(rock.RockError):
            rock.RockKernel(f16 + "-attn_elementwise " + bad)


def test_every_problem_of_the_reference_e2e_lists_resolves(rock):
    """mlir/test/e2e/*.toml, expanded as mlir/test/e2e/generateE2ETest.py expands them (tests/e2e_lists.py): each of
    the 2278 option strings -- "-p" default problems, layouts without g or with a third spatial letter of extent
    one, left / right padding given apart, --reverse_grid, split-K perf_configs, --store-method=atomic_add --
    gives a handle whose every kernel has a code object, and the handle describes tensors of the sizes the
    option string implies.  The one exception is refused with a message: the twelve gradient problems with
    unequal left and right padding (conv_regression_bwd.toml's 4x4 / 2x2 / stride 2 / padding 2,1 and 2,0 case)."""
    import numpy as np
    from tests.e2e_lists import problems
    from tests.test_gpu_e2e_lists import parse_options
    lists, kernels, refused = set(), 0, []
    for name, opts in problems():
        try:
            first = rock.RockKernel(opts)
        except rock.RockError as e:
            refused.append((name, opts, str(e)))
            continue
        lists.add(name)
        kernels += first.kernel_count
        if first.kernel_count > 1:    # the last kernel of a plan too (conversions first, reductions last)
            rock.RockKernel("%s --kernel_id %d" % (opts, first.kernel_count - 1))
        o = parse_options(opts)
        if o["operation"] in ("gemm", "attention"):
            continue
        g = int(o.get("groupsize", 1))
        n, c, k = int(o["batchsize"]), int(o["in_channels"]) // g, int(o["out_channels"]) // g
        hi, wi, y, x = int(o["in_h"]), int(o["in_w"]), int(o["fil_h"]), int(o["fil_w"])
        sh, sw = int(o.get("conv_stride_h", 1)), int(o.get("conv_stride_w", 1))
        dh, dw = int(o.get("dilation_h", 1)), int(o.get("dilation_w", 1))
        p_h, p_w = int(o.get("padding_h", 0)), int(o.get("padding_w", 0))
        pl = (int(o.get("padding_h_l", p_h)), int(o.get("padding_w_l", p_w)))
        pr = (int(o.get("padding_h_r", p_h)), int(o.get("padding_w_r", p_w)))
        ho = (hi + pl[0] + pr[0] - (y - 1) * dh - 1) // sh + 1
        wo = (wi + pl[1] + pr[1] - (x - 1) * dw - 1) // sw + 1
        sizes = [int(np.prod(dims)) for _, dims in first.arguments()[:3]]
        assert sizes == [g * k * c * y * x, n * g * c * hi * wi, n * g * k * ho * wo], opts
    assert len(lists) == 19 and kernels > 2278
    assert len(refused) == 12 and all(name == "conv_regression_bwd.toml" and "symmetric padding" in msg and
                                      "-padding_h_l=2 -padding_h_r=1" in opts for name, opts, msg in refused)


def test_binding_refuses_a_tensor_shorter_than_the_plan_addresses(rock):
    """rockamdCheckArgumentSizes, which the binding asks before anything is launched: a tensor shorter than the
    kernel list addresses is an error on the host, not a fault on the device."""
    import torch
    k = rock.RockKernel("-operation gemm -arch gfx950 -t f16 -g 2 -m 100 -n 60 -k 72")
    a, b, c = (torch.empty(n, dtype=torch.float16) for n in (2 * 100 * 72, 2 * 72 * 60, 2 * 100 * 60))
    rest = (None,) if k.caller_pointers == 4 else (None, torch.empty(max(k.workspace_bytes, 16), dtype=torch.uint8))
    k._check_sizes((a, b, c) + rest)
    with pytest.raises(rock.RockError, match="argument 1 holds 17278 bytes, the kernel list addresses 17280"):
        k._check_sizes((a, b[:-1], c) + rest)
    with pytest.raises(rock.RockError, match="one size per pointer"):
        k._check_sizes((a, b))
    conv = rock.RockKernel("-operation conv_bwd_data -arch gfx950 -t f32 -groupsize 1 -batchsize 4 -in_channels 8 "
                           "-out_channels 16 -in_h 9 -in_w 9 -fil_h 3 -fil_w 3 -padding_h 1 -padding_w 1 "
                           "-fil_layout kcyx -in_layout nchw -out_layout nkhw")
    sizes = [16 * 8 * 9, 4 * 8 * 81, 4 * 16 * 81]
    tensors = [torch.empty(n, dtype=torch.float32) for n in sizes] + [None]
    if conv.caller_pointers == 5:
        tensors.append(torch.empty(max(conv.workspace_bytes, 16), dtype=torch.uint8))
    conv._check_sizes(tuple(tensors))
    tensors[1] = torch.empty(sizes[1] - 1, dtype=torch.float32)
    with pytest.raises(rock.RockError, match="argument 1"):
        conv._check_sizes(tuple(tensors))
