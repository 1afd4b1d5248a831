"""The contraction kernels compiled for the CPU and stepped through whole plans, every block and thread, with
every address checked (tests/kernel_host/: the stand-in for the device environment and the runner).

What the model does and does not show: a thread forms the same addresses as on the GPU (they never depend on data
in these kernels), buffer loads are range-checked like the hardware's, every tensor lies between canary pages and
inaccessible regions, and a 16-byte access that is not 16-byte aligned traps.  The values are not computed (the
matrix instructions do nothing and threads do not run in step), so results are the GPU tests' business.

The plans come from the C ABI exactly as a caller gets them: kernel name, grid, block, parameter block and
pointer map per kernel id, tensor sizes from rockamdGetArgumentInfo.
"""
import ctypes as C
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "rocmlir_amd", "csrc")
HOST = os.path.join(HERE, "kernel_host")
sys.path.insert(0, ROOT)

from rocmlir_amd import _build  # noqa: E402

CLANG = next((c for c in ("/opt/rocm/llvm/bin/clang++", shutil.which("clang++") or "") if c and os.path.exists(c)), None)
pytestmark = pytest.mark.skipif(CLANG is None, reason="the host build uses clang's vector extensions")

# operand types of the model
_TYPES = {0: "f32", 1: "f16"}
# every kernel but the twins with the rolled epilogue ("_e": same loads, same tiles, their own store code)
_LEFT_OUT = ("_e",)
_DTYPE_BYTES = {0: 4, 1: 2, 2: 2, 3: 1, 4: 1, 5: 1, 6: 4}


def _params_type(macro):
    if macro.startswith("RK_GEMM"):
        return "RockGemmParams"
    return "RockConvBwdWeightParams" if "BWD_WEIGHT" in macro else "RockConvParams"


def _model_source(code):
    t = _TYPES[code]
    kernels = [(n, m) for n, m in _build.contraction_kernels(code) if not n.endswith(_LEFT_OUT)]
    lines = ["#define ROCK_DT %d" % code, "#define ROCK_DTNAME %s" % t, '#include "gemm_conv_instances.h"',
             '#include "kernel_table.h"']
    lines += [m for _, m in kernels]
    for n, m in kernels:
        lines.append("static void call_%s(void **q, const void *params) { %s p; std::memcpy(&p, params, sizeof p); "
                     "%s(q[0], q[1], q[2], q[3], q[4], p); }" % (n, _params_type(m), n))
    lines.append("static const HmEntry table[] = {")
    lines += ['  {"%s", call_%s},' % (n, n) for n, _ in kernels]
    lines += ["  {nullptr, nullptr}};", "const HmEntry *hm_table_%s() { return table; }" % t]
    return "\n".join(lines) + "\n"


def _table_source():
    lines = ['#include "kernel_table.h"', "#include <vector>"]
    lines += ["const HmEntry *hm_table_%s();" % t for t in _TYPES.values()]
    lines += ["const HmEntry *hm_kernel_table() {", "  static std::vector<HmEntry> all;", "  if (all.empty()) {"]
    lines += ["    for (const HmEntry *e = hm_table_%s(); e->name; ++e) all.push_back(*e);" % t for t in _TYPES.values()]
    lines += ["    all.push_back({nullptr, nullptr});", "  }", "  return all.data();", "}"]
    return "\n".join(lines) + "\n"


def build_model(d):
    """Compiles the model into directory d and returns the loaded library."""
    units = {"kernel_table": _table_source()}
    units.update({"model_%s" % t: _model_source(code) for code, t in _TYPES.items()})
    for name, text in units.items():
        with open(os.path.join(d, name + ".cpp"), "w") as f:
            f.write(text)
    flags = [CLANG, "-O1", "-std=c++17", "-fPIC", "-w", "-I", HOST, "-I", CSRC]
    jobs = [subprocess.Popen(flags + ["-c", os.path.join(d, n + ".cpp"), "-o", os.path.join(d, n + ".o")],
                             stderr=subprocess.PIPE) for n in units]
    jobs.append(subprocess.Popen(flags + ["-c", os.path.join(HOST, "runner.cpp"), "-o", os.path.join(d, "runner.o")],
                                 stderr=subprocess.PIPE))
    for j in jobs:
        err = j.communicate()[1]
        assert j.returncode == 0, err.decode()[-3000:]
    so = os.path.join(d, "libkernel_host.so")
    # (the kernels' headers define one non-inline helper; every device code object holds one kernel, here they share a library)
    subprocess.check_call([CLANG, "-shared", "-Wl,-z,muldefs", "-o", so, os.path.join(d, "runner.o")] +
                          [os.path.join(d, n + ".o") for n in units])
    lib = C.CDLL(so)
    lib.hm_alloc.restype = C.c_void_p
    lib.hm_alloc.argtypes = [C.c_size_t, C.c_char_p]
    lib.hm_canaries.restype = C.c_long
    lib.hm_canaries.argtypes = [C.c_void_p, C.c_size_t]
    lib.hm_knows.argtypes = [C.c_char_p]
    lib.hm_run.restype = C.c_long
    lib.hm_run.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p), C.c_uint, C.c_uint, C.c_char_p, C.c_size_t]
    return lib


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    return build_model(str(tmp_path_factory.mktemp("kernel_host")))


@pytest.fixture(scope="module")
def rock():
    import rocmlir_amd
    rocmlir_amd.load_library()
    return rocmlir_amd


def _pointer_map(rock, k):
    ncall, nk = C.c_int(), C.c_int()
    src, off = (C.c_int32 * 8)(), (C.c_int64 * 8)()
    assert rock.load_library().rockamdGetPointerMap(k._h, C.byref(ncall), C.byref(nk), src, off) == 0
    return [(src[i], off[i]) for i in range(nk.value)]


def run_plan(model, rock, opts, shrink=None):
    """Steps every kernel of the plan that the model holds.  shrink = (caller index, bytes): that tensor is
    allocated short by so many bytes (to show that the model notices).  Returns (kernel names stepped, problems)."""
    first = rock.RockKernel(opts)
    model.hm_clear()
    tensors = []
    for i, (dt, dims) in enumerate(first.arguments()):
        nbytes = int(np.prod(dims, dtype=np.int64)) * (1 if dt < 0 else _DTYPE_BYTES[dt])
        if shrink and shrink[0] == i:
            nbytes -= shrink[1]
        nbytes = max(nbytes, 16)
        tensors.append((model.hm_alloc(nbytes, b"argument %d" % i), nbytes))
    stepped, problems = [], []
    for kid in range(first.kernel_count):
        k = first if kid == 0 else rock.RockKernel(opts + " --kernel_id %d" % kid)
        name = k.kernel_name.encode()
        if not model.hm_knows(name):
            continue
        ptrs = (C.c_void_p * 8)()
        for j, (src, off) in enumerate(_pointer_map(rock, k)):
            ptrs[j] = None if src < 0 else tensors[src][0] + off
        text = C.create_string_buffer(512)
        bad = model.hm_run(name, k.params(), ptrs, k.grid_size, k.block_size, text, 512)
        assert bad >= 0, "the model could not run " + k.kernel_name
        stepped.append(k.kernel_name)
        if bad:
            problems.append("%s: %d, first: %s" % (k.kernel_name, bad, text.value.decode()))
        for i, (p, n) in enumerate(tensors):
            changed = model.hm_canaries(p, n)
            if changed:
                problems.append("%s wrote %d bytes beside argument %d" % (k.kernel_name, changed, i))
    return stepped, problems


def _conv(op, t, n, c, k, hw, f, pad, layouts="kcyx nchw nkhw", stride=1, extra=""):
    fl, il, ol = layouts.split()
    return ("-operation %s -arch gfx950 -t %s -groupsize 1 -batchsize %d -in_channels %d -out_channels %d -in_h %d "
            "-in_w %d -fil_h %d -fil_w %d -padding_h %d -padding_w %d -conv_stride_h %d -conv_stride_w %d "
            "-fil_layout %s -in_layout %s -out_layout %s %s" % (op, t, n, c, k, hw, hw, f, f, pad, pad, stride, stride,
                                                               fl, il, ol, extra))


def test_the_model_notices_a_short_tensor(model, rock):
    """The input gradient of a 1x1 convolution written 16 bytes short: the last store lands on the canary."""
    opts = _conv("conv_bwd_data", "f32", 16, 32, 32, 14, 1, 1)
    stepped, problems = run_plan(model, rock, opts)
    assert stepped == ["rock_conv_f32_64x64_fast"] and not problems, problems
    stepped, problems = run_plan(model, rock, opts, shrink=(1, 16))
    assert problems and "beside argument 1" in problems[0], problems


def test_the_model_notices_a_short_operand(model, rock):
    """A GEMM operand allocated one chunk short: the direct-to-LDS load of its last chunk is out of the tensor."""
    opts = "-operation gemm -arch gfx950 -t f16 -g 1 -m 128 -n 128 -k 256"
    stepped, problems = run_plan(model, rock, opts)
    assert stepped and not problems, (stepped, problems)
    stepped, problems = run_plan(model, rock, opts, shrink=(0, 16))
    assert problems and "buffer load into LDS outside the tensors" in problems[0], problems


# (operation, type, batch, c, k, image, filter, padding, layouts, stride): what the reference's backward regression
# list runs, at batches the CPU steps through in seconds, plus forward layers over the same kernels
_PLANS = [
    # input gradient written channel-major by the window-resident kernel: tiles of 7 rows of 28 pixels start on
    # odd multiples of 8 bytes in f16, so the vectors of 8 pixels would straddle images and tiles
    ("conv_bwd_data", "f16", 4, 256, 128, 28, 3, 1, "kcyx nchw nkhw", 1),
    ("conv_bwd_data", "f16", 4, 256, 64, 56, 3, 1, "kcyx nchw nkhw", 1),
    ("conv_bwd_data", "f16", 4, 256, 128, 28, 3, 1, "kyxc nhwc nhwk", 1),
    ("conv", "f16", 4, 128, 128, 28, 3, 1, "kyxc nhwc nhwk", 1),
    ("conv", "f16", 4, 128, 128, 28, 3, 1, "kcyx nchw nkhw", 1),
    ("conv_bwd_data", "f32", 16, 32, 32, 14, 1, 1, "kcyx nchw nkhw", 1),
    ("conv_bwd_data", "f16", 16, 32, 32, 14, 1, 1, "kyxc nhwc nhwk", 1),
    ("conv_bwd_weight", "f32", 16, 32, 32, 14, 1, 1, "kcyx nchw nkhw", 1),
    ("conv_bwd_weight", "f16", 8, 64, 64, 14, 3, 1, "kyxc nhwc nhwk", 1),
    ("conv_bwd_weight", "f16", 2, 256, 256, 56, 1, 0, "kcyx nchw nkhw", 1),
    ("conv_bwd_data", "f16", 4, 64, 64, 56, 1, 0, "kyxc nhwc nhwk", 2),
    ("conv_bwd_data", "f32", 4, 64, 128, 17, 3, 1, "kcyx nchw nkhw", 2),
    ("conv_bwd_weight", "f32", 4, 64, 128, 17, 3, 1, "kyxc nhwc nhwk", 2),
    ("conv", "f32", 4, 64, 64, 15, 3, 0, "kyxc nhwc nhwk", 1),
]


@pytest.mark.parametrize("plan", _PLANS, ids=lambda p: "%s-%s-%dx%d-%d-%s" % (p[0], p[1], p[5], p[5], p[6], p[8].split()[1]))
def test_every_address_of_the_plan_lies_in_its_tensors(model, rock, plan):
    op, t, n, c, k, hw, f, pad, layouts, stride = plan
    stepped, problems = run_plan(model, rock, _conv(op, t, n, c, k, hw, f, pad, layouts, stride))
    assert stepped, "no kernel of this plan is in the model"
    assert not problems, problems
