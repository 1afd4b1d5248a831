"""The kernels' own sources built for the CPU (hip/hip_runtime.h and runner.cpp in this directory) and the loop
that runs a plan on them: build_model() compiles the kernels of the chosen operand types into a library,
run_plan() takes an options string and the caller's tensors, asks the C ABI for the plan exactly as a caller gets
it (kernel name, grid, block, parameter block and pointer map per kernel id, tensor sizes from
rockamdGetArgumentInfo) and runs every kernel in order.  Test infrastructure only."""
import ctypes as C
import os
import shutil
import subprocess
import sys

import numpy as np

HOST = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HOST))
CSRC = os.path.join(ROOT, "rocmlir_amd", "csrc")
sys.path.insert(0, ROOT)

from rocmlir_amd import _build  # noqa: E402

CLANG = next((c for c in ("/opt/rocm/llvm/bin/clang++", shutil.which("clang++") or "") if c and os.path.exists(c)), None)

_DTYPE_BYTES = {0: 4, 1: 2, 2: 2, 3: 1, 4: 1, 5: 1, 6: 4}   # RockDType -> element size
ALL_TYPES = tuple(_build.GEMM_TYPES)   # operand type codes of csrc/mfma_gfx950.h: f32, f16, bf16, i8, fp8, bf8, mixed


def _params_type(macro):
    if macro.startswith("RK_GEMM"):
        return "RockGemmParams"
    return "RockConvBwdWeightParams" if "BWD_WEIGHT" in macro else "RockConvParams"


def _model_sources(code, rolled, parts=3):
    """The contraction kernels of one operand type as `parts` translation units (they compile side by side)."""
    t = _build.GEMM_TYPES[code]
    kernels = [(n, m) for n, m in _build.contraction_kernels(code) if rolled or not n.endswith("_e")]
    units = {}
    for part in range(parts):
        mine = kernels[part::parts]
        lines = ["#define ROCK_DT %d" % code, "#define ROCK_DTNAME %s" % t, '#include "gemm_conv_instances.h"',
                 '#include "kernel_table.h"']
        lines += [m for _, m in mine]
        for n, m in mine:
            lines.append("static void call_%s(void **q, const void *params) { %s p; std::memcpy(&p, params, sizeof p); "
                         "%s(q[0], q[1], q[2], q[3], q[4], p); }" % (n, _params_type(m), n))
        lines.append("static const HmEntry table[] = {")
        lines += ['  {"%s", call_%s},' % (n, n) for n, _ in mine]
        lines += ["  {nullptr, nullptr}};", "const HmEntry *hm_table_%s_%d() { return table; }" % (t, part)]
        units["model_%s_%d" % (t, part)] = "\n".join(lines) + "\n"
    return units


# the kernels of csrc/relayout_kernels.hip: name -> (parameter block, pointers)
_UTILITY = {"rock_relayout_b1": ("RockRelayoutParams", 2), "rock_relayout_b2": ("RockRelayoutParams", 2),
            "rock_relayout_b4": ("RockRelayoutParams", 2), "rock_fill_zero": ("RockFillParams", 1),
            "rock_reduce_splits": ("RockReduceParams", 2), "rock_softmax_rows": ("RockSoftmaxParams", 5),
            "rock_relayout_pair_b1": ("RockRelayoutPairParams", 4), "rock_relayout_pair_b2": ("RockRelayoutPairParams", 4),
            "rock_relayout_pair_b4": ("RockRelayoutPairParams", 4), "rock_fold_depth": ("RockFoldDepthParams", 2)}
_CASTS = {"rock_reduce_splits": ["(const float *)", ""], "rock_softmax_rows": ["(float *)", "", "", "", ""]}


def _utility_source():
    lines = ['#include "relayout_kernels.hip"', '#include "kernel_table.h"', "#include <cstring>"]
    for n, (ptype, count) in _UTILITY.items():
        casts = _CASTS.get(n, [""] * count)
        args = ", ".join("%sq[%d]" % (casts[i], i) for i in range(count))
        lines.append("static void call_%s(void **q, const void *params) { %s p; std::memcpy(&p, params, sizeof p); "
                     "%s(%s, p); }" % (n, ptype, n, args))
    lines.append("static const HmEntry table[] = {")
    lines += ['  {"%s", call_%s},' % (n, n) for n in _UTILITY]
    lines += ["  {nullptr, nullptr}};", "const HmEntry *hm_table_utility() { return table; }"]
    return "\n".join(lines) + "\n"


def _attention_sources(parts=4):
    """The fused attention kernels (csrc/attention_kernels.h): Q, K, V, scale tensor, bias, mask, other, O."""
    kernels = _build.attention_kernels()
    units = {}
    for part in range(parts):
        mine = kernels[part::parts]
        lines = ['#include "attention_kernels.h"', '#include "kernel_table.h"', "#include <cstring>"]
        lines += [m for _, m in mine]
        for n, _ in mine:
            lines.append("static void call_%s(void **q, const void *params) { RockAttentionParams p; "
                         "std::memcpy(&p, params, sizeof p); %s(q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7], p); }"
                         % (n, n))
        lines.append("static const HmEntry table[] = {")
        lines += ['  {"%s", call_%s},' % (n, n) for n, _ in mine]
        lines += ["  {nullptr, nullptr}};", "const HmEntry *hm_table_attention_%d() { return table; }" % part]
        units["model_attention_%d" % part] = "\n".join(lines) + "\n"
    return units


def _table_source(tables):
    lines = ['#include "kernel_table.h"', "#include <vector>"]
    lines += ["const HmEntry *%s();" % t for t in tables]
    lines += ["const HmEntry *hm_kernel_table() {", "  static std::vector<HmEntry> all;", "  if (all.empty()) {"]
    lines += ["    for (const HmEntry *e = %s(); e->name; ++e) all.push_back(*e);" % t for t in tables]
    lines += ["    all.push_back({nullptr, nullptr});", "  }", "  return all.data();", "}"]
    return "\n".join(lines) + "\n"


def build_model(d, types=(0, 1), rolled=False, attention=True):
    """Compiles the model into directory d and returns the loaded library.  types: operand type codes (f32 and
    f16 by default; ALL_TYPES for every one); rolled: the kernels with the rolled epilogue ("_e": same loads and
    tiles, their own store code) too; attention: the fused attention kernels."""
    assert CLANG, "the host build uses clang's vector extensions"
    units = {"model_utility": _utility_source()}
    for code in types:
        units.update(_model_sources(code, rolled))
    if attention:
        units.update(_attention_sources())
    units["kernel_table"] = _table_source(["hm_table_" + n[len("model_"):] for n in units])
    for name, text in units.items():
        with open(os.path.join(d, name + ".cpp"), "w") as f:
            f.write(text)
    flags = [CLANG, "-O1", "-std=c++17", "-fPIC", "-w", "-I", HOST, "-I", CSRC]
    todo = [(os.path.join(d, n + ".cpp"), os.path.join(d, n + ".o")) for n in units]
    todo.append((os.path.join(HOST, "runner.cpp"), os.path.join(d, "runner.o")))
    running, limit = [], max(2, os.cpu_count() or 2)
    while todo or running:
        while todo and len(running) < limit:
            src, obj = todo.pop()
            running.append(subprocess.Popen(flags + ["-c", src, "-o", obj], stderr=subprocess.PIPE))
        job = running.pop(0)
        err = job.communicate()[1]
        assert job.returncode == 0, err.decode()[-3000:]
    so = os.path.join(d, "libkernel_host.so")
    # (the kernels' headers define one non-inline helper; every device code object holds one kernel, here they share a library)
    subprocess.check_call([CLANG, "-shared", "-Wl,-z,muldefs", "-o", so, os.path.join(d, "runner.o")] +
                          [os.path.join(d, n + ".o") for n in units])
    return load_model(so)


def load_model(so):
    """The library that build_model() left at `so`."""
    lib = C.CDLL(so)
    lib.hm_alloc.restype = C.c_void_p
    lib.hm_alloc.argtypes = [C.c_size_t, C.c_char_p]
    lib.hm_canaries.restype = C.c_long
    lib.hm_canaries.argtypes = [C.c_void_p, C.c_size_t]
    lib.hm_knows.argtypes = [C.c_char_p]
    lib.hm_run.restype = C.c_long
    lib.hm_run.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p), C.c_uint, C.c_uint, C.c_char_p, C.c_size_t]
    lib.hm_set_late_loads.argtypes = [C.c_int]
    lib.hm_set_thread_order.argtypes = [C.c_int]
    lib.hm_set_blocks.argtypes = [C.c_uint, C.c_uint]
    lib.hm_set_owner_check.argtypes = [C.c_int]
    lib.hm_run_direct.restype = C.c_long
    lib.hm_run_direct.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p), C.c_uint, C.c_uint, C.c_int]
    return lib


def pointer_map(rock, k):
    ncall, nk = C.c_int(), C.c_int()
    src, off = (C.c_int32 * 8)(), (C.c_int64 * 8)()
    assert rock.load_library().rockamdGetPointerMap(k._h, C.byref(ncall), C.byref(nk), src, off) == 0
    return [(src[i], off[i]) for i in range(nk.value)]


def run_plan(model, rock, opts, inputs=None, shrink=None):
    """Runs every kernel of the plan in order.  inputs = {caller index: numpy array}, copied into that tensor as
    it lies (the other tensors start as 0xEE bytes); shrink = (caller index, bytes): that tensor is allocated
    short by so many bytes (to show that the model notices).  Returns (kernel names, problems, tensors) with the
    tensors as uint8 views of the model's memory."""
    first = rock.RockKernel(opts)
    model.hm_clear()
    tensors = []
    for i, (dt, dims) in enumerate(first.arguments()):
        nbytes = int(np.prod(dims, dtype=np.int64)) * (1 if dt < 0 else _DTYPE_BYTES[dt])
        if shrink and shrink[0] == i:
            nbytes -= shrink[1]
        nbytes = max(nbytes, 16)
        at = model.hm_alloc(nbytes, b"argument %d" % i)
        view = np.ctypeslib.as_array((C.c_uint8 * nbytes).from_address(at))
        view[:] = 0xEE
        if inputs and i in inputs:
            raw = np.ascontiguousarray(inputs[i]).view(np.uint8).ravel()
            view[:raw.size] = raw
        tensors.append((at, nbytes, view))
    names, problems = [], []
    for kid in range(first.kernel_count):
        k = first if kid == 0 else rock.RockKernel(opts + " --kernel_id %d" % kid)
        name = k.kernel_name.encode()
        assert model.hm_knows(name), "the model does not hold " + k.kernel_name
        ptrs = (C.c_void_p * 8)()
        for j, (src, off) in enumerate(pointer_map(rock, k)):
            ptrs[j] = None if src < 0 else tensors[src][0] + off
        text = C.create_string_buffer(512)
        bad = model.hm_run(name, k.params(), ptrs, k.grid_size, k.block_size, text, 512)
        assert bad >= 0, "the model could not run " + k.kernel_name
        names.append(k.kernel_name)
        if bad:
            problems.append("%s: %d, first: %s" % (k.kernel_name, bad, text.value.decode()))
        for i, (at, n, _) in enumerate(tensors):
            changed = model.hm_canaries(at, n)
            if changed:
                problems.append("%s wrote %d bytes beside argument %d" % (k.kernel_name, changed, i))
    return names, problems, [v for _, _, v in tensors]




def harness_device(model, rock):
    """What the end-to-end harness (tests/test_gpu_e2e_lists.py: run_conv, run_gemm, run_attention) takes in place
    of the binding: a RockProgram whose launch() runs the plan on the model, for torch tensors on the CPU.
    Device.kernels holds the kernel names of the last launch."""
    import torch

    class Program:
        def __init__(self, opts):
            self.opts = opts
            first = rock.RockKernel(opts)
            self.kernels = [first] + [rock.RockKernel("%s --kernel_id %d" % (opts, i)) for i in range(1, first.kernel_count)]

        def launch(self, *args):
            inputs = {i: a.contiguous().view(torch.uint8).numpy() for i, a in enumerate(args) if a is not None}
            names, problems, out = run_plan(model, rock, self.opts, inputs)
            Device.kernels = names
            assert not problems, (self.opts, names, problems)
            for i, a in enumerate(args):
                if a is not None:
                    flat = a.view(torch.uint8).view(-1)
                    flat.copy_(torch.from_numpy(out[i][:flat.numel()].copy()))

    class Device:
        RockProgram = Program
        kernels = []

    return Device
