"""Build recipe for librocmlir_amd.so: compiles every gfx950 kernel into a code
object of its own with hipcc, embeds the code objects, and links the host
library.

One kernel per code object is the reference's contract for what its library
hands out (mlir/tools/rocmlir-lib/rocmlir-lib.cpp:292-316: one `extern "C"`
kernel per hsaco; MIGraphX stores one code object per fused operator), so
miirBufferGet returns the selected kernel alone.  This file holds the list of
kernels; the sources under csrc/ hold the kernel bodies and the macros that
instantiate them."""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

from ._elf import kernel_symbols

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
BUILD = os.path.join(PKG, "_build")
GEN = os.path.join(BUILD, "gen")
LIB = os.path.join(PKG, "librocmlir_amd.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# operand-type code (mfma_gfx950.h) -> kernel-name part
GEMM_TYPES = {0: "f32", 1: "f16", 2: "bf16", 3: "i8", 4: "fp8", 5: "bf8",
              7: "fp8_bf8", 8: "bf8_fp8"}
CONV_TYPES = (0, 1, 2, 3, 4, 5)      # the mixed 8-bit float pairs are GEMM-only

DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "--cuda-device-only", "--no-gpu-bundle-output", "-I", CSRC,
]

SPILL_WARN = 32  # spilled vector registers above which the build prints a warning

# (block tile rows, columns, waves along M, waves along N) of the tiled kernels
TILES = {"_256x256": (256, 256, 2, 4), "_256x128": (256, 128, 4, 2),
         "_128x128": (128, 128, 2, 2), "_64x64": (64, 64, 2, 2)}
ROWS, COLS = "rk::LD_ROWS_FAST", "rk::LD_COLS_FAST"


def contraction_kernels(type_code):
    """[(kernel name, macro invocation)] for one operand type: the macros of
    csrc/gemm_conv_instances.h."""
    t = GEMM_TYPES[type_code]
    out = []

    def gemm_dl(suffix, tile, la, lb):
        bm, bn, wm, wn = TILES[tile]
        for rich, e in ((False, ""), (True, "_e")):
            name = tile + suffix + e
            out.append(("rock_gemm_%s%s" % (t, name),
                        "RK_GEMM_DL(%s, %d, %d, %d, %d, 128, %s, %s, %s)"
                        % (name, bm, bn, wm, wn, la, lb, "true" if rich else "false")))

    for tile in TILES:                                   # K-contiguous operands
        gemm_dl("_fast", tile, ROWS, ROWS)
    for tile in ("_256x256", "_128x128", "_64x64"):      # K-major operands: how A and B are stored
        gemm_dl("_fast_nn", tile, ROWS, COLS)
        gemm_dl("_fast_tn", tile, COLS, COLS)
        gemm_dl("_fast_tt", tile, COLS, ROWS)
    out.append(("rock_gemm_%s_64x64_generic" % t,
                "RK_GEMM(_64x64_generic, 64, 64, 2, 2, rk::LD_ROWS_GENERIC, rk::LD_ROWS_GENERIC)"))
    out.append(("rock_gemm_%s_32x32_splitk" % t, "RK_GEMM_SPLITK(_32x32_splitk, false)"))
    out.append(("rock_gemm_%s_32x32_splitk_e" % t, "RK_GEMM_SPLITK(_32x32_splitk_e, true)"))
    if type_code in CONV_TYPES:
        for tile in ("_256x128", "_128x128", "_64x64"):
            bm, bn, wm, wn = TILES[tile]
            for rich, e in ((False, ""), (True, "_e")):
                name = tile + "_fast" + e
                out.append(("rock_conv_%s%s" % (t, name), "RK_CONV_DL(%s, %d, %d, %d, %d, 128, %s)"
                            % (name, bm, bn, wm, wn, "true" if rich else "false")))
        if t != "f32":   # rows of taps over narrow pixels (32-bit pixels of 4 channels are whole chunks)
            for rich, e in ((False, ""), (True, "_e")):
                out.append(("rock_conv_%s_64x64_fast_runs%s" % (t, e),
                            "RK_CONV_DL_RUNS(_64x64_fast_runs%s, 64, 64, 2, 2, 128, %s)" % (e, "true" if rich else "false")))
        out.append(("rock_conv_%s_64x64_generic" % t,
                    "RK_CONV(_64x64_generic, 64, 64, 2, 2, rk::LD_CONV_IN_GENERIC, rk::LD_CONV_FIL_GENERIC)"))
        if t in ("f32", "f16", "bf16"):   # filter gradient as one K-major GEMM over the tensors as they lie
            out.append(("rock_conv_bwd_weight_%s_128x128" % t, "RK_CONV_BWD_WEIGHT(_128x128, 128, 128, 2, 2)"))
            out.append(("rock_conv_bwd_weight_%s_64x64" % t, "RK_CONV_BWD_WEIGHT(_64x64, 64, 64, 2, 2)"))
        out.append(("rock_conv_%s_direct224" % t, "RK_CONV_DIRECT(_direct224, false)"))
        out.append(("rock_conv_%s_direct224_e" % t, "RK_CONV_DIRECT(_direct224_e, true)"))
    return out


def attention_kernels():
    out = []
    for t, code in (("f16", "MM_F16"), ("bf16", "MM_BF16")):
        for d in (128, 64):
            out.append(("rock_attention_%s_d%dx%d_fast" % (t, d, d), "RK_ATTN_DL(%s, %s, %d, fast, true)" % (t, code, d)))
            out.append(("rock_attention_%s_d%dx%d_fast_bias" % (t, d, d),
                        "RK_ATTN_DL(%s, %s, %d, fast_bias, false)" % (t, code, d)))
            # K stored [d][seq_k]
            out.append(("rock_attention_%s_d%dx%d_fast_kt" % (t, d, d), "RK_ATTN_DL_KT(%s, %s, %d, fast_kt, true, 2)" % (t, code, d)))
            out.append(("rock_attention_%s_d%dx%d_fast_bias_kt" % (t, d, d),
                        "RK_ATTN_DL_KT(%s, %s, %d, fast_bias_kt, false, 2)" % (t, code, d)))
            out.append(("rock_attention_%s_d%dx%d_generic" % (t, d, d),
                        "RK_ATTN(%s, %s, %d, %d, generic, false)" % (t, code, d, d)))
        out.append(("rock_attention_%s_d256x256_fast_bias" % t, "RK_ATTN_DL_WIDE(%s, %s, 256)" % (t, code)))
        out.append(("rock_attention_%s_d256x256_fast_bias_kt" % t, "RK_ATTN_DL_KT(%s, %s, 256, fast_bias_kt, false, 1)" % (t, code)))
    for d in (128, 64):   # int8 Q and K, f16 V and output
        out.append(("rock_attention_i8_d%dx%d_fast" % (d, d), "RK_ATTN_DL_I8(%d, fast, true)" % d))
        out.append(("rock_attention_i8_d%dx%d_fast_bias" % (d, d), "RK_ATTN_DL_I8(%d, fast_bias, false)" % d))
    return out


# translation units of the host side (csrc/<unit>.cpp)
HOST_UNITS = ["rock_options", "plan_gemm", "plan_relayout", "plan_conv", "plan_conv_bwd_data", "plan_conv_bwd_weight",
              "plan_conv3d", "plan_attention", "rock_handle", "rock_launch", "miir_api", "bench_api"]

# kernels of csrc/relayout_kernels.hip in file order (-DROCK_KERNEL=<position>)
RELAYOUT_KERNELS = ["rock_relayout_b1", "rock_relayout_b2", "rock_relayout_b4", "rock_fill_zero",
                    "rock_reduce_splits", "rock_softmax_rows", "rock_relayout_pair_b1", "rock_relayout_pair_b2",
                    "rock_relayout_pair_b4", "rock_fold_depth"]
# kernels of csrc/probe_kernels.hip by operand-type code (-DROCK_KERNEL=<code>)
PROBE_KERNELS = {0: "rock_probe_mfma_f32", 1: "rock_probe_mfma_f16", 2: "rock_probe_mfma_bf16",
                 3: "rock_probe_mfma_i8", 4: "rock_probe_mfma_fp8"}


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True)
    if res.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + res.stdout + "\n")
        raise RuntimeError("build step failed: " + cmd[-1])
    return res.stdout


def device_jobs():
    """[(kernel name, source path, generated source text or None, extra flags)]"""
    jobs = []
    for code, t in GEMM_TYPES.items():
        for name, macro in contraction_kernels(code):
            text = ("// generated by rocmlir_amd/_build.py\n#define ROCK_DT %d\n#define ROCK_DTNAME %s\n"
                    "#include \"gemm_conv_instances.h\"\n%s\n" % (code, t, macro))
            jobs.append((name, os.path.join(GEN, name + ".hip"), text, []))
    for name, macro in attention_kernels():
        text = "// generated by rocmlir_amd/_build.py\n#include \"attention_kernels.h\"\n%s\n" % macro
        jobs.append((name, os.path.join(GEN, name + ".hip"), text, []))
    for i, name in enumerate(RELAYOUT_KERNELS):
        jobs.append((name, os.path.join(CSRC, "relayout_kernels.hip"), None, ["-DROCK_KERNEL=%d" % i]))
    for code, name in PROBE_KERNELS.items():
        jobs.append((name, os.path.join(CSRC, "probe_kernels.hip"), None, ["-DROCK_KERNEL=%d" % code]))
    return jobs


def kernel_names():
    return [j[0] for j in device_jobs()]


def _newest_source():
    return max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC))


def _check(name):
    """The code object must hold exactly the kernel it is named for."""
    out = os.path.join(BUILD, name + ".hsaco")
    with open(out, "rb") as f:
        syms = kernel_symbols(f.read())
    if syms != [name]:
        raise RuntimeError("%s holds the kernels %s" % (out, syms))


def _compile(job):
    name, src, text, flags = job
    out = os.path.join(BUILD, name + ".hsaco")
    if text is not None:
        with open(src, "w") as f:
            f.write(text)
    log = _run([HIPCC] + DEVICE_FLAGS + flags + ["-Rpass-analysis=kernel-resource-usage", "-o", out, src])
    _check(name)
    # registers spilled to scratch memory: a handful outside the main loop is
    # harmless, hundreds mean a kernel that lost its registers to a code change
    spilled = [int(m) for m in re.findall(r"VGPRs Spill: (\d+)", log)]
    if spilled and max(spilled) > SPILL_WARN:
        sys.stderr.write("warning: %s spills %d vector registers\n" % (name, max(spilled)))
    return "\n".join(l for l in log.splitlines() if ("warning:" in l or "error:" in l) and "-Rpass" not in l)


def build(jobs=8, verbose=False, host_only=False, only=None, incremental=False):
    """host_only: recompile the host units and relink against the code objects already built;
    only: rebuild just the code objects whose kernel name contains this string;
    incremental: skip code objects newer than every file under csrc/."""
    os.makedirs(GEN, exist_ok=True)
    todo = [] if host_only else [j for j in device_jobs() if only is None or only in j[0]]
    if incremental:
        newest = max(_newest_source(), os.path.getmtime(__file__))
        todo = [j for j in todo if not os.path.exists(os.path.join(BUILD, j[0] + ".hsaco"))
                or os.path.getmtime(os.path.join(BUILD, j[0] + ".hsaco")) < newest]
    # longest first: the big tiles with the unrolled epilogue take the longest to compile
    todo.sort(key=lambda j: (0 if "256x" in j[0] else 1, 0 if j[0].endswith("_e") else 1))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for out in pool.map(_compile, todo):
            if verbose and out.strip():
                print(out)
    names = kernel_names()
    missing = [n for n in names if not os.path.exists(os.path.join(BUILD, n + ".hsaco"))]
    if missing:
        raise RuntimeError("code objects missing (build without host_only / only first): %s" % missing[:5])
    for n in names:
        _check(n)
    # table of the embedded code objects for rock_options.cpp, and the assembly that places them
    with open(os.path.join(BUILD, "blobs.inc"), "w") as f:
        f.write("// generated by rocmlir_amd/_build.py: one gfx950 code object per kernel\n")
        f.writelines("ROCK_BLOB(%s)\n" % n for n in names)
    with open(os.path.join(BUILD, "blobs_list.S"), "w") as f:
        f.writelines("    ROCK_BLOB %s\n" % n for n in names)
    blobs_o = os.path.join(BUILD, "blobs.o")
    _run(["gcc", "-c", "-x", "assembler-with-cpp", "-I", BUILD,
          os.path.join(CSRC, "blobs.S"), "-o", blobs_o])
    # the one source with host and device code in one object: the static workspace
    static_o = os.path.join(BUILD, "static_workspace.o")
    _run([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-c", os.path.join(CSRC, "static_workspace.hip"), "-o", static_o])
    # the host side: one object per translation unit, compiled as plain C++ against the HIP runtime API
    host_objects = []

    def host_compile(unit):
        obj = os.path.join(BUILD, unit + ".o")
        _run([HIPCC, "-O2", "-std=c++17", "-fPIC", "-x", "c++", "-D__HIP_PLATFORM_AMD__", "-fvisibility=hidden",
              "-I", os.path.join(ROCM, "include"), "-I", BUILD, "-c", os.path.join(CSRC, unit + ".cpp"), "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        host_objects = list(pool.map(host_compile, HOST_UNITS))
    _run([HIPCC, "-fPIC", "-shared", *host_objects, blobs_o, static_o,
          "-L", os.path.join(ROCM, "lib"), "-lamdhip64",
          "-Wl,-rpath," + os.path.join(ROCM, "lib"),
          "-o", LIB])
    return LIB


if __name__ == "__main__":
    only = [a.split("=", 1)[1] for a in sys.argv[1:] if a.startswith("--only=")]
    print(build(verbose=True, host_only="--host-only" in sys.argv[1:], only=only[0] if only else None,
                incremental="--incremental" in sys.argv[1:]))
