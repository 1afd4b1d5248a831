"""Build recipe for librocmlir_amd.so: compiles every gfx950 kernel to a code
object with hipcc, embeds the code objects, and links the host library."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
BUILD = os.path.join(PKG, "_build")
LIB = os.path.join(PKG, "librocmlir_amd.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# operand-type code (mfma_gfx950.h) -> kernel-name suffix
GEMM_TYPES = {0: "f32", 1: "f16", 2: "bf16", 3: "i8", 4: "fp8", 5: "bf8",
              7: "fp8_bf8", 8: "bf8_fp8"}

DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "--cuda-device-only", "--no-gpu-bundle-output",
]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True)
    if res.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + res.stdout + "\n")
        raise RuntimeError("build step failed: " + cmd[-1])
    return res.stdout


def device_jobs():
    jobs = []
    src = os.path.join(CSRC, "gemm_conv_kernels.hip")
    for code, name in GEMM_TYPES.items():
        out = os.path.join(BUILD, "gemm_%s.hsaco" % name)
        jobs.append([HIPCC] + DEVICE_FLAGS +
                    ["-DROCK_DT=%d" % code, "-DROCK_DTNAME=%s" % name,
                     "-o", out, src])
    jobs.append([HIPCC] + DEVICE_FLAGS +
                ["-o", os.path.join(BUILD, "attention.hsaco"),
                 os.path.join(CSRC, "attention_kernels.hip")])
    jobs.append([HIPCC] + DEVICE_FLAGS +
                ["-o", os.path.join(BUILD, "relayout.hsaco"),
                 os.path.join(CSRC, "relayout_kernels.hip")])
    jobs.append([HIPCC] + DEVICE_FLAGS +
                ["-o", os.path.join(BUILD, "probe.hsaco"),
                 os.path.join(CSRC, "probe_kernels.hip")])
    return jobs


def build(jobs=8, verbose=False, host_only=False, only=None):
    """host_only: relink rock_api.cpp against the code objects already built;
    only: rebuild just the code objects whose file name contains this string."""
    os.makedirs(BUILD, exist_ok=True)
    todo = [] if host_only else [j for j in device_jobs() if only is None or only in os.path.basename(j[-2])]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for out in pool.map(_run, todo):
            if verbose and out.strip():
                print(out)
    # the one source with host and device code in one object: the static workspace
    static_o = os.path.join(BUILD, "static_workspace.o")
    _run([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-c", os.path.join(CSRC, "static_workspace.hip"), "-o", static_o])
    blobs_o = os.path.join(BUILD, "blobs.o")
    _run(["gcc", "-c", "-x", "assembler-with-cpp", "-I", BUILD,
          os.path.join(CSRC, "blobs.S"), "-o", blobs_o])
    _run([HIPCC, "-O2", "-std=c++17", "-fPIC", "-shared", "-x", "c++",
          "-D__HIP_PLATFORM_AMD__", "-fvisibility=hidden",
          "-I", os.path.join(ROCM, "include"),
          os.path.join(CSRC, "rock_api.cpp"), "-x", "none", blobs_o, static_o,
          "-L", os.path.join(ROCM, "lib"), "-lamdhip64",
          "-Wl,-rpath," + os.path.join(ROCM, "lib"),
          "-o", LIB])
    return LIB


if __name__ == "__main__":
    only = [a.split("=", 1)[1] for a in sys.argv[1:] if a.startswith("--only=")]
    print(build(verbose=True, host_only="--host-only" in sys.argv[1:], only=only[0] if only else None))
