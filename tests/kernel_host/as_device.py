"""pytest plugin: the GPU tests with the CPU build of the kernels in place of the device.

  python -m pytest -p tests.kernel_host.as_device tests/test_gpu_conv.py -m gpu

The binding's launch is replaced by one that runs the kernel on the model in this process, on the tensors' own
memory (torch tensors on the CPU: the `gpu` fixture hands out the CPU device); a launch that has not finished
after ROCK_HOST_LAUNCH_SECONDS (150) is skipped, and so is everything that measures time.  ROCK_HOST_LATE_LOADS=1
makes loads into LDS land at the wait that covers them, ROCK_HOST_THREAD_ORDER=1|2 changes the order in which a
block's threads take their turns (descending, waves rotated).  The model is built for
every operand type with the rolled-epilogue kernels into ROCK_HOST_BUILD_DIR (ten minutes the first time, kept
while the sources are unchanged).  Not for the full-size configurations, and not for the entry point that takes
its workspace from the library's device image."""
import ctypes as C
import os
import struct

import pytest
import torch

import rocmlir_amd.api as api
from tests.kernel_host import model as km
from tests.kernel_host.sweep import source_stamp

_SECONDS = int(os.environ.get("ROCK_HOST_LAUNCH_SECONDS", "150"))
_model = None


def _the_model():
    global _model
    if _model is None:
        base = os.environ.get("ROCK_HOST_BUILD_DIR", os.path.join(os.environ.get("TMPDIR", "/tmp"), "rock_kernel_host"))
        d = os.path.join(base, "%s-%s-1" % (source_stamp(), "_".join(str(t) for t in km.ALL_TYPES)))
        so = os.path.join(d, "libkernel_host.so")
        if not os.path.exists(so):
            os.makedirs(d, exist_ok=True)
            km.build_model(d, types=km.ALL_TYPES, rolled=True)
        _model = km.load_model(so)
        _model.hm_set_late_loads(int(os.environ.get("ROCK_HOST_LATE_LOADS", "0")))
        _model.hm_set_thread_order(int(os.environ.get("ROCK_HOST_THREAD_ORDER", "0")))
    return _model


def _pointer_array(self, args):
    if len(args) != self.caller_pointers:
        raise api.RockError("kernel %s takes %d pointer arguments, got %d" % (self.kernel_name, self.caller_pointers, len(args)))
    self._check_sizes(args)
    return [None if a is None else a if isinstance(a, int) else a.data_ptr() for a in args]


def _launch(self, *args, stream=None):
    caller = _pointer_array(self, args)
    lib = api.load_library()
    ptrs = (C.c_void_p * 8)()
    for j, (src, off) in enumerate(km.pointer_map(api, self)):
        ptrs[j] = None if src < 0 or caller[src] is None else caller[src] + off
    # tensors whose addresses the kernel takes from its parameter block
    params = bytearray(self.params())
    count, at, source = C.c_int(0), (C.c_int32 * 16)(), (C.c_int32 * 16)()
    if lib.rockamdGetParamPointers(self._h, C.byref(count), at, source) == 0:
        for i in range(count.value):
            struct.pack_into("<Q", params, at[i], caller[source[i]] or 0)
    name = self.kernel_name.encode()
    model = _the_model()
    if not model.hm_knows(name):
        pytest.skip("the model does not hold " + self.kernel_name)
    bad = model.hm_run_direct(name, bytes(params), ptrs, self.grid_size, self.block_size, _SECONDS)
    if bad == -3:
        pytest.skip("too long for the model: " + self.kernel_name)
    if bad:
        raise api.RockError("%d accesses outside the tensors in %s" % (bad, self.kernel_name))


def _no_timing(*args, **kwargs):
    pytest.skip("timing is not the model's business")


api.RockKernel.launch = _launch
api.RockKernel._pointer_array = _pointer_array
api.RockKernel.benchmark = _no_timing
api.mfma_rate = _no_timing
import rocmlir_amd  # noqa: E402
rocmlir_amd.mfma_rate = _no_timing
torch.cuda.synchronize = lambda *args, **kwargs: None


@pytest.hookimpl(tryfirst=True)
def pytest_fixture_setup(fixturedef, request):
    if fixturedef.argname == "gpu":
        device = torch.device("cpu")
        fixturedef.cached_result = (device, fixturedef.cache_key(request), None)
        return device
