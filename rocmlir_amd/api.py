"""ctypes binding of librocmlir_amd.so and torch-tensor front ends.

The option strings built here use the reference's own flag names
(rocmlir-gen.cpp:90-561 for gemm / attention, ConvGenerator.cpp:492-661 for
convolution), so a problem reads the same as on a rocmlir-gen command line.
"""
import ctypes as C
import os
import threading

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG, "librocmlir_amd.so")
_lib = None
_lock = threading.Lock()

MIIR_SUCCESS = 0
MIIR_INVALID_PARAM = 1
MIIR_INVALID_MODULE = 2
MIIR_BUILD_FAILURE = 3


class RockError(RuntimeError):
    pass


def library_path():
    return _LIB_PATH


def load_library():
    """Loads librocmlir_amd.so; raises RockError when it has not been built."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise RockError(
                "librocmlir_amd.so is missing (%s): run "
                "`python -c 'import __graft_entry__ as g; g.build()'` "
                "or `python -m rocmlir_amd._build`" % _LIB_PATH)
        L = C.CDLL(_LIB_PATH)
        vp, sz = C.c_void_p, C.c_size_t
        L.miirCreateHandle.restype = vp
        L.miirCreateHandle.argtypes = [C.c_char_p]
        for name in ("miirGetKernelCount", "miirGetWorkspaceSize",
                     "miirLowerTuningParams", "miirLowerBin",
                     "miirDestroyHandle"):
            getattr(L, name).restype = C.c_int
            getattr(L, name).argtypes = [vp]
        L.rockamdGetWorkspaceSize64.restype = sz
        L.rockamdGetWorkspaceSize64.argtypes = [vp]
        L.rockamdGetArgumentInfo.restype = C.c_int
        L.rockamdGetArgumentInfo.argtypes = [vp, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                             C.POINTER(C.c_int64)]
        L.miirBufferGet.restype = C.c_int
        L.miirBufferGet.argtypes = [vp, C.c_char_p, C.POINTER(sz)]
        L.miirGetExecutionDims.restype = C.c_int
        L.miirGetExecutionDims.argtypes = [vp, C.POINTER(sz), C.POINTER(sz)]
        L.rockamdGetKernelName.restype = C.c_int
        L.rockamdGetKernelName.argtypes = [vp, C.c_char_p, C.POINTER(sz)]
        L.rockamdGetKernelAttrs.restype = C.c_int
        L.rockamdGetKernelAttrs.argtypes = [vp, C.POINTER(C.c_uint32)]
        L.rockamdGetKernelArgs.restype = C.c_int
        L.rockamdGetKernelArgs.argtypes = [vp, C.POINTER(C.c_int), vp,
                                           C.POINTER(sz)]
        L.rockamdGetPerfConfig.restype = sz
        L.rockamdGetPerfConfig.argtypes = [vp, C.c_char_p, sz]
        L.rockamdGetProblemKey.restype = sz
        L.rockamdGetProblemKey.argtypes = [vp, C.c_char_p, sz]
        L.rockamdSetScale.restype = C.c_int
        L.rockamdSetScale.argtypes = [vp, C.c_float]
        L.rockamdSetZeroPoint.restype = C.c_int
        L.rockamdSetZeroPoint.argtypes = [vp, C.c_int32]
        L.rockamdLaunch.restype = C.c_int
        L.rockamdLaunch.argtypes = [vp, C.POINTER(vp), C.c_int, vp]
        L.rockamdLaunchStaticWorkspace.restype = C.c_int
        L.rockamdLaunchStaticWorkspace.argtypes = [vp, C.POINTER(vp), C.c_int, vp]
        L.rockamdBenchmark.restype = C.c_int
        L.rockamdBenchmark.argtypes = [vp, C.POINTER(vp), C.c_int, vp, C.c_int,
                                       C.c_int, C.POINTER(C.c_float)]
        L.rockamdMeasureMfmaRate.restype = C.c_int
        L.rockamdMeasureMfmaRate.argtypes = [C.c_int, C.c_int, vp,
                                             C.POINTER(C.c_double)]
        L.rockamdGetLastError.restype = C.c_char_p
        L.rockamdGetLastError.argtypes = []
        L.rockamdTuningSpaceCreate.restype = vp
        L.rockamdTuningSpaceCreate.argtypes = [vp, C.c_int]
        L.rockamdTuningGetNumParams.restype = C.c_uint
        L.rockamdTuningGetNumParams.argtypes = [vp]
        L.rockamdTuningParamToString.restype = sz
        L.rockamdTuningParamToString.argtypes = [vp, C.c_uint, C.c_char_p, sz]
        L.rockamdTuningSpaceDestroy.restype = None
        L.rockamdTuningSpaceDestroy.argtypes = [vp]
        L.rockamdTuningSetFromStr.restype = C.c_int
        L.rockamdTuningSetFromStr.argtypes = [vp, C.c_char_p]
        L.rockamdTuningTableCreate.restype = vp
        L.rockamdTuningTableCreate.argtypes = []
        L.rockamdTuningTableDestroy.restype = None
        L.rockamdTuningTableDestroy.argtypes = [vp]
        L.rockamdTuningUpdateTable.restype = C.c_int
        L.rockamdTuningUpdateTable.argtypes = [vp, C.c_char_p, C.c_char_p,
                                               C.c_float]
        L.rockamdTuningSetFromTable.restype = C.c_int
        L.rockamdTuningSetFromTable.argtypes = [vp, vp]
        L.rockamdGetPointerMap.restype = C.c_int
        L.rockamdGetPointerMap.argtypes = [vp, C.POINTER(C.c_int),
                                           C.POINTER(C.c_int),
                                           C.POINTER(C.c_int32),
                                           C.POINTER(C.c_int64)]
        L.rockamdCheckArgumentSizes.restype = C.c_int
        L.rockamdCheckArgumentSizes.argtypes = [vp, C.POINTER(sz), C.c_int]
        L.rockamdGetParamPointers.restype = C.c_int
        L.rockamdGetParamPointers.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.rockamdIsFusible.restype = C.c_int
        L.rockamdIsFusible.argtypes = [vp, C.c_char_p]
        L.rockamdGetNumPrefillArgs.restype = sz
        L.rockamdGetNumPrefillArgs.argtypes = [vp]
        L.rockamdGetPrefillArgsInfo.restype = None
        L.rockamdGetPrefillArgsInfo.argtypes = [vp, C.POINTER(sz), C.POINTER(C.c_float), sz]
        L.rockamdIsSplitKFaster.restype = C.c_int
        L.rockamdIsSplitKFaster.argtypes = [C.c_int64] * 5 + [C.c_int]
        _lib = L
        return _lib


def last_error():
    return load_library().rockamdGetLastError().decode()


_DTYPE_CODES = {"f32": 0, "f16": 1, "bf16": 2, "i8": 3, "fp8": 4}


def mfma_rate(dtype, random_data=False, stream=None):
    """Sustained 32x32 MFMA issue rate in TFLOP/s (TOP/s) on the current GPU
    for operand type `dtype`, with constant or hashed operand bits."""
    out = C.c_double(0)
    rc = load_library().rockamdMeasureMfmaRate(
        _DTYPE_CODES[dtype], int(bool(random_data)),
        getattr(stream, "cuda_stream", stream), C.byref(out))
    if rc != 0:
        raise RockError("rate probe failed (hip error %d): %s" % (rc, last_error()))
    return out.value


class RockKernel:
    """One problem -> one launchable kernel (a MiirHandle).

    Follows the reference client's call order (rocmlir-lib-test.cpp:31-96):
    create, lower tuning params, lower bin, read the binary and the launch
    dimensions."""

    def __init__(self, options):
        L = load_library()
        self.options = options
        self._h = L.miirCreateHandle(options.encode())
        if not self._h:
            raise RockError("miirCreateHandle failed: %s [%s]"
                            % (last_error(), options))
        self._refresh()

    def _refresh(self):
        """(Re)reads what describes the resolved kernel; called after
        creation and after a perf_config has been applied."""
        L = load_library()
        if L.miirLowerTuningParams(self._h) != MIIR_SUCCESS:
            raise RockError("miirLowerTuningParams failed")
        if L.miirLowerBin(self._h) != MIIR_SUCCESS:
            raise RockError("miirLowerBin failed")
        attrs = (C.c_uint32 * 2)()
        L.rockamdGetKernelAttrs(self._h, attrs)
        self.block_size, self.grid_size = int(attrs[0]), int(attrs[1])
        n = C.c_size_t(0)
        L.rockamdGetKernelName(self._h, None, C.byref(n))
        buf = C.create_string_buffer(n.value)
        L.rockamdGetKernelName(self._h, buf, C.byref(n))
        self.kernel_name = buf.value.decode()
        npt, psz = C.c_int(0), C.c_size_t(0)
        L.rockamdGetKernelArgs(self._h, C.byref(npt), None, C.byref(psz))
        self.num_pointers = npt.value
        self.params_size = psz.value
        # multi-kernel problems: kernels of the problem, its workspace, and the
        # caller pointer list every one of its kernels is launched with
        self.kernel_count = L.miirGetKernelCount(self._h)
        self.workspace_bytes = L.rockamdGetWorkspaceSize64(self._h)
        ncall = C.c_int(0)
        L.rockamdGetPointerMap(self._h, C.byref(ncall), None, None, None)
        self.caller_pointers = ncall.value

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.miirDestroyHandle(h)

    # ---- description ------------------------------------------------------
    def _string(self, fn):
        buf = C.create_string_buffer(2048)
        n = fn(self._h, buf, 2048)
        if n == C.c_size_t(-1).value:
            raise RockError("string query failed")
        return buf.value.decode()

    @property
    def perf_config(self):
        return self._string(load_library().rockamdGetPerfConfig)

    @property
    def problem_key(self):
        return self._string(load_library().rockamdGetProblemKey)

    def code_object(self):
        L = load_library()
        n = C.c_size_t(0)
        if L.miirBufferGet(self._h, None, C.byref(n)) != MIIR_SUCCESS:
            raise RockError("miirBufferGet(size) failed")
        buf = C.create_string_buffer(n.value)
        if L.miirBufferGet(self._h, buf, C.byref(n)) != MIIR_SUCCESS:
            raise RockError("miirBufferGet failed")
        return buf.raw[:n.value]

    def params(self):
        L = load_library()
        n = C.c_size_t(self.params_size)
        buf = C.create_string_buffer(n.value)
        npt = C.c_int(0)
        L.rockamdGetKernelArgs(self._h, C.byref(npt), buf, C.byref(n))
        return buf.raw

    def execution_dims(self):
        g, l = C.c_size_t(0), C.c_size_t(0)
        rc = load_library().miirGetExecutionDims(self._h, C.byref(g),
                                                 C.byref(l))
        if rc != MIIR_SUCCESS:
            raise RockError("miirGetExecutionDims failed (%d)" % rc)
        return g.value, l.value

    # ---- tuning (mlir-c/Dialect/Rock.h:39-117) -------------------------------
    TUNING_KINDS = {"quick": 0, "full": 1, "exhaustive": 2}

    def tuning_space(self, kind="full"):
        """perf_config strings of the kernels this problem can run on; the
        first is the built-in table's choice.  kind: "quick" (at most three
        entries), "full" (every kernel) or "exhaustive" (RockEnums.h:19-23)."""
        L = load_library()
        sp = L.rockamdTuningSpaceCreate(self._h, self.TUNING_KINDS[kind])
        if not sp:
            raise RockError("rockamdTuningSpaceCreate failed")
        try:
            out = []
            for i in range(L.rockamdTuningGetNumParams(sp)):
                buf = C.create_string_buffer(128)
                n = L.rockamdTuningParamToString(sp, i, buf, 128)
                if n == C.c_size_t(-1).value or n >= 128:
                    raise RockError("rockamdTuningParamToString failed")
                out.append(buf.value.decode())
            return out
        finally:
            L.rockamdTuningSpaceDestroy(sp)

    def set_perf_config(self, perf_config):
        """Re-resolves the kernel under `perf_config`
        (mlirRockTuningSetFromStr); unknown strings fall back to the table."""
        if not load_library().rockamdTuningSetFromStr(self._h,
                                                      perf_config.encode()):
            raise RockError("rockamdTuningSetFromStr(%r) failed: %s"
                            % (perf_config, last_error()))
        self._refresh()

    def arguments(self):
        """[(dtype code, dims)] for every pointer launch() takes (rockamdGetArgumentInfo)."""
        out = []
        for i in range(self.caller_pointers):
            dt, rank, dims = C.c_int(), C.c_int(), (C.c_int64 * 6)()
            if load_library().rockamdGetArgumentInfo(self._h, i, C.byref(dt), C.byref(rank), dims) != 0:
                raise RockError("rockamdGetArgumentInfo(%d) failed" % i)
            out.append((dt.value, list(dims[:rank.value])))
        return out

    def set_scale(self, scale):
        load_library().rockamdSetScale(self._h, float(scale))

    def set_zero_point(self, zp):
        load_library().rockamdSetZeroPoint(self._h, int(zp))

    # ---- launch --------------------------------------------------------------
    def _check_sizes(self, args):
        """Every tensor argument must hold at least the bytes the kernel list addresses in it
        (rockamdCheckArgumentSizes): a short one is an error here, not a fault on the device."""
        sizes = (C.c_size_t * len(args))()
        for i, a in enumerate(args):
            sizes[i] = 0 if a is None or isinstance(a, int) else a.numel() * a.element_size()
        if load_library().rockamdCheckArgumentSizes(self._h, sizes, len(args)) != MIIR_SUCCESS:
            raise RockError("%s: %s" % (self.kernel_name, last_error()))

    def _pointer_array(self, args):
        if len(args) != self.caller_pointers:
            raise RockError("kernel %s takes %d pointer arguments, got %d"
                            % (self.kernel_name, self.caller_pointers, len(args)))
        self._check_sizes(args)
        arr = (C.c_void_p * len(args))()
        for i, a in enumerate(args):
            if a is None:
                arr[i] = None
            elif isinstance(a, int):
                arr[i] = a
            else:  # torch tensor
                if not a.is_cuda:
                    raise RockError("tensor arguments must live on the GPU")
                arr[i] = a.data_ptr()
        return arr

    @staticmethod
    def _stream(stream):
        if stream is None:
            import torch
            return torch.cuda.current_stream().cuda_stream
        return getattr(stream, "cuda_stream", stream)

    def launch(self, *args, stream=None):
        arr = self._pointer_array(args)
        rc = load_library().rockamdLaunch(self._h, arr, len(args),
                                          self._stream(stream))
        if rc != 0:
            raise RockError("launch of %s failed (hip error %d): %s"
                            % (self.kernel_name, rc, last_error()))

    def benchmark(self, *args, warmup=3, iters=20, stream=None):
        """Average milliseconds per launch (HIP events on the launch stream)."""
        arr = self._pointer_array(args)
        ms = C.c_float(0)
        rc = load_library().rockamdBenchmark(self._h, arr, len(args),
                                             self._stream(stream), warmup,
                                             iters, C.byref(ms))
        if rc != 0:
            raise RockError("benchmark of %s failed (hip error %d): %s"
                            % (self.kernel_name, rc, last_error()))
        return ms.value


class RockProgram:
    """All kernels of one problem (miirGetKernelCount handles, one per
    --kernel_id) plus the workspace they share; launch() runs them in order
    on one stream.  Single-kernel problems behave like their RockKernel."""

    def __init__(self, options):
        self.options = options
        self._build(options)

    def _build(self, options):
        first = RockKernel(options)
        self.kernels = [first] + [RockKernel("%s --kernel_id %d" % (options, i))
                                  for i in range(1, first.kernel_count)]
        self.workspace_bytes = first.workspace_bytes
        self._workspace = None

    @property
    def main(self):
        """The contraction kernel: the last GEMM, convolution or attention kernel of the list (conversion
        kernels may run in front of it, the reduction of split partial sums behind it)."""
        for k in reversed(self.kernels):
            if k.kernel_name.startswith(("rock_gemm_", "rock_conv_", "rock_attention_")):
                return k
        return self.kernels[-1]

    # what rocmlir_amd.tuning.tune() uses, so that problems of several kernels tune like single ones
    kernel_name = property(lambda self: self.main.kernel_name)
    perf_config = property(lambda self: self.main.perf_config)
    problem_key = property(lambda self: self.main.problem_key)

    def tuning_space(self, kind="full"):
        return self.kernels[0].tuning_space(kind)

    def set_perf_config(self, perf_config):
        """Plans the problem again under `perf_config` (the kernel list can
        change: a request may add or drop conversion kernels)."""
        self._build(self.options + (" --perf_config %s" % perf_config if perf_config else ""))

    def _args(self, args):
        if self.kernels[0].caller_pointers == len(args):
            return args   # no workspace pointer in this problem's caller list
        if self._workspace is None:
            import torch
            dev = next(a.device for a in args if a is not None and not isinstance(a, int))
            self._workspace = torch.empty(max(self.workspace_bytes, 16), dtype=torch.uint8, device=dev)
        return tuple(args) + (self._workspace,)

    def launch(self, *args, stream=None):
        full = self._args(args)
        for k in self.kernels:
            k.launch(*full, stream=stream)

    def benchmark(self, *args, warmup=3, iters=20, stream=None):
        """Sum of the kernels' average times in milliseconds."""
        return sum(ms for _, ms in self.benchmark_each(*args, warmup=warmup, iters=iters, stream=stream))

    def benchmark_sequence(self, *args, warmup=2, iters=5):
        """Average milliseconds for the whole list launched in order, back to back (events on torch's current
        stream, where launch() puts the kernels): what a caller of a many-kernel problem waits for, gaps between
        the kernels and the state of the caches they leave each other included."""
        import torch
        full = self._args(args)
        for _ in range(warmup):
            self.launch(*args)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            for k in self.kernels:
                k.launch(*full)
        stop.record()
        stop.synchronize()
        return start.elapsed_time(stop) / iters

    def benchmark_each(self, *args, warmup=3, iters=20, stream=None):
        """[(kernel name, average time in milliseconds)] in launch order."""
        full = self._args(args)
        return [(k.kernel_name, k.benchmark(*full, warmup=warmup, iters=iters, stream=stream)) for k in self.kernels]


# ---------------------------------------------------------------------------
# torch front ends
# ---------------------------------------------------------------------------
_kernel_cache = {}


def _kernel(options):
    k = _kernel_cache.get(options)
    if k is None:
        k = _kernel_cache[options] = RockKernel(options)
    return k


_program_cache = {}


def _program(options):
    p = _program_cache.get(options)
    if p is None:
        p = _program_cache[options] = RockProgram(options)
    return p


def _dtype_name(dt):
    import torch
    names = {torch.float32: "f32", torch.float16: "f16", torch.bfloat16: "bf16",
             torch.int8: "i8", torch.int32: "i32"}
    if hasattr(torch, "float8_e4m3fn"):
        names[torch.float8_e4m3fn] = "fp8"
        names[torch.float8_e5m2] = "bf8"
    try:
        return names[dt]
    except KeyError:
        raise RockError("unsupported tensor dtype %s" % dt)


def _torch_dtype(name):
    import torch
    return {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16,
            "i8": torch.int8, "i32": torch.int32,
            "fp8": torch.float8_e4m3fn, "bf8": torch.float8_e5m2}[name]


def _is_tensor(x):
    return hasattr(x, "data_ptr")


def _channel_vectors(scale, zero_point, quant_scale, out_zero_point):
    """The per-channel quantisation vectors among the four epilogue values, in
    the order the library takes them behind the problem's own tensors, and the
    flags that announce them (a torch tensor instead of a number means one
    value per output channel: f32 scales, int32 or int8 zero points)."""
    import torch
    flags, vectors = "", []
    for name, val, is_zp in (("scale_vector", scale, False), ("zero_point_vector", zero_point, True),
                             ("quant_scale_vector", quant_scale, False),
                             ("out_zero_point_vector", out_zero_point, True)):
        if not _is_tensor(val):
            continue
        if is_zp:
            if val.dtype not in (torch.int8, torch.int32):
                raise RockError("%s: int32 or int8 elements" % name)
            flags += " -%s %s" % (name, "i8" if val.dtype == torch.int8 else "i32")
        else:
            if val.dtype != torch.float32:
                raise RockError("%s: f32 elements" % name)
            flags += " -%s true" % name
        vectors.append(val.contiguous())
    return flags, vectors


def _epilogue_flags(scale, zero_point, bias, relu, quant_scale, out_zero_point,
                    activation=None, clip=None, residual=None, residual_op="add"):
    s = ""
    if scale is not None and not _is_tensor(scale):
        s += " -scale %.9g" % scale
    if not _is_tensor(zero_point) and zero_point:
        s += " -zero_point %d" % zero_point
    if quant_scale is not None and not _is_tensor(quant_scale):
        s += " -quant_scale %.9g" % quant_scale
    if not _is_tensor(out_zero_point) and out_zero_point:
        s += " -out_zero_point %d" % out_zero_point
    s += _channel_vectors(scale, zero_point, quant_scale, out_zero_point)[0]
    if bias is not None:
        s += " -bias true"
    if relu:
        s += " -relu true"
    if activation:
        s += " -activation %s" % activation
    if clip is not None:
        s += " -activation clip -clip_min %.9g -clip_max %.9g" % tuple(clip)
    if residual is not None:
        s += " -residual %s" % residual_op
    return s


def gemm(a, b, *, transA=False, transB=False, transC=False, out_dtype=None,
         scale=None, zero_point=0, bias=None, relu=False, quant_scale=None,
         out_zero_point=0, activation=None, clip=None, residual=None,
         residual_op="add", out=None, perf_config=None, stream=None,
         info=None, split_k=True, layout_conversion=True, accumulate=False):
    """C = epilogue(A x B) with the reference's storage conventions
    (rocmlir-gen.cpp:2058-2080): a is [G,M,K] ([G,K,M] if transA), b is
    [G,K,N] ([G,N,K] if transB), result [G,M,N] ([G,N,M] if transC).
    2-D inputs mean G = 1.  `scale`, `zero_point`, `quant_scale` and
    `out_zero_point` are numbers (per tensor) or torch tensors with one element
    per column of the result (per channel: f32 scales, int32 / int8 zero
    points).  The epilogue runs scale / zero point, per-column
    `bias`, `residual` (a tensor shaped and typed like the result, combined by
    `residual_op` "add" or "mul"), then `activation` ("relu", "sigmoid",
    "tanh", "erf", "gelu", "exp") or `clip=(lo, hi)`, then the narrowing to
    the output type.  A dict passed as `info` receives the name and
    perf_config of the GEMM kernel that ran and the names of all kernels of
    the problem (operands that are not whole 16-byte chunks are first copied
    into padded ones unless `layout_conversion` is False; a long reduction
    over few output tiles is split over blocks unless `split_k` is False).
    `accumulate=True` (rocmlir-gen's -store-method atomic_add) adds the
    result into `out` instead of overwriting it."""
    import torch
    if accumulate and (out is None or residual is not None):
        raise RockError("gemm: accumulate=True adds into `out` and takes no residual")
    a3 = a if a.dim() == 3 else a.unsqueeze(0)
    b3 = b if b.dim() == 3 else b.unsqueeze(0)
    a3, b3 = a3.contiguous(), b3.contiguous()
    G = a3.shape[0]
    M, K = (a3.shape[2], a3.shape[1]) if transA else (a3.shape[1], a3.shape[2])
    Kb, N = (b3.shape[2], b3.shape[1]) if transB else (b3.shape[1], b3.shape[2])
    if Kb != K or b3.shape[0] != G:
        raise RockError("gemm: operand shapes do not match")
    ta, tb = _dtype_name(a3.dtype), _dtype_name(b3.dtype)
    t = ta if ta == tb else "%s_%s" % (ta, tb)
    opts = ("-operation gemm -arch gfx950 -t %s -g %d -m %d -n %d -k %d"
            " -transA %s -transB %s -transC %s"
            % (t, G, M, N, K, str(bool(transA)).lower(),
               str(bool(transB)).lower(), str(bool(transC)).lower()))
    if out_dtype is not None:
        opts += " -out_datatype %s" % out_dtype
    if perf_config:
        opts += " -perf_config %s" % perf_config
    if not split_k:
        opts += " -split_k false"
    if not layout_conversion:
        opts += " -layout_conversion false"
    if accumulate:
        opts += " -store-method atomic_add"
    opts += _epilogue_flags(scale, zero_point, bias, relu, quant_scale,
                            out_zero_point, activation, clip, residual,
                            residual_op)
    prog = _program(opts)   # one kernel, or several: padded operand copies, a reduction split over blocks
    k = next(x for x in prog.kernels if x.kernel_name.startswith("rock_gemm_"))
    if info is not None:
        info["kernel_name"] = k.kernel_name
        info["perf_config"] = k.perf_config
        info["kernels"] = [x.kernel_name for x in prog.kernels]
    if out_dtype is None:
        out_dtype = {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(ta, ta)
    shape = (G, N, M) if transC else (G, M, N)
    if out is None:
        out = torch.empty(shape, dtype=_torch_dtype(out_dtype), device=a.device)
    vectors = _channel_vectors(scale, zero_point, quant_scale, out_zero_point)[1]
    if any(v.numel() != N for v in vectors):
        raise RockError("gemm: a per-channel vector holds one element per column of the result")
    if residual is None:
        prog.launch(a3, b3, out, bias, *vectors, stream=stream)
    else:
        if residual.dtype != out.dtype or residual.numel() != out.numel():
            raise RockError("gemm: the residual must have the result's type and size")
        prog.launch(a3, b3, out, bias, residual.contiguous(), *vectors, stream=stream)
    return out if a.dim() == 3 else out.squeeze(0)


def conv2d(fil, inp, *, fil_layout, in_layout, out_layout, batchsize,
           in_channels, out_channels, in_h, in_w, fil_h, fil_w, groupsize=1,
           stride=(1, 1), padding=(0, 0), dilation=(1, 1), out_dtype=None,
           scale=None, zero_point=0, bias=None, relu=False, quant_scale=None,
           out_zero_point=0, activation=None, clip=None, residual=None,
           residual_op="add", out=None, perf_config=None, stream=None,
           info=None, padding_r=None, layout_conversion=True):
    """Forward convolution; tensors are flat device buffers laid out as the
    layout strings say (Miir / rocmlir-gen spelling, e.g. 'gkyxc', 'nhwgc',
    'NGCHW').  Epilogue arguments as for gemm(); the residual is laid out
    like the output.  `padding` is the top / left padding and, unless
    `padding_r` gives the bottom / right one (--padding_h_r / --padding_w_r),
    that one too.  Returns the flat output tensor.  A dict passed as `info`
    receives the name and perf_config of the kernel that ran.
    `layout_conversion=False` keeps the tensors where they lie (no conversion
    kernels in front; the element-wise kernel where the vector ones cannot read them)."""
    import torch
    t = _dtype_name(inp.dtype)
    pr = padding if padding_r is None else padding_r
    ho = (in_h + padding[0] + pr[0] - (fil_h - 1) * dilation[0] - 1) // stride[0] + 1
    wo = (in_w + padding[1] + pr[1] - (fil_w - 1) * dilation[1] - 1) // stride[1] + 1
    opts = ("--operation conv --arch gfx950 --in_type %s --fil_type %s"
            " --fil_layout %s --in_layout %s --out_layout %s --batchsize %d"
            " --groupsize %d --in_channels %d --out_channels %d --in_h %d"
            " --in_w %d --out_h %d --out_w %d --fil_h %d --fil_w %d"
            " --dilation_h %d --dilation_w %d --conv_stride_h %d"
            " --conv_stride_w %d --padding_h %d --padding_w %d"
            % (t, _dtype_name(fil.dtype), fil_layout, in_layout, out_layout,
               batchsize, groupsize, in_channels, out_channels, in_h, in_w, ho,
               wo, fil_h, fil_w, dilation[0], dilation[1], stride[0], stride[1],
               padding[0], padding[1]))
    if padding_r is not None:
        opts += " --padding_h_r %d --padding_w_r %d" % (pr[0], pr[1])
    if out_dtype is not None:
        opts += " --out_type %s" % out_dtype
    if perf_config:
        opts += " --perf_config %s" % perf_config
    if not layout_conversion:
        opts += " --layout_conversion false"
    opts += _epilogue_flags(scale, zero_point, bias, relu, quant_scale,
                            out_zero_point, activation, clip, residual,
                            residual_op)
    prog = _program(opts)
    k = prog.main
    if info is not None:
        info["kernel_name"] = k.kernel_name
        info["perf_config"] = k.perf_config
        info["kernels"] = [x.kernel_name for x in prog.kernels]
    if out_dtype is None:
        out_dtype = {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(t, t)
    if out is None:
        out = torch.empty(batchsize * out_channels * ho * wo,
                          dtype=_torch_dtype(out_dtype), device=inp.device)
    vectors = _channel_vectors(scale, zero_point, quant_scale, out_zero_point)[1]
    if any(v.numel() != out_channels for v in vectors):
        raise RockError("conv2d: a per-channel vector holds one element per output channel")
    if residual is None:
        prog.launch(fil.contiguous(), inp.contiguous(), out, bias, *vectors, stream=stream)
    else:
        if residual.dtype != out.dtype or residual.numel() != out.numel():
            raise RockError("conv2d: the residual must have the output's type and size")
        prog.launch(fil.contiguous(), inp.contiguous(), out, bias, residual.contiguous(), *vectors, stream=stream)
    return out


def attention(q, k, v, *, scale=1.0, bias=None, scale_tensor=None, mask=None, other=None, zero_point=0,
              transQ=False, transK=False, transV=False, transO=False, out=None, stream=None, info=None,
              score_workspace_limit=None, program=None, inputs=(), layout_conversion=True):
    """O = softmax(scale * scale_tensor * Q K + bias) V (bias and scale_tensor
    optional [G,seq_q,seq_k] tensors, rocmlir-gen's -with-attn-bias /
    -with-attn-scale).  `mask` (int8 or bool, [G,seq_q,seq_k]) with `other`
    (same shape, v's type) puts migraphx.where(mask, scores, other) in front of
    the softmax (mixr-attn-where.mlir:11): a zero in the mask replaces the score
    by other's element.  Storage follows the reference's
    conventions (rocmlir-gen.cpp:2149-2200): q [G,seq_q,d] ([G,d,seq_q] if
    transQ); k [G,d,seq_k] ([G,seq_k,d] if transK -- the usual row-major keys);
    v [G,seq_k,dv] ([G,dv,seq_k] if transV); result [G,seq_q,dv]
    ([G,dv,seq_q] if transO).  int8 q and k (with f16 v, bias, scale_tensor)
    select the quantised first GEMM: the scores are (acc - zero_point) * scale.
    A dict passed as `info` receives the names of the kernels that ran.
    `score_workspace_limit` (bytes) bounds the score chunk of the three-kernel
    form (f32, head dimensions above 256); the default is 32 MiB.
    `program` is a pre-softmax element-wise tree in postfix form over the score
    `x`, the tensors `inputs` (`t0`, `t1`, ...; each [G,seq_q,seq_k], any of
    f32 / f16 / bf16 / int8) and constants `c:<number>`, e.g.
    "x,t0,mul,exp,t1,add" (the region of rock.attention, RockOps.td:208-254);
    it replaces scale, bias, scale_tensor and mask."""
    import torch
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    G = q.shape[0]
    sq, dqk = (q.shape[2], q.shape[1]) if transQ else (q.shape[1], q.shape[2])
    sk = k.shape[1] if transK else k.shape[2]
    dv = v.shape[1] if transV else v.shape[2]
    t = _dtype_name(q.dtype)
    tf = lambda b: str(bool(b)).lower()  # noqa: E731
    opts = ("-operation attention -arch gfx950 -t %s -g %d -seq_len_q %d"
            " -seq_len_k %d -head_dim_qk %d -head_dim_v %d -transQ %s"
            " -transK %s -transV %s -transO %s -scale %.9g"
            % (t, G, sq, sk, dqk, dv, tf(transQ), tf(transK), tf(transV),
               tf(transO), scale))
    if bias is not None:
        opts += " -with-attn-bias true"
    if scale_tensor is not None:
        opts += " -with-attn-scale true"
    if zero_point:
        opts += " -zero_point %d" % zero_point
    if (mask is None) != (other is None):
        raise RockError("attention: mask and other come together")
    if mask is not None:
        opts += " -with-attn-mask true"
        if tuple(mask.shape) != (G, sq, sk) or tuple(other.shape) != (G, sq, sk) or other.dtype != v.dtype:
            raise RockError("attention: mask and other are [G, seq_q, seq_k]; other has v's type")
        mask = mask.to(torch.int8).contiguous()
    if not layout_conversion:   # no copies in front of or behind the kernel: tensors are read as they lie
        opts += " -layout_conversion false"
    if score_workspace_limit is not None:
        opts += " -score_workspace_limit %d" % score_workspace_limit
    if program:
        if bias is not None or scale_tensor is not None or mask is not None or scale != 1.0:
            raise RockError("attention: a program replaces scale, bias, scale_tensor and mask")
        opts += " -attn_elementwise %s" % program.replace(" ", "")
        if inputs:
            opts += " -attn_inputs %s" % ",".join(_dtype_name(t.dtype) for t in inputs)
    kern = _program(opts)   # one fused kernel, or three for head dimensions above 128 and f32
    if info is not None:
        info["kernels"] = [k.kernel_name for k in kern.kernels]
    shape = (G, dv, sq) if transO else (G, sq, dv)
    if out is None:
        out = torch.empty(shape, dtype=v.dtype, device=q.device)
    pre = ([] if scale_tensor is None else [scale_tensor.contiguous()]) + [bias]
    if mask is not None:
        pre += [mask, other.contiguous()]
    if program:
        pre = [t.contiguous() for t in inputs]
    kern.launch(q, k, v, *pre, out, stream=stream)
    return out


def conv3d(fil, inp, *, fil_layout, in_layout, out_layout, batchsize, in_channels, out_channels, in_size,
           fil_size, groupsize=1, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1), out_dtype=None,
           scale=None, zero_point=0, bias=None, relu=False, quant_scale=None, out_zero_point=0,
           activation=None, clip=None, residual=None, residual_op="add", out=None, perf_config=None,
           stream=None, info=None):
    """Forward convolution over three spatial dimensions.  Sizes, strides,
    padding and dilation are (h, w, d) triples; the layout strings have six
    letters ('ngc012' / 'gkc012' / 'ngk012' in rocmlir-gen's spelling, h w d
    and y x z accepted for 0 1 2).  Epilogue arguments as for conv2d(); the
    residual is laid out like the output.  Returns the flat output tensor."""
    import torch
    t = _dtype_name(inp.dtype)
    outs = [(in_size[a] + 2 * padding[a] - (fil_size[a] - 1) * dilation[a] - 1) // stride[a] + 1 for a in range(3)]
    opts = ("--operation conv --arch gfx950 --in_type %s --fil_type %s --fil_layout %s --in_layout %s"
            " --out_layout %s --batchsize %d --groupsize %d --in_channels %d --out_channels %d"
            % (t, _dtype_name(fil.dtype), fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels,
               out_channels))
    for a, s in enumerate("hwd"):
        opts += (" --in_%s %d --fil_%s %d --out_%s %d --dilation_%s %d --conv_stride_%s %d --padding_%s %d"
                 % (s, in_size[a], s, fil_size[a], s, outs[a], s, dilation[a], s, stride[a], s, padding[a]))
    if out_dtype is not None:
        opts += " --out_type %s" % out_dtype
    if perf_config:
        opts += " --perf_config %s" % perf_config
    opts += _epilogue_flags(scale, zero_point, bias, relu, quant_scale, out_zero_point, activation, clip, residual,
                            residual_op)
    prog = _program(opts)
    if info is not None:
        info["kernels"] = [x.kernel_name for x in prog.kernels]
        info["workspace_bytes"] = prog.workspace_bytes
    if out_dtype is None:
        out_dtype = {"i8": "i32", "fp8": "f32", "bf8": "f32"}.get(t, t)
    if out is None:
        out = torch.empty(batchsize * out_channels * outs[0] * outs[1] * outs[2], dtype=_torch_dtype(out_dtype),
                          device=inp.device)
    if residual is None:
        prog.launch(fil.contiguous(), inp.contiguous(), out, bias, stream=stream)
    else:
        if residual.dtype != out.dtype or residual.numel() != out.numel():
            raise RockError("conv3d: the residual must have the output's type and size")
        prog.launch(fil.contiguous(), inp.contiguous(), out, bias, residual.contiguous(), stream=stream)
    return out


def _conv3d_options(operation, t, fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels,
                    out_channels, in_size, fil_size, stride, padding, dilation):
    opts = ("--operation %s --arch gfx950 --in_type %s --fil_type %s --out_type %s --fil_layout %s --in_layout %s"
            " --out_layout %s --batchsize %d --groupsize %d --in_channels %d --out_channels %d"
            % (operation, t, t, t, fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels,
               out_channels))
    for a, s in enumerate("hwd"):
        opts += (" --in_%s %d --fil_%s %d --dilation_%s %d --conv_stride_%s %d --padding_%s %d"
                 % (s, in_size[a], s, fil_size[a], s, dilation[a], s, stride[a], s, padding[a]))
    return opts


def conv3d_bwd_data(fil, dout, *, fil_layout, in_layout, out_layout, batchsize, in_channels, out_channels, in_size,
                    fil_size, groupsize=1, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1), out=None,
                    stream=None, info=None):
    """Gradient of conv3d with respect to its input (operation conv_bwd_data
    with the in_d / fil_d keys): `dout` is the gradient of the output, laid
    out as `out_layout` says; returns the flat input-shaped gradient."""
    import torch
    t = _dtype_name(dout.dtype)
    prog = _program(_conv3d_options("conv_bwd_data", t, fil_layout, in_layout, out_layout, batchsize, groupsize,
                                    in_channels, out_channels, in_size, fil_size, stride, padding, dilation))
    if info is not None:
        info["kernels"] = [k.kernel_name for k in prog.kernels]
        info["workspace_bytes"] = prog.workspace_bytes
    if out is None:
        out = torch.empty(batchsize * in_channels * in_size[0] * in_size[1] * in_size[2], dtype=dout.dtype,
                          device=dout.device)
    prog.launch(fil.contiguous(), out, dout.contiguous(), None, stream=stream)
    return out


def conv3d_bwd_weight(inp, dout, *, fil_layout, in_layout, out_layout, batchsize, in_channels, out_channels,
                      in_size, fil_size, groupsize=1, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1),
                      out=None, stream=None, info=None):
    """Gradient of conv3d with respect to its filter (operation
    conv_bwd_weight with the in_d / fil_d keys); returns the flat
    filter-shaped gradient."""
    import torch
    t = _dtype_name(dout.dtype)
    prog = _program(_conv3d_options("conv_bwd_weight", t, fil_layout, in_layout, out_layout, batchsize, groupsize,
                                    in_channels, out_channels, in_size, fil_size, stride, padding, dilation))
    if info is not None:
        info["kernels"] = [k.kernel_name for k in prog.kernels]
        info["workspace_bytes"] = prog.workspace_bytes
    if out is None:
        out = torch.empty(out_channels * (in_channels // groupsize) * fil_size[0] * fil_size[1] * fil_size[2],
                          dtype=dout.dtype, device=dout.device)
    prog.launch(out, inp.contiguous(), dout.contiguous(), None, stream=stream)
    return out


def _conv_options(operation, t, fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels, out_channels,
                  in_h, in_w, fil_h, fil_w, stride, padding, dilation):
    return ("--operation %s --arch gfx950 --in_type %s --fil_type %s --out_type %s"
            " --fil_layout %s --in_layout %s --out_layout %s --batchsize %d"
            " --groupsize %d --in_channels %d --out_channels %d --in_h %d"
            " --in_w %d --fil_h %d --fil_w %d --dilation_h %d --dilation_w %d"
            " --conv_stride_h %d --conv_stride_w %d --padding_h %d --padding_w %d"
            % (operation, t, t, t, fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels,
               out_channels, in_h, in_w, fil_h, fil_w, dilation[0], dilation[1], stride[0], stride[1],
               padding[0], padding[1]))


def conv2d_bwd_data(fil, dout, *, fil_layout, in_layout, out_layout, batchsize, in_channels, out_channels, in_h,
                    in_w, fil_h, fil_w, groupsize=1, stride=(1, 1), padding=(0, 0), dilation=(1, 1), out=None,
                    layout_conversion=True, stream=None, info=None):
    """Gradient of conv2d with respect to its input (rocmlir-gen / Miir
    operation conv_bwd_data): `dout` is the gradient of the output, laid out
    as `out_layout` says; returns the flat input-shaped gradient."""
    import torch
    t = _dtype_name(dout.dtype)
    opts = _conv_options("conv_bwd_data", t, fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels,
                         out_channels, in_h, in_w, fil_h, fil_w, stride, padding, dilation)
    if not layout_conversion:
        opts += " --layout_conversion false"
    prog = _program(opts)
    if info is not None:
        info["kernels"] = [k.kernel_name for k in prog.kernels]
        info["workspace_bytes"] = prog.workspace_bytes
    if out is None:
        out = torch.empty(batchsize * in_channels * in_h * in_w, dtype=dout.dtype, device=dout.device)
    prog.launch(fil.contiguous(), out, dout.contiguous(), None, stream=stream)
    return out


def conv2d_bwd_weight(inp, dout, *, fil_layout, in_layout, out_layout, batchsize, in_channels, out_channels, in_h,
                      in_w, fil_h, fil_w, groupsize=1, stride=(1, 1), padding=(0, 0), dilation=(1, 1), out=None,
                      layout_conversion=True, stream=None, info=None, as_gemm=True):
    """Gradient of conv2d with respect to its filter (operation
    conv_bwd_weight); returns the flat filter-shaped gradient.  as_gemm=False
    keeps channels-last problems off the single K-major GEMM over the tensors
    as they lie (--bwd_weight_gemm false)."""
    import torch
    t = _dtype_name(dout.dtype)
    opts = _conv_options("conv_bwd_weight", t, fil_layout, in_layout, out_layout, batchsize, groupsize, in_channels,
                         out_channels, in_h, in_w, fil_h, fil_w, stride, padding, dilation)
    if not layout_conversion:
        opts += " --layout_conversion false"
    if not as_gemm:
        opts += " --bwd_weight_gemm false"
    prog = _program(opts)
    if info is not None:
        info["kernels"] = [k.kernel_name for k in prog.kernels]
        info["workspace_bytes"] = prog.workspace_bytes
    if out is None:
        out = torch.empty(out_channels * (in_channels // groupsize) * fil_h * fil_w, dtype=dout.dtype,
                          device=dout.device)
    prog.launch(out, inp.contiguous(), dout.contiguous(), None, stream=stream)
    return out
