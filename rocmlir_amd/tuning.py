"""In-process tuner and tuning table over the C ABI.

The loop of the reference's rocmlir-tuning-driver
(mlir/tools/rocmlir-tuning-driver/rocmlir-tuning-driver.cpp:234-397): for
every entry of the problem's tuning space, apply the perf_config, time the
kernel on the caller's buffers, and record the best in a table keyed by the
reference's problem key (mlirRockTuningUpdateTable / SetFromTable,
mlir-c/Dialect/Rock.h:94-117).  The table can be saved in the reference's
tab-separated ".tuning" text form ("<arch>\t<numCU>\t<problem>\t<perf_config>",
read back by read_tuning_db, mlir/utils/performance/perfRunner.py:174-199).
"""
import ctypes as C

from .api import RockError, load_library


class TuningTable:
    """Problem key -> best perf_config seen (and its time in ms)."""

    def __init__(self):
        self._t = load_library().rockamdTuningTableCreate()
        if not self._t:
            raise RockError("rockamdTuningTableCreate failed")
        self._entries = {}  # mirror for save(): the C table has no iteration

    def __del__(self):
        t, self._t = getattr(self, "_t", None), None
        if t:
            load_library().rockamdTuningTableDestroy(t)

    def update(self, problem_key, perf_config, time_ms):
        """True if the entry was stored, False if a faster one exists."""
        stored = bool(load_library().rockamdTuningUpdateTable(
            self._t, problem_key.encode(), perf_config.encode(),
            C.c_float(time_ms)))
        if stored:
            self._entries[problem_key] = (perf_config, float(time_ms))
        return stored

    def apply(self, kernel):
        """Sets the kernel's perf_config from the table; False if the problem
        is not in it (the kernel keeps the built-in choice)."""
        found = bool(load_library().rockamdTuningSetFromTable(self._t,
                                                              kernel._h))
        if found:
            kernel._refresh()
        return found

    def __len__(self):
        return len(self._entries)

    def entries(self):
        return dict(self._entries)

    def save(self, path):
        with open(path, "w") as f:
            for key in sorted(self._entries):
                f.write("%s\t%s\n" % (key, self._entries[key][0]))

    @classmethod
    def load(cls, path):
        t = cls()
        with open(path) as f:
            for line in f:
                line = line.rstrip("\n")
                if not line or line.startswith("#"):
                    continue
                key, _, perf = line.rpartition("\t")
                t.update(key, perf, 0.0)
        return t


def tune(kernel, *args, table=None, warmup=5, iters=20, stream=None, kind="full"):
    """Times every entry of `kernel`'s tuning space (of the given kind) on the
    given device buffers, leaves the fastest applied, records it in `table` if
    given, and returns [(perf_config, kernel_name, ms), ...] fastest first."""
    results = []
    for perf in kernel.tuning_space(kind):
        kernel.set_perf_config(perf)
        ms = kernel.benchmark(*args, warmup=warmup, iters=iters, stream=stream)
        results.append((kernel.perf_config, kernel.kernel_name, ms))
    results.sort(key=lambda r: r[2])
    kernel.set_perf_config(results[0][0])
    if table is not None:
        table.update(kernel.problem_key, results[0][0], results[0][2])
    return results
