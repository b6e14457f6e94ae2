"""Python host side of ark::Executor over the C ABI.

Lifecycle as in the reference (ark/api/executor.cpp, python/ark/runtime.py):
Executor(plan) -> compile() -> launch() -> run(n) -> wait() -> stop().
Tensor I/O goes through numpy arrays (bf16 as uint16 bit patterns) or torch
tensors on the host.
"""
import ctypes
import json

import numpy as np

from ._lib import lib, check

_ELEM = {"fp32": 4, "fp16": 2, "bf16": 2, "int32": 4, "uint32": 4, "int8": 1, "uint8": 1, "byte": 1}
_NP = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16, "int32": np.int32,
       "uint32": np.uint32, "int8": np.int8, "uint8": np.uint8, "byte": np.uint8}


class ExecInfo(ctypes.Structure):
    _fields_ = [("device_id", ctypes.c_int), ("stream", ctypes.c_void_p),
                ("num_processors", ctypes.c_int), ("threads_per_processor", ctypes.c_int),
                ("lds_bytes", ctypes.c_int), ("arena_bytes", ctypes.c_size_t),
                ("num_steps", ctypes.c_int), ("num_barriers", ctypes.c_int),
                ("barriers_elided", ctypes.c_int), ("kernel_families", ctypes.c_int),
                ("compiled", ctypes.c_int), ("launched", ctypes.c_int),
                ("destroyed", ctypes.c_int), ("loop_mode", ctypes.c_int),
                ("iterations_done", ctypes.c_int), ("barriers_local", ctypes.c_int),
                ("iteration_sync", ctypes.c_int), ("barriers_counted", ctypes.c_int),
                ("gemv_chains", ctypes.c_int), ("gemv_claimed", ctypes.c_int)]


def _i64(v):
    return (ctypes.c_int64 * len(v))(*[int(x) for x in v])


def plan_schedule(plan):
    """The barrier / task-sequence schedule a plan compiles to (no GPU needed)."""
    out = ctypes.c_char_p()
    check(lib().arkmi_plan_schedule(plan.encode(), ctypes.byref(out)))
    try:
        return json.loads(ctypes.string_at(out).decode())
    finally:
        lib().arkmi_free(out)


def plan_analysis(plan, dep_counters=-1):
    """What compile() decides for the plan (no GPU needed): barriers kept, elided, made local or
    replaced by dependency counters, and the counters' wait and signal tables."""
    out = ctypes.c_char_p()
    check(lib().arkmi_plan_analysis(plan.encode(), ctypes.c_int(dep_counters), ctypes.byref(out)))
    try:
        return json.loads(ctypes.string_at(out).decode())
    finally:
        lib().arkmi_free(out)


def schedule_tasks(plan, step, block, slot):
    """Task ids (block, slot) runs in schedule step `step` (no GPU needed)."""
    n = ctypes.c_int()
    check(lib().arkmi_schedule_tasks(plan.encode(), step, block, slot, None, 0, ctypes.byref(n)))
    buf = (ctypes.c_int64 * max(1, n.value))()
    check(lib().arkmi_schedule_tasks(plan.encode(), step, block, slot, buf, n.value, ctypes.byref(n)))
    return list(buf[:n.value])


class Executor:
    def __init__(self, plan, device_id=0, stream=None, name="Executor", loop_mode=True, trace=False):
        self._h = ctypes.c_void_p()
        check(lib().arkmi_exec_create(ctypes.c_int(device_id), ctypes.c_void_p(stream or 0),
                                      name.encode(), plan.encode(), ctypes.c_int(int(loop_mode)),
                                      ctypes.byref(self._h)))
        if trace:
            check(lib().arkmi_exec_enable_trace(self._h))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().arkmi_exec_destroy(self._h)
            self._h = None

    def close(self):
        self.__del__()

    def info(self):
        i = ExecInfo()
        check(lib().arkmi_exec_info(self._h, ctypes.byref(i)))
        return {f: getattr(i, f) for f, _ in ExecInfo._fields_}

    def plan(self):
        out = ctypes.c_char_p()
        check(lib().arkmi_exec_plan(self._h, ctypes.byref(out)))
        try:
            return ctypes.string_at(out).decode()
        finally:
            lib().arkmi_free(out)

    def compile(self):
        check(lib().arkmi_exec_compile(self._h))
        return self

    def launch(self):
        check(lib().arkmi_exec_launch(self._h))
        return self

    def run(self, iters=1):
        check(lib().arkmi_exec_run(self._h, ctypes.c_int(iters)))

    def run_separate(self, iters=1):
        """The plan's ops as separate kernel launches (asynchronous, on the
        executor's stream); the loop kernel must not be launched."""
        check(lib().arkmi_exec_run_separate(self._h, ctypes.c_int(iters)))

    def wait(self, max_spin_count=-1):
        check(lib().arkmi_exec_wait(self._h, ctypes.c_int64(max_spin_count)))

    def stop(self, max_spin_count=-1):
        ms = ctypes.c_float()
        check(lib().arkmi_exec_stop(self._h, ctypes.c_int64(max_spin_count), ctypes.byref(ms)))
        return ms.value

    def destroy(self):
        check(lib().arkmi_exec_release(self._h))

    def tensor_address(self, tensor):
        a = ctypes.c_size_t()
        check(lib().arkmi_exec_buffer_address(self._h, ctypes.c_uint64(tensor.buffer_id), ctypes.byref(a)))
        return a.value

    def _copy(self, tensor, ptr, nbytes, to_device, is_d2d=False, stream=None):
        check(lib().arkmi_exec_copy(self._h, ctypes.c_uint64(tensor.buffer_id),
                                    ctypes.c_int(len(tensor.shape)), _i64(tensor.shape),
                                    _i64(tensor.strides), _i64(tensor.offsets),
                                    ctypes.c_int(_ELEM[tensor.dtype]), ctypes.c_void_p(ptr),
                                    ctypes.c_size_t(nbytes), ctypes.c_void_p(stream or 0),
                                    ctypes.c_int(int(to_device)), ctypes.c_int(int(is_d2d))))

    def tensor_write(self, tensor, array):
        """array: numpy array of the tensor's storage type and shape (dense)."""
        a = np.ascontiguousarray(array)
        if a.dtype != _NP[tensor.dtype]:
            raise TypeError(f"expected {_NP[tensor.dtype]} for {tensor.dtype}, got {a.dtype}")
        self._copy(tensor, a.ctypes.data, a.nbytes, True)

    def tensor_read(self, tensor):
        a = np.empty(tensor.shape, dtype=_NP[tensor.dtype])
        self._copy(tensor, a.ctypes.data, a.nbytes, False)
        return a

    def tensor_write_device(self, tensor, torch_tensor):
        """Device-to-device write from a dense torch tensor on the same GPU."""
        t = torch_tensor.contiguous()
        self._copy(tensor, t.data_ptr(), t.numel() * t.element_size(), True, is_d2d=True)

    def tensor_read_device(self, tensor, torch_tensor):
        if not torch_tensor.is_contiguous():
            raise ValueError("destination must be contiguous")
        self._copy(tensor, torch_tensor.data_ptr(), torch_tensor.numel() * torch_tensor.element_size(),
                   False, is_d2d=True)

    def read_trace(self, task_group):
        """[(block, slot, order)] per task of the task group, by task index."""
        n = ctypes.c_int()
        check(lib().arkmi_exec_read_trace(self._h, task_group, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_int32 * (3 * max(1, n.value)))()
        check(lib().arkmi_exec_read_trace(self._h, task_group, buf, n.value, ctypes.byref(n)))
        return [(buf[3 * i], buf[3 * i + 1], buf[3 * i + 2]) for i in range(n.value)]

    def read_step_times(self):
        """Microseconds block 0 spent in each schedule step of the last iteration
        (tracing must be enabled)."""
        n = ctypes.c_int()
        check(lib().arkmi_exec_read_step_times(self._h, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_double * max(1, n.value))()
        check(lib().arkmi_exec_read_step_times(self._h, buf, n.value, ctypes.byref(n)))
        return list(buf[:n.value])

    def read_step_clocks(self):
        """(clocks_us[block][step], n_steps): when each workgroup entered each
        schedule step of the last iteration, in microseconds of GPU wall clock."""
        nb, ns, rate = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        check(lib().arkmi_exec_read_step_clocks(self._h, None, 0, ctypes.byref(nb), ctypes.byref(ns),
                                                ctypes.byref(rate)))
        n = nb.value * (ns.value + 1)
        buf = (ctypes.c_uint64 * n)()
        check(lib().arkmi_exec_read_step_clocks(self._h, buf, n, ctypes.byref(nb), ctypes.byref(ns),
                                                ctypes.byref(rate)))
        a = np.frombuffer(buf, dtype=np.uint64).reshape(nb.value, ns.value + 1).astype(np.float64)
        return a * 1000.0 / rate.value, ns.value
