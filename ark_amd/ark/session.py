"""Planner, runtime, modules and state-dict files of the `ark` surface.

Follows python/ark/planner.py:110-230, runtime.py:15-168, module.py:13-89, init.py:10-17 and
serialize.py:8-28: same names, same state machine, same messages for misuse.
"""
import copy as _copy
import json
import logging
import pickle
from enum import Enum

from .. import executor as _x
from .. import model as _m
from .frontend import Model, Parameter

__all__ = ["Plan", "PlannerContext", "Planner", "Executor", "Runtime", "Module", "init",
           "save", "load"]


class Plan:
    """A parsed plan file; str() is the text Executor takes."""

    def __init__(self, plan):
        if plan is None:
            plan = {"Rank": 0, "WorldSize": 1, "Architecture": "ANY", "NumProcessors": 1,
                    "NumWarpsPerProcessor": 1, "TaskInfos": [], "ProcessorGroups": []}
        else:
            plan = _copy.deepcopy(plan)
        self.plan = plan

    def __str__(self):
        return json.dumps(self.plan)

    rank = property(lambda self: self.plan["Rank"])
    world_size = property(lambda self: self.plan["WorldSize"])
    architecture = property(lambda self: self.plan["Architecture"])
    num_processors = property(lambda self: self.plan["NumProcessors"])
    num_warps_per_processor = property(lambda self: self.plan["NumWarpsPerProcessor"])
    task_infos = property(lambda self: self.plan["TaskInfos"])
    processor_groups = property(lambda self: self.plan["ProcessorGroups"])

    @staticmethod
    def from_str(plan_str):
        return Plan(json.loads(plan_str))

    @staticmethod
    def from_file(file_path):
        with open(file_path, "r") as f:
            return Plan(json.load(f))


class PlannerContext(_m.PlannerContext):
    """`with ark.PlannerContext(processor_range=[0, 128], sync=False, config={...}):` on the
    global model.  `sync` defaults to True, which leaves the enclosing setting alone."""

    def __init__(self, **kwargs):
        if kwargs.get("sync", True) is not False:
            kwargs.pop("sync", None)
        super().__init__(Model.get_model(), **kwargs)


class Planner:
    """Planner of the global model for one device.  `arch` / `num_processors` plan for a named
    architecture without touching a GPU (an addition; the reference always asks the device)."""

    def __init__(self, device_id=0, arch=None, num_processors=0):
        self._model = Model.get_model().compress()
        self._device_id, self._arch, self._num_processors = device_id, arch, num_processors
        self._rules = []

    def install_config_rule(self, rule):
        """rule(op_json: str, arch_name: str) -> config JSON str ('' to pass)."""
        self._rules.append(rule)

    def plan(self):
        return Plan.from_str(self._model.plan(self._device_id, self._arch, self._num_processors,
                                              self._rules, pretty=False))


class Executor(_x.Executor):
    """ark.Executor(device_id, stream, name, plan, loop_mode): the reference's argument order."""

    def __init__(self, device_id, stream, name, plan, loop_mode=True):
        super().__init__(str(plan), device_id, stream, name, loop_mode)

    def destroyed(self):
        return bool(self.info()["destroyed"])

    def barrier(self):
        """Barrier over ranks; one rank here, so nothing to wait for."""

    def tensor_read(self, tensor, ndarray=None, stream=0):
        t = tensor._tensor
        if ndarray is None:
            return super().tensor_read(t)
        self._copy(t, ndarray.ctypes.data, ndarray.nbytes, False, stream=stream)
        return ndarray

    def tensor_write(self, tensor, ndarray, stream=0):
        self._copy(tensor._tensor, ndarray.ctypes.data, ndarray.nbytes, True, stream=stream)


class _RuntimeState:
    runtime = None
    executor = None


class Runtime:
    """Init -> launch() -> LaunchedNotRunning -> run() -> Running -> wait() -> LaunchedNotRunning;
    stop() keeps the executor for another launch(), reset() destroys it."""

    class State(Enum):
        Init = 0
        LaunchedNotRunning = 1
        Running = 2

    @staticmethod
    def get_runtime():
        if _RuntimeState.runtime is None:
            _RuntimeState.runtime = Runtime()
        return _RuntimeState.runtime

    def __init__(self):
        self.executor = None
        self.state = Runtime.State.Init
        _RuntimeState.runtime = self

    def __del__(self):
        try:
            self.reset()
        except Exception:  # interpreter shutdown: the library may already be gone
            pass

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        self.reset()

    def launched(self):
        return self.state in (Runtime.State.LaunchedNotRunning, Runtime.State.Running)

    def running(self):
        return self.state == Runtime.State.Running

    def launch(self, plan=None, device_id=0, stream=0, loop_mode=True):
        if self.launched():
            logging.warning("Runtime is already launched, skip launching")
            return
        plan = Planner(device_id).plan() if plan is None else plan
        if self.state == Runtime.State.Init:
            old = _RuntimeState.executor
            if old is not None and not old.destroyed():
                logging.warning("Destroying an old executor")
                old.destroy()
            _RuntimeState.executor = Executor(device_id, stream, "ArkRuntime", str(plan), loop_mode)
            self.executor = _RuntimeState.executor
            self.executor.compile()
        self.executor.launch()
        self.state = Runtime.State.LaunchedNotRunning

    def run(self, iter=1, non_blocking=False):
        if self.state != Runtime.State.LaunchedNotRunning:
            logging.error("ARK runtime is not launched")
            raise RuntimeError("ARK runtime is not launched")
        self.state = Runtime.State.Running
        self.executor.run(iter)
        if not non_blocking:
            self.wait()

    def barrier(self):
        if self.state != Runtime.State.LaunchedNotRunning:
            logging.error("ARK runtime is not launched")
            raise RuntimeError("ARK runtime is not launched")
        self.executor.barrier()

    def wait(self):
        if self.state != Runtime.State.Running:
            logging.warning("ARK runtime is not running, skip waiting")
            return
        self.executor.wait()
        self.state = Runtime.State.LaunchedNotRunning

    def stop(self):
        """Stops the kernel; returns the elapsed milliseconds.  launch() starts it again."""
        if not self.launched():
            logging.warning("ARK runtime is never launched, skip stopping")
            return None
        elapsed = self.executor.stop()
        self.state = Runtime.State.LaunchedNotRunning
        return elapsed

    def reset(self):
        if self.launched():
            self.stop()
        if self.executor is not None:
            if not self.executor.destroyed():
                self.executor.destroy()
            self.executor = None
        self.state = Runtime.State.Init


class Module:
    """Tree of modules and parameters; attribute assignment registers them."""

    def __init__(self):
        self.sub_modules = {}
        self.parameters = {}

    def __setattr__(self, name, value):
        if isinstance(value, Module):
            self.register_module(name, value)
        elif isinstance(value, Parameter):
            self.register_parameter(name, value)
        super().__setattr__(name, value)

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)

    def register_module(self, name, module):
        if not isinstance(module, Module):
            raise TypeError("module must be a Module")
        self.sub_modules[name] = module

    def register_parameter(self, name, param):
        if not isinstance(param, Parameter):
            raise TypeError("param must be a Parameter")
        self.parameters[name] = param

    def params_dict(self, prefix=""):
        out = {}
        for name, sub in self.sub_modules.items():
            if sub is not None:
                out.update(sub.params_dict(prefix=prefix + name + "."))
        for name, p in self.parameters.items():
            out[prefix + name] = p
        return out

    def load_state_dict(self, state_dict, prefix=""):
        """Copies arrays to the parameters' device memory; the runtime must be launched."""
        unused = set(state_dict.keys())
        for name, p in self.params_dict(prefix).items():
            p.from_numpy(state_dict[name])
            unused.remove(name)
        if unused:
            logging.warning(f"{len(unused)} unused parameter(s) in state_dict")

    def state_dict(self, prefix=""):
        return {k: v.to_numpy() for k, v in self.params_dict(prefix).items()}

    def forward(self, *args, **kwargs):
        ...

    def backward(self, *args, **kwargs):
        ...


def init():
    """Drops the global model, destroys a live executor and reads the ARK_* environment again."""
    from .._lib import lib, check
    check(lib().arkmi_init())
    Model.reset()
    ex = _RuntimeState.executor
    if ex is not None:
        if not ex.destroyed():
            ex.destroy()
    _RuntimeState.executor = None
    if _RuntimeState.runtime is not None:
        _RuntimeState.runtime.executor = None
        _RuntimeState.runtime.state = Runtime.State.Init


def save(state_dict, state_dict_file_path):
    """Writes a state dict in the reference's file format (a pickled dict of numpy arrays)."""
    if not isinstance(state_dict, dict):
        logging.warning("Invalid state_dict saved to %s", state_dict_file_path)
    with open(state_dict_file_path, "wb") as f:
        pickle.dump(state_dict, f)


def load(state_dict_file_path):
    """Reads a file save() wrote.  Unpickling runs code from the file: load your own files only."""
    with open(state_dict_file_path, "rb") as f:
        state_dict = pickle.load(f)
    if not isinstance(state_dict, dict):
        logging.warning("Invalid state_dict file")
    return state_dict
