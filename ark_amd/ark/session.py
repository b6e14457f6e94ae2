"""Planner, runtime, modules and state-dict files of the `ark` surface.

Behaviour to match: python/ark/planner.py:110-230 (plan objects and the planner),
runtime.py:27-168 (the three-state life cycle), module.py:13-89 (module trees and state
dicts), init.py:10-17 and serialize.py:8-28 (state-dict files).  The runtime is written as a
transition table, the module as one ordered registry of named members, and state-dict files
are read by an unpickler that constructs numpy arrays and plain containers only.
"""
import copy as _copy
import io
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


_log = logging.getLogger("ark")


class _Live:
    """What outlives a Runtime object: the process-wide runtime and the one executor that may
    hold device memory at a time."""
    runtime = None
    executor = None

    @classmethod
    def retire_executor(cls):
        ex, cls.executor = cls.executor, None
        if ex is not None and not ex.destroyed():
            ex.destroy()


class Runtime:
    """The life cycle of the global model on one device.

    Three states; each public call looks its (state, call) pair up in `_TABLE`, which names the
    step to take and the state to end in.  A pair mapped to `_refuse` raises, one mapped to
    `_skip` logs and returns None.

        state               launch        run          wait        barrier     stop
        Init                build+start   refuse       skip        refuse      skip
        LaunchedNotRunning  skip          start iters  skip        barrier     halt
        Running             skip          refuse       complete    refuse      halt

    `stop()` halts the kernel but leaves the state at LaunchedNotRunning with the executor (and
    its device memory) alive, so tensors stay readable; `reset()` returns to Init and frees it.
    """

    class State(Enum):
        Init = 0
        LaunchedNotRunning = 1
        Running = 2

    # -- the steps ---------------------------------------------------------------------------
    def _build_and_start(self, plan=None, device_id=0, stream=0, loop_mode=True):
        if plan is None:
            plan = Planner(device_id).plan()
        if _Live.executor is not None and not _Live.executor.destroyed():
            _log.warning("Destroying an old executor")
        _Live.retire_executor()
        self.executor = _Live.executor = Executor(device_id, stream, "ArkRuntime", str(plan), loop_mode)
        self.executor.compile()
        self.executor.launch()

    def _start_iterations(self, iter=1, non_blocking=False):
        self.executor.run(iter)
        return non_blocking

    def _complete(self):
        self.executor.wait()

    def _barrier(self):
        self.executor.barrier()

    def _halt(self):
        return self.executor.stop()

    def _refuse(self, *args, **kwargs):
        _log.error("ARK runtime is not launched")
        raise RuntimeError("ARK runtime is not launched")

    _SKIP_NOTES = {
        "launch": "Runtime is already launched, skip launching",
        "wait": "ARK runtime is not running, skip waiting",
        "stop": "ARK runtime is never launched, skip stopping",
    }

    _I, _L, _R = State.Init, State.LaunchedNotRunning, State.Running
    _TABLE = {
        (_I, "launch"): (_build_and_start, _L), (_L, "launch"): (None, _L), (_R, "launch"): (None, _R),
        (_I, "run"): (_refuse, _I), (_L, "run"): (_start_iterations, _R), (_R, "run"): (_refuse, _R),
        (_I, "wait"): (None, _I), (_L, "wait"): (None, _L), (_R, "wait"): (_complete, _L),
        (_I, "barrier"): (_refuse, _I), (_L, "barrier"): (_barrier, _L), (_R, "barrier"): (_refuse, _R),
        (_I, "stop"): (None, _I), (_L, "stop"): (_halt, _L), (_R, "stop"): (_halt, _L),
    }
    del _I, _L, _R

    def _step(self, call, *args, **kwargs):
        action, after = Runtime._TABLE[(self.state, call)]
        if action is None:
            _log.warning(Runtime._SKIP_NOTES[call])
            return None
        out = action(self, *args, **kwargs)
        self.state = after
        return out

    # -- the public calls --------------------------------------------------------------------
    @staticmethod
    def get_runtime():
        return _Live.runtime if _Live.runtime is not None else Runtime()

    def __init__(self):
        self.executor = None
        self.state = Runtime.State.Init
        _Live.runtime = self   # the newest runtime is the one tensors talk to

    def launched(self):
        return self.state is not Runtime.State.Init

    def running(self):
        return self.state is Runtime.State.Running

    def launch(self, plan=None, device_id=0, stream=0, loop_mode=True):
        """Plans the global model (unless a plan is given), allocates and starts the kernel."""
        self._step("launch", plan, device_id, stream, loop_mode)

    def run(self, iter=1, non_blocking=False):
        if not self._step("run", iter, non_blocking):
            self.wait()

    def wait(self):
        self._step("wait")

    def barrier(self):
        self._step("barrier")

    def stop(self):
        """Halts the kernel; elapsed milliseconds since the launch, or None if never launched."""
        return self._step("stop")

    def reset(self):
        """Back to Init: the kernel halted, the executor and its device memory released."""
        if self.launched():
            self.stop()
        ex, self.executor = self.executor, None
        if ex is not None:
            if ex is _Live.executor:
                _Live.retire_executor()
            elif not ex.destroyed():
                ex.destroy()
        self.state = Runtime.State.Init

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.reset()

    def __del__(self):
        try:
            self.reset()
        except Exception:  # interpreter shutdown: the native library may be gone already
            pass


class Module:
    """A node of a model tree.  Assigning a Module or a Parameter to an attribute enters it in
    the node's registry under the attribute's name (assigning again replaces the entry);
    `sub_modules` and `parameters` are the two views of that registry, in order of entry."""

    def _members(self):
        return self.__dict__.setdefault("_registry", {})

    def __setattr__(self, name, value):
        if isinstance(value, (Module, Parameter)):
            self._members()[name] = value
        object.__setattr__(self, name, value)

    @property
    def sub_modules(self):
        return {k: v for k, v in self._members().items() if isinstance(v, Module)}

    @property
    def parameters(self):
        return {k: v for k, v in self._members().items() if isinstance(v, Parameter)}

    def register_module(self, name, module):
        if not isinstance(module, Module):
            raise TypeError("module must be a Module")
        self._members()[name] = module

    def register_parameter(self, name, param):
        if not isinstance(param, Parameter):
            raise TypeError("param must be a Parameter")
        self._members()[name] = param

    def _walk(self, prefix):
        """(dotted name, Parameter) of every parameter below this node: sub-modules first, in
        order of entry, then the node's own parameters."""
        for name, sub in self.sub_modules.items():
            yield from sub._walk(f"{prefix}{name}.")
        for name, p in self.parameters.items():
            yield prefix + name, p

    def params_dict(self, prefix=""):
        return dict(self._walk(prefix))

    def state_dict(self, prefix=""):
        """Every parameter read back as a numpy array (shapes only before the launch)."""
        return {name: p.to_numpy() for name, p in self._walk(prefix)}

    def load_state_dict(self, state_dict, prefix=""):
        """Writes the arrays to the parameters' device memory (after `Runtime.launch()`); a
        parameter without an array is a KeyError, arrays without a parameter are reported."""
        used = set()
        for name, p in self._walk(prefix):
            p.from_numpy(state_dict[name])
            used.add(name)
        extra = len(set(state_dict) - used)
        if extra:
            _log.warning("%d unused parameter(s) in state_dict", extra)

    def forward(self, *args, **kwargs):
        """What the module appends to the global model; a subclass defines it."""
        return None

    def backward(self, *args, **kwargs):
        """Placeholder, as in the reference: nothing here differentiates."""
        return None

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)


def init():
    """Starts over: the `ARK_*` environment is read again, the global model is dropped, a live
    executor is destroyed and the runtime returns to Init."""
    from .._lib import lib, check
    check(lib().arkmi_init())
    Model.reset()
    _Live.retire_executor()
    rt = _Live.runtime
    if rt is not None:
        rt.executor, rt.state = None, Runtime.State.Init


# ---- state-dict files -------------------------------------------------------------------------
# The file format is the reference's: one pickled dict of numpy arrays.  Unpickling a file runs
# whatever callables it names, so the reader resolves only the few that numpy arrays and plain
# containers are made of and refuses every other global.
_ARRAY_GLOBALS = {
    ("numpy", "ndarray"), ("numpy", "dtype"),
    ("numpy.core.multiarray", "_reconstruct"), ("numpy._core.multiarray", "_reconstruct"),
    ("numpy.core.multiarray", "scalar"), ("numpy._core.multiarray", "scalar"),
    ("numpy.core.numeric", "_frombuffer"), ("numpy._core.numeric", "_frombuffer"),
    ("collections", "OrderedDict"),
}


class _ArrayUnpickler(pickle.Unpickler):
    def find_class(self, module, name):
        if (module, name) not in _ARRAY_GLOBALS:
            raise pickle.UnpicklingError(f"state-dict files hold numpy arrays only; refusing {module}.{name}")
        return super().find_class(module, name)


def save(state_dict, state_dict_file_path):
    """Writes `{name: numpy array}` to a file `load()` (and the reference's) can read."""
    if not isinstance(state_dict, dict):
        _log.warning("Invalid state_dict saved to %s", state_dict_file_path)
    payload = pickle.dumps(state_dict, protocol=4)
    _ArrayUnpickler(io.BytesIO(payload)).load()   # nothing is written that load() would refuse
    with open(state_dict_file_path, "wb") as f:
        f.write(payload)


def load(state_dict_file_path):
    """Reads a state-dict file without running code from it: a file that names anything but
    numpy's array constructors raises `pickle.UnpicklingError`."""
    with open(state_dict_file_path, "rb") as f:
        state_dict = _ArrayUnpickler(f).load()
    if not isinstance(state_dict, dict):
        _log.warning("Invalid state_dict file")
    return state_dict
