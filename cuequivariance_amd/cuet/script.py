"""``torch.jit.script`` for the modules of this package.

The reference's test harness runs every operation in a ``script`` mode too (``cuequivariance_torch/_tests/utils.py:150-154``:
``torch.jit.script``, ``torch.jit.save``, ``torch.jit.load``, call).  The modules here are ordinary Python (plans, tables, calls
through ctypes), which TorchScript cannot compile; what it compiles instead is a small stand-in that every module hands out
through ``__prepare_scriptable__``: a module with the same ``forward`` signature (and the same ``weight`` parameter, if any)
whose body is one call of the operator ``cuequivariance_amd::module_call`` with the arguments as a list of tensors.  The operator
finds the Python module by a key and runs its eager ``forward``; its gradient runs that ``forward`` once more with autograd
switched on and differentiates it (first derivatives only).  The key names a module of THIS process: a scripted module that was
saved runs again after ``torch.jit.load`` as long as the module it was scripted from is alive in the process (as in the
reference's harness); for programs that must load elsewhere use ``torch.export`` or ``torch.jit.trace``, whose graphs name what
they launch by value.
"""

import collections
import itertools
from typing import Dict, List, Optional

import torch
import torch.nn as nn

__all__ = ["scriptable"]

# The modules that were scripted, by key.  A scripted program cannot hold a Python object, so this table keeps the modules
# alive (the last 256 of them: a program whose module has been dropped raises an error that says so).
_live: "collections.OrderedDict[str, nn.Module]" = collections.OrderedDict()
_serial = itertools.count()


def _key_of(mod: nn.Module) -> str:
    key = getattr(mod, "_script_key", None)
    if key is None:
        key = f"{type(mod).__name__}#{next(_serial)}"
        object.__setattr__(mod, "_script_key", key)
    _live[key] = mod
    _live.move_to_end(key)
    while len(_live) > 256:
        _live.popitem(last=False)
    return key


def _call(mod: nn.Module, tensors: List[torch.Tensor], present: List[int], ints: List[int]):
    """The eager ``forward`` of ``mod`` on the arguments a stand-in packed: ``present[k]`` 0 = argument k left out, 1 = given,
    2 = the stand-in's own ``weight`` parameter (takes the place of the module's)."""
    names, int_names = mod._script_args
    if names == "polynomial":  # ints: the number of inputs, then per dictionary its number of entries followed by their keys
        n, pos, at = ints[0], 1, ints[0]
        dicts = []
        for _ in range(3):
            count = ints[pos]
            dicts.append({int(k): tensors[at + j] for j, k in enumerate(ints[pos + 1:pos + 1 + count])})
            pos, at = pos + 1 + count, at + count
        return list(mod(list(tensors[:n]), *dicts))
    kwargs, own = {}, None
    for name, t, p in zip(names, tensors, present):
        if p == 1:
            kwargs[name] = t
        elif p == 2:
            own = t
    for name, v in zip(int_names, ints):
        if v >= 0:
            kwargs[name] = int(v)
    if own is not None:
        out = torch.func.functional_call(mod, {"weight": own}, args=(), kwargs=kwargs)
    else:
        out = mod(**kwargs)
    return list(out) if isinstance(out, (list, tuple)) else [out]


@torch.library.custom_op("cuequivariance_amd::module_call", mutates_args=())
def _module_call(key: str, tensors: List[torch.Tensor], present: List[int], ints: List[int]) -> List[torch.Tensor]:
    mod = _live.get(key)
    if mod is None:
        raise RuntimeError(f"cuequivariance_amd::module_call: the module {key} this scripted program was made from is not alive in "
                           "this process (scripted programs name their module by a key of the process; use torch.export or "
                           "torch.jit.trace for programs that are loaded elsewhere)")
    with torch.no_grad():
        outs = _call(mod, list(tensors), list(present), list(ints))
    taken = {t.data_ptr() for t in tensors}
    return [o.clone() if o.data_ptr() in taken else o for o in outs]  # (results of an operator may not alias its arguments)


@_module_call.register_fake
def _module_call_fake(key, tensors, present, ints):
    raise NotImplementedError("cuequivariance_amd::module_call is the call of a scripted stand-in; trace the module itself instead")


def _setup(ctx, inputs, output):
    key, tensors, present, ints = inputs
    ctx.key, ctx.present, ctx.ints = key, list(present), list(ints)
    ctx.save_for_backward(*tensors)


def _backward(ctx, grads):
    mod = _live.get(ctx.key)
    if mod is None:
        raise RuntimeError(f"cuequivariance_amd::module_call: the module {ctx.key} is not alive in this process")
    with torch.enable_grad():
        ins = [t.detach().requires_grad_(t.is_floating_point()) for t in ctx.saved_tensors]
        outs = _call(mod, ins, ctx.present, ctx.ints)
        wanted = [k for k, t in enumerate(ins) if t.requires_grad]
        pairs = [(o, g) for o, g in zip(outs, grads) if g is not None and o.requires_grad]
        got = torch.autograd.grad([o for o, _ in pairs], [ins[k] for k in wanted], [g for _, g in pairs], allow_unused=True) if pairs else ()
    out: List[Optional[torch.Tensor]] = [None] * len(ins)
    for k, g in zip(wanted, got):
        out[k] = g
    return None, out, None, None


torch.library.register_autograd("cuequivariance_amd::module_call", _backward, setup_context=_setup)


def _empty(like: torch.Tensor) -> torch.Tensor:
    return torch.empty(0, device=like.device)


class _WithWeight(nn.Module):
    """Stand-in of a module ``forward(x1, x2, weight=None, indices_1=None, indices_2=None, indices_out=None, size_out=None)``
    (the channel-wise and the fully connected product; the latter takes no ``indices_2``)."""

    weight: Optional[torch.Tensor]

    def __init__(self, key: str, weight: Optional[nn.Parameter]):
        super().__init__()
        self.key = key
        self.register_parameter("weight", weight)

    def forward(self, x1: torch.Tensor, x2: torch.Tensor, weight: Optional[torch.Tensor] = None,
                indices_1: Optional[torch.Tensor] = None, indices_2: Optional[torch.Tensor] = None,
                indices_out: Optional[torch.Tensor] = None, size_out: Optional[int] = None) -> torch.Tensor:
        tensors: List[torch.Tensor] = [x1, x2]
        present: List[int] = [1, 1]
        own = self.weight
        if own is not None:
            if weight is not None:
                raise ValueError("Internal weights are used, weight should be None")
            tensors.append(own)
            present.append(2)
        elif weight is not None:
            tensors.append(weight)
            present.append(1)
        else:
            raise ValueError("Internal weights are not used, weight should not be None")
        for t in [indices_1, indices_2, indices_out]:
            if t is not None:
                tensors.append(t)
                present.append(1)
            else:
                tensors.append(_empty(x1))
                present.append(0)
        ints: List[int] = [size_out if size_out is not None else -1]
        return torch.ops.cuequivariance_amd.module_call(self.key, tensors, present, ints)[0]


class _LinearLike(nn.Module):
    """Stand-in of ``Linear.forward(x, weight=None, weight_indices=None)``."""

    weight: Optional[torch.Tensor]

    def __init__(self, key: str, weight: Optional[nn.Parameter]):
        super().__init__()
        self.key = key
        self.register_parameter("weight", weight)

    def forward(self, x: torch.Tensor, weight: Optional[torch.Tensor] = None, weight_indices: Optional[torch.Tensor] = None) -> torch.Tensor:
        tensors: List[torch.Tensor] = [x]
        present: List[int] = [1]
        own = self.weight
        if own is not None:
            if weight is not None:
                raise ValueError("Internal weights are used, weight should be None")
            tensors.append(own)
            present.append(2)
        elif weight is not None:
            tensors.append(weight)
            present.append(1)
        else:
            raise ValueError("Weights should not be None")
        if weight_indices is not None:
            tensors.append(weight_indices)
            present.append(1)
        else:
            tensors.append(_empty(x))
            present.append(0)
        ints: List[int] = [-1]  # (never empty: the gradient of the operator wants the same structure back)
        return torch.ops.cuequivariance_amd.module_call(self.key, tensors, present, ints)[0]


class _Contraction(nn.Module):
    """Stand-in of ``SymmetricContraction.forward(x, indices)`` (the weights are always the module's own)."""

    def __init__(self, key: str, weight: nn.Parameter):
        super().__init__()
        self.key = key
        self.weight = weight

    def forward(self, x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        tensors: List[torch.Tensor] = [x, indices, self.weight]
        present: List[int] = [1, 1, 2]
        ints: List[int] = [-1]  # (never empty: the gradient of the operator wants the same structure back)
        return torch.ops.cuequivariance_amd.module_call(self.key, tensors, present, ints)[0]


class _OneTensor(nn.Module):
    """Stand-in of a module ``forward(x)`` without parameters (spherical harmonics, inversion, layout change)."""

    def __init__(self, key: str):
        super().__init__()
        self.key = key

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        tensors: List[torch.Tensor] = [x]
        present: List[int] = [1]
        ints: List[int] = [-1]  # (never empty: the gradient of the operator wants the same structure back)
        return torch.ops.cuequivariance_amd.module_call(self.key, tensors, present, ints)[0]


class _FourTensors(nn.Module):
    """Stand-in of ``Rotation.forward(gamma, beta, alpha, x)``."""

    def __init__(self, key: str):
        super().__init__()
        self.key = key

    def forward(self, gamma: torch.Tensor, beta: torch.Tensor, alpha: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
        tensors: List[torch.Tensor] = [gamma, beta, alpha, x]
        present: List[int] = [1, 1, 1, 1]
        ints: List[int] = [-1]  # (never empty: the gradient of the operator wants the same structure back)
        return torch.ops.cuequivariance_amd.module_call(self.key, tensors, present, ints)[0]


class _Polynomial(nn.Module):
    """Stand-in of ``SegmentedPolynomial.forward(inputs, input_indices=None, output_shapes=None, output_indices=None)``."""

    def __init__(self, key: str):
        super().__init__()
        self.key = key

    def forward(self, inputs: List[torch.Tensor], input_indices: Optional[Dict[int, torch.Tensor]] = None,
                output_shapes: Optional[Dict[int, torch.Tensor]] = None,
                output_indices: Optional[Dict[int, torch.Tensor]] = None) -> List[torch.Tensor]:
        tensors: List[torch.Tensor] = []
        for t in inputs:
            tensors.append(t)
        ints: List[int] = [len(inputs)]
        for d in [input_indices, output_shapes, output_indices]:
            if d is not None:
                ints.append(len(d))
                for k in d.keys():
                    ints.append(k)
                for v in d.values():
                    tensors.append(v)
            else:
                ints.append(0)
        present: List[int] = [1]
        return torch.ops.cuequivariance_amd.module_call(self.key, tensors, present, ints)


_STAND_INS = {
    "with_weight": (_WithWeight, (["x1", "x2", "weight", "indices_1", "indices_2", "indices_out"], ["size_out"])),
    "fully_connected": (_WithWeight, (["x1", "x2", "weight", "indices_1", "_unused", "indices_out"], ["size_out"])),
    "linear": (_LinearLike, (["x", "weight", "weight_indices"], [])),
    "contraction": (_Contraction, (["x", "indices", "weight"], [])),
    "vectors": (_OneTensor, (["vectors"], [])),
    "x": (_OneTensor, (["x"], [])),
    "rotation": (_FourTensors, (["gamma", "beta", "alpha", "x"], [])),
    "polynomial": (_Polynomial, ("polynomial", [])),
}


def scriptable(kind: str):
    """Class decorator: gives a module ``__prepare_scriptable__``, which ``torch.jit.script`` calls and then compiles what it
    returns - the stand-in of ``kind`` - in place of the module."""
    stand_in, args = _STAND_INS[kind]

    def decorate(cls):
        cls._script_args = args

        def prepare(self):
            key = _key_of(self)
            if stand_in in (_WithWeight, _LinearLike):
                return stand_in(key, getattr(self, "weight", None))
            if stand_in is _Contraction:
                return stand_in(key, self.weight)
            return stand_in(key)

        cls.__prepare_scriptable__ = prepare
        return cls

    return decorate
