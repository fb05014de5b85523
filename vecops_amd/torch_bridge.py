"""Torch registration facade for the HIP operators - the counterpart of vecops'
``vecops.ops.torch.register`` (python/vecops/ops/torch.py:35-86) for operators whose
recipes resolve to prebuilt gfx950 artifacts instead of JIT-compiled sources.

``register("library::name", operator)`` defines one mutable ``torch.ops`` operator
(outputs are caller-allocated ``Tensor(a!)`` arguments, python/vecops/_schema_bridge.py:954-1002)
and returns a public callable that, unlike the raw ``torch.ops`` symbol, accepts named
specialization values and gives back the caller's own output tensors.  Tensors on a ROCm
device ("cuda" in torch) enter the operator as ``VECOPS_DEVICE_PRIVATE`` views and run on
``torch.cuda.current_stream()``; host tensors enter as ``VECOPS_DEVICE_CPU`` views and are
staged by the artifact.  Device workspace comes from torch's allocator; calls whose tensors all live on the device are
stream-ordered (they return once enqueued on the current stream), calls with host tensors wait for their results.
Every call enters the Operator through the native bridge entry ``vecops_operator_bridge_invoke_v1``
(runtime/OperatorBridgeAbi.h:69-71) of libvecops_hip_host.so.  Like the
reference's process-local bridge (docs/Runtime.md:196-206) the wrapper keeps up to eight
call signatures per thread - tensor kind, dtype, device, shape, strides, optional
presence and specialization values, never addresses or scalar payloads - and reuses the
workspace size found for a signature instead of resolving the call a second time.
"""
from __future__ import annotations

import threading
from types import SimpleNamespace

from . import host_api as H

# Positional parameters of the operators this package ships (name, kind); kind is
# "in", "in?" (optional tensor), "out", "out?" (optional output), "int" or "float".  Specialization values are
# keyword-only integers on the torch operator (-1 = not given); "dtype" ones take a
# torch dtype or a VecopsDType number on the public callable.
SIGNATURES = {
    "vecops::matmul": ([("a", "in"), ("b", "in"), ("c_in", "in?"), ("c", "out")], {"ComputeType": "dtype"}),
    "vecops::matmul_i8_dequant": ([("a", "in"), ("b", "in"), ("row_scales", "in"), ("column_scales", "in"),
                                   ("correction", "in?"), ("c", "out")], {}),
    "vecops::matmul_w8a16_group": ([("x", "in"), ("w", "in"), ("scales", "in"), ("y", "out")], {"G": "int"}),
    "vecops::matmul_fused": ([("a", "in"), ("b", "in"), ("c_in", "in?"), ("row_scales", "in?"),
                              ("column_scales", "in?"), ("activation", "int"), ("scale", "float"), ("shift", "float"),
                              ("clamp_lo", "float"), ("clamp_hi", "float"), ("c", "out")], {}),
    "vecops::matmul_pack_b": ([("b", "in"), ("a_zero_point", "int"), ("packed", "out"), ("compensation", "out?")],
                              {"ComputeType": "dtype"}),
    "vecops::matmul_packed_b": ([("a", "in"), ("packed_b", "in"), ("c_in", "in?"), ("c", "out")],
                                {"PackedType": "dtype", "ComputeType": "dtype"}),
    "vecops::matmul_pack_a": ([("a", "in"), ("packed", "out")], {"ComputeType": "dtype"}),
    "vecops::matmul_packed_a": ([("packed_a", "in"), ("b", "in"), ("c_in", "in?"), ("c", "out")],
                                {"PackedType": "dtype", "ComputeType": "dtype"}),
    "vecops::matmul_runtime_quant": ([("a", "in"), ("b", "in"), ("multipliers", "in"), ("zero_point", "int"),
                                      ("row_scales", "in"), ("column_scales", "in"), ("correction", "in?"),
                                      ("c", "out")], {}),
}

_PREPARED_CALLS = 8          # signatures kept per thread (docs/Runtime.md:196-206)
_libraries: dict[str, SimpleNamespace] = {}
_registrations: dict[tuple[str, str], "_Registration"] = {}
_lock = threading.Lock()
_host_library = None


def _name(qualified_name: str) -> tuple[str, str]:
    """Validate and split a ``library::operator`` registration name."""
    if qualified_name.count("::") != 1:
        raise ValueError("Torch operator name must use the 'library::name' form")
    library, name = qualified_name.split("::")
    if not library or not name:
        raise ValueError("Torch operator library and name must not be empty")
    if not library.isidentifier() or not name.isidentifier():
        raise ValueError("Torch operator library and name must be identifiers")
    return library, name


def _dtype_code(value) -> int:
    import torch
    if isinstance(value, int):
        return value
    return {torch.int8: H.I8, torch.uint8: H.U8, torch.int32: H.I32, torch.float16: H.F16, torch.bfloat16: H.BF16,
            torch.float32: H.F32}[value]


class _Registration:
    def __init__(self, library, name, operator, params, specs, return_outputs):
        self.library, self.name, self.operator = library, name, operator
        self.params, self.specs, self.return_outputs = params, specs, return_outputs
        self.outputs = tuple(i for i, (_, kind) in enumerate(params) if kind in ("out", "out?"))
        self.local = threading.local()
        self.torch_op = None
        self.wrapper = None

    # -- the torch.ops side ---------------------------------------------------------------
    def schema(self) -> str:
        parts = []
        alias = iter("abcdefgh")
        for pname, kind in self.params:
            if kind in ("out", "out?"):
                parts.append(f"Tensor({next(alias)}!){'?' if kind == 'out?' else ''} {pname}")
            else:
                parts.append({"in": "Tensor", "in?": "Tensor?", "int": "int", "float": "float"}[kind] + " " + pname)
        if self.specs:
            parts.append("*")
            parts += [f"int {sname}=-1" for sname in self.specs]
        returns = "(" + ", ".join("Tensor?" if self.params[i][1] == "out?" else "Tensor" for i in self.outputs) + ")" \
            if self.return_outputs else "()"
        return f"{self.name}({', '.join(parts)}) -> {returns}"

    def signature(self, values, spec_values):
        sig = []
        for v, (_, kind) in zip(values, self.params):
            if kind in ("int", "float"):
                sig.append(kind)                                   # the payload stays out of the signature
            elif v is None:
                sig.append(None)
            else:
                sig.append((v.dtype, v.device, tuple(v.shape), tuple(v.stride())))
        return tuple(sig), tuple(sorted(spec_values.items()))

    def invoke(self, *args, **spec_ints):
        import torch
        values = list(args)
        for i, (pname, kind) in enumerate(self.params):
            if kind == "float":
                values[i] = float(values[i])
            elif kind == "int":
                values[i] = int(values[i])
        specs = {}
        for sname, skind in self.specs.items():
            raw = spec_ints.get(sname, -1)
            if raw != -1:
                specs[sname] = ("dtype", raw) if skind == "dtype" else raw
        frame = H.Frame(values, outputs=self.outputs)
        tensors = [v for v in values if isinstance(v, torch.Tensor)]
        on_device = any(t.is_cuda for t in tensors)
        stream = None
        workspace, workspace_size = None, 0
        if on_device:
            device = next(t.device for t in tensors if t.is_cuda)
            stream = torch.cuda.current_stream(device).cuda_stream
            cache = getattr(self.local, "prepared", None)
            if cache is None:
                cache = self.local.prepared = {}
            sig = self.signature(values, {k: v for k, v in spec_ints.items() if v != -1})
            need = cache.get(sig)
            if need is None:
                need = self.operator.workspace(frame, specs)      # resolves and validates once per signature
                if len(cache) >= _PREPARED_CALLS:
                    cache.pop(next(iter(cache)))
                cache[sig] = need
            if need:
                scratch = torch.empty(need, dtype=torch.uint8, device=device)
                workspace, workspace_size = scratch.data_ptr(), need
        # One foreign call through the process-local bridge entry (vecops_operator_bridge_invoke_v1); ctypes drops the
        # interpreter lock for its duration.  Device tensors: the work is ordered on torch's current stream, where
        # the scratch was allocated, so the call returns once the kernels are enqueued.
        self.operator.bridge_invoke(frame, specs, workspace=workspace, workspace_size=workspace_size, stream=stream,
                                    stream_ordered=on_device and not any(not t.is_cuda for t in tensors))
        if self.return_outputs:
            outs = tuple(values[i] for i in self.outputs)
            return outs
        return None

    def define(self):
        import torch
        lib = torch.library.Library(self.library, "FRAGMENT")
        lib.define(self.schema())
        outputs = self.outputs
        return_outputs = self.return_outputs

        def meta(*args, **kwargs):
            return tuple(args[i] for i in outputs) if return_outputs else None

        lib.impl(self.name, self.invoke, "CUDA")
        lib.impl(self.name, self.invoke, "CPU")
        lib.impl(self.name, meta, "Meta")
        self._library = lib                                         # keeps the definitions alive
        self.torch_op = getattr(getattr(torch.ops, self.library), self.name)

    # -- the public callable --------------------------------------------------------------
    def public(self, *args, **kwargs):
        if len(args) != len(self.params):
            raise TypeError(f"{self.library}::{self.name} expects {len(self.params)} positional arguments, "
                            f"got {len(args)}")
        unknown = set(kwargs) - set(self.specs)
        if unknown:
            raise TypeError(f"{self.library}::{self.name} got unknown specialization value(s): {sorted(unknown)}")
        spec_ints = {}
        for sname, skind in self.specs.items():
            if sname in kwargs:
                spec_ints[sname] = _dtype_code(kwargs[sname]) if skind == "dtype" else int(kwargs[sname])
        self.torch_op(*args, **spec_ints)
        outs = tuple(args[i] for i in self.outputs if args[i] is not None)
        return outs[0] if len(outs) == 1 else outs


def host_library() -> H.HostLibrary:
    global _host_library
    if _host_library is None:
        _host_library = H.HostLibrary()
    return _host_library


def register(qualified_name: str, dispatch=None, *, operator_name: str | None = None, return_outputs: bool = False,
             artifact_directory: str = H.ARTIFACT_DIR):
    """Register one Torch operator backed by a HIP ``Operator`` and return its public callable.

    ``qualified_name`` must use ``"library::operator"`` form.  ``dispatch`` is an existing
    ``host_api.HostOperator``; when omitted, the operator ``operator_name`` (default
    ``vecops::<operator>``) is created over ``artifact_directory``.  Registration is idempotent per
    ``(library, name)`` in this process.  Pass ``return_outputs=True`` when a consumer needs the mutable
    operator to return its output tensors rather than ``()``; the public callable returns the caller's
    own output objects in either mode.
    """
    library, name = _name(qualified_name)
    vecops_name = operator_name or f"vecops::{name}"
    if vecops_name not in SIGNATURES:
        raise ValueError(f"no HIP operator named {vecops_name}")
    if dispatch is not None and not isinstance(dispatch, H.HostOperator):
        raise TypeError("dispatch must be a host_api.HostOperator")
    with _lock:
        key = (library, name)
        if key in _registrations:
            return _registrations[key].wrapper
        operator = dispatch if dispatch is not None else host_library().operator(vecops_name, artifact_directory)
        params, specs = SIGNATURES[vecops_name]
        reg = _Registration(library, name, operator, params, specs, return_outputs)
        reg.define()
        reg.wrapper = reg.public
        _registrations[key] = reg
        namespace = _libraries.setdefault(library, SimpleNamespace())
        setattr(namespace, name, reg.wrapper)
        return reg.wrapper


def register_all(library: str = "vecops_hip") -> SimpleNamespace:
    """Register every operator of this package under one torch library; returns its namespace."""
    for vecops_name in SIGNATURES:
        register(f"{library}::{vecops_name.split('::')[1]}")
    return _libraries[library]


def __getattr__(name: str):
    """Return a previously registered library namespace or raise AttributeError."""
    try:
        return _libraries[name]
    except KeyError as error:
        raise AttributeError(name) from error


__all__ = ["register", "register_all", "host_library", "SIGNATURES"]
