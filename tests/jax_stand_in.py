"""Stand-ins that let `axlearn_amd/flash_attention/jax_ffi.py` be imported and run where jax is not installed.

jax_ffi.py is the JAX side of the XLA FFI binding: it needs `jax`, the reference's own modules
(`axlearn.common...`) and the compiled shim `libaxl_attn_ffi.so`, none of which exist in this
environment.  `installed()` puts the handful of names it uses into `sys.modules` for the duration of a
`with` block:

  * arrays are torch tensors (`jax.numpy` maps onto torch, `Tensor.astype` onto `Tensor.to`);
  * `axlearn.common.attention_bias`, `...flash_attention.common`, `...flash_attention.remat` and
    `...utils` map onto this package's host mirrors of those modules;
  * `jax.custom_vjp`, `jax.jit`, `jax.ShapeDtypeStruct` and `checkpoint_name` are the obvious eager
    forms (`custom_vjp` keeps the pair given to `defvjp`, `vjp()` below runs it; `checkpoint_name`
    returns its argument and records the name it was given);
  * `jax.ffi.ffi_call(target, result_types)(*operands, **attributes)` allocates the results (a workspace
    is a result of exactly the declared size; an aliased result is the donated operand), builds the call
    frame and runs the handler of that target in `csrc/ffi_shim.cc` itself, compiled against a stand-in
    for jaxlib's `xla/ffi/api/ffi.h` (tests/xla_ffi_stand_in/): operands and results as dense buffers with
    dtype and dimensions, scalars as named attributes of exact type.  Every call is also appended to
    `State.calls`.

What this cannot show: XLA, jax's tracing and differentiation machinery, and the shim against the real
header.  What it does show: that the module imports with the names it uses, that the shim compiles and
its handlers fill the C-ABI structures correctly from what the JAX side passes, that the classes and the
custom_vjp pair run to completion on the real kernels with the workspace sizes computed on the JAX side,
and that the results are those of the torch-side mirror.
"""

from __future__ import annotations

import contextlib
import ctypes
import importlib
import os
import sys
import types

import numpy as np
import torch

from axlearn_amd import _lib

JAX_SIDE = "axlearn_amd.flash_attention.jax_ffi"


class State:
    """What the stand-ins saw."""

    def __init__(self):
        self.registered = []      # (target, platform)
        self.calls = []           # (target, [operand shapes], {attribute: value}, [result shapes])
        self.checkpoint_names = []
        self.execute = True       # False: results are allocated (on the operands' device) but no kernel runs
        self.device = "cuda"      # where the module's own constants (jnp.zeros, jnp.arange, random masks) live


class ShapeDtypeStruct:
    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(int(s) for s in shape), dtype


class CustomVjp:
    """`jax.custom_vjp(fun, nondiff_argnums)`: calling it evaluates `fun`."""

    def __init__(self, fun, nondiff_argnums=()):
        self.fun, self.nondiff_argnums = fun, tuple(nondiff_argnums)
        self.fwd = self.bwd = None
        self.__doc__ = fun.__doc__

    def defvjp(self, fwd, bwd):
        self.fwd, self.bwd = fwd, bwd

    def __call__(self, *args):
        return self.fun(*args)

    def vjp(self, *args):
        """(primal output, cotangent -> gradients of the differentiable arguments), by the rules given to
        `defvjp`: fwd gets every argument, bwd the non-differentiable ones first, then residuals and the
        cotangent."""
        out, residuals = self.fwd(*args)
        nondiff = [args[i] for i in self.nondiff_argnums]
        return out, lambda cotangent: self.bwd(*nondiff, residuals, cotangent)


def _jit(fun=None, **_):
    return fun if fun is not None else (lambda f: f)


TARGETS = ("AxlFlashFwd", "AxlFlashBwd", "AxlDecode", "AxlPagedDecode", "AxlPagedKvInsert")
SHIM_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "xla_ffi_stand_in")
SHIM_PATH = os.path.join(SHIM_DIR, "libaxl_attn_ffi_standin.so")
# xla::ffi::DataType
_DATA_TYPE = {torch.bool: 1, torch.int32: 4, torch.int64: 5, torch.uint8: 6, torch.float16: 10, torch.float32: 11,
              torch.bfloat16: 16}
_ERROR_CODE = {3: "INVALID_ARGUMENT", 12: "UNIMPLEMENTED", 13: "INTERNAL"}


class _Buffer(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("rank", ctypes.c_int32),
                ("dims", ctypes.POINTER(ctypes.c_int64))]


class _Attr(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("kind", ctypes.c_int32), ("i32", ctypes.c_int32), ("f32", ctypes.c_float)]


class _CallFrame(ctypes.Structure):
    _fields_ = [("stream", ctypes.c_void_p), ("n_args", ctypes.c_int32), ("args", ctypes.POINTER(_Buffer)),
                ("n_rets", ctypes.c_int32), ("rets", ctypes.POINTER(_Buffer)), ("n_attrs", ctypes.c_int32),
                ("attrs", ctypes.POINTER(_Attr)), ("error_code", ctypes.c_int32), ("error", ctypes.c_char * 1024)]


class FfiError(RuntimeError):
    """A handler of the shim returned an xla::ffi::Error."""

    def __init__(self, code: int, message: str):
        super().__init__(f"{_ERROR_CODE.get(code, code)}: {message}")
        self.code = code


_shim = None


def load_shim() -> ctypes.CDLL:
    """csrc/ffi_shim.cc built against the stand-in header (tests/xla_ffi_stand_in/Makefile; `build()` of
    __graft_entry__.py makes it)."""
    global _shim
    if _shim is None:
        if not os.path.exists(SHIM_PATH):
            raise RuntimeError(f"{SHIM_PATH} is missing: make -C {SHIM_DIR}")
        _lib.load()
        shim = ctypes.CDLL(SHIM_PATH)
        if shim.axl_ffi_shim_abi_version() != _lib.ABI_VERSION:
            raise RuntimeError(f"{SHIM_PATH} was built against ABI {shim.axl_ffi_shim_abi_version()}, "
                               f"the library has {_lib.ABI_VERSION}: make -C {SHIM_DIR}")
        _shim = shim
    return _shim


def _buffers(tensors, keep):
    arr = (_Buffer * len(tensors))()
    for slot, t in zip(arr, tensors):
        dims = (ctypes.c_int64 * max(t.dim(), 1))(*t.shape)
        keep.append(dims)
        slot.data, slot.dtype, slot.rank, slot.dims = t.data_ptr() if t.numel() else None, _DATA_TYPE[t.dtype], t.dim(), dims
    return arr


def _run_handler(target, operands, results, attributes):
    """One custom call: the frame XLA would hand to the handler, then the handler itself."""
    keep = []
    attrs = (_Attr * max(len(attributes), 1))()
    for slot, (name, value) in zip(attrs, attributes.items()):
        slot.name = name.encode()
        if type(value) is np.int32:       # XLA FFI decodes scalars by exact type: no conversions
            slot.kind, slot.i32 = 0, int(value)
        elif type(value) is np.float32:
            slot.kind, slot.f32 = 1, float(value)
        else:
            raise TypeError(f"{target}: attribute {name} must be np.int32 or np.float32, got {type(value)}")
    stream = _lib.current_stream_ptr() if torch.cuda.is_available() else None
    frame = _CallFrame(stream=stream, n_args=len(operands), args=_buffers(operands, keep),
                       n_rets=len(results), rets=_buffers(results, keep), n_attrs=len(attributes), attrs=attrs)
    handler = getattr(load_shim(), target)
    handler.restype, handler.argtypes = ctypes.c_int, [ctypes.POINTER(_CallFrame)]
    if handler(ctypes.byref(frame)) != 0:
        raise FfiError(frame.error_code, frame.error.decode())


def _ffi_call(state: State):
    def ffi_call(target, result_types, input_output_aliases=None):
        assert any(t == target for t, _ in state.registered), f"{target} was never registered"

        def call(*operands, **attributes):
            device = operands[0].device
            alias_of = {r: o for o, r in (input_output_aliases or {}).items()}
            results = []
            for i, rt in enumerate(result_types):
                if i in alias_of:   # a donated operand: XLA hands its buffer back as the result
                    src = operands[alias_of[i]]
                    assert tuple(src.shape) == rt.shape and src.dtype == rt.dtype
                    results.append(src)
                else:
                    results.append(torch.empty(rt.shape, dtype=rt.dtype, device=device))
            state.calls.append((target, [tuple(o.shape) for o in operands],
                                {k: v.item() for k, v in attributes.items()}, [tuple(r.shape) for r in results]))
            if state.execute:
                for o in operands:   # XLA buffers are dense and live on the device
                    assert o.numel() == 0 or (o.device.type == "cuda" and o.is_contiguous()), (target, o.shape, o.device)
                _run_handler(target, operands, results, attributes)
            return tuple(results)

        return call

    return ffi_call


def _numpy_like(state: State):
    jnp = types.ModuleType("jax.numpy")
    for name in ("bfloat16", "float16", "float32", "int32", "uint8", "bool"):
        setattr(jnp, name, getattr(torch, name))
    jnp.dtype = lambda d: d
    jnp.zeros = lambda shape, dtype=torch.float32: torch.zeros(shape, dtype=dtype, device=state.device)
    jnp.arange = lambda n: torch.arange(n, device=state.device)
    jnp.broadcast_to = lambda x, shape: torch.broadcast_to(x, shape).contiguous()

    def where(cond, a, b):
        a = a if isinstance(a, torch.Tensor) else torch.tensor(a, device=cond.device)
        b = b if isinstance(b, torch.Tensor) else torch.tensor(b, device=cond.device)
        return torch.where(cond, a, b)

    jnp.where = where

    def pad(x, pad_width):   # ((before, after), ...) per dimension, zeros
        flat = [n for pair in reversed(pad_width) for n in pair]
        return torch.nn.functional.pad(x, flat) if any(flat) else x

    jnp.pad = pad
    return jnp


@contextlib.contextmanager
def installed():
    """Yields (the freshly imported jax_ffi module, State).  Everything put into `sys.modules`,
    `ctypes.CDLL` and `torch.Tensor.astype` is taken out again on exit."""
    from axlearn_amd import attention_bias
    from axlearn_amd.flash_attention import common, hip_attention

    state = State()
    jax = types.ModuleType("jax")
    jax.numpy = _numpy_like(state)
    jax.random = types.ModuleType("jax.random")

    def bernoulli(key, p, shape):   # key: an int seed here
        g = torch.Generator().manual_seed(int(key))
        return (torch.rand(tuple(shape), generator=g) < p).to(state.device)

    jax.random.bernoulli = bernoulli
    jax.custom_vjp = CustomVjp
    jax.jit = _jit
    jax.ShapeDtypeStruct = ShapeDtypeStruct
    jax.ffi = types.ModuleType("jax.ffi")
    jax.ffi.pycapsule = lambda symbol: symbol
    jax.ffi.register_ffi_target = lambda name, capsule, platform: state.registered.append((name, platform))
    jax.ffi.ffi_call = _ffi_call(state)
    jax.ad_checkpoint = types.ModuleType("jax.ad_checkpoint")

    def checkpoint_name(x, name):
        state.checkpoint_names.append(name)
        return x

    jax.ad_checkpoint.checkpoint_name = checkpoint_name
    remat = types.ModuleType("axlearn.common.flash_attention.remat")
    remat.FLASH_ATTN_RESIDUAL_NAME = hip_attention.FLASH_ATTN_RESIDUAL_NAME
    utils = types.ModuleType("axlearn.common.utils")
    utils.Nested, utils.Tensor = dict, torch.Tensor
    fakes = {
        "jax": jax, "jax.numpy": jax.numpy, "jax.ffi": jax.ffi, "jax.ad_checkpoint": jax.ad_checkpoint,
        "jax.random": jax.random,
        "axlearn": types.ModuleType("axlearn"), "axlearn.common": types.ModuleType("axlearn.common"),
        "axlearn.common.attention_bias": attention_bias,
        "axlearn.common.flash_attention": types.ModuleType("axlearn.common.flash_attention"),
        "axlearn.common.flash_attention.common": common,
        "axlearn.common.flash_attention.remat": remat,
        "axlearn.common.utils": utils,
    }
    assert not any(name in sys.modules for name in fakes), "a real jax / axlearn is importable: use it instead"

    real_cdll = ctypes.CDLL

    def cdll(path, *args, **kwargs):
        if str(path).endswith("libaxl_attn_ffi.so"):   # the compiled shim: its handler symbols are only registered
            return types.SimpleNamespace(axl_ffi_shim_abi_version=load_shim().axl_ffi_shim_abi_version,
                                         **{target: target for target in TARGETS})
        return real_cdll(path, *args, **kwargs)

    sys.modules.update(fakes)
    sys.modules.pop(JAX_SIDE, None)
    ctypes.CDLL = cdll
    torch.Tensor.astype = lambda self, dtype: self.to(dtype)
    try:
        yield importlib.import_module(JAX_SIDE), state
    finally:
        del torch.Tensor.astype
        ctypes.CDLL = real_cdll
        for name in list(fakes) + [JAX_SIDE]:
            sys.modules.pop(name, None)
        pkg = sys.modules.get("axlearn_amd.flash_attention")
        if pkg is not None and hasattr(pkg, "jax_ffi"):
            delattr(pkg, "jax_ffi")
