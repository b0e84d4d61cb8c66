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
  * `jax.ffi.ffi_call(target, result_types)(*operands, **attributes)` allocates the results and runs the
    C-ABI entry point that `csrc/ffi_shim.cc` binds to `target`, filling the parameter structure from
    operand shapes and attributes the way the shim does (dense row-major strides, a zero-element buffer
    for an absent operand, workspaces as extra results of exactly the declared size), through the ctypes
    mirror of include/axl_attn.h.  Every call is also appended to `State.calls`.

What this cannot show: XLA, jax's tracing and differentiation machinery, and the compiled shim.  What it
does show: that the module imports with the names it uses, that its classes and its custom_vjp pair run
to completion on the real kernels with the workspace sizes it computes, and that the results are those
of the torch-side mirror.
"""

from __future__ import annotations

import contextlib
import ctypes
import importlib
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


def _elements(t):
    return 0 if t is None else t.numel()


def _or_null(t):
    return None if _elements(t) == 0 else t.data_ptr()


def _dense4(shape):
    return _lib.AxlStrides(shape[1] * shape[2] * shape[3], shape[2] * shape[3], shape[3])


def _fill_aux(bias, drop, rate):
    aux = _lib.AxlAttnAux()
    if _elements(bias):
        d = bias.shape
        assert len(d) == 4
        aux.bias, aux.bias_dtype = bias.data_ptr(), _lib.dtype_code(bias.dtype)
        aux.bias_row_stride = d[3]
        aux.bias_head_stride = 0 if d[1] == 1 else d[2] * d[3]
        aux.bias_batch_stride = 0 if d[0] == 1 else d[1] * d[2] * d[3]
    if _elements(drop):
        d = drop.shape
        assert len(d) == 4 and drop.dtype == torch.uint8
        aux.dropout_mask, aux.dropout_rate = drop.data_ptr(), rate
        aux.drop_row_stride, aux.drop_head_stride, aux.drop_batch_stride = d[3], d[2] * d[3], d[1] * d[2] * d[3]
    return aux


def _fill_decode_bias(bias):
    out = _lib.AxlDecodeBias()
    if _elements(bias):
        d = bias.shape
        assert len(d) == 3
        out.bias, out.dtype = bias.data_ptr(), _lib.dtype_code(bias.dtype)
        out.head_stride = 0 if d[1] == 1 else d[2]
        out.batch_stride = 0 if d[0] == 1 else d[1] * d[2]
    return out


def _flash_fwd(ops, res, at):
    q, k, v, segment_ids, logit_sink, bias, dropout_mask, q_pos_offsets = ops
    out, lse = res
    p = _lib.AxlFlashFwdParams(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), out=out.data_ptr(), lse=lse.data_ptr(),
        segment_ids=_or_null(segment_ids), q_strides=_dense4(q.shape), k_strides=_dense4(k.shape),
        v_strides=_dense4(v.shape), out_strides=_dense4(out.shape), batch=q.shape[0], q_len=q.shape[1],
        num_q_heads=q.shape[2], head_dim=q.shape[3], kv_len=k.shape[1], num_kv_heads=k.shape[2],
        dtype=_lib.dtype_code(q.dtype), mask_kind=at["mask_kind"], sliding_window=at["sliding_window"],
        q_pos_offset=at["q_pos_offset"], softmax_scale=at["softmax_scale"], logit_sink=_or_null(logit_sink),
        q_pos_offsets=_or_null(q_pos_offsets), aux=_fill_aux(bias, dropout_mask, at["dropout_rate"]))
    return "axl_flash_fwd", p


def _flash_bwd(ops, res, at):
    q, k, v, out, d_out, lse, segment_ids, logit_sink, bias, dropout_mask = ops
    dq, dk, dv, d_sink, workspace = res
    p = _lib.AxlFlashBwdParams(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), out=out.data_ptr(), d_out=d_out.data_ptr(), lse=lse.data_ptr(),
        dq=dq.data_ptr(), dk=dk.data_ptr(), dv=dv.data_ptr(), segment_ids=_or_null(segment_ids),
        q_strides=_dense4(q.shape), k_strides=_dense4(k.shape), v_strides=_dense4(v.shape),
        out_strides=_dense4(out.shape), d_out_strides=_dense4(d_out.shape), dq_strides=_dense4(dq.shape),
        dk_strides=_dense4(dk.shape), dv_strides=_dense4(dv.shape), batch=q.shape[0], q_len=q.shape[1],
        num_q_heads=q.shape[2], head_dim=q.shape[3], kv_len=k.shape[1], num_kv_heads=k.shape[2],
        dtype=_lib.dtype_code(q.dtype), mask_kind=at["mask_kind"], sliding_window=at["sliding_window"],
        q_pos_offset=at["q_pos_offset"], softmax_scale=at["softmax_scale"], workspace=_or_null(workspace),
        workspace_bytes=workspace.numel(), logit_sink=_or_null(logit_sink), d_logit_sink=_or_null(d_sink),
        aux=_fill_aux(bias, dropout_mask, at["dropout_rate"]), flags=at["flags"])
    return "axl_flash_bwd", p


def _decode(ops, res, at):
    q, k, v, lengths, bias = ops
    out, workspace = res
    assert q.dim() == 3 and k.dim() == 4
    p = _lib.AxlDecodeParams(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), lengths=lengths.data_ptr(), out=out.data_ptr(),
        k_strides=_dense4(k.shape), v_strides=_dense4(v.shape), batch=q.shape[0], num_q_heads=q.shape[1],
        head_dim=q.shape[2], kv_len=k.shape[1], num_kv_heads=k.shape[2], dtype=_lib.dtype_code(q.dtype),
        sliding_window=at["sliding_window"], softmax_scale=at["softmax_scale"], workspace=_or_null(workspace),
        workspace_bytes=workspace.numel(), flags=at["flags"] & _lib.DECODE_DETERMINISTIC, bias=_fill_decode_bias(bias))
    return "axl_decode", p


def _paged_decode(ops, res, at):
    q, k_pages, v_pages, page_tables, lengths, bias = ops
    out, workspace = res
    assert q.dim() == 3 and k_pages.dim() == 4 and page_tables.dim() == 2
    p = _lib.AxlPagedDecodeParams(
        q=q.data_ptr(), k_pages=k_pages.data_ptr(), v_pages=v_pages.data_ptr(), page_tables=page_tables.data_ptr(),
        lengths=lengths.data_ptr(), out=out.data_ptr(), batch=q.shape[0], num_q_heads=q.shape[1], head_dim=q.shape[2],
        num_kv_heads=k_pages.shape[0], num_pages=k_pages.shape[1], page_size=k_pages.shape[2],
        pages_per_seq=page_tables.shape[1], dtype=_lib.dtype_code(q.dtype), sliding_window=at["sliding_window"],
        softmax_scale=at["softmax_scale"], workspace=_or_null(workspace), workspace_bytes=workspace.numel(),
        flags=at["flags"] & _lib.DECODE_DETERMINISTIC, bias=_fill_decode_bias(bias))
    return "axl_paged_decode", p


def _page_insert(ops, res, at):
    del at
    k_pages, v_pages, k_proj, v_proj, page_indices, key_positions = ops
    k_out, v_out = res
    assert k_out.data_ptr() == k_pages.data_ptr() and v_out.data_ptr() == v_pages.data_ptr()  # aliased
    pd, jd, idd = k_pages.shape, k_proj.shape, page_indices.shape
    assert len(pd) == 4 and len(jd) == 4 and len(idd) == 2
    p = _lib.AxlPageInsertParams(
        k_pages=k_out.data_ptr(), v_pages=v_out.data_ptr(), k_proj=k_proj.data_ptr(), v_proj=v_proj.data_ptr(),
        page_indices=page_indices.data_ptr(), key_positions=key_positions.data_ptr(),
        k_proj_batch_stride=jd[3], v_proj_batch_stride=jd[3], k_proj_head_stride=jd[1] * jd[2] * jd[3],
        v_proj_head_stride=jd[1] * jd[2] * jd[3], batch=idd[0], pages_per_seq=idd[1], num_kv_heads=pd[0],
        num_pages=pd[1], page_size=pd[2], head_dim=pd[3], dtype=_lib.dtype_code(k_pages.dtype),
        broadcast_positions=int(key_positions.numel() == 1 and idd[0] > 1))
    return "axl_paged_kv_insert", p


# target -> (handler, operands, results, attributes with the type the shim binds them as)
HANDLERS = {
    "AxlFlashFwd": (_flash_fwd, 8, 2, dict(softmax_scale=np.float32, mask_kind=np.int32, sliding_window=np.int32,
                                           q_pos_offset=np.int32, dropout_rate=np.float32)),
    "AxlFlashBwd": (_flash_bwd, 10, 5, dict(softmax_scale=np.float32, mask_kind=np.int32, sliding_window=np.int32,
                                            q_pos_offset=np.int32, dropout_rate=np.float32, flags=np.int32)),
    "AxlDecode": (_decode, 5, 2, dict(softmax_scale=np.float32, sliding_window=np.int32, flags=np.int32)),
    "AxlPagedDecode": (_paged_decode, 6, 2, dict(softmax_scale=np.float32, sliding_window=np.int32, flags=np.int32)),
    "AxlPagedKvInsert": (_page_insert, 6, 2, {}),
}


def _ffi_call(state: State):
    def ffi_call(target, result_types, input_output_aliases=None):
        handler, n_operands, n_results, attr_types = HANDLERS[target]
        assert any(t == target for t, _ in state.registered), f"{target} was never registered"

        def call(*operands, **attributes):
            assert len(operands) == n_operands and len(result_types) == n_results, target
            assert list(attributes) == list(attr_types), (target, list(attributes))
            for name, value in attributes.items():  # XLA FFI decodes attributes by exact type
                assert type(value) is attr_types[name], (target, name, type(value))
            device = operands[0].device
            aliases = input_output_aliases or {}
            alias_of = {r: o for o, r in aliases.items()}
            results = []
            for i, rt in enumerate(result_types):
                if i in alias_of:
                    src = operands[alias_of[i]]
                    assert tuple(src.shape) == rt.shape and src.dtype == rt.dtype
                    results.append(src)
                else:
                    results.append(torch.empty(rt.shape, dtype=rt.dtype, device=device))
            state.calls.append((target, [tuple(o.shape) for o in operands],
                                {k: v.item() for k, v in attributes.items()}, [tuple(r.shape) for r in results]))
            if state.execute:
                for o in operands:
                    assert o.numel() == 0 or (o.device.type == "cuda" and o.is_contiguous()), (target, o.shape, o.device)
                entry, params = handler(operands, results, {k: v.item() for k, v in attributes.items()})
                _lib.check(getattr(_lib.load(), entry)(ctypes.byref(params), _lib.current_stream_ptr()))
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
        if str(path).endswith("libaxl_attn_ffi.so"):   # the compiled shim: its symbols are only registered
            return types.SimpleNamespace(**{target: target for target in HANDLERS})
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
