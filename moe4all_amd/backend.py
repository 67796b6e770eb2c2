"""ctypes binding of ``include/infr_hip.h`` shaped like the reference's Rust interface.

Reference counterparts: ``infr_core::backend::{Backend, Buffer, Plan, Bindings, BufferUsage}``
(crates/infr-core/src/backend.rs:384-1088) and ``infr_core::graph::{Graph, Op, TensorKind}``
(crates/infr-core/src/graph.rs).  Errors map to exceptions the way the reference's
``infr_core::Error`` variants would surface (crates/infr-core/src/error.rs:11-31).
"""
from __future__ import annotations

import ctypes as C
import enum
import os
import subprocess
from dataclasses import dataclass
from typing import Iterable, Optional, Sequence

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_PKG, "csrc")
_LIB = os.path.join(_PKG, "libinfr_hip.so")

NO_TENSOR = 0xFFFFFFFF


class BackendError(RuntimeError):
    """infr_core::Error::Backend / Other (status 1, 3, 4)."""


class Unsupported(BackendError):
    """infr_core::Error::Unsupported (status 2)."""


class DType(enum.IntEnum):
    # ordinals of infr_core::DType (crates/infr-core/src/tensor.rs:7-57)
    F32 = 0
    F16 = 1
    Bf16 = 2
    I32 = 3
    U32 = 4
    Q4_0 = 5
    Q4_1 = 6
    Q5_0 = 7
    Q5_1 = 8
    Q8_0 = 9
    Q2K = 10
    Q3K = 11
    Q4K = 12
    Q5K = 13
    Q6K = 14
    Iq1S = 15
    Iq1M = 16
    Iq2Xxs = 17
    Iq2Xs = 18
    Iq2S = 19
    Iq3Xxs = 20
    Iq3S = 21
    Iq4Nl = 22
    Iq4Xs = 23
    Tq1_0 = 24
    Tq2_0 = 25
    I2S = 26
    Q2_0 = 27
    Mxfp4 = 28
    Nvfp4 = 29


class BufferUsage(enum.IntEnum):
    Weights = 0
    Activations = 1
    KvCache = 2
    Staging = 3
    Readback = 4
    HostWeights = 5


class TensorKind(enum.IntEnum):
    Input = 0
    Weight = 1
    Internal = 2
    Output = 3


class Activation(enum.IntEnum):
    Silu = 0
    Gelu = 1
    Sigmoid = 2


class MoeGating(enum.IntEnum):
    Softmax = 0
    Sigmoid = 1
    SqrtSoftplus = 2


_BLOCK = {DType.F32: (1, 4), DType.I32: (1, 4), DType.U32: (1, 4), DType.F16: (1, 2), DType.Bf16: (1, 2),
          DType.Q8_0: (32, 34), DType.Q4K: (256, 144), DType.Q6K: (256, 210), DType.Q4_0: (32, 18), DType.Q4_1: (32, 20),
          DType.Q5_0: (32, 22), DType.Q5_1: (32, 24), DType.Q2K: (256, 84), DType.Q3K: (256, 110), DType.Q5K: (256, 176),
          DType.Iq4Nl: (32, 18), DType.Iq4Xs: (256, 136), DType.Tq1_0: (256, 54), DType.Tq2_0: (256, 66), DType.Q2_0: (64, 18),
          DType.Mxfp4: (32, 17), DType.Nvfp4: (64, 36),
          DType.Iq1S: (256, 50), DType.Iq1M: (256, 56), DType.Iq2Xxs: (256, 66), DType.Iq2Xs: (256, 74), DType.Iq2S: (256, 82),
          DType.Iq3Xxs: (256, 98), DType.Iq3S: (256, 110)}


def bytes_for(dtype: DType, numel: int) -> int:
    e, b = _BLOCK[DType(dtype)]
    if numel % e:
        raise ValueError(f"{numel} elements is not a whole number of {DType(dtype).name} blocks")
    return numel // e * b


# ----------------------------------------------------------------------------- C structs
class _TensorDecl(C.Structure):
    _fields_ = [("rank", C.c_uint32), ("shape", C.c_uint64 * 4), ("dtype", C.c_int32), ("kind", C.c_int32)]


class _OpMoeFfn(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("x", "router_x", "router", "gate_exps", "up_exps", "down_exps",
                                          "down_scale", "fused_gate_up", "dst", "ne", "n_expert", "n_used",
                                          "n_ff_exp")] + [
        ("scale", C.c_float), ("act", C.c_int32), ("has_swiglu_clamp", C.c_uint32), ("swiglu_clamp", C.c_float),
        ("gating", C.c_int32), ("norm_w", C.c_uint32), ("weight_before", C.c_uint32), ("has_ep_band", C.c_uint32),
        ("ep_base", C.c_uint32), ("ep_n_local", C.c_uint32), ("exp_probs_b", C.c_uint32),
        ("n_expert_groups", C.c_uint32), ("n_expert_groups_used", C.c_uint32), ("expert_ids", C.c_uint32)]


class _OpLinear(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("x", "weight", "dst", "m", "in_f", "out_f", "w_off")]


class _OpGatedAct(C.Structure):
    _fields_ = [("gate", C.c_uint32), ("up", C.c_uint32), ("dst", C.c_uint32), ("rows", C.c_uint32),
                ("nff", C.c_uint32), ("act", C.c_int32), ("up_off", C.c_uint32), ("up_stride", C.c_uint32),
                ("gate_stride", C.c_uint32), ("gate_block_width", C.c_uint32), ("has_swiglu_clamp", C.c_uint32),
                ("swiglu_clamp", C.c_float)]


class _OpAdd(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("a", "b", "dst", "n")]


class _OpSharedAdd(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("moe", "shexp", "gate", "dst", "rows", "n")]


class _OpCopy(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("src", "src_off", "src_stride", "dst", "dst_off", "dst_stride", "rows", "n")]


class _OpRmsNorm(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("x", "weight", "dst", "rows", "dim")] + [("eps", C.c_float)]


class _OpUnion(C.Union):
    _fields_ = [("moe_ffn", _OpMoeFfn), ("linear", _OpLinear), ("gated_act", _OpGatedAct), ("add", _OpAdd),
                ("moe_shared_expert_add", _OpSharedAdd), ("copy", _OpCopy), ("rms_norm", _OpRmsNorm)]


class _Op(C.Structure):
    _fields_ = [("kind", C.c_int32), ("u", _OpUnion)]


class _Graph(C.Structure):
    _fields_ = [("tensors", C.POINTER(_TensorDecl)), ("n_tensors", C.c_uint32), ("ops", C.POINTER(_Op)),
                ("n_ops", C.c_uint32)]


class _Binding(C.Structure):
    _fields_ = [("tensor", C.c_uint32), ("buffer", C.c_void_p)]


class _Caps(C.Structure):
    _fields_ = [("name", C.c_char * 64)] + [(n, C.c_uint32) for n in (
        "f16", "bf16", "i8", "i8_dot", "subgroup_min", "subgroup_max", "integrated", "compute_units",
        "buffer_device_address", "max_shared_memory_bytes", "unified_memory", "decode_replay", "combined_gu",
        "graph_input_inplace")] + [("device_memory_bytes", C.c_uint64)]


class _Config(C.Structure):
    _fields_ = [("disable_graph_replay", C.c_uint32), ("moe_batched_min_rows", C.c_uint32),
                ("disable_op_fusion", C.c_uint32), ("disable_single_launch_moe", C.c_uint32),
                ("single_launch_spin_limit", C.c_uint32), ("single_launch_logits", C.c_uint32),
                ("single_launch_guess_skew", C.c_uint32), ("disable_single_launch_guess", C.c_uint32)]


class _MoeFfnStaticArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("router", C.c_void_p), ("gate_exps", C.c_void_p), ("up_exps", C.c_void_p),
                ("down_exps", C.c_void_p), ("dst", C.c_void_p),
                ("gate_dtype", C.c_int32), ("up_dtype", C.c_int32), ("down_dtype", C.c_int32),
                ("rows", C.c_uint32), ("ne", C.c_uint32), ("n_expert", C.c_uint32), ("n_used", C.c_uint32),
                ("n_ff_exp", C.c_uint32)]


STATIC_SCRATCH_BYTES = 1 << 20   # INFR_HIP_STATIC_SCRATCH_BYTES


class _ProfEntry(C.Structure):
    _fields_ = [("kernel", C.c_char * 64), ("launches", C.c_uint64), ("total_ms", C.c_double),
                ("min_ms", C.c_double), ("max_ms", C.c_double)]


# Every symbol include/infr_hip.h declares, with its ctypes signature.
_V = C.c_void_p
_SIGNATURES = {
    "infr_hip_create": ([C.c_int, C.POINTER(_Config), C.POINTER(_V)], C.c_int),
    "infr_hip_destroy": ([_V], None),
    "infr_hip_name": ([_V], C.c_char_p),
    "infr_hip_capabilities_get": ([_V, C.POINTER(_Caps)], C.c_int),
    "infr_hip_alloc": ([_V, C.c_size_t, C.c_int32, C.POINTER(_V)], C.c_int),
    "infr_hip_alloc_uninit": ([_V, C.c_size_t, C.c_int32, C.POINTER(_V)], C.c_int),
    "infr_hip_buffer_len": ([_V], C.c_size_t),
    "infr_hip_buffer_device_addr": ([_V], C.c_uint64),
    "infr_hip_buffer_free": ([_V], None),
    "infr_hip_upload": ([_V, _V, _V, C.c_size_t], C.c_int),
    "infr_hip_download": ([_V, _V, _V, C.c_size_t], C.c_int),
    "infr_hip_upload_range": ([_V, _V, C.c_size_t, _V, C.c_size_t], C.c_int),
    "infr_hip_download_range": ([_V, _V, C.c_size_t, _V, C.c_size_t], C.c_int),
    "infr_hip_copy_buffer": ([_V, _V, _V, C.c_size_t], C.c_int),
    "infr_hip_compile": ([_V, C.POINTER(_Graph), C.POINTER(_V)], C.c_int),
    "infr_hip_plan_free": ([_V], None),
    "infr_hip_execute": ([_V, _V, C.POINTER(_Binding), C.c_uint32], C.c_int),
    "infr_hip_sync": ([_V], C.c_int),
    "infr_hip_last_error": ([], C.c_char_p),
    "infr_hip_prof_enable": ([_V, C.c_int], C.c_int),
    "infr_hip_probe_grouped_loads_only": ([_V, C.c_int], C.c_int),
    "infr_hip_prof_read": ([_V, C.POINTER(_ProfEntry), C.c_uint32, C.POINTER(C.c_uint32)], C.c_int),
    "infr_hip_plan_moe_routing": ([_V, _V, C.c_uint32, _V, _V, _V, _V], C.c_int),
    "infr_hip_plan_moe_bucketing": ([_V, _V, C.c_uint32, _V, _V, _V], C.c_int),
    "infr_hip_dequant": ([_V, _V, C.c_int32, C.c_uint64, _V], C.c_int),
    "infr_hip_moe_ffn_static": ([_V, C.POINTER(_MoeFfnStaticArgs)], C.c_int),
    "infr_hip_probe_late_experts": ([_V, C.POINTER(C.c_uint64)], C.c_int),
    "infr_hip_probe_alloc_calls": ([C.POINTER(C.c_uint64)], C.c_int),
    "infr_hip_probe_dependent_reads": ([_V, _V, C.POINTER(C.c_uint64), C.c_uint32, C.c_uint32, C.POINTER(C.c_double),
                                        C.POINTER(C.c_double)], C.c_int),
}

_lib: Optional[C.CDLL] = None


def library_path() -> str:
    return _LIB


def build_library(jobs: int = 8) -> str:
    """Compile libinfr_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    subprocess.check_call(["make", "-C", _CSRC, "-B", f"-j{jobs}"], stdout=subprocess.DEVNULL,
                          stderr=subprocess.DEVNULL)
    return _LIB


def load_library() -> C.CDLL:
    """Load the HIP backend.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise BackendError(f"{_LIB} is missing: build it with moe4all_amd.build_library() "
                               "(hipcc --offload-arch=gfx950); this backend has no CPU fallback")
        lib = C.CDLL(_LIB)
        for name, (args, res) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = res
        _lib = lib
    return _lib


def _check(st: int) -> None:
    if st == 0:
        return
    msg = load_library().infr_hip_last_error().decode("utf-8", "replace")
    if st == 2:
        raise Unsupported(f"unsupported: {msg}")
    if st == 3:
        raise BackendError("aborted: shutdown requested")
    raise BackendError(f"backend: {msg}")


# ----------------------------------------------------------------------------- graph IR
@dataclass(frozen=True)
class TensorDesc:
    shape: tuple
    dtype: DType

    def __init__(self, shape, dtype):
        shape = (shape,) if isinstance(shape, int) else tuple(int(s) for s in shape)
        object.__setattr__(self, "shape", shape)
        object.__setattr__(self, "dtype", DType(dtype))

    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    def nbytes(self) -> int:
        return bytes_for(self.dtype, self.numel())


class Graph:
    """Ordered op list over declared tensors (crates/infr-core/src/graph.rs:2056-2262)."""

    def __init__(self):
        self.tensors: list = []   # (TensorDesc, TensorKind)
        self.ops: list = []       # _Op
        self.inputs: list = []
        self.weights: list = []
        self.outputs: list = []

    def _decl(self, desc: TensorDesc, kind: TensorKind) -> int:
        self.tensors.append((desc, kind))
        return len(self.tensors) - 1

    def input(self, desc: TensorDesc) -> int:
        i = self._decl(desc, TensorKind.Input)
        self.inputs.append(i)
        return i

    def weight(self, desc: TensorDesc) -> int:
        i = self._decl(desc, TensorKind.Weight)
        self.weights.append(i)
        return i

    def internal(self, desc: TensorDesc) -> int:
        return self._decl(desc, TensorKind.Internal)

    def output(self, desc: TensorDesc) -> int:
        i = self._decl(desc, TensorKind.Output)
        self.outputs.append(i)
        return i

    def desc(self, tid: int) -> TensorDesc:
        return self.tensors[tid][0]

    # ---- Op constructors, field names as in the reference's Op variants
    def moe_ffn(self, *, x, router, gate_exps, up_exps, down_exps, dst, ne, n_expert, n_used, n_ff_exp,
                router_x=None, down_scale=None, fused_gate_up=False, scale=1.0, act=Activation.Silu,
                swiglu_clamp=None, gating=MoeGating.Softmax, norm_w=True, weight_before=False, ep_band=None,
                exp_probs_b=None, n_expert_groups=0, n_expert_groups_used=0, expert_ids=None) -> None:
        op = _Op(kind=0)
        m = op.u.moe_ffn
        m.x, m.router_x, m.router = x, x if router_x is None else router_x, router
        m.gate_exps, m.up_exps, m.down_exps = gate_exps, gate_exps if up_exps is None else up_exps, down_exps
        m.down_scale = NO_TENSOR if down_scale is None else down_scale
        m.fused_gate_up = int(fused_gate_up)
        m.dst, m.ne, m.n_expert, m.n_used, m.n_ff_exp = dst, ne, n_expert, n_used, n_ff_exp
        m.scale, m.act = scale, int(act)
        m.has_swiglu_clamp, m.swiglu_clamp = int(swiglu_clamp is not None), swiglu_clamp or 0.0
        m.gating, m.norm_w, m.weight_before = int(gating), int(norm_w), int(weight_before)
        m.has_ep_band = int(ep_band is not None)
        m.ep_base, m.ep_n_local = ep_band if ep_band is not None else (0, 0)
        m.exp_probs_b = NO_TENSOR if exp_probs_b is None else exp_probs_b
        m.n_expert_groups, m.n_expert_groups_used = n_expert_groups, n_expert_groups_used
        m.expert_ids = NO_TENSOR if expert_ids is None else expert_ids
        self.ops.append(op)

    def linear(self, *, x, weight, dst, m, in_f, out_f, w_off=0) -> None:
        op = _Op(kind=1)
        l = op.u.linear
        l.x, l.weight, l.dst, l.m, l.in_f, l.out_f, l.w_off = x, weight, dst, m, in_f, out_f, w_off
        self.ops.append(op)

    def gated_act(self, *, gate, up, dst, rows, nff, act=Activation.Silu, up_off=0, up_stride=0, gate_stride=0,
                  gate_block_width=0, swiglu_clamp=None) -> None:
        op = _Op(kind=2)
        a = op.u.gated_act
        a.gate, a.up, a.dst, a.rows, a.nff, a.act = gate, up, dst, rows, nff, int(act)
        a.up_off, a.up_stride, a.gate_stride, a.gate_block_width = up_off, up_stride, gate_stride, gate_block_width
        a.has_swiglu_clamp, a.swiglu_clamp = int(swiglu_clamp is not None), swiglu_clamp or 0.0
        self.ops.append(op)

    def add(self, *, a, b, dst, n) -> None:
        op = _Op(kind=3)
        op.u.add.a, op.u.add.b, op.u.add.dst, op.u.add.n = a, b, dst, n
        self.ops.append(op)

    def moe_shared_expert_add(self, *, moe, shexp, gate, dst, rows, n) -> None:
        op = _Op(kind=4)
        s = op.u.moe_shared_expert_add
        s.moe, s.shexp, s.gate, s.dst, s.rows, s.n = moe, shexp, gate, dst, rows, n
        self.ops.append(op)

    def copy(self, *, src, src_off, dst, dst_off, n) -> None:
        """Op::Copy (crates/infr-core/src/graph.rs:1230-1237)."""
        op = _Op(kind=5)
        c = op.u.copy
        c.src, c.src_off, c.dst, c.dst_off, c.rows, c.n = src, src_off, dst, dst_off, 1, n
        self.ops.append(op)

    def copy_strided(self, *, src, src_off, src_stride, dst, dst_off, dst_stride, rows, n) -> None:
        """Op::CopyStrided (crates/infr-core/src/graph.rs:1238-1251)."""
        op = _Op(kind=6)
        c = op.u.copy
        c.src, c.src_off, c.src_stride, c.dst, c.dst_off, c.dst_stride, c.rows, c.n = (
            src, src_off, src_stride, dst, dst_off, dst_stride, rows, n)
        self.ops.append(op)

    def rms_norm(self, *, x, weight, dst, rows, dim, eps, add=False) -> None:
        """Op::RmsNorm (crates/infr-core/src/graph.rs:160-169); add=True is Op::RmsNormAdd (:170-179)."""
        op = _Op(kind=8 if add else 7)
        r = op.u.rms_norm
        r.x, r.weight, r.dst, r.rows, r.dim, r.eps = x, weight, dst, rows, dim, eps
        self.ops.append(op)

    def push_raw(self, kind: int) -> None:
        """Append an op of an arbitrary kind code (used to test the Unsupported path)."""
        self.ops.append(_Op(kind=kind))

    def _as_c(self):
        nt, no = len(self.tensors), len(self.ops)
        decls = (_TensorDecl * max(nt, 1))()
        for i, (d, k) in enumerate(self.tensors):
            if len(d.shape) > 4:
                raise ValueError("tensor rank > 4")
            decls[i].rank = len(d.shape)
            for j, s in enumerate(d.shape):
                decls[i].shape[j] = s
            decls[i].dtype, decls[i].kind = int(d.dtype), int(k)
        ops = (_Op * max(no, 1))(*self.ops)
        g = _Graph(tensors=decls, n_tensors=nt, ops=ops, n_ops=no)
        return g, (decls, ops)


# ----------------------------------------------------------------------------- runtime objects
class Buffer:
    """Opaque device allocation (crates/infr-core/src/backend.rs:423-452)."""

    def __init__(self, be: "Backend", handle: int):
        self._be, self._h = be, handle

    def len_bytes(self) -> int:
        return load_library().infr_hip_buffer_len(self._h)

    def device_addr(self) -> int:
        return load_library().infr_hip_buffer_device_addr(self._h)

    def free(self) -> None:
        if self._h:
            load_library().infr_hip_buffer_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()   # safe after Backend.close(): a buffer keeps its backend object alive until it is freed
        except Exception:
            pass


class Plan:
    def __init__(self, be: "Backend", handle: int, graph: Graph):
        self._be, self._h, self.graph = be, handle, graph

    def free(self) -> None:
        if self._h:
            load_library().infr_hip_plan_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()   # safe after Backend.close(), as for buffers
        except Exception:
            pass


class Bindings:
    """tensor id -> buffer for one execute (crates/infr-core/src/backend.rs:522-620)."""

    def __init__(self):
        self._slots: dict = {}

    def bind(self, tid: int, buf: Buffer) -> "Bindings":
        self._slots[int(tid)] = buf
        return self

    def get(self, tid: int) -> Optional[Buffer]:
        return self._slots.get(int(tid))

    def _as_c(self):
        n = len(self._slots)
        arr = (_Binding * max(n, 1))()
        for i, (t, b) in enumerate(self._slots.items()):
            arr[i].tensor, arr[i].buffer = t, b._h
        return arr, n


class Backend:
    """The gfx950 compute device (crates/infr-core/src/backend.rs:630 `trait Backend`)."""

    def __init__(self, device: int = 0, *, disable_graph_replay: bool = False, moe_batched_min_rows: int = 0,
                 disable_op_fusion: bool = False, disable_single_launch_moe: bool = False,
                 single_launch_spin_limit: int = 0, single_launch_logits: int = 0, single_launch_guess_skew: int = 0,
                 disable_single_launch_guess: bool = False):
        self._h = None
        lib = load_library()
        cfg = _Config(disable_graph_replay=int(disable_graph_replay), moe_batched_min_rows=moe_batched_min_rows,
                      disable_op_fusion=int(disable_op_fusion), disable_single_launch_moe=int(disable_single_launch_moe),
                      single_launch_spin_limit=single_launch_spin_limit, single_launch_logits=single_launch_logits,
                      single_launch_guess_skew=single_launch_guess_skew,
                      disable_single_launch_guess=int(disable_single_launch_guess))
        h = _V()
        _check(lib.infr_hip_create(device, C.byref(cfg), C.byref(h)))
        self._h = h.value
        self._lib = lib

    def close(self) -> None:
        if self._h:
            self._lib.infr_hip_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def name(self) -> str:
        return self._lib.infr_hip_name(self._h).decode()

    def capabilities(self) -> dict:
        caps = _Caps()
        _check(self._lib.infr_hip_capabilities_get(self._h, C.byref(caps)))
        out = {n: getattr(caps, n) for n, _ in _Caps._fields_}
        out["name"] = caps.name.decode()
        return out

    # ---- memory
    def alloc(self, nbytes: int, usage: BufferUsage = BufferUsage.Activations) -> Buffer:
        h = _V()
        _check(self._lib.infr_hip_alloc(self._h, nbytes, int(usage), C.byref(h)))
        return Buffer(self, h.value)

    def alloc_uninit(self, nbytes: int, usage: BufferUsage = BufferUsage.Weights) -> Buffer:
        h = _V()
        _check(self._lib.infr_hip_alloc_uninit(self._h, nbytes, int(usage), C.byref(h)))
        return Buffer(self, h.value)

    @staticmethod
    def _bytes(a) -> np.ndarray:
        if isinstance(a, (bytes, bytearray, memoryview)):
            return np.frombuffer(a, dtype=np.uint8)
        return np.ascontiguousarray(a).view(np.uint8).reshape(-1)

    def upload(self, dst: Buffer, src) -> None:
        b = self._bytes(src)
        _check(self._lib.infr_hip_upload(self._h, dst._h, b.ctypes.data_as(_V), b.size))

    def upload_range(self, dst: Buffer, offset: int, src) -> None:
        b = self._bytes(src)
        _check(self._lib.infr_hip_upload_range(self._h, dst._h, offset, b.ctypes.data_as(_V), b.size))

    def download(self, src: Buffer, nbytes: Optional[int] = None, dtype=np.uint8) -> np.ndarray:
        n = src.len_bytes() if nbytes is None else nbytes
        out = np.empty(n, np.uint8)
        _check(self._lib.infr_hip_download(self._h, src._h, out.ctypes.data_as(_V), n))
        return out.view(dtype)

    def download_range(self, src: Buffer, offset: int, nbytes: int, dtype=np.uint8) -> np.ndarray:
        out = np.empty(nbytes, np.uint8)
        _check(self._lib.infr_hip_download_range(self._h, src._h, offset, out.ctypes.data_as(_V), nbytes))
        return out.view(dtype)

    def copy_buffer(self, src: Buffer, dst: Buffer, nbytes: int) -> None:
        _check(self._lib.infr_hip_copy_buffer(self._h, src._h, dst._h, nbytes))

    def buffer_from(self, data, usage: BufferUsage = BufferUsage.Weights) -> Buffer:
        """alloc_uninit + upload, the GPU weight binder's sequence
        (crates/infr-llama/src/seam/mod.rs:597-608)."""
        b = self._bytes(data)
        buf = self.alloc_uninit(b.size, usage)
        self.upload(buf, b)
        return buf

    # ---- graphs
    def compile(self, graph: Graph) -> Plan:
        g, keep = graph._as_c()
        h = _V()
        _check(self._lib.infr_hip_compile(self._h, C.byref(g), C.byref(h)))
        del keep
        return Plan(self, h.value, graph)

    def execute(self, plan: Plan, bindings: Bindings) -> None:
        arr, n = bindings._as_c()
        _check(self._lib.infr_hip_execute(self._h, plan._h, arr, n))

    def sync(self) -> None:
        _check(self._lib.infr_hip_sync(self._h))

    # ---- taps
    def prof_enable(self, on: bool = True) -> None:
        _check(self._lib.infr_hip_prof_enable(self._h, int(on)))

    def probe_grouped_loads_only(self, on: bool = True) -> None:
        """Measurement only: the batched path's grouped GEMMs move their data but skip unpacking and matrix work."""
        _check(self._lib.infr_hip_probe_grouped_loads_only(self._h, int(on)))

    def prof_read(self) -> dict:
        n = C.c_uint32()
        _check(self._lib.infr_hip_prof_read(self._h, None, 0, C.byref(n)))
        arr = (_ProfEntry * max(n.value, 1))()
        _check(self._lib.infr_hip_prof_read(self._h, arr, n.value, C.byref(n)))
        return {arr[i].kernel.decode(): {"launches": arr[i].launches, "total_ms": arr[i].total_ms,
                                          "min_ms": arr[i].min_ms, "max_ms": arr[i].max_ms}
                for i in range(n.value)}

    def moe_routing(self, plan: Plan, op_index: int = 0) -> dict:
        m = plan.graph.ops[op_index].u.moe_ffn
        rows = plan.graph.desc(m.x).numel() // m.ne
        ids = np.zeros((rows, m.n_used), np.int32)
        w = np.zeros((rows, m.n_used), np.float32)
        logits = np.zeros((rows, m.n_expert), np.float32)
        probs = np.zeros((rows, m.n_expert), np.float32)
        _check(self._lib.infr_hip_plan_moe_routing(self._h, plan._h, op_index, ids.ctypes.data_as(_V),
                                                   w.ctypes.data_as(_V), logits.ctypes.data_as(_V),
                                                   probs.ctypes.data_as(_V)))
        return {"idx": ids, "w": w, "logits": logits, "probs": probs}

    def moe_bucketing(self, plan: Plan, op_index: int = 0) -> dict:
        """Bucketing of the last execution of a MoeFfn op that took the batched path
        (crates/infr-cpu/src/lib.rs:3874-3908): `offsets` [n_expert+1], `pair_row` / `pair_rank`
        [rows*n_used] in bucket order, `slot_pair` [rows, n_used] bucket position of each pair."""
        m = plan.graph.ops[op_index].u.moe_ffn
        rows = plan.graph.desc(m.x).numel() // m.ne
        offsets = np.zeros(m.n_expert + 1, np.int32)
        src = np.zeros(rows * m.n_used, np.int32)
        slot = np.zeros((rows, m.n_used), np.int32)
        _check(self._lib.infr_hip_plan_moe_bucketing(self._h, plan._h, op_index, offsets.ctypes.data_as(_V),
                                                     src.ctypes.data_as(_V), slot.ctypes.data_as(_V)))
        return {"offsets": offsets, "pair_row": src // m.n_used, "pair_rank": src % m.n_used, "slot_pair": slot}

    def moe_ffn_static(self, *, x: Buffer, router: Buffer, gate_exps: Buffer, up_exps: Buffer, down_exps: Buffer,
                       dst: Buffer, gate_dtype: DType, down_dtype: DType, rows: int, ne: int, n_expert: int, n_used: int,
                       n_ff_exp: int, up_dtype: Optional[DType] = None) -> None:
        """infr_hip_moe_ffn_static: one plain Op::MoeFfn on the caller's buffers; allocates nothing."""
        a = _MoeFfnStaticArgs(x=x._h, router=router._h, gate_exps=gate_exps._h, up_exps=up_exps._h, down_exps=down_exps._h,
                              dst=dst._h, gate_dtype=int(gate_dtype), up_dtype=int(gate_dtype if up_dtype is None else up_dtype),
                              down_dtype=int(down_dtype), rows=rows, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff_exp)
        _check(self._lib.infr_hip_moe_ffn_static(self._h, C.byref(a)))

    def late_experts(self) -> int:
        """infr_hip_probe_late_experts: experts the single-launch kernel's guess missed and loaded late, so far."""
        n = C.c_uint64()
        _check(self._lib.infr_hip_probe_late_experts(self._h, C.byref(n)))
        return int(n.value)

    def alloc_calls(self) -> int:
        """infr_hip_probe_alloc_calls: allocating runtime calls this library has made in this process so far."""
        n = C.c_uint64()
        _check(self._lib.infr_hip_probe_alloc_calls(C.byref(n)))
        return int(n.value)

    def probe_dependent_reads(self, pool: Buffer, stage_bytes: Sequence[int], iters: int = 200) -> dict:
        """infr_hip_probe_dependent_reads: microseconds of each stage alone and of the whole chain."""
        n = len(stage_bytes)
        sizes = (C.c_uint64 * n)(*[int(b) for b in stage_bytes])
        per = (C.c_double * n)()
        chain = C.c_double()
        _check(self._lib.infr_hip_probe_dependent_reads(self._h, pool._h, sizes, n, iters, per, C.byref(chain)))
        return {"stage_us": [float(v) for v in per], "chain_us": float(chain.value)}

    def dequant(self, src: Buffer, dtype: DType, numel: int) -> np.ndarray:
        dst = self.alloc(numel * 4, BufferUsage.Readback)
        try:
            _check(self._lib.infr_hip_dequant(self._h, src._h, int(dtype), numel, dst._h))
            return self.download(dst, numel * 4, np.float32)
        finally:
            dst.free()


def run_graph(be: Backend, g: Graph, bound: Sequence, out: int, out_n: int, keep: Optional[list] = None) -> np.ndarray:
    """The reference's one-op harness (crates/infr-testkit/src/lib.rs:170-201): compile,
    alloc(max(len,4)) + upload every bound id, alloc the output, bind, execute, download."""
    plan = be.compile(g)
    bufs = []
    b = Bindings()
    for tid, data in bound:
        raw = Backend._bytes(data)
        kind = g.tensors[tid][1]
        buf = be.alloc(max(raw.size, 4), BufferUsage.Weights if kind == TensorKind.Weight else BufferUsage.Activations)
        be.upload(buf, raw)
        bufs.append(buf)
        b.bind(tid, buf)
    ob = b.get(out)   # an output the caller pre-filled (an op that accumulates, or runs in place)
    own = ob is None
    if own:
        ob = be.alloc(out_n * 4, BufferUsage.Readback)
        b.bind(out, ob)
    be.execute(plan, b)
    res = be.download(ob, out_n * 4, np.float32).copy()
    if keep is not None:
        keep.extend([plan, b, bufs, ob])
    else:
        for buf in bufs:
            buf.free()
        if own:
            ob.free()
        plan.free()
    return res
