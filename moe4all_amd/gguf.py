"""GGUF weight source: host-side mirror of the reference's `infr_gguf::Gguf`
(crates/infr-gguf/src/lib.rs:82-110) over the C ABI in include/infr_gguf.h, plus the slice of
the model loader that the routed-expert FFN path needs: the per-layer tensor names and the
hyperparameter keys of a qwen3moe-style model (crates/infr-llama/src/seam/runner.rs:2519-2565,
crates/infr-llama/src/config.rs:1155-1283).

Nothing is decoded on the host.  Tensors are uploaded as the raw block bytes of the file.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np

from . import backend as B
from .backend import Backend, Bindings, Buffer, DType, Graph, TensorDesc

_V = C.c_void_p


class LoaderError(B.BackendError):
    """infr_core::Error::Loader / ::Io (crates/infr-core/src/error.rs:11-31)."""


class _Tensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype", C.c_int32), ("ggml_type", C.c_uint32), ("rank", C.c_uint32),
                ("shape", C.c_uint64 * 4), ("numel", C.c_uint64), ("offset", C.c_uint64), ("nbytes", C.c_uint64)]


_SIGS = {
    "infr_gguf_open": ([C.c_char_p, C.POINTER(_V)], C.c_int),
    "infr_gguf_close": ([_V], None),
    "infr_gguf_last_error": ([], C.c_char_p),
    "infr_gguf_tensor_count": ([_V], C.c_uint64),
    "infr_gguf_tensor_at": ([_V, C.c_uint64, C.POINTER(_Tensor)], C.c_int),
    "infr_gguf_tensor_find": ([_V, C.c_char_p, C.POINTER(_Tensor)], C.c_int),
    "infr_gguf_tensor_bytes": ([_V, C.c_char_p, C.POINTER(_V), C.POINTER(C.c_uint64)], C.c_int),
    "infr_gguf_shard_count": ([_V], C.c_uint32),
    "infr_gguf_meta_u64": ([_V, C.c_char_p, C.POINTER(C.c_uint64)], C.c_int),
    "infr_gguf_meta_i64": ([_V, C.c_char_p, C.POINTER(C.c_int64)], C.c_int),
    "infr_gguf_meta_f64": ([_V, C.c_char_p, C.POINTER(C.c_double)], C.c_int),
    "infr_gguf_meta_bool": ([_V, C.c_char_p, C.POINTER(C.c_int32)], C.c_int),
    "infr_gguf_meta_str": ([_V, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(C.c_uint64)], C.c_int),
    "infr_gguf_meta_array_len": ([_V, C.c_char_p, C.POINTER(C.c_uint64)], C.c_int),
    "infr_gguf_block_layout": ([C.c_int32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)], C.c_int),
    "infr_gguf_bind_weight": ([_V, C.c_char_p, _V, C.POINTER(_V), C.POINTER(C.c_int32), C.POINTER(C.c_uint64)], C.c_int),
}
_bound = False


def _lib() -> C.CDLL:
    global _bound
    lib = B.load_library()
    if not _bound:
        for name, (args, res) in _SIGS.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = res
        # the string pointer of meta_str is not NUL-terminated: take it as a raw address
        lib.infr_gguf_meta_str.argtypes = [_V, C.c_char_p, C.POINTER(_V), C.POINTER(C.c_uint64)]
        _bound = True
    return lib


def _check(st: int) -> None:
    if st == 0:
        return
    msg = _lib().infr_gguf_last_error().decode("utf-8", "replace")
    if st == 2:
        raise B.Unsupported(msg)
    if st in (5, 6):
        raise LoaderError(msg)
    raise B.BackendError(msg)


@dataclass(frozen=True)
class TensorInfo:
    """infr_core::loader::TensorInfo: shape in file order (shape[0] varies fastest)."""
    name: str
    dtype: int          # infr_dtype ordinal
    ggml_type: int
    shape: tuple
    numel: int
    offset: int
    nbytes: int


def block_layout(dtype: int) -> tuple:
    e, b = C.c_uint32(), C.c_uint32()
    _check(_lib().infr_gguf_block_layout(int(dtype), C.byref(e), C.byref(b)))
    return e.value, b.value


class Gguf:
    """An opened model: one file or a whole gguf-split shard set (Gguf::open, lib.rs:484-493)."""

    def __init__(self, path: str):
        self._h = None
        h = _V()
        _check(_lib().infr_gguf_open(str(path).encode(), C.byref(h)))
        self._h = h.value

    def close(self) -> None:
        if self._h:
            _lib().infr_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _info(t: _Tensor) -> TensorInfo:
        return TensorInfo(t.name.decode(), t.dtype, t.ggml_type, tuple(t.shape[d] for d in range(t.rank)), t.numel,
                          t.offset, t.nbytes)

    @property
    def n_shards(self) -> int:
        return _lib().infr_gguf_shard_count(self._h)

    def tensors(self) -> List[TensorInfo]:
        out = []
        t = _Tensor()
        for i in range(_lib().infr_gguf_tensor_count(self._h)):
            _check(_lib().infr_gguf_tensor_at(self._h, i, C.byref(t)))
            out.append(self._info(t))
        return out

    def find(self, name: str) -> TensorInfo:
        t = _Tensor()
        _check(_lib().infr_gguf_tensor_find(self._h, name.encode(), C.byref(t)))
        return self._info(t)

    def has(self, name: str) -> bool:
        t = _Tensor()
        return _lib().infr_gguf_tensor_find(self._h, name.encode(), C.byref(t)) == 0

    def tensor_bytes(self, name: str) -> np.ndarray:
        """A copy of the tensor's raw bytes (the mapping itself stays private to the library)."""
        p, n = _V(), C.c_uint64()
        _check(_lib().infr_gguf_tensor_bytes(self._h, name.encode(), C.byref(p), C.byref(n)))
        if n.value == 0:
            return np.zeros(0, np.uint8)
        return np.ctypeslib.as_array((C.c_uint8 * n.value).from_address(p.value)).copy()

    # ---- metadata
    def meta_u64(self, key: str) -> Optional[int]:
        v = C.c_uint64()
        return v.value if _lib().infr_gguf_meta_u64(self._h, key.encode(), C.byref(v)) == 0 else None

    def meta_i64(self, key: str) -> Optional[int]:
        v = C.c_int64()
        return v.value if _lib().infr_gguf_meta_i64(self._h, key.encode(), C.byref(v)) == 0 else None

    def meta_f64(self, key: str) -> Optional[float]:
        v = C.c_double()
        return v.value if _lib().infr_gguf_meta_f64(self._h, key.encode(), C.byref(v)) == 0 else None

    def meta_bool(self, key: str) -> Optional[bool]:
        v = C.c_int32()
        return bool(v.value) if _lib().infr_gguf_meta_bool(self._h, key.encode(), C.byref(v)) == 0 else None

    def meta_str(self, key: str) -> Optional[str]:
        p, n = _V(), C.c_uint64()
        if _lib().infr_gguf_meta_str(self._h, key.encode(), C.byref(p), C.byref(n)) != 0:
            return None
        return C.string_at(p.value, n.value).decode("utf-8", "replace") if n.value else ""

    def meta_array_len(self, key: str) -> Optional[int]:
        v = C.c_uint64()
        return v.value if _lib().infr_gguf_meta_array_len(self._h, key.encode(), C.byref(v)) == 0 else None

    # ---- device
    def bind_weight(self, be: Backend, name: str):
        """alloc_uninit(Weights) + upload of the raw bytes (crates/infr-llama/src/seam/mod.rs:597-608).
        Returns (Buffer, dtype ordinal, numel)."""
        h, dt, n = _V(), C.c_int32(), C.c_uint64()
        _check(_lib().infr_gguf_bind_weight(self._h, name.encode(), be._h, C.byref(h), C.byref(dt), C.byref(n)))
        return Buffer(be, h.value), dt.value, n.value


@dataclass
class MoeHyper:
    """The MoeConfig fields the FFN sublayer needs (crates/infr-llama/src/config.rs:1223-1283)."""
    arch: str
    n_layer: int
    ne: int
    n_expert: int
    n_used: int
    n_ff_exp: int
    eps: float
    shexp_ff: int = 0   # {arch}.expert_shared_feed_forward_length (config.rs:1189, :1508); 0 = no shared expert


def moe_hyper(g: Gguf) -> MoeHyper:
    arch = g.meta_str("general.architecture")
    if arch is None:
        raise LoaderError("GGUF: no general.architecture")

    def need(key):
        v = g.meta_u64(f"{arch}.{key}")
        if v is None:
            raise LoaderError(f"GGUF: missing {arch}.{key}")
        return v

    eps = g.meta_f64(f"{arch}.attention.layer_norm_rms_epsilon")
    return MoeHyper(arch, need("block_count"), need("embedding_length"), need("expert_count"), need("expert_used_count"),
                    need("expert_feed_forward_length"), 1e-6 if eps is None else eps,
                    g.meta_u64(f"{arch}.expert_shared_feed_forward_length") or 0)


class MoeFfnLayer:
    """One layer's FFN sublayer built from a GGUF file:  y = x + MoeFfn(rmsnorm(x) * ffn_norm).

    Tensor names (runner.rs:2519-2565): blk.{l}.ffn_norm.weight, ffn_gate_inp.weight (router),
    ffn_gate_exps / ffn_up_exps / ffn_down_exps.weight.  qwen3moe parameterisation
    (config.rs:1270-1272): softmax gating, renormalised weights, scale 1.  GGUF lists a tensor's
    fastest axis first, so ffn_gate_exps [ne, n_ff, n_expert] is the row-major [n_expert, n_ff, ne]
    bank Op::MoeFfn reads.

    With a shared expert (`expert_shared_feed_forward_length` > 0; runner.rs:2586-2596, :8089-8174) the
    layer also binds ffn_{gate,up,down}_shexp.weight and emits Linear, Linear, GatedAct, Linear on the same
    normalised input, combined by Op::MoeSharedExpertAdd when the file carries ffn_gate_inp_shexp.weight
    (a per-token sigmoid gate, qwen35moe) and by a plain Op::Add otherwise (llama4)."""

    ROLES = {"norm": "ffn_norm.weight", "router": "ffn_gate_inp.weight", "gate": "ffn_gate_exps.weight",
             "up": "ffn_up_exps.weight", "down": "ffn_down_exps.weight"}
    SHARED = {"sh_gate": "ffn_gate_shexp.weight", "sh_up": "ffn_up_shexp.weight", "sh_down": "ffn_down_shexp.weight"}

    def __init__(self, be: Backend, g: Gguf, layer: int, rows: int, hyper: Optional[MoeHyper] = None):
        hp = hyper or moe_hyper(g)
        self.be, self.hyper, self.rows, self.layer = be, hp, rows, layer
        self.buffers: Dict[str, Buffer] = {}
        infos = {}
        roles = dict(self.ROLES)
        self.gated = False
        if hp.shexp_ff:
            roles.update(self.SHARED)
            self.gated = g.has(f"blk.{layer}.ffn_gate_inp_shexp.weight")
            if self.gated:
                roles["sh_gate_inp"] = "ffn_gate_inp_shexp.weight"
        for role, suffix in roles.items():
            name = f"blk.{layer}.{suffix}"
            info = g.find(name)
            infos[role] = info
            self.buffers[role], _, _ = g.bind_weight(be, name)
        want = {"norm": (hp.ne,), "router": (hp.ne, hp.n_expert), "gate": (hp.ne, hp.n_ff_exp, hp.n_expert),
                "up": (hp.ne, hp.n_ff_exp, hp.n_expert), "down": (hp.n_ff_exp, hp.ne, hp.n_expert)}
        if hp.shexp_ff:
            want.update({"sh_gate": (hp.ne, hp.shexp_ff), "sh_up": (hp.ne, hp.shexp_ff), "sh_down": (hp.shexp_ff, hp.ne)})
            if self.gated and infos["sh_gate_inp"].numel != hp.ne:
                raise LoaderError(f"GGUF: blk.{layer}.ffn_gate_inp_shexp.weight has {infos['sh_gate_inp'].numel} elements, "
                                  f"the model's hyperparameters need {hp.ne}")
        for role, shape in want.items():
            if infos[role].shape != shape:
                raise LoaderError(f"GGUF: blk.{layer}.{roles[role]} has shape {infos[role].shape}, the model's "
                                  f"hyperparameters need {shape}")
        gr = Graph()
        self.x = gr.input(TensorDesc([rows, hp.ne], DType.F32))
        self.t = {
            "norm": gr.weight(TensorDesc([hp.ne], DType(infos["norm"].dtype))),
            "router": gr.weight(TensorDesc([hp.n_expert, hp.ne], DType(infos["router"].dtype))),
            "gate": gr.weight(TensorDesc([hp.n_expert, hp.n_ff_exp, hp.ne], DType(infos["gate"].dtype))),
            "up": gr.weight(TensorDesc([hp.n_expert, hp.n_ff_exp, hp.ne], DType(infos["up"].dtype))),
            "down": gr.weight(TensorDesc([hp.n_expert, hp.ne, hp.n_ff_exp], DType(infos["down"].dtype))),
        }
        self.xn = gr.internal(TensorDesc([rows, hp.ne], DType.F32))
        sub = gr.internal(TensorDesc([rows, hp.ne], DType.F32))
        self.y = gr.output(TensorDesc([rows, hp.ne], DType.F32))
        gr.rms_norm(x=self.x, weight=self.t["norm"], dst=self.xn, rows=rows, dim=hp.ne, eps=hp.eps)
        moe_dst = gr.internal(TensorDesc([rows, hp.ne], DType.F32)) if hp.shexp_ff else sub
        gr.moe_ffn(x=self.xn, router=self.t["router"], gate_exps=self.t["gate"], up_exps=self.t["up"],
                   down_exps=self.t["down"], dst=moe_dst, ne=hp.ne, n_expert=hp.n_expert, n_used=hp.n_used,
                   n_ff_exp=hp.n_ff_exp)
        if hp.shexp_ff:
            sff = hp.shexp_ff
            self.t["sh_gate"] = gr.weight(TensorDesc([sff, hp.ne], DType(infos["sh_gate"].dtype)))
            self.t["sh_up"] = gr.weight(TensorDesc([sff, hp.ne], DType(infos["sh_up"].dtype)))
            self.t["sh_down"] = gr.weight(TensorDesc([hp.ne, sff], DType(infos["sh_down"].dtype)))
            gbuf, ubuf = gr.internal(TensorDesc([rows, sff], DType.F32)), gr.internal(TensorDesc([rows, sff], DType.F32))
            act, d_out = gr.internal(TensorDesc([rows, sff], DType.F32)), gr.internal(TensorDesc([rows, hp.ne], DType.F32))
            if self.gated:   # the gate logit comes first, as the reference emits it (runner.rs:8104-8114)
                self.t["sh_gate_inp"] = gr.weight(TensorDesc([1, hp.ne], DType(infos["sh_gate_inp"].dtype)))
                gate_logit = gr.internal(TensorDesc([rows, 1], DType.F32))
                gr.linear(x=self.xn, weight=self.t["sh_gate_inp"], dst=gate_logit, m=rows, in_f=hp.ne, out_f=1)
            gr.linear(x=self.xn, weight=self.t["sh_gate"], dst=gbuf, m=rows, in_f=hp.ne, out_f=sff)
            gr.linear(x=self.xn, weight=self.t["sh_up"], dst=ubuf, m=rows, in_f=hp.ne, out_f=sff)
            gr.gated_act(gate=gbuf, up=ubuf, dst=act, rows=rows, nff=sff)
            gr.linear(x=act, weight=self.t["sh_down"], dst=d_out, m=rows, in_f=sff, out_f=hp.ne)
            if self.gated:
                gr.moe_shared_expert_add(moe=moe_dst, shexp=d_out, gate=gate_logit, dst=sub, rows=rows, n=hp.ne)
            else:
                gr.add(a=moe_dst, b=d_out, dst=sub, n=rows * hp.ne)
        gr.add(a=self.x, b=sub, dst=self.y, n=rows * hp.ne)
        self.graph = gr
        self.moe_op = 1
        self.plan = be.compile(gr)

    def forward(self, x: np.ndarray) -> np.ndarray:
        hp = self.hyper
        x = np.ascontiguousarray(x, np.float32).reshape(self.rows, hp.ne)
        xb, yb = self.be.buffer_from(x, B.BufferUsage.Activations), self.be.alloc(self.rows * hp.ne * 4)
        b = Bindings()
        b.bind(self.x, xb).bind(self.y, yb)
        for role, tid in self.t.items():
            b.bind(tid, self.buffers[role])
        try:
            self.be.execute(self.plan, b)
            return self.be.download(yb, self.rows * hp.ne * 4, np.float32).reshape(self.rows, hp.ne).copy()
        finally:
            xb.free()
            yb.free()

    def free(self) -> None:
        self.plan.free()
        for buf in self.buffers.values():
            buf.free()
        self.buffers = {}
