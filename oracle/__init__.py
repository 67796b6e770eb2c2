"""CPU oracle for the routed-expert MoE FFN path (test infrastructure only).

ctypes view of ``libinfr_oracle.so`` (built by ``oracle/Makefile`` from ``infr_oracle.c``).
Only tests, the smoke check and the benchmark's CPU-baseline leg import this package; the
HIP backend in ``moe4all_amd`` never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libinfr_oracle.so")

# infr_core::DType ordinals (crates/infr-core/src/tensor.rs:7-57)
F32, F16, BF16, I32, U32 = 0, 1, 2, 3, 4
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K = 5, 6, 7, 8, 9, 10, 11, 12, 13, 14
IQ1_S, IQ1_M, IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S = 15, 16, 17, 18, 19, 20, 21
IQ4_NL, IQ4_XS, TQ1_0, TQ2_0, Q2_0, MXFP4, NVFP4 = 22, 23, 24, 25, 27, 28, 29
ACT_SILU, ACT_GELU, ACT_SIGMOID = 0, 1, 2
GATE_SOFTMAX, GATE_SIGMOID, GATE_SQRT_SOFTPLUS = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile the oracle with the committed Makefile (gcc only, no GPU code)."""
    src = os.path.join(_HERE, "infr_oracle.c")
    hdr = os.path.join(_HERE, "infr_oracle.h")
    grids = os.path.join(_HERE, "..", "moe4all_amd", "csrc", "iquant_grids.h")
    stale = (not os.path.exists(_LIB_PATH)
             or os.path.getmtime(_LIB_PATH) < max(os.path.getmtime(f) for f in (src, hdr, grids)))
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libinfr_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _MoeArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("router_x", C.c_void_p), ("rows", C.c_int),
        ("router", C.c_void_p), ("router_dtype", C.c_int), ("router_bytes", C.c_size_t),
        ("gate", C.c_void_p), ("gate_dtype", C.c_int), ("gate_bytes", C.c_size_t),
        ("up", C.c_void_p), ("up_dtype", C.c_int), ("up_bytes", C.c_size_t),
        ("down", C.c_void_p), ("down_dtype", C.c_int), ("down_bytes", C.c_size_t),
        ("down_scale", C.c_void_p),
        ("fused_gate_up", C.c_int),
        ("ne", C.c_int), ("n_expert", C.c_int), ("n_used", C.c_int), ("n_ff_exp", C.c_int),
        ("scale", C.c_float),
        ("act", C.c_int),
        ("has_swiglu_clamp", C.c_int), ("swiglu_clamp", C.c_float),
        ("gating", C.c_int), ("norm_w", C.c_int), ("weight_before", C.c_int),
        ("exp_probs_b", C.c_void_p),
        ("n_expert_groups", C.c_int), ("n_expert_groups_used", C.c_int),
        ("expert_ids", C.c_void_p),
        ("n_threads", C.c_int),
        ("dst", C.c_void_p),
        ("logits_out", C.c_void_p), ("probs_out", C.c_void_p),
        ("idx_out", C.c_void_p), ("w_out", C.c_void_p),
        ("n_buckets_out", C.c_void_p), ("bucket_expert_out", C.c_void_p),
        ("bucket_p0_out", C.c_void_p), ("bucket_count_out", C.c_void_p),
        ("pair_row_out", C.c_void_p), ("slot_pair_out", C.c_void_p),
        ("production", C.c_int),
    ]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        L.orc_block_geometry.argtypes = [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.orc_bytes_for.argtypes = [C.c_int, C.c_int64]
        L.orc_bytes_for.restype = C.c_int64
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_k4.argtypes = [C.c_int, C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
        L.orc_k4.restype = None
        L.orc_dequant.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
        L.orc_dequant.restype = C.c_int64
        L.orc_dot.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.orc_dot.restype = C.c_float
        L.orc_act.argtypes = [C.c_int, C.c_float]
        L.orc_act.restype = C.c_float
        L.orc_gated_act.argtypes = [C.c_int, C.c_int, C.c_float, C.c_float, C.c_float]
        L.orc_gated_act.restype = C.c_float
        L.orc_route_row.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float,
                                    C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                    C.c_void_p, C.c_void_p]
        L.orc_moe_ffn.argtypes = [C.POINTER(_MoeArgs)]
        L.orc_linear.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_int64, C.c_int,
                                 C.c_int, C.c_int, C.c_int64, C.c_int, C.c_void_p]
        L.orc_gated_act_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                         C.c_float, C.c_void_p]
        L.orc_gated_act_rows.restype = None
        L.orc_add.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
        L.orc_add.restype = None
        L.orc_moe_shared_expert_add.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                                C.c_void_p]
        L.orc_moe_shared_expert_add.restype = None
        L.orc_rms_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p]
        L.orc_rms_norm.restype = None
        L.orc_quantize_q8.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_quantize_q8.restype = None
        L.orc_vec_dot_q8.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.orc_vec_dot_q8.restype = C.c_float
        L.orc_hw_threads.restype = C.c_int
        L.orc_grid_entry.argtypes = [C.c_int, C.c_int, C.c_void_p]
        L.orc_ksigns.argtypes = [C.c_int]
        L.orc_ksigns.restype = C.c_uint8
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint8).reshape(-1)


def block_geometry(dtype: int):
    e, b = C.c_int(), C.c_int()
    if lib().orc_block_geometry(dtype, C.byref(e), C.byref(b)) != 0:
        raise ValueError(f"oracle: unsupported dtype {dtype}")
    return e.value, b.value


def bytes_for(dtype: int, numel: int) -> int:
    n = lib().orc_bytes_for(dtype, numel)
    if n < 0:
        raise ValueError(f"oracle: {numel} elements is not a whole number of dtype-{dtype} blocks")
    return n


def f16_to_f32(h: int) -> float:
    return lib().orc_f16_to_f32(h)


def k4(j: int, scales) -> tuple:
    s = _u8(scales)
    sc, m = C.c_uint32(), C.c_uint32()
    lib().orc_k4(j, _p(s), C.byref(sc), C.byref(m))
    return sc.value, m.value


GRID_NAMES = ("iq2xxs", "iq2xs", "iq2s", "iq3xxs", "iq3s", "iq1s")
GRID_SIZES = (256, 512, 1024, 256, 512, 2048)


def grid(which: int) -> np.ndarray:
    """Lattice codebook `which` (index into GRID_NAMES) as [entries, 8 or 4] int8, one signed byte per element as in
    crates/infr-core/src/iquant_grids.rs."""
    buf = np.zeros(8, np.int8)
    rows = []
    for e in range(GRID_SIZES[which]):
        n = lib().orc_grid_entry(which, e, _p(buf))
        rows.append(buf[:n].copy())
    assert lib().orc_grid_entry(which, GRID_SIZES[which], _p(buf)) == -1
    return np.stack(rows)


def ksigns() -> np.ndarray:
    return np.array([lib().orc_ksigns(i) for i in range(128)], np.uint8)


def dequant(dtype: int, data) -> np.ndarray:
    b = _u8(data)
    be, bb = block_geometry(dtype)
    out = np.empty(b.size // bb * be, dtype=np.float32)
    n = lib().orc_dequant(dtype, _p(b), b.size, _p(out))
    if n != out.size:
        raise ValueError("oracle: dequant failed")
    return out


def dot(a, b) -> np.float32:
    a, b = _f32(a), _f32(b)
    assert a.size == b.size
    return np.float32(lib().orc_dot(_p(a), _p(b), a.size))


def act(kind: int, g: float) -> np.float32:
    return np.float32(lib().orc_act(kind, g))


def gated_act(kind: int, gate: float, up: float, clamp=None) -> np.float32:
    return np.float32(lib().orc_gated_act(kind, clamp is not None, clamp or 0.0, gate, up))


def route_row(logits, n_used, gating=GATE_SOFTMAX, norm_w=True, scale=1.0, exp_probs_b=None,
              n_groups=0, n_groups_used=0, hash_ids=None):
    lg = _f32(logits)
    n = lg.size
    probs = np.empty(n, np.float32)
    idx = np.empty(n_used, np.int32)
    w = np.empty(n_used, np.float32)
    b = None if exp_probs_b is None else _f32(exp_probs_b)
    h = None if hash_ids is None else _f32(hash_ids)
    rc = lib().orc_route_row(_p(lg), n, n_used, gating, int(norm_w), scale, _p(b), n_groups,
                             n_groups_used, _p(h), _p(probs), _p(idx), _p(w))
    if rc != 0:
        raise ValueError("oracle: routing undefined (NaN or id out of range)")
    return probs, idx, w


def moe_ffn(x, router, gate, up, down, *, ne, n_expert, n_used, n_ff_exp,
            router_dtype=F32, gate_dtype=F32, up_dtype=None, down_dtype=None, router_x=None,
            scale=1.0, act=ACT_SILU, gating=GATE_SOFTMAX, norm_w=True, weight_before=False,
            fused_gate_up=False, down_scale=None, swiglu_clamp=None, exp_probs_b=None,
            n_expert_groups=0, n_expert_groups_used=0, expert_ids=None, n_threads=0, production=False):
    """Run Op::MoeFfn in reference numerics.  Weights are raw GGUF bytes (any array; viewed as u8).

    production=True: the CPU backend's batch numerics (int8 activations for Q4_K / Q6_K / Q8_0 banks from two
    rows on) - for the timed CPU baseline only, not a parity reference.

    Returns a dict with dst [rows, ne] plus the routing/bucketing captures.
    """
    x = _f32(x).reshape(-1, ne)
    rows = x.shape[0]
    rx = x if router_x is None else _f32(router_x).reshape(-1, ne)
    rb, gb, db = _u8(router), _u8(gate), _u8(down)
    ub = None if fused_gate_up else _u8(up)
    up_dtype = gate_dtype if up_dtype is None else up_dtype
    down_dtype = gate_dtype if down_dtype is None else down_dtype
    ds = None if down_scale is None else _f32(down_scale)
    eb = None if exp_probs_b is None else _f32(exp_probs_b)
    ids = None if expert_ids is None else _f32(expert_ids)
    out = {
        "dst": np.zeros((rows, ne), np.float32),
        "logits": np.zeros((rows, n_expert), np.float32),
        "probs": np.zeros((rows, n_expert), np.float32),
        "idx": np.zeros((rows, n_used), np.int32),
        "w": np.zeros((rows, n_used), np.float32),
        "n_buckets": np.zeros(1, np.int32),
        "bucket_expert": np.zeros(n_expert, np.int32),
        "bucket_p0": np.zeros(n_expert, np.int32),
        "bucket_count": np.zeros(n_expert, np.int32),
        "pair_row": np.zeros(max(rows * n_used, 1), np.int32),
        "slot_pair": np.zeros((max(rows, 1), n_used), np.int32),
    }
    a = _MoeArgs(
        x=_p(x), router_x=_p(rx), rows=rows,
        router=_p(rb), router_dtype=router_dtype, router_bytes=rb.size,
        gate=_p(gb), gate_dtype=gate_dtype, gate_bytes=gb.size,
        up=_p(ub), up_dtype=up_dtype, up_bytes=0 if ub is None else ub.size,
        down=_p(db), down_dtype=down_dtype, down_bytes=db.size,
        down_scale=_p(ds), fused_gate_up=int(fused_gate_up),
        ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=n_ff_exp, scale=scale, act=act,
        has_swiglu_clamp=int(swiglu_clamp is not None), swiglu_clamp=swiglu_clamp or 0.0,
        gating=gating, norm_w=int(norm_w), weight_before=int(weight_before),
        exp_probs_b=_p(eb), n_expert_groups=n_expert_groups,
        n_expert_groups_used=n_expert_groups_used, expert_ids=_p(ids), n_threads=n_threads,
        dst=_p(out["dst"]), logits_out=_p(out["logits"]), probs_out=_p(out["probs"]),
        idx_out=_p(out["idx"]), w_out=_p(out["w"]), n_buckets_out=_p(out["n_buckets"]),
        bucket_expert_out=_p(out["bucket_expert"]), bucket_p0_out=_p(out["bucket_p0"]),
        bucket_count_out=_p(out["bucket_count"]), pair_row_out=_p(out["pair_row"]),
        slot_pair_out=_p(out["slot_pair"]), production=int(production),
    )
    rc = lib().orc_moe_ffn(C.byref(a))
    if rc != 0:
        raise ValueError(f"oracle: orc_moe_ffn failed ({rc})")
    nb = int(out["n_buckets"][0])
    out["n_buckets"] = nb
    for k in ("bucket_expert", "bucket_p0", "bucket_count"):
        out[k] = out[k][:nb]
    out["pair_row"] = out["pair_row"][: rows * n_used]
    out["slot_pair"] = out["slot_pair"][:rows]
    return out


def linear(x, w, w_dtype, in_f, out_f, w_off=0, w_numel=None, n_threads=0) -> np.ndarray:
    x = _f32(x).reshape(-1, in_f)
    wb = _u8(w)
    if w_numel is None:
        be, bb = block_geometry(w_dtype)
        w_numel = wb.size // bb * be
    dst = np.empty((x.shape[0], out_f), np.float32)
    rc = lib().orc_linear(_p(x), _p(wb), w_dtype, wb.size, w_numel, x.shape[0], in_f, out_f, w_off,
                          n_threads, _p(dst))
    if rc != 0:
        raise ValueError(f"oracle: orc_linear failed ({rc})")
    return dst


def gated_act_rows(gate, up, act=ACT_SILU, clamp=None) -> np.ndarray:
    g, u = _f32(gate), _f32(up)
    rows, nff = g.reshape(-1, g.shape[-1]).shape
    dst = np.empty_like(g)
    lib().orc_gated_act_rows(_p(g), _p(u), rows, nff, act, clamp is not None, clamp or 0.0, _p(dst))
    return dst


def add(a, b) -> np.ndarray:
    a, b = _f32(a), _f32(b)
    dst = np.empty_like(a)
    lib().orc_add(_p(a), _p(b), a.size, _p(dst))
    return dst


def moe_shared_expert_add(moe, shexp, gate) -> np.ndarray:
    m, s, g = _f32(moe), _f32(shexp), _f32(gate).reshape(-1)
    rows = g.size
    dst = np.empty_like(m)
    lib().orc_moe_shared_expert_add(_p(m), _p(s), _p(g), rows, m.size // rows, _p(dst))
    return dst


def rms_norm(x, weight, eps, add_to=None) -> np.ndarray:
    """Op::RmsNorm; with add_to, Op::RmsNormAdd applied to a copy of add_to."""
    x, w = _f32(x), _f32(weight).reshape(-1)
    dim = w.size
    rows = x.size // dim
    dst = np.empty_like(x) if add_to is None else _f32(add_to).copy()
    lib().orc_rms_norm(_p(x), _p(w), rows, dim, eps, add_to is not None, _p(dst))
    return dst


def quantize_q8(x):
    """quantize_q8 of one row (length a multiple of 256): (int8 codes, f32 scale per 256, i32 sums per 32)."""
    x = _f32(x).reshape(-1)
    nb = x.size // 256
    qs, d, bs = np.zeros(nb * 256, np.int8), np.zeros(nb, np.float32), np.zeros(nb * 8, np.int32)
    lib().orc_quantize_q8(_p(x), x.size, _p(qs), _p(d), _p(bs))
    return qs, d, bs


def vec_dot_q8(dtype, row, q8) -> np.float32:
    """One quantised weight row against one quantize_q8 activation row (the int8 production dot)."""
    qs, d, bs = q8
    r = _u8(row)
    return np.float32(lib().orc_vec_dot_q8(dtype, _p(r), _p(qs), _p(d), _p(bs), qs.size))


def hw_threads() -> int:
    return lib().orc_hw_threads()
