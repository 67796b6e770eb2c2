"""Seeded synthetic workloads of the MoE FFN benchmark configurations.

Weights are N(0, 0.02) streams quantised with ggml-compatible quantisers (``include/infr_synth.h``);
the same bytes come out of the host generator and the device generator, so small cases can be
built on the CPU, large ones directly in HBM.  Every tensor of a layer has its own stream:
``stream_seed(seed0, layer, role)``.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import numpy as np

from .backend import Backend, Buffer, BufferUsage, DType, _check, bytes_for, load_library

_V = C.c_void_p
_bound = False

ROLE_ROUTER, ROLE_GATE, ROLE_UP, ROLE_DOWN, ROLE_X = 1, 2, 3, 4, 5
ROLE_SH_GATE, ROLE_SH_UP, ROLE_SH_DOWN, ROLE_SH_GATE_INP = 6, 7, 8, 9


def _lib():
    global _bound
    lib = load_library()
    if not _bound:
        lib.infr_synth_normal_host.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, _V]
        lib.infr_synth_normal_host.restype = C.c_int
        lib.infr_synth_quantize_host.argtypes = [C.c_int32, _V, C.c_uint64, _V]
        lib.infr_synth_quantize_host.restype = C.c_int64
        lib.infr_synth_weights_host.argtypes = [C.c_int32, C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, _V, C.c_int]
        lib.infr_synth_weights_host.restype = C.c_int64
        lib.infr_synth_weights_device.argtypes = [_V, _V, C.c_size_t, C.c_int32, C.c_uint64, C.c_uint64, C.c_uint64,
                                                  C.c_double]
        lib.infr_synth_weights_device.restype = C.c_int
        _bound = True
    return lib


def stream_seed(seed0: int, layer: int, role: int) -> int:
    """One SplitMix64 stream per (layer, tensor role)."""
    z = (seed0 * 0x9E3779B97F4A7C15 + layer * 0xD1B54A32D192ED03 + role * 0x8CB92BA72F3D8DD7) & 0xFFFFFFFFFFFFFFFF
    z ^= z >> 29
    return (z * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF


def normal(seed: int, n: int, sigma: float = 1.0, offset: int = 0) -> np.ndarray:
    out = np.empty(n, np.float32)
    if _lib().infr_synth_normal_host(seed, offset, n, sigma, out.ctypes.data_as(_V)) != 0:
        raise ValueError("synth: normal failed")
    return out


def quantize(dtype: DType, w) -> np.ndarray:
    w = np.ascontiguousarray(w, np.float32).reshape(-1)
    out = np.empty(bytes_for(dtype, w.size), np.uint8)
    if _lib().infr_synth_quantize_host(int(dtype), w.ctypes.data_as(_V), w.size, out.ctypes.data_as(_V)) != out.size:
        raise ValueError("synth: quantize failed")
    return out


def weights_host(dtype: DType, seed: int, numel: int, sigma: float = 0.02, offset: int = 0, n_threads: int = 0) -> np.ndarray:
    out = np.empty(bytes_for(dtype, numel), np.uint8)
    n = _lib().infr_synth_weights_host(int(dtype), seed, offset, numel, sigma, out.ctypes.data_as(_V), n_threads)
    if n != out.size:
        raise ValueError("synth: weights_host failed (numel and offset must be multiples of 256)")
    return out.view(np.float32) if dtype == DType.F32 else out


def weights_device(be: Backend, buf: Buffer, dtype: DType, seed: int, numel: int, sigma: float = 0.02, offset: int = 0,
                   byte_offset: int = 0) -> None:
    _check(_lib().infr_synth_weights_device(be._h, buf._h, byte_offset, int(dtype), seed, offset, numel, sigma))


def zipf_bias(n_expert: int, s: float, seed: int) -> np.ndarray:
    """Per-expert logit bias ln(rank^-s / Z) under a seeded permutation: softmax(bias) is a Zipf(s)
    popularity.  Injected through the op's own inputs (x[:,0] = 1, router[e,0] = bias_e)."""
    rng = np.random.default_rng(seed)
    rank = rng.permutation(n_expert) + 1
    p = rank.astype(np.float64) ** (-s)
    return np.log(p / p.sum()).astype(np.float32)


@dataclass(frozen=True)
class MoeShape:
    name: str
    n_layer: int
    ne: int
    n_expert: int
    n_used: int
    n_ff: int
    gate_dtype: DType
    down_dtype: DType
    shared_ff: int = 0   # intermediate size of the always-on shared expert (0 = none)

    def expert_bytes(self) -> int:
        return 2 * bytes_for(self.gate_dtype, self.n_ff * self.ne) + bytes_for(self.down_dtype, self.ne * self.n_ff)

    def shared_bytes(self) -> int:
        if not self.shared_ff:
            return 0
        return 2 * bytes_for(self.gate_dtype, self.shared_ff * self.ne) + bytes_for(self.down_dtype, self.ne * self.shared_ff)

    def router_bytes(self) -> int:
        return self.n_expert * self.ne * 4

    def layer_resident_bytes(self) -> int:
        return self.n_expert * self.expert_bytes() + self.shared_bytes() + self.router_bytes()

    def algorithmic_bytes(self, batch: int, distinct_experts: Optional[int] = None) -> int:
        """Bytes one MoE layer must move for `batch` tokens: every distinct selected expert once,
        the shared expert, the router, activations in and out."""
        u = self.n_used * batch if distinct_experts is None else distinct_experts
        return u * self.expert_bytes() + self.shared_bytes() + self.router_bytes() + batch * self.ne * 4 * 2


# The benchmark configurations (hidden / experts / top-k / expert intermediate, quant mix).
CONFIG_1 = MoeShape("c1-single-layer-q8_0", 1, 2048, 128, 8, 768, DType.Q8_0, DType.Q8_0)
CONFIG_2 = MoeShape("c2-qwen3-30b-a3b-q4k-q6k-48L", 48, 2048, 128, 8, 768, DType.Q4K, DType.Q6K)
CONFIG_5 = MoeShape("c5-large-moe-256e-shared-q4k-q6k-40L", 40, 4096, 256, 8, 1536, DType.Q4K, DType.Q6K, shared_ff=1536)
# the routed-expert shape of gpt-oss-120b (hidden and intermediate 2880, 128 experts, top-4, 36 layers) with its MXFP4
# expert banks as they lie in a GGUF file: 60.9 GB resident
CONFIG_MXFP4 = MoeShape("gptoss-120b-shape-mxfp4-36L", 36, 2880, 128, 4, 2880, DType.Mxfp4, DType.Mxfp4)


class LayerWeights:
    """Device-resident weights of one synthetic MoE layer."""

    def __init__(self, be: Backend, shape: MoeShape, seed0: int, layer: int, on_device: bool = True):
        s = shape
        self.shape = s
        self.router = be.alloc_uninit(s.router_bytes(), BufferUsage.Weights)
        self.gate = be.alloc_uninit(bytes_for(s.gate_dtype, s.n_expert * s.n_ff * s.ne), BufferUsage.Weights)
        self.up = be.alloc_uninit(bytes_for(s.gate_dtype, s.n_expert * s.n_ff * s.ne), BufferUsage.Weights)
        self.down = be.alloc_uninit(bytes_for(s.down_dtype, s.n_expert * s.ne * s.n_ff), BufferUsage.Weights)
        gen = weights_device if on_device else self._host_fill
        gen(be, self.router, DType.F32, stream_seed(seed0, layer, ROLE_ROUTER), s.n_expert * s.ne)
        gen(be, self.gate, s.gate_dtype, stream_seed(seed0, layer, ROLE_GATE), s.n_expert * s.n_ff * s.ne)
        gen(be, self.up, s.gate_dtype, stream_seed(seed0, layer, ROLE_UP), s.n_expert * s.n_ff * s.ne)
        gen(be, self.down, s.down_dtype, stream_seed(seed0, layer, ROLE_DOWN), s.n_expert * s.ne * s.n_ff)
        self.shared = None
        if s.shared_ff:
            sg = be.alloc_uninit(bytes_for(s.gate_dtype, s.shared_ff * s.ne), BufferUsage.Weights)
            su = be.alloc_uninit(bytes_for(s.gate_dtype, s.shared_ff * s.ne), BufferUsage.Weights)
            sd = be.alloc_uninit(bytes_for(s.down_dtype, s.ne * s.shared_ff), BufferUsage.Weights)
            gen(be, sg, s.gate_dtype, stream_seed(seed0, layer, ROLE_SH_GATE), s.shared_ff * s.ne)
            gen(be, su, s.gate_dtype, stream_seed(seed0, layer, ROLE_SH_UP), s.shared_ff * s.ne)
            gen(be, sd, s.down_dtype, stream_seed(seed0, layer, ROLE_SH_DOWN), s.ne * s.shared_ff)
            self.shared = (sg, su, sd)

    @staticmethod
    def _host_fill(be, buf, dtype, seed, numel, sigma=0.02):
        be.upload(buf, weights_host(dtype, seed, numel, sigma))

    def buffers(self):
        out = [self.router, self.gate, self.up, self.down]
        if self.shared:
            out += list(self.shared)
        return out

    def free(self):
        for b in self.buffers():
            b.free()
