"""The entry point that allocates nothing (infr_hip_moe_ffn_static) against infr_hip_execute, through the C ABI.

Two calls in a row on one backend, the second with a smaller input: the static scratch keeps the first
call's contents, so anything the second call read without writing it first would show.  Bar: the bits
infr_hip_execute writes for the same op (same kernels, same operands), and the oracle's bar beside it."""
import ctypes as C

import numpy as np
import pytest

import helpers as H
import moe4all_amd as M
import oracle as O
from moe4all_amd import DType, TensorDesc
from test_gpu_parity import _realistic, bits, moe_graph, run_moe, MAX_ABS, REL_L2

pytestmark = pytest.mark.gpu


def _case(rows, ne, E, K, nff, gdt, ddt, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, nff, ne, gdt)
    down = _realistic(rng, E, ne, nff, ddt)
    return dict(x=x, router=router, gate=gate, up=up, down=down)


def _free_device_bytes():
    """hipMemGetInfo through the HIP runtime the library itself is linked against."""
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def _static(be, d, rows, ne, E, K, nff, gdt, ddt, calls=1):
    bufs = {k: be.buffer_from(v) for k, v in d.items()}
    dst = be.alloc(rows * ne * 4)
    be.upload(dst, np.full(rows * ne, np.nan, np.float32))   # every element has to be written
    try:
        be.sync()
        before = (be.alloc_calls(), _free_device_bytes())
        for _ in range(calls):
            be.moe_ffn_static(x=bufs["x"], router=bufs["router"], gate_exps=bufs["gate"], up_exps=bufs["up"],
                              down_exps=bufs["down"], dst=dst, gate_dtype=DType(gdt), down_dtype=DType(ddt), rows=rows, ne=ne,
                              n_expert=E, n_used=K, n_ff_exp=nff)
        be.sync()
        # the property the entry point exists for: no allocating call by the library, no device memory taken
        assert (be.alloc_calls(), _free_device_bytes()) == before
        return be.download(dst, rows * ne * 4, np.float32).reshape(rows, ne).copy()
    finally:
        for b in list(bufs.values()) + [dst]:
            b.free()


def test_static_scratch_entry_point_writes_the_bits_of_execute_twice_in_a_row():
    be = M.Backend(0)
    try:
        # a larger call first (several rows, large rows of h), then a smaller one on the same scratch
        for rows, ne, E, K, nff, gdt, ddt, seed in ((3, 2048, 32, 8, 768, H.Q4K, H.Q6K, 11), (1, 512, 8, 2, 256, H.Q8_0, H.Q4K, 12)):
            d = _case(rows, ne, E, K, nff, gdt, ddt, seed)
            got = _static(be, d, rows, ne, E, K, nff, gdt, ddt, calls=3)
            g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
            want, _ = run_moe(be, g, ids, d, rows, ne)
            assert np.array_equal(bits(got), bits(want)), (rows, H.max_abs(got, want))
            ref = O.moe_ffn(d["x"], d["router"], d["gate"], d["up"], d["down"], ne=ne, n_expert=E, n_used=K, n_ff_exp=nff,
                            gate_dtype=gdt, down_dtype=ddt)["dst"]
            assert H.rel_l2(got, ref) < REL_L2 and H.max_abs(got, ref) < MAX_ABS
    finally:
        be.close()


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    be = M.Backend(0)
    try:
        tiny = be.alloc(64)
        args = dict(x=tiny, router=tiny, gate_exps=tiny, up_exps=tiny, down_exps=tiny, dst=tiny, gate_dtype=DType.Q4K,
                    down_dtype=DType.Q6K)
        with pytest.raises(M.BackendError, match="hold"):    # operands smaller than the shapes
            be.moe_ffn_static(**args, rows=1, ne=2048, n_expert=8, n_used=2, n_ff_exp=768)
        with pytest.raises(M.Unsupported, match="rows"):      # more rows than the per-token path takes
            be.moe_ffn_static(**args, rows=16, ne=2048, n_expert=8, n_used=2, n_ff_exp=768)
        # rows * n_used * (n_ff_exp + ne) * 4 bytes beyond the static scratch: refused on the shapes alone, before the
        # operands' extents are looked at, so no operand of that size is needed here
        big = dict(rows=15, ne=8192, n_expert=64, n_used=8, n_ff_exp=8192)
        need = 15 * 8 * (8192 + 8192) * 4
        assert need > M.backend.STATIC_SCRATCH_BYTES
        with pytest.raises(M.Unsupported, match="scratch"):
            be.moe_ffn_static(**{**args, "down_dtype": DType.Q4K}, **big)
        tiny.free()
    finally:
        be.close()
