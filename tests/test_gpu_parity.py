"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same
seeded inputs and against the committed golden fixtures.

Bars: bit-exact for decoded weights, router logits, probabilities, expert ids and routing
weights; layer outputs within max-abs 2e-3 and relative L2 1e-3 (f32 accumulation)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers as H
import moe4all_amd as M
import oracle as O
from moe4all_amd import DType, TensorDesc
from moe4all_amd import backend as B

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")

MAX_ABS, REL_L2 = 2e-3, 1e-3


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def moe_graph(rows, ne, E, K, nff, gdt, ddt, rdt=DType.F32, **opts):
    g = M.Graph()
    x = g.input(TensorDesc([rows, ne], DType.F32))
    router = g.weight(TensorDesc([E, ne], rdt))
    fused = opts.get("fused_gate_up", False)
    gate = g.weight(TensorDesc([E, (2 if fused else 1) * nff, ne], gdt))
    up = None if fused else g.weight(TensorDesc([E, nff, ne], gdt))
    down = g.weight(TensorDesc([E, ne, nff], ddt))
    extra = {}
    for name, shape, dt in (("down_scale", [E], DType.F32), ("exp_probs_b", [E], DType.F32),
                            ("expert_ids", [rows, K], DType.I32)):
        if opts.pop("with_" + name, False):
            extra[name] = g.weight(TensorDesc(shape, dt)) if name != "expert_ids" else g.input(TensorDesc(shape, dt))
    dst = g.output(TensorDesc([rows, ne], DType.F32))
    g.moe_ffn(x=x, router=router, gate_exps=gate, up_exps=up, down_exps=down, dst=dst, ne=ne, n_expert=E, n_used=K,
              n_ff_exp=nff, **extra, **opts)
    return g, dict(x=x, router=router, gate=gate, up=up, down=down, dst=dst, **extra)


def run_moe(be, g, ids, data, rows, ne):
    keep = []
    bound = [(ids[k], v) for k, v in data.items() if ids.get(k) is not None and v is not None]
    out = M.run_graph(be, g, bound, ids["dst"], rows * ne, keep=keep)
    routing = be.moe_routing(keep[0], 0)
    for buf in keep[2]:
        buf.free()
    keep[3].free()
    keep[0].free()
    return out.reshape(rows, ne), routing


# ------------------------------------------------------------------ decode
def test_backend_identity(be):
    assert be.name() == "hip-gfx950"
    caps = be.capabilities()
    assert caps["subgroup_min"] == 64 and caps["compute_units"] >= 64 and not caps["unified_memory"]


def test_alloc_is_zeroed_and_transfers_roundtrip(be):
    buf = be.alloc(1000)
    assert buf.len_bytes() == 1000 and not be.download(buf).any()
    tiny = be.alloc(0)
    assert tiny.len_bytes() == 4  # reference: vec![0u8; bytes.max(4)]
    data = np.arange(1000, dtype=np.uint8)
    be.upload(buf, data[:600])
    got = be.download(buf)
    assert np.array_equal(got[:600], data[:600]) and not got[600:].any()
    be.upload_range(buf, 900, data[:100])
    assert np.array_equal(be.download_range(buf, 900, 100), data[:100])
    other = be.alloc(1000)
    be.copy_buffer(buf, other, 700)
    assert np.array_equal(be.download(other)[:700], be.download(buf)[:700])
    with pytest.raises(M.BackendError):
        be.upload(buf, np.zeros(1001, np.uint8))
    with pytest.raises(M.BackendError):
        be.download_range(buf, 990, 20)
    for b in (buf, tiny, other):
        b.free()


def test_dequant_matches_golden_bits(be):
    g = np.load(os.path.join(GOLD, "dequant.npz"))
    for n in sorted({k.rsplit(".", 1)[0] for k in g.files}):
        dt, raw = int(g[n + ".dtype"]), g[n + ".bytes"]
        e, b = H.BLOCK[dt]
        buf = be.buffer_from(raw)
        got = be.dequant(buf, DType(dt), raw.size // b * e)
        buf.free()
        assert np.array_equal(bits(got), g[n + ".bits"]), n


AFFINE = [H.Q4_0, H.Q4_1, H.Q5_0, H.Q5_1, H.Q8_0, H.Q2K, H.Q3K, H.Q4K, H.Q5K, H.Q6K]
DECODED = AFFINE + list(H.SCALE_CODE) + list(H.GRID_IQUANTS)   # every block format the device decodes


@pytest.mark.parametrize("dt", DECODED)
def test_dequant_matches_oracle_bits_on_a_large_tensor(be, dt):
    e, b = H.BLOCK[dt]
    raw = H.synth_weight(dt, e * 4099, seed=dt)
    buf = be.buffer_from(raw)
    got = be.dequant(buf, DType(dt), e * 4099)
    buf.free()
    assert np.array_equal(bits(got), bits(O.dequant(dt, raw)))


@pytest.mark.parametrize("dt,in_f", [(H.Q4K, 2048), (H.Q4K, 4096), (H.Q4K, 256), (H.Q4K, 1024), (H.Q6K, 768),
                                     (H.Q6K, 1536), (H.Q6K, 256), (H.Q6K, 4096), (H.Q8_0, 2048), (H.Q8_0, 768),
                                     (H.Q8_0, 4096), (H.Q8_0, 96), (H.Q4K, 5120), (H.F16, 100), (H.Q4_0, 96), (H.Q4_1, 2048),
                                     (H.Q5_0, 160), (H.Q5_1, 1024), (H.Q2K, 512), (H.Q3K, 768), (H.Q5K, 2048),
                                     (H.IQ4_NL, 96), (H.IQ4_XS, 512), (H.TQ1_0, 256), (H.TQ1_0, 1024), (H.TQ2_0, 768),
                                     (H.Q2_0, 192), (H.MXFP4, 2880), (H.MXFP4, 160), (H.NVFP4, 320), (H.IQ1_S, 512),
                                     (H.IQ1_M, 256), (H.IQ2_XXS, 768), (H.IQ2_XS, 256), (H.IQ2_S, 1024), (H.IQ3_XXS, 512),
                                     (H.IQ3_S, 2048)])
def test_one_hot_gemv_reads_back_the_decoded_weight(be, dt, in_f):
    """x = e_c makes y[o] = W[o][c]: the in-register unpacking of the GEMV kernels must reproduce
    the reference decode exactly (same trick as crates/infr-vulkan/tests/weight_dequant_parity.rs)."""
    out_f = 37
    e, b = H.BLOCK[dt]
    if dt == H.F16:
        raw = (np.random.default_rng(1).standard_normal(out_f * in_f)).astype(np.float16).view(np.uint8)
    else:
        raw = H.synth_weight(dt, out_f * in_f, seed=7 + in_f)
    W = O.dequant(dt, raw).reshape(out_f, in_f)
    rng = np.random.default_rng(in_f)
    cols = sorted(set([0, 1, 15, 16, 31, 32, 33, 63, 64, 95, in_f // 2, in_f - 33, in_f - 1]) |
                  set(int(c) for c in rng.integers(0, in_f, 24)))
    cols = [c for c in cols if 0 <= c < in_f]
    m = len(cols)
    x = np.zeros((m, in_f), np.float32)
    x[np.arange(m), cols] = 1.0
    g = M.Graph()
    xi = g.input(TensorDesc([m, in_f], DType.F32))
    wi = g.weight(TensorDesc([out_f, in_f], DType(dt)))
    yi = g.output(TensorDesc([m, out_f], DType.F32))
    g.linear(x=xi, weight=wi, dst=yi, m=m, in_f=in_f, out_f=out_f)
    y = M.run_graph(be, g, [(xi, x), (wi, raw)], yi, m * out_f).reshape(m, out_f)
    want = W[:, cols].T
    assert np.array_equal(y, want), f"first mismatch at {np.argwhere(y != want)[:3]}"


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("rows,ne,E,K,rdt", [(1, 2048, 128, 8, H.F32), (4, 2048, 128, 8, H.F32),
                                             (33, 256, 64, 6, H.F32), (3, 100, 10, 3, H.F32),
                                             (1, 4096, 256, 8, H.F32), (5, 512, 16, 4, H.Q8_0),
                                             (2, 256, 8, 2, H.F16), (70, 2048, 100, 8, H.F32),
                                             (16, 160, 40, 4, H.F32), (1030, 512, 256, 8, H.F32), (500, 288, 128, 4, H.F32),
                                             (2050, 288, 100, 4, H.F32), (1024, 640, 256, 8, H.F32)])
def test_router_logits_probs_ids_weights_bit_exact(be, rows, ne, E, K, rdt):
    rng = np.random.default_rng(rows * 7 + ne)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    rf = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    router = {H.F32: rf, H.Q8_0: H.quantize_q8_0(rf) if ne % 32 == 0 else None, H.F16: rf.astype(np.float16)}[rdt]
    nff = 32
    z = np.zeros(E * nff * ne, np.float32)
    g, ids = moe_graph(rows, ne, E, K, nff, DType.F32, DType.F32, rdt=DType(rdt))
    out, r = run_moe(be, g, ids, dict(x=x, router=router, gate=z, up=z, down=z), rows, ne)
    ref = O.moe_ffn(x, router, z, z, z, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, router_dtype=rdt)
    assert np.array_equal(bits(r["logits"]), bits(ref["logits"]))
    assert np.array_equal(bits(r["probs"]), bits(ref["probs"]))
    assert np.array_equal(r["idx"], ref["idx"])
    assert np.array_equal(bits(r["w"]), bits(ref["w"]))
    assert not out.any()


@pytest.mark.parametrize("rows", [1, 64, 2048])
def test_router_logits_keep_subnormal_terms(be, rows):
    """Products and sums around 1e-39 are subnormal f32 numbers: the logits kernels of every batch size (per-row chains
    on the vector ALUs, the two forms of the matrix-core kernel) must keep them as the CPU's fused multiply-add does."""
    ne, E, K, nff = 256, 128, 8, 32
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((rows, ne)) * 1e-22).astype(np.float32)
    rf = (rng.standard_normal((E, ne)) * 1e-18).astype(np.float32)
    z = np.zeros(E * nff * ne, np.float32)
    g, ids = moe_graph(rows, ne, E, K, nff, DType.F32, DType.F32)
    _, r = run_moe(be, g, ids, dict(x=x, router=rf, gate=z, up=z, down=z), rows, ne)
    ref = O.moe_ffn(x, rf, z, z, z, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff)
    assert np.abs(ref["logits"]).max() < 1.1754944e-38 and ref["logits"].any()
    assert np.array_equal(bits(r["logits"]), bits(ref["logits"]))
    assert np.array_equal(r["idx"], ref["idx"])


def test_routing_variants_bit_exact_ids(be):
    ne, E, K, nff, rows = 64, 16, 4, 32, 6
    rng = np.random.default_rng(11)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = rng.standard_normal((E, ne)).astype(np.float32) * 0.3
    z = np.zeros(E * nff * ne, np.float32)
    bias = rng.uniform(-0.3, 0.3, E).astype(np.float32)
    # sigmoid gating, bias, 4 groups keep 2, no renorm, scale
    g, ids = moe_graph(rows, ne, E, K, nff, DType.F32, DType.F32, gating=M.MoeGating.Sigmoid, norm_w=False, scale=2.5,
                       with_exp_probs_b=True, n_expert_groups=4, n_expert_groups_used=2)
    _, r = run_moe(be, g, ids, dict(x=x, router=router, gate=z, up=z, down=z, exp_probs_b=bias), rows, ne)
    ref = O.moe_ffn(x, router, z, z, z, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gating=O.GATE_SIGMOID, norm_w=False,
                    scale=2.5, exp_probs_b=bias, n_expert_groups=4, n_expert_groups_used=2)
    assert np.array_equal(r["idx"], ref["idx"]) and np.array_equal(bits(r["w"]), bits(ref["w"]))
    # ties: identical router rows -> identical probabilities -> ascending ids
    router_t = np.tile(router[:1], (E, 1))
    g, ids = moe_graph(rows, ne, E, K, nff, DType.F32, DType.F32)
    _, r = run_moe(be, g, ids, dict(x=x, router=router_t, gate=z, up=z, down=z), rows, ne)
    assert np.array_equal(r["idx"], np.tile(np.arange(K, dtype=np.int32), (rows, 1)))
    # hash routing: supplied ids, weights from the router's own probabilities
    hid = rng.integers(0, E, (rows, K)).astype(np.int32)
    g, ids = moe_graph(rows, ne, E, K, nff, DType.F32, DType.F32, with_expert_ids=True)
    _, r = run_moe(be, g, ids, dict(x=x, router=router, gate=z, up=z, down=z, expert_ids=hid), rows, ne)
    ref = O.moe_ffn(x, router, z, z, z, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, expert_ids=hid.astype(np.float32))
    assert np.array_equal(r["idx"], hid) and np.array_equal(bits(r["w"]), bits(ref["w"]))


# ------------------------------------------------------------------ Op::MoeFfn
def test_moe_ffn_golden_cases_of_the_reference_tests(be):
    gold = np.load(os.path.join(GOLD, "moe_small.npz"))
    for name, c in H.moe_cases().items():
        dt = DType(c["dtype"])
        opts = dict(gating=M.MoeGating(c["gating"]))
        if "bias" in c:
            opts.update(with_exp_probs_b=True, n_expert_groups=c["n_groups"], n_expert_groups_used=c["n_groups_used"])
        g, ids = moe_graph(1, c["ne"], c["n_expert"], c["n_used"], c["n_ff"], dt, dt, **opts)
        data = dict(x=c["x"], router=c["router"], gate=c["gate"], up=c["up"], down=c["down"], exp_probs_b=c.get("bias"))
        out, r = run_moe(be, g, ids, data, 1, c["ne"])
        if c["gating"] != 2:  # sqrt-softplus probabilities use the device logf: ids only
            assert np.array_equal(r["idx"], gold[name + ".idx"]), name
        else:
            assert sorted(r["idx"][0]) == sorted(gold[name + ".idx"][0]), name
        # the reference's own device tolerances: 1e-3 (seam_op_parity.rs / metal parity.rs)
        assert H.elem_rel_err(out, gold[name + ".want"]) < 1e-3, name
        assert H.rel_l2(out, gold[name + ".want"]) < 1e-5, name


def _realistic(rng, E, rows_out, cols, dt):
    """N(0, 0.02) weights in the magnitude band of BASELINE's configs; Q8_0 via the reference's
    test quantiser, K-quants as synthetic valid blocks rescaled to the same band."""
    if dt == H.Q8_0:
        return H.quantize_q8_0((rng.standard_normal(E * rows_out * cols) * 0.02).astype(np.float32))
    raw = H.synth_weight(dt, E * rows_out * cols, int(rng.integers(1, 1 << 30)))
    e, b = H.BLOCK[dt]
    blk = raw.reshape(-1, b)
    if dt == H.Q4K:  # d*sc*q - dmin*m with sc,m <= 63, q <= 15: centre and shrink to ~0.02
        blk[:, 0:2] = H.f16_bytes(0.0001)
        blk[:, 2:4] = H.f16_bytes(0.00075)
    else:
        blk[:, 208:210] = H.f16_bytes(0.00001)
    return blk.reshape(-1)


@pytest.mark.parametrize("rows,ne,E,K,nff,gdt,ddt", [
    (1, 2048, 128, 8, 768, H.Q8_0, H.Q8_0),    # config 1
    (1, 2048, 128, 8, 768, H.Q4K, H.Q6K),      # one layer of config 2
    (4, 2048, 128, 8, 768, H.Q8_0, H.Q8_0),    # config 3, batch 4
    (16, 2048, 128, 8, 768, H.Q4K, H.Q6K),     # config 3 shape with the K-quant mix
    (1, 4096, 256, 8, 1536, H.Q4K, H.Q6K),     # one layer of config 5
    (1, 512, 384, 15, 1280, H.Q4K, H.Q6K),     # 8 candidates per lane and 16 selection rounds in the two-wave routing; 8 rows per wave
    (3, 256, 8, 3, 256, H.Q6K, H.Q4K),         # small, several weight rows per wavefront
    (2, 512, 8, 2, 1024, H.Q8_0, H.Q4K),
    (2, 96, 6, 2, 64, H.Q8_0, H.Q8_0),         # shape-generic kernels (96 is not a multiple of 256)
])
def test_moe_ffn_matches_oracle(be, rows, ne, E, K, nff, gdt, ddt):
    rng = np.random.default_rng(ne + rows + gdt)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, nff, ne, gdt)
    down = _realistic(rng, E, ne, nff, ddt)
    g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
    out, r = run_moe(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), rows, ne)
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    assert np.array_equal(r["idx"], ref["idx"])
    assert np.array_equal(bits(r["w"]), bits(ref["w"]))
    scale = float(np.abs(ref["dst"]).max())
    assert scale > 1e-4, "degenerate case"
    assert H.rel_l2(out, ref["dst"]) < REL_L2, H.rel_l2(out, ref["dst"])
    assert H.max_abs(out, ref["dst"]) < MAX_ABS, (H.max_abs(out, ref["dst"]), scale)


def _bank_weights(rng, E, nff, ne, gdt, ddt):
    """Q4_K / Q6_K / Q8_0 banks as the other tests make them; any other affine format as centred synthetic blocks."""
    if gdt in (H.Q4K, H.Q6K, H.Q8_0) and ddt in (H.Q4K, H.Q6K, H.Q8_0):
        return _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, ne, nff, ddt)
    return (H.centred_weight(gdt, E * nff * ne, 1), H.centred_weight(gdt, E * nff * ne, 2),
            H.centred_weight(ddt, E * ne * nff, 3))


@pytest.mark.parametrize("rows", [1, 5, 40])
@pytest.mark.parametrize("gdt,ddt", [(H.IQ2_XXS, H.IQ3_S), (H.IQ1_M, H.IQ2_S), (H.IQ3_XXS, H.IQ2_XS), (H.IQ1_S, H.IQ4_XS)])
def test_moe_ffn_with_grid_iquant_experts_matches_oracle(be, gdt, ddt, rows):
    """Expert banks in the lattice-codebook formats (the 1- to 3-bit quantisations MoE checkpoints ship in), one token,
    a decode batch and a prefill-sized chunk."""
    ne, E, K, nff = 512, 8, 3, 256
    rng = np.random.default_rng(rows + gdt)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = rng.standard_normal((E, ne)).astype(np.float32) * 0.05
    gate, up, down = _bank_weights(rng, E, nff, ne, gdt, ddt)
    g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
    be.prof_enable(True)
    out, r = run_moe(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), rows, ne)
    be.sync()
    names = set(be.prof_read())
    be.prof_enable(False)
    # the 32-element unit decoders, not the element-wise kernels: GEMV forms for decode, matrix cores for the chunk
    want_names = {"moe_grouped_units_gate_up", "moe_grouped_units_down"} if rows >= 32 else \
        {"moe_route_gate_up_units", "moe_down_combine_units"} if rows == 1 else {"moe_route_gate_up_units", "moe_down_units"}
    assert want_names <= names, names
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    assert np.array_equal(r["idx"], ref["idx"])
    assert float(np.abs(ref["dst"]).max()) > 1e-4, "degenerate case"
    tol = REL_L2_MFMA if rows >= 32 else REL_L2
    for row in range(rows):
        assert H.rel_l2(out.reshape(rows, ne)[row], ref["dst"].reshape(rows, ne)[row]) < tol, row


@pytest.mark.parametrize("rows", [3, 1])   # one row: the unit formats' down stage and combine are one launch
@pytest.mark.parametrize("gdt,ddt", [(H.Q4K, H.Q6K), (H.Q5K, H.Q4_0)])
def test_moe_ffn_option_variants_match_oracle(be, gdt, ddt, rows):
    ne, E, K, nff = 256, 8, 3, 256
    rng = np.random.default_rng(21)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = rng.standard_normal((E, ne)).astype(np.float32) * 0.05
    gate, up, down = _bank_weights(rng, E, nff, ne, gdt, ddt)
    ds = rng.uniform(0.5, 1.5, E).astype(np.float32)
    base = dict(ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)

    def check(gopts, oopts, data_extra=None, fused=False):
        g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt), **gopts)
        data = dict(x=x, router=router, gate=gate, up=up, down=down)
        ogate, oup = gate, up
        if fused:
            gu = np.concatenate([gate.reshape(E, -1), up.reshape(E, -1)], axis=1).reshape(-1)
            data.update(gate=gu, up=None)
            ogate, oup = gu, None
        data.update(data_extra or {})
        out, r = run_moe(be, g, ids, data, rows, ne)
        ref = O.moe_ffn(x, router, ogate, oup, down, **base, **oopts)
        assert np.array_equal(r["idx"], ref["idx"])
        assert H.rel_l2(out, ref["dst"]) < REL_L2, (gopts, H.rel_l2(out, ref["dst"]))

    check(dict(weight_before=True, gating=M.MoeGating.Sigmoid, norm_w=False),
          dict(weight_before=True, gating=O.GATE_SIGMOID, norm_w=False))
    check(dict(with_down_scale=True, scale=1.7), dict(down_scale=ds, scale=1.7), dict(down_scale=ds))
    check(dict(swiglu_clamp=0.05, act=M.Activation.Gelu), dict(swiglu_clamp=0.05, act=O.ACT_GELU))
    check(dict(fused_gate_up=True), dict(fused_gate_up=True), fused=True)


def test_buffers_and_plans_may_outlive_their_backend():
    """infr_hip_destroy first, frees afterwards: the reference's buffers keep their device alive, so this order is legal.
    Every other call with the destroyed handle is refused with a status."""
    be2 = M.Backend(0)
    buf = be2.alloc(4096)
    g, ids = moe_graph(1, 256, 4, 2, 256, DType.Q4K, DType.Q4K)
    plan = be2.compile(g)
    handle = be2._h
    be2.close()
    lib = M.load_library()
    out = C.c_void_p()
    assert lib.infr_hip_alloc(handle, 16, 1, C.byref(out)) != 0 and b"bad handle" in lib.infr_hip_last_error()
    assert lib.infr_hip_upload(handle, buf._h, (C.c_char * 4)(), 4) != 0
    plan.free()
    buf.free()


def test_no_exception_crosses_the_abi(be):
    """A graph whose op count cannot be allocated: std::bad_alloc inside infr_hip_compile comes back as a status."""
    gr = B._Graph()
    op = B._Op(kind=3)
    gr.ops, gr.n_ops = C.pointer(op), 0xFFFFFFFF
    out = C.c_void_p()
    st = M.load_library().infr_hip_compile(be._h, C.byref(gr), C.byref(out))
    assert st == 1 and not out.value, st
    assert b"infr_hip_compile" in M.load_library().infr_hip_last_error()


def test_execute_is_repeatable_and_rebinding_works(be):
    rows, ne, E, K, nff = 1, 2048, 32, 8, 768
    rng = np.random.default_rng(4)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = (_realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K),
                      _realistic(rng, E, ne, nff, H.Q6K))
    g, ids = moe_graph(rows, ne, E, K, nff, DType.Q4K, DType.Q6K)
    plan = be.compile(g)
    wb = {k: be.buffer_from(v) for k, v in (("router", router), ("gate", gate), ("up", up), ("down", down))}
    xb, yb = be.alloc(ne * 4), be.alloc(ne * 4, M.BufferUsage.Readback)
    b = M.Bindings()
    for k, buf in wb.items():
        b.bind(ids[k], buf)
    b.bind(ids["x"], xb).bind(ids["dst"], yb)
    outs = []
    for t in range(3):
        x = rng.standard_normal((1, ne)).astype(np.float32)
        be.upload(xb, x)
        be.execute(plan, b)
        be.execute(plan, b)  # same inputs twice: identical bits
        got = be.download(yb, ne * 4, np.float32).copy()
        ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K,
                        down_dtype=H.Q6K)
        assert H.rel_l2(got, ref["dst"]) < REL_L2
        outs.append(got)
    assert not np.array_equal(outs[0], outs[1])
    # an unbound weight is an error value, not a crash (reference: "unbound Weight")
    b2 = M.Bindings().bind(ids["x"], xb).bind(ids["dst"], yb)
    with pytest.raises(M.BackendError, match="unbound"):
        be.execute(plan, b2)
    # a too-small output buffer is refused before any kernel runs
    small = be.alloc(16)
    b.bind(ids["dst"], small)
    with pytest.raises(M.BackendError, match="bound buffer holds"):
        be.execute(plan, b)
    for buf in list(wb.values()) + [xb, yb, small]:
        buf.free()
    plan.free()


def test_compile_refuses_what_the_path_does_not_cover(be):
    g = M.Graph()
    g.push_raw(17)
    with pytest.raises(M.Unsupported):
        be.compile(g)
    g, _ = moe_graph(1, 256, 8, 2, 256, DType.I32, DType.I32)   # an integer table is not a weight format
    with pytest.raises(M.Unsupported, match="I32"):
        be.compile(g)
    g, _ = moe_graph(1, 256, 8, 2, 256, DType.Q4K, DType.Q4K, ep_band=(6, 4))   # band past the last expert
    with pytest.raises(M.BackendError, match="ep_band"):
        be.compile(g)
    g, _ = moe_graph(1, 256, 8, 2, 256, DType.Q4K, DType.Q4K, ep_band=(0, 4))   # tensors hold 8 experts, the band says 4
    with pytest.raises(M.BackendError, match="gate_exps"):
        be.compile(g)
    g, _ = moe_graph(1, 256, 8, 2, 256, DType.Q4K, DType.Q4K, swiglu_clamp=1.0, weight_before=True)
    with pytest.raises(M.BackendError):
        be.compile(g)
    g, _ = moe_graph(1, 100, 8, 2, 256, DType.Q4K, DType.Q4K)  # 100 is not a whole number of blocks
    with pytest.raises(M.BackendError):
        be.compile(g)


# ------------------------------------------------------------------ shared-expert neighbours
def test_shared_expert_branch_matches_oracle(be):
    """The op sequence the reference emits around MoeFfn for a shared expert
    (crates/infr-llama/src/seam/runner.rs:8088-8175): Linear(out_f=1) gate logit, Linear gate,
    Linear up, GatedAct, Linear down, MoeSharedExpertAdd."""
    rows, ne, nff = 2, 1024, 512
    rng = np.random.default_rng(8)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    moe = rng.standard_normal((rows, ne)).astype(np.float32)
    wg, wu = _realistic(rng, 1, nff, ne, H.Q4K), _realistic(rng, 1, nff, ne, H.Q4K)
    wd = _realistic(rng, 1, ne, nff, H.Q6K)
    wgi = (rng.standard_normal(ne) * 0.05).astype(np.float32)
    g = M.Graph()
    xi, mi = g.input(TensorDesc([rows, ne], DType.F32)), g.input(TensorDesc([rows, ne], DType.F32))
    wgt, wut = g.weight(TensorDesc([nff, ne], DType.Q4K)), g.weight(TensorDesc([nff, ne], DType.Q4K))
    wdt, wgit = g.weight(TensorDesc([ne, nff], DType.Q6K)), g.weight(TensorDesc([1, ne], DType.F32))
    gl, gt, ut = (g.internal(TensorDesc([rows, 1], DType.F32)), g.internal(TensorDesc([rows, nff], DType.F32)),
                  g.internal(TensorDesc([rows, nff], DType.F32)))
    at, st = g.internal(TensorDesc([rows, nff], DType.F32)), g.internal(TensorDesc([rows, ne], DType.F32))
    yi = g.output(TensorDesc([rows, ne], DType.F32))
    g.linear(x=xi, weight=wgit, dst=gl, m=rows, in_f=ne, out_f=1)
    g.linear(x=xi, weight=wgt, dst=gt, m=rows, in_f=ne, out_f=nff)
    g.linear(x=xi, weight=wut, dst=ut, m=rows, in_f=ne, out_f=nff)
    g.gated_act(gate=gt, up=ut, dst=at, rows=rows, nff=nff)
    g.linear(x=at, weight=wdt, dst=st, m=rows, in_f=nff, out_f=ne)
    g.moe_shared_expert_add(moe=mi, shexp=st, gate=gl, dst=yi, rows=rows, n=ne)
    got = M.run_graph(be, g, [(xi, x), (mi, moe), (wgt, wg), (wut, wu), (wdt, wd), (wgit, wgi)], yi, rows * ne)
    og = O.linear(x, wg, H.Q4K, ne, nff)
    ou = O.linear(x, wu, H.Q4K, ne, nff)
    oa = O.gated_act_rows(og, ou)
    osx = O.linear(oa, wd, H.Q6K, nff, ne)
    ogl = O.linear(x, wgi, H.F32, ne, 1)
    want = O.moe_shared_expert_add(moe, osx, ogl)
    assert H.rel_l2(got, want) < REL_L2 and H.max_abs(got, want) < MAX_ABS
    # Op::Add variant (llama4: ungated)
    g2 = M.Graph()
    a, b = g2.input(TensorDesc([rows * ne], DType.F32)), g2.input(TensorDesc([rows * ne], DType.F32))
    d = g2.output(TensorDesc([rows * ne], DType.F32))
    g2.add(a=a, b=b, dst=d, n=rows * ne)
    got2 = M.run_graph(be, g2, [(a, x), (b, moe)], d, rows * ne)
    assert np.array_equal(got2, O.add(x, moe).ravel())


def test_copy_and_copy_strided_follow_the_cpu_semantics(be):
    """Op::Copy / Op::CopyStrided (crates/infr-cpu/src/lib.rs:3532-3583): windows counted in elements,
    the rest of dst untouched, and a copy inside one tensor reads its source window before it
    writes (overlapping windows included)."""
    rng = np.random.default_rng(5)
    a = rng.standard_normal(4096).astype(np.float32)
    g = M.Graph()
    src = g.input(TensorDesc([4096], DType.F32))
    dst = g.output(TensorDesc([6, 100], DType.F32))
    mid = g.internal(TensorDesc([4096], DType.F32))
    g.copy(src=src, src_off=0, dst=mid, dst_off=0, n=4096)
    g.copy(src=mid, src_off=10, dst=mid, dst_off=50, n=1000)             # overlapping, forward
    g.copy_strided(src=mid, src_off=3, src_stride=300, dst=mid, dst_off=7, dst_stride=300, rows=5, n=250)  # overlapping rows
    g.copy_strided(src=mid, src_off=20, src_stride=64, dst=dst, dst_off=10, dst_stride=100, rows=6, n=37)
    got = M.run_graph(be, g, [(src, a)], dst, 600).reshape(6, 100)
    m = a.copy()
    m[50:1050] = m[10:1010].copy()
    snap = m.copy()
    for r in range(5):
        m[7 + 300 * r:7 + 300 * r + 250] = snap[3 + 300 * r:3 + 300 * r + 250]
    want = np.zeros((6, 100), np.float32)
    for r in range(6):
        want[r, 10:47] = m[20 + 64 * r:20 + 64 * r + 37]
    assert np.array_equal(bits(got), bits(want))
    g2 = M.Graph()
    s2, d2 = g2.input(TensorDesc([8], DType.F32)), g2.output(TensorDesc([8], DType.F32))
    g2.copy(src=s2, src_off=4, dst=d2, dst_off=0, n=5)   # reads past the source
    with pytest.raises(M.BackendError):
        be.compile(g2)


@pytest.mark.parametrize("rows,act", [(1, M.Activation.Silu), (5, M.Activation.Gelu)])
def test_fused_dense_ffn_launches_give_the_bits_of_the_separate_ops(be, rows, act):
    """Linear+Linear+GatedAct and Linear+Add collapse into one launch each when their temporaries are
    single-use Internal tensors; declaring the temporaries as Outputs keeps the ops separate.  Both
    run the same inner products in the same rounding order, so the results must be identical bits."""
    ne, nff = 1024, 512
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    res = rng.standard_normal((rows, ne)).astype(np.float32)
    wg, wu = _realistic(rng, 1, nff, ne, H.Q4K), _realistic(rng, 1, nff, ne, H.Q4K)
    wd = _realistic(rng, 1, ne, nff, H.Q6K)

    def run(fusable):
        g = M.Graph()
        mk = g.internal if fusable else g.output
        xi, ri = g.input(TensorDesc([rows, ne], DType.F32)), g.input(TensorDesc([rows, ne], DType.F32))
        wgt, wut = g.weight(TensorDesc([nff, ne], DType.Q4K)), g.weight(TensorDesc([nff, ne], DType.Q4K))
        wdt = g.weight(TensorDesc([ne, nff], DType.Q6K))
        gt, ut = mk(TensorDesc([rows, nff], DType.F32)), mk(TensorDesc([rows, nff], DType.F32))
        at, st = g.internal(TensorDesc([rows, nff], DType.F32)), mk(TensorDesc([rows, ne], DType.F32))
        yi = g.output(TensorDesc([rows, ne], DType.F32))
        g.linear(x=xi, weight=wut, dst=ut, m=rows, in_f=ne, out_f=nff)       # up first: either order fuses
        g.linear(x=xi, weight=wgt, dst=gt, m=rows, in_f=ne, out_f=nff)
        g.gated_act(gate=gt, up=ut, dst=at, rows=rows, nff=nff, act=act)
        g.linear(x=at, weight=wdt, dst=st, m=rows, in_f=nff, out_f=ne)
        g.add(a=ri, b=st, dst=yi, n=rows * ne)
        plan = be.compile(g)
        bufs = [be.buffer_from(v) for v in (x, res, wg, wu, wd)]
        b = M.Bindings()
        for tid, buf in zip((xi, ri, wgt, wut, wdt), bufs):
            b.bind(tid, buf)
        extra = []
        if not fusable:
            for tid, n in ((gt, rows * nff), (ut, rows * nff), (st, rows * ne)):
                extra.append(be.alloc(n * 4))
                b.bind(tid, extra[-1])
        yb = be.alloc(rows * ne * 4)
        b.bind(yi, yb)
        be.prof_enable(True)
        be.execute(plan, b)
        out = be.download(yb, rows * ne * 4, np.float32)
        names = set(be.prof_read())
        be.prof_enable(False)
        for buf in bufs + extra + [yb]:
            buf.free()
        plan.free()
        return out, names

    fused, fused_names = run(True)
    plain, plain_names = run(False)
    assert {"linear_gate_up_act", "linear_add"} <= fused_names
    assert "gated_act" in plain_names and "add" in plain_names
    assert np.array_equal(bits(fused), bits(plain))
    og, ou = O.linear(x, wg, H.Q4K, ne, nff), O.linear(x, wu, H.Q4K, ne, nff)
    want = O.add(res, O.linear(O.gated_act_rows(og, ou, act=int(act)), wd, H.Q6K, nff, ne))
    assert H.rel_l2(fused.reshape(rows, ne), want.reshape(rows, ne)) < REL_L2


@pytest.mark.parametrize("rows,K,opts", [(1, 4, {}), (1, 8, {"weight_before": True}), (1, 6, {"with_down_scale": True}),
                                         (3, 8, {}),
                                         # tiles of several weight rows per wavefront: the streamed decode kernels
                                         (1, 4, {"with_dims": (2048, 2048)}),
                                         (1, 8, {"weight_before": True, "with_dims": (2048, 2048)}),
                                         (1, 6, {"with_down_scale": True, "with_dims": (2048, 1536)}),
                                         # a decode batch past 16 rows that stays on the per-token kernels (its pairs
                                         # are expected on too many distinct experts for bucketing to pay)
                                         (20, 2, {"with_experts": 64})])
def test_shared_expert_as_an_extra_slot_gives_the_bits_of_the_separate_ops(be, rows, K, opts):
    """MoeFfn followed by an ungated shared expert (Linear, Linear, GatedAct, Linear, Add —
    crates/infr-llama/src/seam/runner.rs:8116-8174) runs as one more slot of the two routed decode
    kernels when the routed sum is a single-use Internal tensor, for one token row and for the few rows of a decode
    batch on the per-token kernels.  Declaring that tensor an Output keeps MoeFfn and the dense FFN apart; both must
    give identical bits."""
    (ne, nff), E = opts.get("with_dims", (1024, 512)), opts.get("with_experts", 16)
    rng = np.random.default_rng(100 + rows)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    eg, eu = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
    ed = _realistic(rng, E, ne, nff, H.Q6K)
    wg, wu = _realistic(rng, 1, nff, ne, H.Q4K), _realistic(rng, 1, nff, ne, H.Q4K)
    wd = _realistic(rng, 1, ne, nff, H.Q6K)
    dscale = (0.5 + rng.random(E)).astype(np.float32) if opts.get("with_down_scale") else None
    mopts = {k: v for k, v in opts.items() if not k.startswith("with_")}

    def run(fusable):
        g = M.Graph()
        xi = g.input(TensorDesc([rows, ne], DType.F32))
        rt = g.weight(TensorDesc([E, ne], DType.F32))
        egt, eut = g.weight(TensorDesc([E, nff, ne], DType.Q4K)), g.weight(TensorDesc([E, nff, ne], DType.Q4K))
        edt = g.weight(TensorDesc([E, ne, nff], DType.Q6K))
        wgt, wut = g.weight(TensorDesc([nff, ne], DType.Q4K)), g.weight(TensorDesc([nff, ne], DType.Q4K))
        wdt = g.weight(TensorDesc([ne, nff], DType.Q6K))
        dst = g.weight(TensorDesc([E], DType.F32)) if dscale is not None else None
        moe = (g.internal if fusable else g.output)(TensorDesc([rows, ne], DType.F32))
        gt, ut = g.internal(TensorDesc([rows, nff], DType.F32)), g.internal(TensorDesc([rows, nff], DType.F32))
        at, st = g.internal(TensorDesc([rows, nff], DType.F32)), g.internal(TensorDesc([rows, ne], DType.F32))
        yi = g.output(TensorDesc([rows, ne], DType.F32))
        g.moe_ffn(x=xi, router=rt, gate_exps=egt, up_exps=eut, down_exps=edt, dst=moe, ne=ne, n_expert=E, n_used=K,
                  n_ff_exp=nff, down_scale=dst, **mopts)
        g.linear(x=xi, weight=wgt, dst=gt, m=rows, in_f=ne, out_f=nff)
        g.linear(x=xi, weight=wut, dst=ut, m=rows, in_f=ne, out_f=nff)
        g.gated_act(gate=gt, up=ut, dst=at, rows=rows, nff=nff)
        g.linear(x=at, weight=wdt, dst=st, m=rows, in_f=nff, out_f=ne)
        g.add(a=moe, b=st, dst=yi, n=rows * ne)
        plan = be.compile(g)
        pairs = [(xi, x), (rt, router), (egt, eg), (eut, eu), (edt, ed), (wgt, wg), (wut, wu), (wdt, wd)]
        if dscale is not None:
            pairs.append((dst, dscale))
        bufs, b = [], M.Bindings()
        for tid, v in pairs:
            bufs.append(be.buffer_from(v))
            b.bind(tid, bufs[-1])
        if not fusable:
            bufs.append(be.alloc(rows * ne * 4))
            b.bind(moe, bufs[-1])
        yb = be.alloc(rows * ne * 4)
        b.bind(yi, yb)
        be.prof_enable(True)
        be.execute(plan, b)
        out = be.download(yb, rows * ne * 4, np.float32)
        names = set(be.prof_read())
        be.prof_enable(False)
        routing = be.moe_routing(plan, 0)
        for buf in bufs + [yb]:
            buf.free()
        plan.free()
        return out, names, routing

    fused, fused_names, r1 = run(True)
    plain, plain_names, r2 = run(False)
    assert {"moe_route_gate_up_shared", "moe_down_combine_shared"} <= fused_names and "linear_add" not in fused_names
    assert {"moe_route_gate_up", "linear_gate_up_act", "linear_add"} <= plain_names
    assert np.array_equal(r1["idx"], r2["idx"]) and np.array_equal(bits(r1["w"]), bits(r2["w"]))
    assert np.array_equal(bits(fused), bits(plain))
    want_moe = O.moe_ffn(x, router, eg, eu, ed, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K,
                         down_dtype=H.Q6K, down_scale=dscale, **mopts)["dst"]
    og, ou = O.linear(x, wg, H.Q4K, ne, nff), O.linear(x, wu, H.Q4K, ne, nff)
    want = O.add(want_moe, O.linear(O.gated_act_rows(og, ou), wd, H.Q6K, nff, ne))
    assert H.rel_l2(fused.reshape(rows, ne), want.reshape(rows, ne)) < REL_L2


@pytest.mark.parametrize("rows,dim,add,inplace", [(1, 2048, False, False), (5, 100, False, False), (3, 8192, True, False),
                                                  (2, 4096, False, True), (1, 6, True, False), (0, 64, False, False)])
def test_rms_norm_and_rms_norm_add_match_the_oracle(be, rows, dim, add, inplace):
    """Op::RmsNorm / Op::RmsNormAdd (crates/infr-cpu/src/lib.rs:1046-1093): dims with and without
    a 16-byte row pitch, several passes per thread, in place, and an empty batch."""
    rng = np.random.default_rng(rows * 131 + dim)
    x = (rng.standard_normal((rows, dim)) * 3).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(dim)).astype(np.float32)
    y0 = rng.standard_normal((rows, dim)).astype(np.float32)
    eps = 1e-6
    g = M.Graph()
    wt = g.weight(TensorDesc([dim], DType.F32))
    if inplace:
        xi = yi = g.output(TensorDesc([rows, dim], DType.F32))
    else:
        xi = g.input(TensorDesc([rows, dim], DType.F32))
        yi = g.output(TensorDesc([rows, dim], DType.F32))
    g.rms_norm(x=xi, weight=wt, dst=yi, rows=rows, dim=dim, eps=eps, add=add)
    bound = [(wt, w), (yi, x if inplace else y0)] + ([] if inplace else [(xi, x)])
    got = M.run_graph(be, g, bound, yi, rows * dim).reshape(rows, dim)
    want = O.rms_norm(x, w, eps, add_to=y0 if add else None).reshape(rows, dim)
    if rows:
        assert H.max_abs(got, want) < 2e-5 * max(1.0, float(np.abs(want).max()))
        assert H.rel_l2(got, want) < 1e-6


@pytest.mark.parametrize("rows,shared", [(1, False), (1, True), (3, False), (20, False), (40, False)])
def test_norm_moe_residual_chain_folds_into_the_moe_kernels(be, rows, shared):
    """RmsNorm -> MoeFfn [-> shared expert -> Add] -> Add(residual), the FFN sublayer the model emits
    (crates/infr-llama/src/seam/runner.rs:8037-8174).  On one token row the norm rides in the logits
    kernel (crates/infr-core/src/fusion.rs:15-19) and on every path the residual Add rides in the combine
    (fusion.rs:20-24); the folded chain must give the bits of the ops run one graph at a time."""
    ne, nff, E, K = 1024, 512, 16, 4
    rng = np.random.default_rng(700 + rows)
    x = (rng.standard_normal((rows, ne)) * 2).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    eg, eu = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
    ed = _realistic(rng, E, ne, nff, H.Q6K)
    wg, wu = _realistic(rng, 1, nff, ne, H.Q4K), _realistic(rng, 1, nff, ne, H.Q4K)
    wd = _realistic(rng, 1, ne, nff, H.Q6K)
    eps = 1e-6

    def graph(folded, xn_given=None):
        """folded: the whole chain in one graph with single-use Internal temporaries.  Otherwise the norm
        has already run (xn_given) and the routed sum is an Output, so nothing folds."""
        g = M.Graph()
        xi = g.input(TensorDesc([rows, ne], DType.F32))
        nwt = g.weight(TensorDesc([ne], DType.F32))
        rt = g.weight(TensorDesc([E, ne], DType.F32))
        egt, eut = g.weight(TensorDesc([E, nff, ne], DType.Q4K)), g.weight(TensorDesc([E, nff, ne], DType.Q4K))
        edt = g.weight(TensorDesc([E, ne, nff], DType.Q6K))
        pairs = [(xi, x), (rt, router), (egt, eg), (eut, eu), (edt, ed)]
        if folded:
            xn = g.internal(TensorDesc([rows, ne], DType.F32))
            g.rms_norm(x=xi, weight=nwt, dst=xn, rows=rows, dim=ne, eps=eps)
            pairs.append((nwt, nw))
        else:
            xn = g.input(TensorDesc([rows, ne], DType.F32))
            pairs.append((xn, xn_given))
        extra_out = []
        moe = g.internal(TensorDesc([rows, ne], DType.F32)) if folded else g.output(TensorDesc([rows, ne], DType.F32))
        if not folded:
            extra_out.append(moe)
        g.moe_ffn(x=xn, router=rt, gate_exps=egt, up_exps=eut, down_exps=edt, dst=moe, ne=ne, n_expert=E, n_used=K,
                  n_ff_exp=nff)
        sub = moe
        if shared:
            wgt, wut = g.weight(TensorDesc([nff, ne], DType.Q4K)), g.weight(TensorDesc([nff, ne], DType.Q4K))
            wdt = g.weight(TensorDesc([ne, nff], DType.Q6K))
            gt, ut = g.internal(TensorDesc([rows, nff], DType.F32)), g.internal(TensorDesc([rows, nff], DType.F32))
            at, st = g.internal(TensorDesc([rows, nff], DType.F32)), g.internal(TensorDesc([rows, ne], DType.F32))
            sub = g.internal(TensorDesc([rows, ne], DType.F32)) if folded else g.output(TensorDesc([rows, ne], DType.F32))
            if not folded:
                extra_out.append(sub)
            g.linear(x=xn, weight=wgt, dst=gt, m=rows, in_f=ne, out_f=nff)
            g.linear(x=xn, weight=wut, dst=ut, m=rows, in_f=ne, out_f=nff)
            g.gated_act(gate=gt, up=ut, dst=at, rows=rows, nff=nff)
            g.linear(x=at, weight=wdt, dst=st, m=rows, in_f=nff, out_f=ne)
            g.add(a=moe, b=st, dst=sub, n=rows * ne)
            pairs += [(wgt, wg), (wut, wu), (wdt, wd)]
        yi = g.output(TensorDesc([rows, ne], DType.F32))
        g.add(a=xi, b=sub, dst=yi, n=rows * ne)
        return g, pairs, extra_out, yi

    def run(folded, xn_given=None):
        g, pairs, extra_out, yi = graph(folded, xn_given)
        plan = be.compile(g)
        bufs, b = [], M.Bindings()
        for tid, v in pairs:
            bufs.append(be.buffer_from(v))
            b.bind(tid, bufs[-1])
        for tid in extra_out + [yi]:
            bufs.append(be.alloc(rows * ne * 4))
            b.bind(tid, bufs[-1])
        be.prof_enable(True)
        be.execute(plan, b)
        out = be.download(bufs[-1], rows * ne * 4, np.float32)
        names = set(be.prof_read())
        be.prof_enable(False)
        moe_op = 1 if folded else 0
        routing = be.moe_routing(plan, moe_op)
        for buf in bufs:
            buf.free()
        plan.free()
        return out, names, routing

    # the norm on its own
    g0 = M.Graph()
    x0, w0 = g0.input(TensorDesc([rows, ne], DType.F32)), g0.weight(TensorDesc([ne], DType.F32))
    y0 = g0.output(TensorDesc([rows, ne], DType.F32))
    g0.rms_norm(x=x0, weight=w0, dst=y0, rows=rows, dim=ne, eps=eps)
    xn_dev = M.run_graph(be, g0, [(x0, x), (w0, nw)], y0, rows * ne).reshape(rows, ne)

    folded, fnames, r1 = run(True)
    plain, pnames, r2 = run(False, xn_dev)
    assert "add" not in fnames and "add" in pnames
    if rows == 1:
        assert "rms_norm_router_logits" in fnames and "rms_norm" not in fnames and "router_logits" not in fnames
        if shared:
            assert {"moe_route_gate_up_shared", "moe_down_combine_shared"} <= fnames and "linear_add" not in fnames
    else:
        assert "rms_norm" in fnames and "router_logits" in fnames
    assert np.array_equal(r1["idx"], r2["idx"]) and np.array_equal(bits(r1["w"]), bits(r2["w"]))
    assert np.array_equal(bits(folded), bits(plain))

    # against the oracle, routed from the device's normalised rows so that a last-place difference
    # of the norm cannot flip a near-tie of the selection
    assert H.rel_l2(xn_dev, O.rms_norm(x, nw, eps).reshape(rows, ne)) < 1e-6
    want = O.moe_ffn(xn_dev, router, eg, eu, ed, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K,
                     down_dtype=H.Q6K)
    assert np.array_equal(r1["idx"], want["idx"])
    sub = want["dst"]
    if shared:
        og, ou = O.linear(xn_dev, wg, H.Q4K, ne, nff), O.linear(xn_dev, wu, H.Q4K, ne, nff)
        sub = O.add(sub, O.linear(O.gated_act_rows(og, ou), wd, H.Q6K, nff, ne))
    want_y = O.add(x, sub).reshape(rows, ne)
    tol = 1e-2 if rows >= 32 else REL_L2
    assert H.rel_l2(folded.reshape(rows, ne) - x, want_y - x) < tol


@pytest.mark.parametrize("m", [1, 3, 6])
def test_linear_sweep_over_every_decoded_weight_format(be, m):
    """The reference's weight-format sweep for Op::Linear (crates/infr-testkit/src/lib.rs:389-403: every
    format as a LinearCase at one shape, seeds 0x201 + i) over the formats this backend decodes, at the
    sweep's 256 x 8 shape and at a decode-sized one; reference-mode tolerance (decode_parity.rs:93-102)."""
    for i, dt in enumerate(DECODED):
        for in_f, out_f in ((256, 8), (2048, 96)):
            raw = H.synth_weight(dt, out_f * in_f, seed=0x201 + i)
            x = H.rand_f32(m * in_f, 0x301 + i).reshape(m, in_f)
            g = M.Graph()
            xi, wi = g.input(TensorDesc([m, in_f], DType.F32)), g.weight(TensorDesc([out_f, in_f], DType(dt)))
            yi = g.output(TensorDesc([m, out_f], DType.F32))
            g.linear(x=xi, weight=wi, dst=yi, m=m, in_f=in_f, out_f=out_f)
            got = M.run_graph(be, g, [(xi, x), (wi, raw)], yi, m * out_f).reshape(m, out_f)
            want = O.linear(x, raw, dt, in_f, out_f)
            assert H.rel_l2(got, want) < 1e-5, (DType(dt).name, in_f)


@pytest.mark.parametrize("dt", [H.F32, H.F16, H.BF16])
@pytest.mark.parametrize("m,in_f,out_f", [(1, 2048, 96), (3, 4096, 37), (6, 264, 8), (1, 100, 5)])
def test_linear_on_float_weights(be, dt, m, in_f, out_f):
    """Unquantised weight matrices (norm-adjacent projections, F16 heads): 16-byte loads when the row pitch
    allows, the element-wise kernel otherwise (in_f = 100: a 200-byte F16 row)."""
    rng = np.random.default_rng(in_f + m)
    w32 = (rng.standard_normal(out_f * in_f) * 0.1).astype(np.float32)
    raw = w32 if dt == H.F32 else w32.astype(np.float16) if dt == H.F16 else (w32.view(np.uint32) >> 16).astype(np.uint16)
    x = rng.standard_normal((m, in_f)).astype(np.float32)
    g = M.Graph()
    xi, wi = g.input(TensorDesc([m, in_f], DType.F32)), g.weight(TensorDesc([out_f, in_f], DType(dt)))
    yi = g.output(TensorDesc([m, out_f], DType.F32))
    g.linear(x=xi, weight=wi, dst=yi, m=m, in_f=in_f, out_f=out_f)
    got = M.run_graph(be, g, [(xi, x), (wi, raw)], yi, m * out_f).reshape(m, out_f)
    want = O.linear(x, raw, dt, in_f, out_f)
    assert H.rel_l2(got, want) < 1e-5


@pytest.mark.parametrize("dt,m,in_f,out_f", [(H.Q4K, 140, 512, 100), (H.Q6K, 300, 768, 2048), (H.Q8_0, 129, 2048, 256),
                                             (H.Q5K, 128, 512, 96), (H.Q4_0, 200, 192, 300), (H.Q3K, 133, 256, 40),
                                             (H.Q4K, 2048, 4096, 1536), (H.Q4_1, 150, 96, 64), (H.F16, 170, 256, 64),
                                             (H.BF16, 130, 320, 100), (H.F32, 260, 128, 300), (H.F16, 140, 100, 64),
                                             (H.Q4K, 100, 512, 64), (H.MXFP4, 160, 2880, 96), (H.IQ4_XS, 130, 512, 64),
                                             (H.NVFP4, 140, 192, 50), (H.TQ2_0, 128, 256, 40), (H.IQ4_NL, 131, 96, 64),
                                             (H.IQ2_XXS, 130, 512, 64), (H.IQ2_XS, 129, 256, 40), (H.IQ2_S, 140, 768, 50),
                                             (H.IQ3_XXS, 128, 256, 96), (H.IQ3_S, 150, 512, 33), (H.IQ1_S, 131, 256, 64),
                                             (H.IQ1_M, 160, 1024, 48)])
def test_linear_with_a_batch_of_rows_runs_on_the_matrix_cores(be, dt, m, in_f, out_f):
    """Op::Linear from 128 rows on (a prefill chunk through a dense projection or the shared expert): the rows
    are one bucket of the grouped GEMMs, f16 operands with a power-of-two scale per row, bar 1e-2 per row.
    Unquantised weights are rounded to f16 operands.  Widths that are no whole 64-k slice stay on the f32 kernels."""
    rng = np.random.default_rng(m + in_f)
    x = rng.standard_normal((m, in_f)).astype(np.float32)
    x[m // 2] *= 3.0e4
    x[m // 3] *= 1.0e-5
    if dt in (H.F16, H.BF16, H.F32):
        w32 = (rng.standard_normal(out_f * in_f) * 0.02).astype(np.float32)
        raw = w32 if dt == H.F32 else w32.astype(np.float16) if dt == H.F16 else (w32.view(np.uint32) >> 16).astype(np.uint16)
    else:
        raw = H.centred_weight(dt, out_f * in_f, 5)
    g = M.Graph()
    xi, wi = g.input(TensorDesc([m, in_f], DType.F32)), g.weight(TensorDesc([out_f, in_f], DType(dt)))
    yi = g.output(TensorDesc([m, out_f], DType.F32))
    g.linear(x=xi, weight=wi, dst=yi, m=m, in_f=in_f, out_f=out_f)
    be.prof_enable(True)
    got = M.run_graph(be, g, [(xi, x), (wi, raw)], yi, m * out_f).reshape(m, out_f)
    be.sync()
    names = set(be.prof_read())
    be.prof_enable(False)
    want = O.linear(x, raw, dt, in_f, out_f)
    mfma = in_f % 64 == 0 and m >= 128
    assert (("linear_grouped" in names or "linear_grouped_units" in names) and "linear" not in names) if mfma else names == {"linear"}
    for r in range(m):
        assert H.rel_l2(got[r], want[r]) < (REL_L2_MFMA if mfma else 1e-5), r


def test_batched_linear_reads_a_row_band_of_a_concatenated_weight(be):
    """w_off selects rows [w_off / in_f, + out_f) of a larger weight tensor (graph.rs:208-211), on the matrix-core
    form as on the GEMV form: both bands of a 2 x out_f matrix, against the oracle and against each other's rows."""
    m, in_f, out_f = 150, 512, 96
    rng = np.random.default_rng(77)
    x = rng.standard_normal((m, in_f)).astype(np.float32)
    raw = H.centred_weight(H.Q4K, 2 * out_f * in_f, 8)
    outs = []
    for band in (0, 1):
        g = M.Graph()
        xi, wi = g.input(TensorDesc([m, in_f], DType.F32)), g.weight(TensorDesc([2 * out_f, in_f], DType.Q4K))
        yi = g.output(TensorDesc([m, out_f], DType.F32))
        g.linear(x=xi, weight=wi, dst=yi, m=m, in_f=in_f, out_f=out_f, w_off=band * out_f * in_f)
        got = M.run_graph(be, g, [(xi, x), (wi, raw)], yi, m * out_f).reshape(m, out_f)
        want = O.linear(x, raw, H.Q4K, in_f, out_f, w_off=band * out_f * in_f)
        assert H.rel_l2(got, want) < REL_L2_MFMA
        outs.append(got)
    assert not np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("gdt,ddt,rows,ne,nff", [
    (H.Q5K, H.Q5K, 1, 512, 256), (H.Q4_0, H.Q5_0, 2, 512, 256), (H.Q2K, H.Q3K, 1, 512, 256), (H.Q4_1, H.Q5_1, 3, 512, 256),
    (H.Q3K, H.Q2K, 5, 512, 256), (H.Q5_1, H.Q4_0, 1, 512, 256),
    (H.Q5K, H.Q6K, 40, 512, 256), (H.Q4_0, H.Q4_1, 77, 512, 256), (H.Q5K, H.Q5K, 300, 512, 256), (H.Q2K, H.Q3K, 130, 256, 512),
    (H.Q5_0, H.Q5_1, 64, 192, 320), (H.Q8_0, H.Q4_0, 33, 2048, 64),
    (H.Q4_0, H.Q5_0, 40, 480, 96), (H.Q4_1, H.Q4_1, 70, 96, 32),
    (H.MXFP4, H.MXFP4, 1, 512, 256), (H.MXFP4, H.MXFP4, 64, 512, 256), (H.IQ4_XS, H.IQ4_NL, 3, 512, 256),
    (H.IQ4_NL, H.IQ4_XS, 40, 512, 256), (H.NVFP4, H.Q2_0, 2, 512, 256), (H.TQ2_0, H.TQ1_0, 5, 512, 256),
    (H.TQ1_0, H.TQ2_0, 50, 256, 256), (H.Q2_0, H.NVFP4, 35, 192, 320), (H.MXFP4, H.IQ4_NL, 40, 480, 96),
    (H.Q4K, H.Q5K, 48, 512, 256), (H.Q8_0, H.Q5K, 40, 512, 256), (H.Q6K, H.Q4_1, 36, 256, 256)])
def test_moe_ffn_with_experts_in_the_other_affine_formats(be, gdt, ddt, rows, ne, nff):
    """Expert banks in formats without an integer-dot kernel.  Up to 31 rows: the 32-element-unit GEMV kernels,
    one block column per (row, rank) pair (f32, bar 1e-3).  From 32 rows: bucketing + the unit-decoder grouped
    GEMM on the matrix cores (f16 operands, bar 1e-2) when both contraction lengths are whole 64-k slices,
    otherwise the unit GEMV over the expert buckets (f32).  Same routing everywhere."""
    E, K = 8, 3
    rng = np.random.default_rng(gdt * 17 + ddt + rows)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    if rows > 4:
        x[rows // 2] *= 2.0e4    # far outside the f16 range: the per-row scale must absorb it
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    gate, up = H.centred_weight(gdt, E * nff * ne, 1), H.centred_weight(gdt, E * nff * ne, 2)
    down = H.centred_weight(ddt, E * ne * nff, 3)
    g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
    keep = []
    got = M.run_graph(be, g, [(ids["x"], x), (ids["router"], router), (ids["gate"], gate), (ids["up"], up),
                              (ids["down"], down)], ids["dst"], rows * ne, keep=keep).reshape(rows, ne)
    routing = be.moe_routing(keep[0], 0)
    want = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    assert np.array_equal(routing["idx"], want["idx"])
    be.prof_enable(True)
    be.execute(keep[0], keep[1])
    be.sync()
    names = set(be.prof_read())
    be.prof_enable(False)
    mfma = rows >= 32 and ne % 64 == 0 and nff % 64 == 0
    wd = want["dst"].reshape(rows, ne)
    for r in range(rows):   # per row: a row scaled by 2e4 must not drown the others
        assert H.rel_l2(got[r], wd[r]) < (REL_L2_MFMA if mfma else REL_L2), r
    if mfma:
        assert {"moe_grouped_units_gate_up", "moe_grouped_units_down", "moe_unbucket_combine"} <= names
        b = be.moe_bucketing(keep[0], 0)
        _check_bucketing(b, want, E)
    elif rows >= 32:   # batches walk the expert buckets on the f32 unit kernels
        assert {"moe_gate_up_units_bucketed", "moe_down_units_bucketed", "moe_unbucket_combine"} <= names
    else:
        # routing rides in the gate/up kernel while rows * n_expert <= 512 (as on the integer-dot kernels)
        assert ("moe_route_gate_up_units" if rows * E <= 512 else "moe_gate_up_units") in names
        assert ("route_topk" in names) == (rows * E > 512) and (("moe_down_combine_units" if rows <= 2 else "moe_down_units") in names or ddt == H.Q6K)
    keep[0].free()
    for buf in keep[2] + [keep[3]]:
        buf.free()


@pytest.mark.parametrize("rows,grouped", [(48, False), (49, True)])
def test_sparse_batches_of_unit_formats_stay_on_the_per_pair_gemv(be, rows, grouped):
    """A batch that selects each expert one and a half times or less (2 * rows * n_used <= 3 * n_expert) fills no
    tile of the grouped GEMM: banks in the unit formats then run the per-pair GEMV (f32, bar 1e-3) whatever the
    row count."""
    ne, nff, E, K = 256, 256, 64, 2
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    gate, up = H.centred_weight(H.MXFP4, E * nff * ne, 1), H.centred_weight(H.MXFP4, E * nff * ne, 2)
    down = H.centred_weight(H.IQ4_XS, E * ne * nff, 3)
    g, ids = moe_graph(rows, ne, E, K, nff, DType.Mxfp4, DType.Iq4Xs)
    keep = []
    be.prof_enable(True)
    got = M.run_graph(be, g, [(ids["x"], x), (ids["router"], router), (ids["gate"], gate), (ids["up"], up),
                              (ids["down"], down)], ids["dst"], rows * ne, keep=keep).reshape(rows, ne)
    be.sync()
    names = set(be.prof_read())
    be.prof_enable(False)
    want = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.MXFP4, down_dtype=H.IQ4_XS)
    assert np.array_equal(be.moe_routing(keep[0], 0)["idx"], want["idx"])
    assert ("moe_grouped_units_gate_up" in names) == grouped and ("moe_gate_up_units" in names) == (not grouped)
    wd = want["dst"].reshape(rows, ne)
    for r in range(rows):
        assert H.rel_l2(got[r], wd[r]) < (REL_L2_MFMA if grouped else REL_L2), r
    keep[0].free()
    for buf in keep[2] + [keep[3]]:
        buf.free()


# ------------------------------------------------------------------ synthetic workloads at full size
from moe4all_amd import synth as S  # noqa: E402


@pytest.mark.parametrize("dt", [DType.F32, DType.Q8_0, DType.Q4K, DType.Q6K, DType.Mxfp4])
def test_device_generator_writes_the_host_generator_bytes(be, dt):
    numel = 256 * 1000
    seed = S.stream_seed(42, 7, int(dt))
    buf = be.alloc_uninit(M.backend.bytes_for(dt, numel))
    S.weights_device(be, buf, dt, seed, numel)
    dev = be.download(buf)
    buf.free()
    host = S.weights_host(dt, seed, numel).view(np.uint8)
    assert np.array_equal(dev, host), f"{int((dev != host).sum())} differing bytes"


@pytest.mark.parametrize("shape,batch", [(S.CONFIG_1, 1), (S.CONFIG_2, 1), (S.CONFIG_1, 4), (S.CONFIG_1, 16),
                                         (S.CONFIG_2, 8), (S.CONFIG_5, 1), (S.CONFIG_5, 8), (S.CONFIG_MXFP4, 1),
                                         (S.CONFIG_MXFP4, 8)])
def test_benchmark_config_layer_matches_oracle_at_full_size(be, shape, batch):
    """One full-size layer of each benchmark configuration: N(0,0.02) weights quantised on the
    device, N(0,1) activations; the oracle runs on the downloaded bytes."""
    lw = S.LayerWeights(be, shape, seed0=77, layer=3, on_device=True)
    s = shape
    x = S.normal(S.stream_seed(78, 3, S.ROLE_X), batch * s.ne, 1.0).reshape(batch, s.ne)
    g = M.Graph()
    xi = g.input(TensorDesc([batch, s.ne], DType.F32))
    ri = g.weight(TensorDesc([s.n_expert, s.ne], DType.F32))
    gi = g.weight(TensorDesc([s.n_expert, s.n_ff, s.ne], s.gate_dtype))
    ui = g.weight(TensorDesc([s.n_expert, s.n_ff, s.ne], s.gate_dtype))
    di = g.weight(TensorDesc([s.n_expert, s.ne, s.n_ff], s.down_dtype))
    yi = g.output(TensorDesc([batch, s.ne], DType.F32))
    b = M.Bindings().bind(ri, lw.router).bind(gi, lw.gate).bind(ui, lw.up).bind(di, lw.down)
    if s.shared_ff:
        moe = g.internal(TensorDesc([batch, s.ne], DType.F32))
        g.moe_ffn(x=xi, router=ri, gate_exps=gi, up_exps=ui, down_exps=di, dst=moe, ne=s.ne, n_expert=s.n_expert,
                  n_used=s.n_used, n_ff_exp=s.n_ff)
        sg, su = g.weight(TensorDesc([s.shared_ff, s.ne], s.gate_dtype)), g.weight(TensorDesc([s.shared_ff, s.ne], s.gate_dtype))
        sd = g.weight(TensorDesc([s.ne, s.shared_ff], s.down_dtype))
        tg, tu, ta = (g.internal(TensorDesc([batch, s.shared_ff], DType.F32)) for _ in range(3))
        ts = g.internal(TensorDesc([batch, s.ne], DType.F32))
        g.linear(x=xi, weight=sg, dst=tg, m=batch, in_f=s.ne, out_f=s.shared_ff)
        g.linear(x=xi, weight=su, dst=tu, m=batch, in_f=s.ne, out_f=s.shared_ff)
        g.gated_act(gate=tg, up=tu, dst=ta, rows=batch, nff=s.shared_ff)
        g.linear(x=ta, weight=sd, dst=ts, m=batch, in_f=s.shared_ff, out_f=s.ne)
        g.add(a=moe, b=ts, dst=yi, n=batch * s.ne)
        b.bind(sg, lw.shared[0]).bind(su, lw.shared[1]).bind(sd, lw.shared[2])
    else:
        g.moe_ffn(x=xi, router=ri, gate_exps=gi, up_exps=ui, down_exps=di, dst=yi, ne=s.ne, n_expert=s.n_expert,
                  n_used=s.n_used, n_ff_exp=s.n_ff)
    plan = be.compile(g)
    xb, yb = be.buffer_from(x, M.BufferUsage.Activations), be.alloc(batch * s.ne * 4, M.BufferUsage.Readback)
    b.bind(xi, xb).bind(yi, yb)
    be.execute(plan, b)
    got = be.download(yb, batch * s.ne * 4, np.float32).reshape(batch, s.ne)
    r = be.moe_routing(plan, 0)
    router = be.download(lw.router, dtype=np.float32)
    gate, up, down = be.download(lw.gate), be.download(lw.up), be.download(lw.down)
    ref = O.moe_ffn(x, router, gate, up, down, ne=s.ne, n_expert=s.n_expert, n_used=s.n_used, n_ff_exp=s.n_ff,
                    gate_dtype=int(s.gate_dtype), down_dtype=int(s.down_dtype))
    want = ref["dst"]
    if s.shared_ff:
        sgb, sub, sdb = (be.download(t) for t in lw.shared)
        a = O.gated_act_rows(O.linear(x, sgb, int(s.gate_dtype), s.ne, s.shared_ff),
                             O.linear(x, sub, int(s.gate_dtype), s.ne, s.shared_ff))
        want = O.add(want, O.linear(a, sdb, int(s.down_dtype), s.shared_ff, s.ne))
    assert np.array_equal(r["idx"], ref["idx"])
    assert np.array_equal(bits(r["w"]), bits(ref["w"]))
    assert 0.01 < float(np.sqrt(np.mean(want ** 2))) < 1.0   # magnitudes of the real workload
    assert H.max_abs(got, want) < MAX_ABS, H.max_abs(got, want)
    assert H.rel_l2(got, want) < REL_L2, H.rel_l2(got, want)
    for buf in (xb, yb):
        buf.free()
    plan.free()
    lw.free()


# ------------------------------------------------------------------ batched path (bucketing + grouped GEMM)
REL_L2_MFMA = 1e-2   # f16 operands on the matrix cores, f32 accumulation


def _check_bucketing(b, ref, E):
    """Bucket order is an integer contract: experts ascending, rows ascending inside a bucket."""
    counts = np.diff(b["offsets"])
    want = np.zeros(E, np.int64)
    want[ref["bucket_expert"]] = ref["bucket_count"]
    assert np.array_equal(counts, want)
    assert np.array_equal(b["offsets"][ref["bucket_expert"]], ref["bucket_p0"])
    assert np.array_equal(b["pair_row"], ref["pair_row"])
    assert np.array_equal(b["slot_pair"], ref["slot_pair"])


def _run_batched(be, g, ids, data, rows, ne):
    keep = []
    bound = [(ids[k], v) for k, v in data.items() if ids.get(k) is not None and v is not None]
    out = M.run_graph(be, g, bound, ids["dst"], rows * ne, keep=keep)
    routing = be.moe_routing(keep[0], 0)
    bucketing = be.moe_bucketing(keep[0], 0)
    for buf in keep[2]:
        buf.free()
    keep[3].free()
    keep[0].free()
    return out.reshape(rows, ne), routing, bucketing


@pytest.mark.parametrize("rows,ne,E,K,nff,gdt,ddt", [
    (64, 512, 8, 2, 256, H.Q4K, H.Q6K),
    (33, 256, 16, 4, 256, H.Q6K, H.Q4K),        # ragged tile, experts without tokens
    (40, 768, 6, 3, 512, H.Q8_0, H.Q8_0),       # three 256-feature down tiles, four 128-feature gate/up tiles
    (300, 256, 4, 2, 256, H.Q4K, H.Q8_0),       # buckets larger than one 128-token tile
    (700, 512, 3, 2, 256, H.Q4K, H.Q4K),        # buckets of 400-500 pairs: 256-token tiles, then 128-token ones, then a ragged one
    (200, 2048, 128, 8, 768, H.Q4K, H.Q6K),     # config-2 layer shape
    (128, 2048, 128, 8, 768, H.Q8_0, H.Q8_0),   # config-1 layer shape
])
def test_batched_moe_ffn_buckets_exactly_and_matches_oracle(be, rows, ne, E, K, nff, gdt, ddt):
    rng = np.random.default_rng(rows + ne + gdt)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    x[rows // 2] *= 3.0e4      # a row far outside f16 range: the per-row scale must absorb it
    x[rows // 3] *= 1.0e-6
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, nff, ne, gdt)
    down = _realistic(rng, E, ne, nff, ddt)
    g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
    out, r, b = _run_batched(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), rows, ne)
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    assert np.array_equal(r["idx"], ref["idx"])
    assert np.array_equal(bits(r["w"]), bits(ref["w"]))
    _check_bucketing(b, ref, E)
    # per-row relative error: rows differ by ten orders of magnitude
    num = np.linalg.norm((out - ref["dst"]).astype(np.float64), axis=1)
    den = np.linalg.norm(ref["dst"].astype(np.float64), axis=1)
    assert (den > 0).all()
    worst = float((num / den).max())
    assert worst < REL_L2_MFMA, worst
    assert H.rel_l2(out, ref["dst"]) < REL_L2_MFMA


@pytest.mark.parametrize("gdt,ddt", [(H.Q4K, H.Q6K), (H.Q5K, H.Q4_0)])
def test_batched_moe_ffn_option_variants_match_oracle(be, gdt, ddt):
    ne, E, K, nff, rows = 256, 8, 3, 256, 48
    rng = np.random.default_rng(23)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = rng.standard_normal((E, ne)).astype(np.float32) * 0.05
    gate, up, down = _bank_weights(rng, E, nff, ne, gdt, ddt)
    ds = rng.uniform(0.5, 1.5, E).astype(np.float32)
    bias = rng.standard_normal(E).astype(np.float32) * 0.1
    eids = rng.integers(0, E, (rows, K)).astype(np.int32)
    base = dict(ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    cases = [
        (dict(weight_before=True), dict(weight_before=True), {}),
        (dict(swiglu_clamp=0.05), dict(swiglu_clamp=0.05), {}),
        (dict(with_down_scale=True), dict(down_scale=ds), dict(down_scale=ds)),
        (dict(gating=M.MoeGating.Sigmoid, norm_w=False, scale=2.5), dict(gating=O.GATE_SIGMOID, norm_w=False, scale=2.5), {}),
        (dict(with_exp_probs_b=True, gating=M.MoeGating.Sigmoid), dict(exp_probs_b=bias, gating=O.GATE_SIGMOID), dict(exp_probs_b=bias)),
        (dict(with_expert_ids=True), dict(expert_ids=eids), dict(expert_ids=eids)),   # duplicates inside a row allowed
        (dict(act=M.Activation.Gelu), dict(act=O.ACT_GELU), {}),
    ]
    for gopts, oopts, extra in cases:
        g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt), **dict(gopts))
        out, r, b = _run_batched(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down, **extra), rows, ne)
        ref = O.moe_ffn(x, router, gate, up, down, **base, **oopts)
        assert np.array_equal(r["idx"], ref["idx"]), gopts
        _check_bucketing(b, ref, E)
        assert H.rel_l2(out, ref["dst"]) < REL_L2_MFMA, (gopts, H.rel_l2(out, ref["dst"]))
    if gdt != H.Q4K:
        # gate and up rows of an expert in one tensor: the unit-decoder GEMM takes that layout on the matrix cores too
        gu = np.concatenate([gate.reshape(E, -1), up.reshape(E, -1)], axis=1).reshape(-1)
        g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt), fused_gate_up=True)
        out, r, b = _run_batched(be, g, ids, dict(x=x, router=router, gate=gu, up=None, down=down), rows, ne)
        ref = O.moe_ffn(x, router, gu, None, down, **base, fused_gate_up=True)
        assert np.array_equal(r["idx"], ref["idx"])
        assert H.rel_l2(out, ref["dst"]) < REL_L2_MFMA


@pytest.mark.parametrize("rows,ne,E,K,nff,gdt,ddt", [
    (16, 512, 8, 2, 256, H.Q4K, H.Q6K),
    (19, 256, 16, 4, 256, H.Q6K, H.Q4K),       # experts without tokens, odd bucket sizes
    (31, 2048, 128, 8, 768, H.Q8_0, H.Q8_0),   # the largest batch below the matrix-core path
    (18, 256, 24, 17, 256, H.Q4K, H.Q6K),      # more ranks than the per-token down kernel combines: bucketed down + combine
    (70, 320, 8, 2, 96, H.Q8_0, H.Q8_0),       # ne is no multiple of 256: no matrix-core path, the bucketed GEMV takes any row count
])
def test_bucketed_decode_batches_bucket_exactly_and_keep_f32_accuracy(be, rows, ne, E, K, nff, gdt, ddt):
    """16..31 token rows: pairs are bucketed by expert and the gate/up rows of an expert serve two tokens
    per read (the down projection streams per pair); the inner product is the per-token kernels', so the
    f32 bar applies."""
    rng = np.random.default_rng(rows * 3 + ne)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, nff, ne, gdt)
    down = _realistic(rng, E, ne, nff, ddt)
    ds = rng.uniform(0.5, 1.5, E).astype(np.float32)
    eids = rng.integers(0, E, (rows, K)).astype(np.int32)
    base = dict(ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    for gopts, oopts, extra in [({}, {}, {}),
                                (dict(weight_before=True, with_down_scale=True), dict(weight_before=True, down_scale=ds), dict(down_scale=ds)),
                                (dict(with_expert_ids=True), dict(expert_ids=eids), dict(expert_ids=eids))]:
        g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt), **dict(gopts))
        out, r, b = _run_batched(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down, **extra), rows, ne)
        ref = O.moe_ffn(x, router, gate, up, down, **base, **oopts)
        assert np.array_equal(r["idx"], ref["idx"])
        _check_bucketing(b, ref, E)
        scale = float(np.abs(ref["dst"]).max())
        assert H.rel_l2(out, ref["dst"]) < REL_L2, (gopts, H.rel_l2(out, ref["dst"]))
        assert H.max_abs(out, ref["dst"]) < MAX_ABS, (gopts, H.max_abs(out, ref["dst"]), scale)


@pytest.mark.parametrize("rows,opts", [(1, {}), (3, {"weight_before": True}), (20, {}), (20, {"weight_before": True}), (40, {}),
                                       (1, {"fmt": (H.Q5K, H.Q5_0)}), (20, {"fmt": (H.Q5K, H.Q5_0)}),
                                       (40, {"fmt": (H.Q5K, H.Q5_0), "weight_before": True})])
def test_expert_parallel_bands_sum_to_the_full_layer(be, rows, opts):
    """ep_band (crates/infr-core/src/graph.rs:1307-1319, crates/infr-vulkan/shaders/moe_ep_band_remap.comp):
    routing stays global, the expert tensors hold one rank's shard, selections of foreign experts become
    (id 0, weight 0).  The partial outputs of all ranks must add up to the single-device layer, and the
    remapped ids / weights must be the shader's."""
    ne, nff, E, K, W = 512, 256, 16, 4, 2
    opts = dict(opts)
    gdt, ddt = opts.pop("fmt", (H.Q4K, H.Q6K))   # the second pair runs on the 32-element-unit kernels
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.05).astype(np.float32)
    if gdt == H.Q4K:
        gate, up = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
        down = _realistic(rng, E, ne, nff, H.Q6K)
    else:
        gate, up = H.centred_weight(gdt, E * nff * ne, 1), H.centred_weight(gdt, E * nff * ne, 2)
        down = H.centred_weight(ddt, E * ne * nff, 3)
    ds = rng.uniform(0.5, 1.5, E).astype(np.float32)

    def run(band):
        n_loc = E if band is None else band[1]
        lo = 0 if band is None else band[0]
        g = M.Graph()
        xi = g.input(TensorDesc([rows, ne], DType.F32))
        rt = g.weight(TensorDesc([E, ne], DType.F32))
        gt, ut = g.weight(TensorDesc([n_loc, nff, ne], DType(gdt))), g.weight(TensorDesc([n_loc, nff, ne], DType(gdt)))
        dt = g.weight(TensorDesc([n_loc, ne, nff], DType(ddt)))
        dst = g.weight(TensorDesc([n_loc], DType.F32))
        yo = g.output(TensorDesc([rows, ne], DType.F32))
        g.moe_ffn(x=xi, router=rt, gate_exps=gt, up_exps=ut, down_exps=dt, dst=yo, ne=ne, n_expert=E, n_used=K,
                  n_ff_exp=nff, down_scale=dst, ep_band=band, **opts)
        shard = lambda raw: raw.reshape(E, -1)[lo:lo + n_loc].reshape(-1)
        keep = []
        out = M.run_graph(be, g, [(xi, x), (rt, router), (gt, shard(gate)), (ut, shard(up)), (dt, shard(down)),
                                  (dst, ds[lo:lo + n_loc].copy())], yo, rows * ne, keep=keep)
        r = be.moe_routing(keep[0], 0)
        for buf in keep[2]:
            buf.free()
        keep[3].free()
        keep[0].free()
        return out.reshape(rows, ne), r

    full, rf = run(None)
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt,
                    down_dtype=ddt, down_scale=ds, **opts)
    assert np.array_equal(rf["idx"], ref["idx"])
    total = np.zeros_like(full)
    for rank in range(W):
        lo, n = rank * (E // W), E // W
        part, rp = run((lo, n))
        own = (rf["idx"] >= lo) & (rf["idx"] < lo + n)
        assert np.array_equal(rp["idx"], np.where(own, rf["idx"] - lo, 0))
        assert np.array_equal(bits(rp["w"]), bits(np.where(own, rf["w"], np.float32(0))))
        total += part
    tol = REL_L2_MFMA if rows >= 32 else REL_L2
    assert H.rel_l2(total, ref["dst"]) < tol
    assert H.rel_l2(total, full) < 1e-5   # the ranks' sum differs from one device only by reassociation


def test_small_batches_keep_the_per_token_path(be):
    g, ids = moe_graph(4, 256, 8, 2, 256, DType.Q4K, DType.Q6K)
    plan = be.compile(g)
    with pytest.raises(M.BackendError):
        be.moe_bucketing(plan, 0)
    plan.free()


@pytest.mark.parametrize("tokens,gdt,ddt", [(512, DType.Q8_0, DType.Q8_0), (512, DType.Q4K, DType.Q6K)])
def test_prefill_chunk_with_skewed_routing_matches_oracle(be, tokens, gdt, ddt):
    """Config-4 shape: one config-1 layer, Zipf(1.1) expert popularity injected through the op's own
    inputs (x[:,0] = 1, router[:,0] = bias), device-generated weights."""
    s = S.MoeShape("c4", 1, 2048, 128, 8, 768, gdt, ddt)
    lw = S.LayerWeights(be, s, seed0=91, layer=0, on_device=True)
    router = be.download(lw.router, dtype=np.float32).reshape(s.n_expert, s.ne).copy()
    router[:, 0] = S.zipf_bias(s.n_expert, 1.1, 5)
    be.upload(lw.router, router)
    x = S.normal(S.stream_seed(92, 0, S.ROLE_X), tokens * s.ne, 1.0).reshape(tokens, s.ne).copy()
    x[:, 0] = 1.0
    g, ids = moe_graph(tokens, s.ne, s.n_expert, s.n_used, s.n_ff, gdt, ddt)
    plan = be.compile(g)
    xb, yb = be.buffer_from(x, M.BufferUsage.Activations), be.alloc(tokens * s.ne * 4, M.BufferUsage.Readback)
    bnd = (M.Bindings().bind(ids["x"], xb).bind(ids["router"], lw.router).bind(ids["gate"], lw.gate)
           .bind(ids["up"], lw.up).bind(ids["down"], lw.down).bind(ids["dst"], yb))
    be.execute(plan, bnd)
    got = be.download(yb, tokens * s.ne * 4, np.float32).reshape(tokens, s.ne)
    r, b = be.moe_routing(plan, 0), be.moe_bucketing(plan, 0)
    gate, up, down = be.download(lw.gate), be.download(lw.up), be.download(lw.down)
    ref = O.moe_ffn(x, router, gate, up, down, ne=s.ne, n_expert=s.n_expert, n_used=s.n_used, n_ff_exp=s.n_ff,
                    gate_dtype=int(gdt), down_dtype=int(ddt))
    assert np.array_equal(r["idx"], ref["idx"])
    _check_bucketing(b, ref, s.n_expert)
    counts = np.diff(b["offsets"])
    assert counts.max() > 4 * max(1, int(np.median(counts))), "routing is not skewed"
    assert H.rel_l2(got, ref["dst"]) < REL_L2_MFMA, H.rel_l2(got, ref["dst"])
    plan.free()


@pytest.mark.parametrize("gdt,ddt", [(DType.Q4K, DType.Q6K), (DType.Q8_0, DType.Q8_0)])
def test_prefill_rows_do_not_depend_on_their_neighbours(be, gdt, ddt):
    """Properties that hold at any size, checked at the full 2048-token chunk of the config-4 shape:
    a token's output row is a function of that row alone, so (1) shuffling the tokens shuffles the output rows
    bit for bit although every expert bucket and GEMM tile is composed differently, (2) a prefix of the chunk
    run on its own gives the bits it gives inside the chunk, and (3) a token repeated in the chunk gives
    the same row each time."""
    tokens = 2048
    s = S.MoeShape("c4", 1, 2048, 128, 8, 768, gdt, ddt)
    lw = S.LayerWeights(be, s, seed0=17, layer=0, on_device=True)
    router = be.download(lw.router, dtype=np.float32).reshape(s.n_expert, s.ne).copy()
    router[:, 0] = S.zipf_bias(s.n_expert, 1.1, 9)
    be.upload(lw.router, router)
    x = S.normal(S.stream_seed(18, 0, S.ROLE_X), tokens * s.ne, 1.0).reshape(tokens, s.ne).copy()
    x[:, 0] = 1.0
    x[1500] = x[3]          # a repeated token
    x[77] *= 1.0e3          # rows of very different magnitude share tiles
    x[78] *= 1.0e-4

    def run(xin):
        n = xin.shape[0]
        g, ids = moe_graph(n, s.ne, s.n_expert, s.n_used, s.n_ff, gdt, ddt)
        plan = be.compile(g)
        xb, yb = be.buffer_from(xin, M.BufferUsage.Activations), be.alloc(n * s.ne * 4, M.BufferUsage.Readback)
        bnd = (M.Bindings().bind(ids["x"], xb).bind(ids["router"], lw.router).bind(ids["gate"], lw.gate)
               .bind(ids["up"], lw.up).bind(ids["down"], lw.down).bind(ids["dst"], yb))
        be.execute(plan, bnd)
        out = be.download(yb, n * s.ne * 4, np.float32).reshape(n, s.ne).copy()
        idx = be.moe_routing(plan, 0)["idx"].copy()
        buckets.append(be.moe_bucketing(plan, 0))
        plan.free()
        xb.free()
        yb.free()
        return out, idx

    buckets = []
    full, idx = run(x)
    assert np.isfinite(full).all()
    # the whole chunk against the oracle: ids and the bucket order of all 2048 tokens bit for bit (they depend on the
    # router alone, so the oracle runs with one-feature dummy experts), and the output rows of a sample of 96 tokens
    # (the oracle on x[sample] alone: rows are independent, which the rest of this test shows for the device)
    dummy = np.zeros(s.n_expert * s.ne, np.float32)
    rt = O.moe_ffn(x, router, dummy, dummy, dummy, ne=s.ne, n_expert=s.n_expert, n_used=s.n_used, n_ff_exp=1)
    assert np.array_equal(idx, rt["idx"])
    _check_bucketing(buckets[0], rt, s.n_expert)
    sample = np.unique(np.concatenate([[0, 3, 77, 78, 1500, tokens - 1], np.random.default_rng(5).choice(tokens, 90, replace=False)]))
    assert len(sample) >= 64
    gate, up, down = be.download(lw.gate), be.download(lw.up), be.download(lw.down)
    ref = O.moe_ffn(x[sample], router, gate, up, down, ne=s.ne, n_expert=s.n_expert, n_used=s.n_used, n_ff_exp=s.n_ff,
                    gate_dtype=int(gdt), down_dtype=int(ddt))
    assert np.array_equal(ref["idx"], idx[sample])
    for i, t in enumerate(sample):
        assert H.rel_l2(full[t], ref["dst"][i]) < REL_L2_MFMA, (int(t), H.rel_l2(full[t], ref["dst"][i]))
    perm = np.random.default_rng(3).permutation(tokens)
    shuffled, idx_p = run(np.ascontiguousarray(x[perm]))
    assert np.array_equal(idx_p, idx[perm])
    assert np.array_equal(bits(shuffled), bits(full[perm]))
    head, _ = run(np.ascontiguousarray(x[:700]))
    assert np.array_equal(bits(head), bits(full[:700]))
    assert np.array_equal(bits(full[1500]), bits(full[3]))


@pytest.mark.parametrize("shape_name", ["c2", "c5"])
def test_decode_rows_give_the_same_bits_in_any_batch(be, shape_name):
    """At the full layer shapes: a token row alone (routing inside the gate/up kernel), inside a batch of 8
    (staged per-token kernels, separate routing launch) and inside a batch of 20 (bucketed GEMV, two tokens of
    an expert share each weight row) runs the same inner products in the same order, so the three outputs
    agree bit for bit; so do ids and routing weights."""
    s = S.CONFIG_2 if shape_name == "c2" else S.MoeShape("c5-routed", 1, 4096, 256, 8, 1536, DType.Q4K, DType.Q6K)
    lw = S.LayerWeights(be, s, seed0=23, layer=0, on_device=True)
    x = S.normal(S.stream_seed(24, 0, S.ROLE_X), 20 * s.ne, 1.0).reshape(20, s.ne).copy()

    def run(xin):
        n = xin.shape[0]
        g, ids = moe_graph(n, s.ne, s.n_expert, s.n_used, s.n_ff, s.gate_dtype, s.down_dtype)
        plan = be.compile(g)
        xb, yb = be.buffer_from(xin, M.BufferUsage.Activations), be.alloc(n * s.ne * 4, M.BufferUsage.Readback)
        bnd = (M.Bindings().bind(ids["x"], xb).bind(ids["router"], lw.router).bind(ids["gate"], lw.gate)
               .bind(ids["up"], lw.up).bind(ids["down"], lw.down).bind(ids["dst"], yb))
        be.execute(plan, bnd)
        out = be.download(yb, n * s.ne * 4, np.float32).reshape(n, s.ne).copy()
        r = be.moe_routing(plan, 0)
        plan.free()
        xb.free()
        yb.free()
        return out, r["idx"].copy(), r["w"].copy()

    full, idx, w = run(x)
    eight, idx8, w8 = run(np.ascontiguousarray(x[:8]))
    assert np.array_equal(idx8, idx[:8]) and np.array_equal(bits(w8), bits(w[:8]))
    assert np.array_equal(bits(eight), bits(full[:8]))
    for r in (0, 7, 19):
        one, idx1, w1 = run(np.ascontiguousarray(x[r:r + 1]))
        assert np.array_equal(idx1[0], idx[r]) and np.array_equal(bits(w1[0]), bits(w[r]))
        assert np.array_equal(bits(one[0]), bits(full[r])), r


def test_batched_threshold_is_configurable_and_the_paths_agree():
    """moe_batched_min_rows moves the switch to the matrix-core path; with it out of reach a 48-row batch
    runs the bucketed f32-accurate kernels and must meet the f32 bar, with it at 1 even two rows take
    the grouped GEMMs; both bucket identically."""
    rows, ne, E, K, nff = 48, 512, 8, 2, 256
    rng = np.random.default_rng(5)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
    down = _realistic(rng, E, ne, nff, H.Q6K)
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
    outs = {}
    for name, min_rows, bar in (("gemv", 1000, REL_L2), ("mfma", 1, REL_L2_MFMA)):
        be2 = M.Backend(0, moe_batched_min_rows=min_rows)
        try:
            g, ids = moe_graph(rows, ne, E, K, nff, DType.Q4K, DType.Q6K)
            out, r, b = _run_batched(be2, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), rows, ne)
            assert np.array_equal(r["idx"], ref["idx"])
            _check_bucketing(b, ref, E)
            assert H.rel_l2(out, ref["dst"]) < bar, (name, H.rel_l2(out, ref["dst"]))
            outs[name] = out
        finally:
            be2.close()
    assert H.rel_l2(outs["mfma"], outs["gemv"]) < REL_L2_MFMA


@pytest.mark.parametrize("three_launch,tie", [(False, False), (True, False), (True, True)])
def test_routing_of_logits_a_few_dozen_ulp_apart_is_the_stable_sort_of_the_probabilities(be, three_launch, tie):
    """Logits 40 ulp apart: inside the selection the higher logit ranks first although its id is higher, and at the
    selection's edge it decides which expert is in.  A selection on truncated or rounded keys would get both wrong;
    the contract is the reference's stable descending sort of the probabilities (crates/infr-cpu/src/lib.rs:3847-3850)."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(77)
    x = np.zeros((1, ne), np.float32)
    x[0, 0] = 1.0                       # logits = router[:, 0]
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    col = (rng.standard_normal(E) * 0.05).astype(np.float32)

    def up_ulps(v, n):
        return (np.float32(v).view(np.uint32) + np.uint32(n)).view(np.float32)

    col[[3, 17, 40, 41, 60]] = [3.0, 2.5, 2.25, 2.0, 1.75]
    col[5] = 2.75
    col[9] = up_ulps(2.75, 40)          # 9 before 5
    col[20] = 1.25
    col[30] = up_ulps(1.25, 40)         # 30 is rank 8 and 20 is out
    want = [3, 9, 5, 17, 40, 41, 60, 30]
    if tie:                             # two equal logits at the selection's edge: the smaller id is in, the other out
        col[60] = col[70] = 1.25
        want = [3, 9, 5, 17, 40, 41, 30, 20]
    router[:, 0] = col
    if three_launch:                    # routing inside the gate/up kernel (sum and selection on two wavefronts)
        be = M.Backend(0, disable_single_launch_moe=True)
    gate, up = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
    down = _realistic(rng, E, ne, nff, H.Q6K)
    g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
    try:
        out, r = run_moe(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), 1, ne)
    finally:
        if three_launch:
            be.close()
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
    assert ref["idx"][0].tolist() == want
    assert np.array_equal(r["idx"], ref["idx"]) and np.array_equal(bits(r["w"]), bits(ref["w"]))
    assert H.rel_l2(out, ref["dst"]) < REL_L2 and H.max_abs(out, ref["dst"]) < MAX_ABS


@pytest.mark.parametrize("rows", [1, 20])
def test_non_finite_activations_reach_the_output(be, rows):
    """An f32 dot product over a NaN or an infinity is not finite (the reference's path, crates/infr-cpu/src/moe.rs:142-173);
    the fixed-point staging of the integer-dot kernels must not turn such an activation into zero.  The router reads a
    clean copy of the rows (Op::MoeFfn.router_x), so the routing stays defined and only the expert dots see them."""
    ne, E, K, nff = 512, 8, 2, 256
    rng = np.random.default_rng(3)
    clean = rng.standard_normal((rows, ne)).astype(np.float32)
    x = clean.copy()
    x[0, 37] = np.nan
    x[rows - 1, 300] = np.inf
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
    down = _realistic(rng, E, ne, nff, H.Q6K)
    g = M.Graph()
    tx, trx = g.input(TensorDesc([rows, ne], DType.F32)), g.input(TensorDesc([rows, ne], DType.F32))
    tr = g.weight(TensorDesc([E, ne], DType.F32))
    tg, tu = g.weight(TensorDesc([E, nff, ne], DType.Q4K)), g.weight(TensorDesc([E, nff, ne], DType.Q4K))
    td = g.weight(TensorDesc([E, ne, nff], DType.Q6K))
    dst = g.output(TensorDesc([rows, ne], DType.F32))
    g.moe_ffn(x=tx, router_x=trx, router=tr, gate_exps=tg, up_exps=tu, down_exps=td, dst=dst, ne=ne, n_expert=E, n_used=K,
              n_ff_exp=nff)
    out = M.run_graph(be, g, [(tx, x), (trx, clean), (tr, router), (tg, gate), (tu, up), (td, down)], dst, rows * ne)
    out = out.reshape(rows, ne)
    with np.errstate(all="ignore"):
        ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K,
                        router_x=clean)["dst"]
    assert not np.isfinite(ref[0]).any() and not np.isfinite(ref[rows - 1]).any()
    assert not np.isfinite(out[0]).any() and not np.isfinite(out[rows - 1]).any()
    if rows > 2:
        assert np.isfinite(out[1:rows - 1]).all()
        assert H.rel_l2(out[1:rows - 1], ref[1:rows - 1]) < REL_L2


@pytest.mark.parametrize("rows,gated", [(1, False), (5, False), (1, True), (4, True)])
def test_disabling_op_fusion_changes_the_launches_not_the_bits(rows, gated):
    """infr_hip_config.disable_op_fusion (the reference keeps the same hatch for its rewrites,
    crates/infr-core/src/fusion.rs:49-52): one launch per op, identical output bits."""
    ne, nff, E, K = 512, 256, 8, 2
    rng = np.random.default_rng(31 + rows)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    eg, eu, ed = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, ne, nff, H.Q6K)
    wg, wu, wd = _realistic(rng, 1, nff, ne, H.Q4K), _realistic(rng, 1, nff, ne, H.Q4K), _realistic(rng, 1, ne, nff, H.Q6K)
    wq = (rng.standard_normal(ne) * 0.05).astype(np.float32)   # gate vector of the gated shared expert
    outs, names = {}, {}
    for off in (False, True):
        be2 = M.Backend(0, disable_op_fusion=off)
        try:
            g = M.Graph()
            xi, nwt = g.input(TensorDesc([rows, ne], DType.F32)), g.weight(TensorDesc([ne], DType.F32))
            rt = g.weight(TensorDesc([E, ne], DType.F32))
            egt, eut = g.weight(TensorDesc([E, nff, ne], DType.Q4K)), g.weight(TensorDesc([E, nff, ne], DType.Q4K))
            edt = g.weight(TensorDesc([E, ne, nff], DType.Q6K))
            wgt, wut = g.weight(TensorDesc([nff, ne], DType.Q4K)), g.weight(TensorDesc([nff, ne], DType.Q4K))
            wdt = g.weight(TensorDesc([ne, nff], DType.Q6K))
            t = lambda n: g.internal(TensorDesc([rows, n], DType.F32))  # noqa: E731
            xn, moe, gt, ut, at, st, sub = t(ne), t(ne), t(nff), t(nff), t(nff), t(ne), t(ne)
            yi = g.output(TensorDesc([rows, ne], DType.F32))
            g.rms_norm(x=xi, weight=nwt, dst=xn, rows=rows, dim=ne, eps=1e-6)
            g.moe_ffn(x=xn, router=rt, gate_exps=egt, up_exps=eut, down_exps=edt, dst=moe, ne=ne, n_expert=E, n_used=K,
                      n_ff_exp=nff)
            extra = []
            if gated:   # sigmoid(gate . x) weighs the shared expert (crates/infr-llama/src/seam/runner.rs:8104-8163)
                wqt = g.weight(TensorDesc([1, ne], DType.F32))
                logit = g.internal(TensorDesc([rows, 1], DType.F32))
                g.linear(x=xn, weight=wqt, dst=logit, m=rows, in_f=ne, out_f=1)
                extra.append((wqt, wq))
            g.linear(x=xn, weight=wgt, dst=gt, m=rows, in_f=ne, out_f=nff)
            g.linear(x=xn, weight=wut, dst=ut, m=rows, in_f=ne, out_f=nff)
            g.gated_act(gate=gt, up=ut, dst=at, rows=rows, nff=nff)
            g.linear(x=at, weight=wdt, dst=st, m=rows, in_f=nff, out_f=ne)
            if gated:
                g.moe_shared_expert_add(moe=moe, shexp=st, gate=logit, dst=sub, rows=rows, n=ne)
            else:
                g.add(a=moe, b=st, dst=sub, n=rows * ne)
            g.add(a=xi, b=sub, dst=yi, n=rows * ne)
            keep = []
            be2.prof_enable(True)
            outs[off] = M.run_graph(be2, g, [(xi, x), (nwt, nw), (rt, router), (egt, eg), (eut, eu), (edt, ed), (wgt, wg),
                                             (wut, wu), (wdt, wd)] + extra, yi, rows * ne, keep=keep)
            be2.sync()
            names[off] = set(be2.prof_read())
        finally:
            be2.close()
    assert np.array_equal(bits(outs[False]), bits(outs[True]))
    assert {"rms_norm", "add", "gated_act", "linear"} <= names[True]
    assert ("moe_shared_expert_add" in names[True]) == gated
    assert "gated_act" not in names[False]
    if rows == 1:   # the gated form keeps one launch for the gate logit
        assert names[False] == {"rms_norm_router_logits", "moe_route_gate_up_shared", "moe_down_combine_shared"} | ({"linear"} if gated else set())
    else:   # a decode batch on the per-token kernels folds the same way; its token rows are normalised by a launch of its own
        # (the routing is a launch of its own only when rows x experts is large)
        assert names[False] - {"route_topk"} == {"rms_norm", "router_logits", "moe_route_gate_up_shared", "moe_down_combine_shared"} | ({"linear"} if gated else set()), names[False]
    # and against the oracle
    xn_o = O.rms_norm(x, nw, 1e-6).reshape(rows, ne)
    moe_o = O.moe_ffn(xn_o, router, eg, eu, ed, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
    sh_o = O.linear(O.gated_act_rows(O.linear(xn_o, wg, H.Q4K, ne, nff), O.linear(xn_o, wu, H.Q4K, ne, nff)), wd, H.Q6K, nff, ne)
    sub_o = O.moe_shared_expert_add(moe_o["dst"], sh_o, O.linear(xn_o, wq, H.F32, ne, 1)) if gated else O.add(moe_o["dst"], sh_o)
    assert H.rel_l2(outs[False].reshape(rows, ne) - x, sub_o.reshape(rows, ne)) < REL_L2


@pytest.mark.gpu
def test_loads_only_probe_moves_data_without_results_and_switches_off_cleanly():
    """infr_hip_probe_grouped_loads_only: the measurement variant of the grouped GEMMs runs (same launches, same
    kernels' names), what it writes is not the layer's output, and after switching it off the backend gives the
    bits it gave before."""
    rows, ne, E, K, nff = 96, 512, 8, 2, 256
    rng = np.random.default_rng(17)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up = _realistic(rng, E, nff, ne, H.Q4K), _realistic(rng, E, nff, ne, H.Q4K)
    down = _realistic(rng, E, ne, nff, H.Q6K)
    be2 = M.Backend(0)
    try:
        data = dict(x=x, router=router, gate=gate, up=up, down=down)
        g, ids = moe_graph(rows, ne, E, K, nff, DType.Q4K, DType.Q6K)
        before, _, _ = _run_batched(be2, g, ids, data, rows, ne)
        be2.probe_grouped_loads_only(True)
        be2.prof_enable(True)
        g2, ids2 = moe_graph(rows, ne, E, K, nff, DType.Q4K, DType.Q6K)
        probed, r, _ = _run_batched(be2, g2, ids2, data, rows, ne)
        names = set(be2.prof_read())
        be2.prof_enable(False)
        be2.probe_grouped_loads_only(False)
        assert {"moe_grouped_gate_up", "moe_grouped_down"} <= names
        assert not np.array_equal(probed, before)          # no matrix work was done
        g3, ids3 = moe_graph(rows, ne, E, K, nff, DType.Q4K, DType.Q6K)
        after, _, _ = _run_batched(be2, g3, ids3, data, rows, ne)
        assert np.array_equal(after.view(np.uint32), before.view(np.uint32))
    finally:
        be2.close()



