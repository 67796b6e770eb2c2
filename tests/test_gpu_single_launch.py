"""Single-token Op::MoeFfn as one launch (moe4all_amd/csrc/k_layer.hip) against the three-launch path of the same
library and against the oracle: same ids, same routing weights, same output bits, for the shapes and options the
kernel takes; and the bounded wait of its in-kernel hand-overs, forced from the host."""
import numpy as np
import pytest

import helpers as H
import moe4all_amd as M
import oracle as O
from moe4all_amd import DType
from test_gpu_parity import _realistic, bits, moe_graph

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be3():
    """The same device with the single-launch kernel switched off."""
    b = M.Backend(0, disable_single_launch_moe=True)
    yield b
    b.close()


def _run(backend, g, ids, data, ne, want_kernel):
    keep = []
    bound = [(ids[k], v) for k, v in data.items() if ids.get(k) is not None and v is not None]
    backend.prof_enable(True)
    out = M.run_graph(backend, g, bound, ids["dst"], ne, keep=keep)
    backend.sync()
    names = set(backend.prof_read())
    backend.prof_enable(False)
    r = backend.moe_routing(keep[0], 0)
    for buf in keep[2]:
        buf.free()
    keep[3].free()
    keep[0].free()
    assert (want_kernel in names), names
    return out, r


def _graph(ne, E, K, nff, gdt, ddt, opts):
    """moe_graph, or for an expert-parallel band the same graph with expert tensors that hold the band only."""
    if "ep_band" not in opts:
        return moe_graph(1, ne, E, K, nff, DType(gdt), DType(ddt), **opts)
    n_loc = opts["ep_band"][1]
    g = M.Graph()
    x = g.input(M.TensorDesc([1, ne], DType.F32))
    router = g.weight(M.TensorDesc([E, ne], DType.F32))
    gate, up = g.weight(M.TensorDesc([n_loc, nff, ne], DType(gdt))), g.weight(M.TensorDesc([n_loc, nff, ne], DType(gdt)))
    down = g.weight(M.TensorDesc([n_loc, ne, nff], DType(ddt)))
    dst = g.output(M.TensorDesc([1, ne], DType.F32))
    g.moe_ffn(x=x, router=router, gate_exps=gate, up_exps=up, down_exps=down, dst=dst, ne=ne, n_expert=E, n_used=K,
              n_ff_exp=nff, **opts)
    return g, dict(x=x, router=router, gate=gate, up=up, down=down, dst=dst)


def _banks(rng, E, nff, ne, gdt, ddt):
    return _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, nff, ne, gdt), _realistic(rng, E, ne, nff, ddt)


@pytest.mark.parametrize("gdt,ddt,E,opts", [
    (H.Q4K, H.Q6K, 128, {}),                                            # one layer of config 2
    (H.Q8_0, H.Q8_0, 128, {}),                                          # config 1
    (H.Q4K, H.Q6K, 256, {}),                                            # eight router rows per workgroup
    (H.Q8_0, H.Q8_0, 256, dict(scale=2.5, norm_w=False)),
    (H.Q4K, H.Q6K, 128, dict(weight_before=True, with_down_scale=True)),
    (H.Q4K, H.Q6K, 128, dict(act=M.Activation.Gelu, swiglu_clamp=0.05)),
    (H.Q4K, H.Q6K, 128, dict(gating=M.MoeGating.Sigmoid)),              # not the plain softmax: the complete routing routine
    (H.Q4K, H.Q6K, 128, dict(with_exp_probs_b=True, n_expert_groups=8, n_expert_groups_used=4)),
    (H.Q4K, H.Q6K, 128, dict(with_expert_ids=True)),
    (H.Q4K, H.Q6K, 128, dict(fused_gate_up=True)),
    (H.Q4K, H.Q6K, 128, dict(ep_band=(32, 64))),                        # foreign selections weigh nothing and are skipped
])
def test_single_launch_gives_the_bits_of_three_launches(be, be3, gdt, ddt, E, opts):
    ne, K, nff = 2048, 8, 768
    rng = np.random.default_rng(E + gdt + len(opts))
    x = rng.standard_normal((1, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    n_local = opts["ep_band"][1] if "ep_band" in opts else E
    gate, up, down = _banks(rng, n_local, nff, ne, gdt, ddt)
    data = dict(x=x, router=router, gate=gate, up=up, down=down)
    if opts.get("fused_gate_up"):
        data.update(gate=np.concatenate([gate.reshape(n_local, -1), up.reshape(n_local, -1)], axis=1).reshape(-1), up=None)
    if opts.get("with_down_scale"):
        data["down_scale"] = rng.uniform(0.5, 1.5, E).astype(np.float32)
    if opts.get("with_exp_probs_b"):
        data["exp_probs_b"] = (rng.standard_normal(E) * 0.01).astype(np.float32)
    if opts.get("with_expert_ids"):
        data["expert_ids"] = rng.choice(E, (1, K), replace=False).astype(np.int32)
    g, ids = _graph(ne, E, K, nff, gdt, ddt, dict(opts))
    one, r1 = _run(be, g, ids, data, ne, "moe_layer")
    g, ids = _graph(ne, E, K, nff, gdt, ddt, dict(opts))
    three, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
    assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
    assert np.array_equal(bits(r1["logits"]), bits(r3["logits"]))
    assert np.array_equal(bits(one), bits(three))
    assert np.abs(three).max() > 1e-5
    if "ep_band" in opts:
        assert (r1["w"] == 0).any() and (r1["w"] != 0).any(), "the band should hold some of the selection, not all"


def test_single_launch_matches_the_oracle_with_tied_and_near_tied_probabilities(be):
    """Two experts with the same router row tie exactly (the lower id ranks first, crates/infr-cpu/src/lib.rs:3847-3850),
    two more are an ulp apart: the selection by exponentials that the kernel runs beside the sum cannot decide these and
    hands over to the complete routine."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(5)
    x = np.zeros((1, ne), np.float32)
    x[0, 0] = 1.0
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    col = (rng.standard_normal(E) * 0.05).astype(np.float32)
    col[[70, 11]] = 3.0                                        # an exact tie at the top: 11 before 70
    col[[90, 33, 64]] = [2.5, 2.25, 2.0]
    col[100] = 1.5
    col[7] = (np.float32(1.5).view(np.uint32) + np.uint32(1)).view(np.float32)
    col[[20, 21]] = 1.0                                        # an exact tie at the edge of the selection: 20 is in, 21 is out
    router[:, 0] = col
    gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
    g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
    out, r = _run(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), ne, "moe_layer")
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
    assert ref["idx"][0].tolist()[:2] == [11, 70] and ref["idx"][0].tolist()[-1] == 20
    assert np.array_equal(r["idx"], ref["idx"]) and np.array_equal(bits(r["w"]), bits(ref["w"]))
    assert np.array_equal(bits(r["probs"]), bits(ref["probs"]))
    assert H.rel_l2(out, ref["dst"]) < 1e-3 and H.max_abs(out, ref["dst"]) < 2e-3


def test_single_launch_with_the_residual_add_folded_in(be, be3):
    """MoeFfn followed by Op::Add of the layer input: the kernel's last step adds the other operand (in place)."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(9)
    x = rng.standard_normal((1, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
    outs = []
    for backend, kernel in ((be, "moe_layer"), (be3, "moe_route_gate_up")):
        g = M.Graph()
        xi = g.input(M.TensorDesc([1, ne], DType.F32))
        rt = g.weight(M.TensorDesc([E, ne], DType.F32))
        gt, ut = g.weight(M.TensorDesc([E, nff, ne], DType.Q4K)), g.weight(M.TensorDesc([E, nff, ne], DType.Q4K))
        dt = g.weight(M.TensorDesc([E, ne, nff], DType.Q6K))
        moe = g.internal(M.TensorDesc([1, ne], DType.F32))
        yi = g.output(M.TensorDesc([1, ne], DType.F32))
        g.moe_ffn(x=xi, router=rt, gate_exps=gt, up_exps=ut, down_exps=dt, dst=moe, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff)
        g.add(a=xi, b=moe, dst=yi, n=ne)
        backend.prof_enable(True)
        y = M.run_graph(backend, g, [(xi, x), (rt, router), (gt, gate), (ut, up), (dt, down)], yi, ne)
        backend.sync()
        names = set(backend.prof_read())
        backend.prof_enable(False)
        assert kernel in names and "add" not in names, names
        outs.append(y)
    assert np.array_equal(bits(outs[0]), bits(outs[1]))
    ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
    assert H.rel_l2(outs[0].reshape(1, ne) - x, ref["dst"]) < 1e-3


def test_a_wait_that_runs_out_is_reported_and_the_backend_falls_back(be3):
    """single_launch_spin_limit = 1: a workgroup gives up a hand-over after its first poll.  Every workgroup still leaves the
    kernel (no wait is unbounded), the next synchronisation reports the error, and from then on the backend runs the
    three-launch path, whose results are the reference ones."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(13)
    x = rng.standard_normal((1, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, H.Q8_0, H.Q8_0)
    data = dict(x=x, router=router, gate=gate, up=up, down=down)
    b = M.Backend(0, single_launch_spin_limit=1)
    try:
        seen = None
        for _ in range(4):   # the first poll of some workgroup finds a peer's record missing: practically always at once
            g, ids = moe_graph(1, ne, E, K, nff, DType.Q8_0, DType.Q8_0)
            try:
                _run(b, g, ids, data, ne, "moe_layer")
            except M.BackendError as err:
                seen = str(err)
                break
        assert seen is not None and "timed out" in seen and "three-launch" in seen
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q8_0, DType.Q8_0)
        after, r = _run(b, g, ids, data, ne, "moe_route_gate_up")
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q8_0, DType.Q8_0)
        want, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
        assert np.array_equal(bits(after), bits(want)) and np.array_equal(r["idx"], r3["idx"])
    finally:
        b.close()


def test_shapes_the_kernel_does_not_take_stay_on_three_launches(be):
    """Six experts per token, or a hidden size above 2048: compile keeps the three-launch path."""
    for ne, E, K, nff in ((2048, 128, 6, 768), (4096, 128, 8, 768)):
        rng = np.random.default_rng(ne + K)
        x = rng.standard_normal((1, ne)).astype(np.float32)
        router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
        gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
        out, r = _run(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), ne, "moe_route_gate_up")
        ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
        assert np.array_equal(r["idx"], ref["idx"]) and H.rel_l2(out, ref["dst"]) < 1e-3
