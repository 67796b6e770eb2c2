"""Single-token Op::MoeFfn as one launch against the three-launch path of the same library and against the oracle: same
ids, same routing weights, same output bits, for the shapes and options the kernels take; and the bounded wait of their
in-kernel hand-overs, forced from the host.  Two kernels: "moe_layer" (moe4all_amd/csrc/k_layer_stream.hip) requests
the expert rows of a guessed selection while the exact routing runs beside the stream, "moe_layer_inorder"
(k_layer.hip) runs the stages in order and takes the routing options the guess cannot serve."""
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


@pytest.fixture(scope="module")
def be_inorder():
    """The same device with the guessing kernel switched off: every shape the in-order kernel takes runs on it."""
    b = M.Backend(0, disable_single_launch_guess=True)
    yield b
    b.close()


GUESS, INORDER = "moe_layer", "moe_layer_inorder"


@pytest.mark.parametrize("gdt,ddt,E,opts,kernel", [
    (H.Q4K, H.Q6K, 128, {}, GUESS),                                     # one layer of config 2
    (H.Q8_0, H.Q8_0, 128, {}, GUESS),                                   # config 1
    (H.Q4K, H.Q6K, 256, {}, GUESS),                                     # every logit computed once for the grid
    (H.Q8_0, H.Q8_0, 256, dict(scale=2.5, norm_w=False), GUESS),
    (H.Q4K, H.Q6K, 128, dict(with_down_scale=True), GUESS),
    (H.Q4K, H.Q6K, 128, dict(weight_before=True, with_down_scale=True), INORDER),   # the weights precede the gate/up stage
    (H.Q4K, H.Q6K, 128, dict(act=M.Activation.Gelu, swiglu_clamp=0.05), GUESS),
    (H.Q4K, H.Q6K, 128, dict(gating=M.MoeGating.Sigmoid), GUESS),       # not the plain softmax: the complete routing routine
    (H.Q4K, H.Q6K, 128, dict(with_exp_probs_b=True, n_expert_groups=8, n_expert_groups_used=4), INORDER),
    (H.Q4K, H.Q6K, 128, dict(with_expert_ids=True), INORDER),
    (H.Q4K, H.Q6K, 128, dict(fused_gate_up=True), GUESS),
    (H.Q4K, H.Q6K, 128, dict(ep_band=(32, 64)), INORDER),               # foreign selections weigh nothing and are skipped
    (H.Q4K, H.Q6K, 128, dict(inorder=True), INORDER),                   # the in-order kernel on the plain shapes
    (H.Q8_0, H.Q8_0, 128, dict(inorder=True), INORDER),
    (H.Q4K, H.Q6K, 256, dict(inorder=True), INORDER),
    (H.Q4K, H.Q6K, 128, dict(inorder=True, gating=M.MoeGating.Sigmoid), INORDER),
])
def test_single_launch_gives_the_bits_of_three_launches(be, be3, be_inorder, gdt, ddt, E, opts, kernel):
    ne, K, nff = 2048, 8, 768
    opts = dict(opts)
    if opts.pop("inorder", False):
        be = be_inorder
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
    one, r1 = _run(be, g, ids, data, ne, kernel)
    g, ids = _graph(ne, E, K, nff, gdt, ddt, dict(opts))
    three, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
    assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
    assert np.array_equal(bits(r1["logits"]), bits(r3["logits"]))
    assert np.array_equal(bits(one), bits(three))
    assert np.abs(three).max() > 1e-5
    if "ep_band" in opts:
        assert (r1["w"] == 0).any() and (r1["w"] != 0).any(), "the band should hold some of the selection, not all"


@pytest.mark.parametrize("kernel", [GUESS, INORDER])
def test_single_launch_matches_the_oracle_with_tied_and_near_tied_probabilities(be, be_inorder, kernel):
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
    out, r = _run(be if kernel == GUESS else be_inorder, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), ne, kernel)
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


@pytest.mark.parametrize("kernel", [GUESS, INORDER])
def test_a_wait_that_runs_out_is_reported_and_the_backend_falls_back(be3, kernel):
    """single_launch_spin_limit = 1: a workgroup gives up a hand-over after its first poll.  Every workgroup still leaves the
    kernel (no wait is unbounded), the next synchronisation reports the error, and from then on the backend runs the
    three-launch path, whose results are the reference ones."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(13)
    x = rng.standard_normal((1, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, H.Q8_0, H.Q8_0)
    data = dict(x=x, router=router, gate=gate, up=up, down=down)
    b = M.Backend(0, single_launch_spin_limit=1, disable_single_launch_guess=kernel == INORDER)
    try:
        seen = None
        for _ in range(4):   # the first poll of some workgroup finds a peer's record missing: practically always at once
            g, ids = moe_graph(1, ne, E, K, nff, DType.Q8_0, DType.Q8_0)
            try:
                _run(b, g, ids, data, ne, kernel)
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
    """Six experts per token, or an intermediate size that is no multiple of 384: compile keeps the three-launch path."""
    for ne, E, K, nff in ((2048, 128, 6, 768), (4096, 128, 8, 1024)):
        rng = np.random.default_rng(ne + K)
        x = rng.standard_normal((1, ne)).astype(np.float32)
        router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
        gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
        out, r = _run(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), ne, "moe_route_gate_up")
        ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
        assert np.array_equal(r["idx"], ref["idx"]) and H.rel_l2(out, ref["dst"]) < 1e-3


def test_hidden_size_4096_with_the_small_intermediate_size(be, be3):
    """ne = 4096 with n_ff = 768: a shape between the two benchmark shapes."""
    ne, E, K, nff = 4096, 128, 8, 768
    data = _plain_case(4096, ne=ne, nff=nff)
    g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
    one, r1 = _run(be, g, ids, data, ne, GUESS)
    g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
    three, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
    assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
    assert np.array_equal(bits(one), bits(three))


def _plain_case(seed, E=128, gdt=H.Q4K, ddt=H.Q6K, ne=2048, nff=768):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((1, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, gdt, ddt)
    return dict(x=x, router=router, gate=gate, up=up, down=down)


@pytest.mark.parametrize("skew,gdt,ddt,E", [(1, H.Q4K, H.Q6K, 128), (3, H.Q4K, H.Q6K, 128), (8, H.Q4K, H.Q6K, 128),
                                            (2, H.Q8_0, H.Q8_0, 128), (2, H.Q4K, H.Q6K, 256)])
def test_an_expert_the_guess_missed_is_loaded_late_and_changes_nothing(be3, skew, gdt, ddt, E):
    """single_launch_guess_skew = n: every guess leaves out the n most likely experts, so n groups of workgroups find
    their expert outside the exact selection, compute the missed one after the routing is known and hand its
    activations over under that expert's tag.  Ids, weights and output bits are those of the three-launch path."""
    ne, K, nff = 2048, 8, 768
    data = _plain_case(100 + skew + E, E, gdt, ddt)
    b = M.Backend(0, single_launch_guess_skew=skew)
    try:
        before = b.late_experts()
        for rep in range(3):   # the same plan shape three times: the records of the launch before are never taken
            g, ids = moe_graph(1, ne, E, K, nff, DType(gdt), DType(ddt))
            late, r1 = _run(b, g, ids, data, ne, GUESS)
            g, ids = moe_graph(1, ne, E, K, nff, DType(gdt), DType(ddt))
            three, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
            assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
            assert np.array_equal(bits(late), bits(three))
        assert b.late_experts() - before == 3 * skew
    finally:
        b.close()


@pytest.mark.parametrize("rows,gdt,ddt,skew", [(2, H.Q4K, H.Q6K, 0), (4, H.Q4K, H.Q6K, 0), (2, H.Q8_0, H.Q8_0, 0), (4, H.Q8_0, H.Q8_0, 0),
                                               (4, H.Q4K, H.Q6K, 2), (2, H.Q8_0, H.Q8_0, 8), (8, H.Q4K, H.Q6K, 0), (8, H.Q4K, H.Q6K, 1)])
def test_two_and_four_token_rows_in_one_launch_give_the_bits_of_three_launches(be3, rows, gdt, ddt, skew):
    """Two, four or eight token rows: every row takes 8 / rows of the XCDs and runs the single-token scheme among its own
    workgroups (its own logits, guess, routing, hand-overs and output rows).  Ids, weights, logits and output bits per row
    are those of the three-launch path, also when every row's guess misses `skew` experts, and a row's bits do not depend
    on its neighbours (row 0 alone gives the same)."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(1000 + rows + gdt + skew)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    x[rows - 1] *= 30.0                                    # rows of different magnitude: nothing is shared between rows
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, gdt, ddt)
    data = dict(x=x, router=router, gate=gate, up=up, down=down)
    b = M.Backend(0, single_launch_guess_skew=skew)
    try:
        before = b.late_experts()
        for rep in range(2):   # twice on the same shape: records of the launch before are never taken
            g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
            one, r1 = _run(b, g, ids, data, rows * ne, GUESS)
            g, ids = moe_graph(rows, ne, E, K, nff, DType(gdt), DType(ddt))
            three, r3 = _run(be3, g, ids, data, rows * ne, "moe_route_gate_up")
            assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
            assert np.array_equal(bits(r1["logits"]), bits(r3["logits"])) and np.array_equal(bits(r1["probs"]), bits(r3["probs"]))
            assert np.array_equal(bits(one), bits(three))
        assert b.late_experts() - before == 2 * rows * skew
        g, ids = moe_graph(1, ne, E, K, nff, DType(gdt), DType(ddt))
        alone, _ = _run(b, g, ids, dict(data, x=x[:1]), ne, GUESS)
        assert np.array_equal(bits(alone.reshape(-1)), bits(one.reshape(rows, ne)[0]))
        ref = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
        assert np.array_equal(r1["idx"], ref["idx"])
        assert H.rel_l2(one.reshape(rows, ne), ref["dst"]) < 1e-3
    finally:
        b.close()


def test_three_token_rows_stay_on_three_launches(be):
    """A row count that does not divide the eight XCDs keeps the per-token kernels."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
    g, ids = moe_graph(3, ne, E, K, nff, DType.Q4K, DType.Q6K)
    _run(be, g, ids, dict(x=x, router=router, gate=gate, up=up, down=down), 3 * ne, "moe_route_gate_up")


def test_a_good_guess_loads_nothing_late(be):
    before = be.late_experts()
    g, ids = moe_graph(1, 2048, 128, 8, 768, DType.Q4K, DType.Q6K)
    _run(be, g, ids, _plain_case(77), 2048, GUESS)
    assert be.late_experts() == before


@pytest.mark.parametrize("mode", [1, 2])
def test_logits_once_for_the_grid_or_once_per_group_give_the_same_bits(be3, mode):
    ne, E, K, nff = 2048, 128, 8, 768
    data = _plain_case(31)
    b = M.Backend(0, single_launch_logits=mode)
    try:
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
        one, r1 = _run(b, g, ids, data, ne, GUESS)
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
        three, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
        assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
        assert np.array_equal(bits(r1["logits"]), bits(r3["logits"])) and np.array_equal(bits(r1["probs"]), bits(r3["probs"]))
        assert np.array_equal(bits(one), bits(three))
    finally:
        b.close()


def test_near_tied_logits_at_the_edge_of_the_selection(be, be3):
    """Router rows that repeat each other up to a last-place change of one element: the eighth and ninth largest logits
    are equal or an ulp apart in many of the tokens, so estimate and exact value may order them differently.  Whatever
    the guess was, the published selection and the output are the three-launch path's."""
    ne, E, K, nff = 2048, 128, 8, 768
    rng = np.random.default_rng(2024)
    gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
    base = (rng.standard_normal(ne) * 0.02).astype(np.float32)
    late0 = be.late_experts()
    for t in range(6):
        router = (rng.standard_normal((E, ne)) * 0.002).astype(np.float32)
        twins = rng.choice(E, 24, replace=False)
        for k, e in enumerate(twins):                      # 24 rows = base with one element moved by k ulps
            row = base.copy()
            j = int(rng.integers(ne))
            row[j] = (row[j].view(np.uint32) + np.uint32(k % 4)).view(np.float32)
            router[e] = row
        x = rng.standard_normal((1, ne)).astype(np.float32)
        x += np.float32(100.0) * base                      # the twins' logit is large and positive: they fill the selection
        data = dict(x=x, router=router, gate=gate, up=up, down=down)
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
        one, r1 = _run(be, g, ids, data, ne, GUESS)
        g, ids = moe_graph(1, ne, E, K, nff, DType.Q4K, DType.Q6K)
        three, r3 = _run(be3, g, ids, data, ne, "moe_route_gate_up")
        assert set(r3["idx"][0].tolist()) <= set(twins.tolist())
        assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
        assert np.array_equal(bits(one), bits(three))
    print("late experts over six near-tied tokens:", be.late_experts() - late0)


_SHARED_CASES = {}


def _shared_graph(ne, E, K, nff, gated, rows=1):
    g = M.Graph()
    T = M.TensorDesc
    x = g.input(T([rows, ne], DType.F32))
    router = g.weight(T([E, ne], DType.F32))
    gate, up = g.weight(T([E, nff, ne], DType.Q4K)), g.weight(T([E, nff, ne], DType.Q4K))
    down = g.weight(T([E, ne, nff], DType.Q6K))
    sg, su, sd = g.weight(T([nff, ne], DType.Q4K)), g.weight(T([nff, ne], DType.Q4K)), g.weight(T([ne, nff], DType.Q6K))
    moe = g.internal(T([rows, ne], DType.F32))
    tg, tu, ta = (g.internal(T([rows, nff], DType.F32)) for _ in range(3))
    ts = g.internal(T([rows, ne], DType.F32))
    dst = g.output(T([rows, ne], DType.F32))
    ids = dict(x=x, router=router, gate=gate, up=up, down=down, sg=sg, su=su, sd=sd, dst=dst)
    g.moe_ffn(x=x, router=router, gate_exps=gate, up_exps=up, down_exps=down, dst=moe, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff)
    if gated:
        wq = g.weight(T([1, ne], DType.F32))
        tq = g.internal(T([rows, 1], DType.F32))
        g.linear(x=x, weight=wq, dst=tq, m=rows, in_f=ne, out_f=1)
        ids["wq"] = wq
    g.linear(x=x, weight=sg, dst=tg, m=rows, in_f=ne, out_f=nff)
    g.linear(x=x, weight=su, dst=tu, m=rows, in_f=ne, out_f=nff)
    g.gated_act(gate=tg, up=tu, dst=ta, rows=rows, nff=nff)
    g.linear(x=ta, weight=sd, dst=ts, m=rows, in_f=nff, out_f=ne)
    if gated:
        g.moe_shared_expert_add(moe=moe, shexp=ts, gate=tq, dst=dst, rows=rows, n=ne)
    else:
        g.add(a=moe, b=ts, dst=dst, n=rows * ne)
    return g, ids


@pytest.mark.parametrize("ne,E,nff,gated,skew,rows", [(4096, 256, 1536, False, 0, 1), (4096, 256, 1536, True, 0, 1),
                                                      (4096, 256, 1536, False, 2, 1), (4096, 256, 1536, False, 0, 2),
                                                      (4096, 256, 1536, True, 1, 4), (2048, 128, 768, False, 0, 1)])
def test_single_launch_with_the_always_on_expert_folded_in(be3, ne, E, nff, gated, skew, rows):
    """The large shape's layer (256 experts, hidden 4096, an always-on expert beside the routed ones) as ONE launch: the
    always-on expert's rows are spread over all workgroups and requested first.  Same bits as the three-launch path,
    within the parity bar of the oracle."""
    K = 8
    if (ne, E, nff) not in _SHARED_CASES:   # one set of banks per shape: the large one is 3 GB
        rng = np.random.default_rng(ne + E)
        d = dict(x=rng.standard_normal((1, ne)).astype(np.float32), router=(rng.standard_normal((E, ne)) * 0.02).astype(np.float32))
        d["gate"], d["up"], d["down"] = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
        d["sg"], d["su"], d["sd"] = (a.reshape(-1) for a in _banks(rng, 1, nff, ne, H.Q4K, H.Q6K))
        d["wq"] = (rng.standard_normal((1, ne)) * 0.02).astype(np.float32)
        _SHARED_CASES.clear()
        _SHARED_CASES[(ne, E, nff)] = d
    data = dict(_SHARED_CASES[(ne, E, nff)])
    if not gated:
        del data["wq"]
    if rows > 1:   # more token rows: each takes 8 / rows of the XCDs, the always-on expert's share per workgroup grows
        data["x"] = np.random.default_rng(rows).standard_normal((rows, ne)).astype(np.float32)
    b = M.Backend(0, single_launch_guess_skew=skew)
    try:
        g, ids = _shared_graph(ne, E, K, nff, gated, rows)
        one, r1 = _run(b, g, ids, data, rows * ne, "moe_layer_shared")
        g, ids = _shared_graph(ne, E, K, nff, gated, rows)
        three, r3 = _run(be3, g, ids, data, rows * ne, "moe_route_gate_up_shared")
        assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
        assert np.array_equal(bits(r1["logits"]), bits(r3["logits"]))
        assert np.array_equal(bits(one), bits(three))
        assert b.late_experts() == skew * rows
    finally:
        b.close()
    ref = O.moe_ffn(data["x"], data["router"], data["gate"], data["up"], data["down"], ne=ne, n_expert=E, n_used=K,
                    n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
    assert np.array_equal(r1["idx"], ref["idx"]) and np.array_equal(bits(r1["w"]), bits(ref["w"]))
    if not gated:
        sh = O.moe_ffn(data["x"], np.zeros((1, ne), np.float32), data["sg"], data["su"], data["sd"], ne=ne, n_expert=1,
                       n_used=1, n_ff_exp=nff, gate_dtype=H.Q4K, down_dtype=H.Q6K)
        want = ref["dst"] + sh["dst"]
        assert H.rel_l2(one.reshape(want.shape), want) < 1e-3 and H.max_abs(one.reshape(want.shape), want) < 2e-3


@pytest.mark.parametrize("gated", [False, True])
def test_two_token_rows_with_the_always_on_expert_folded_in(be, be3, gated):
    """Two rows of the small shape with an always-on expert: each row's share of that expert is spread over the row's 128
    workgroups.  Same bits as the three-launch path, row by row."""
    rows, ne, E, K, nff = 2, 2048, 128, 8, 768
    rng = np.random.default_rng(50 + gated)
    data = dict(x=rng.standard_normal((rows, ne)).astype(np.float32), router=(rng.standard_normal((E, ne)) * 0.02).astype(np.float32))
    data["gate"], data["up"], data["down"] = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
    data["sg"], data["su"], data["sd"] = (a.reshape(-1) for a in _banks(rng, 1, nff, ne, H.Q4K, H.Q6K))
    if gated:
        data["wq"] = (rng.standard_normal((1, ne)) * 0.02).astype(np.float32)
    g, ids = _shared_graph(ne, E, K, nff, gated, rows)
    one, r1 = _run(be, g, ids, data, rows * ne, "moe_layer_shared")
    g, ids = _shared_graph(ne, E, K, nff, gated, rows)
    three, r3 = _run(be3, g, ids, data, rows * ne, "moe_route_gate_up_shared")
    assert np.array_equal(r1["idx"], r3["idx"]) and np.array_equal(bits(r1["w"]), bits(r3["w"]))
    assert np.array_equal(bits(one), bits(three))
    assert np.abs(one.reshape(rows, ne)[1]).max() > 1e-5


@pytest.mark.parametrize("shared", [False, True])
def test_single_launch_with_the_rms_norm_and_the_residual_folded_in(be, shared):
    """The model's whole FFN sublayer for one token, y = x + ffn(rmsnorm(x) * w), as ONE launch: every workgroup
    normalises the raw row itself (the sum of squares in the standalone kernel's order, so the same bits) and one of them
    stores the normalised row where the RmsNorm's dst is.  Same bits as one launch per op, and the normalised row is there."""
    ne, E, K, nff, eps = 2048, 128, 8, 768, 1e-6
    rng = np.random.default_rng(90 + shared)
    x = (rng.standard_normal((1, ne)) * 3.0).astype(np.float32)
    nw = rng.uniform(0.5, 1.5, ne).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.02).astype(np.float32)
    gate, up, down = _banks(rng, E, nff, ne, H.Q4K, H.Q6K)
    sg, su, sd = (a.reshape(-1) for a in _banks(rng, 1, nff, ne, H.Q4K, H.Q6K))
    outs, norms, names = {}, {}, {}
    for off in (False, True):
        b = be if not off else M.Backend(0, disable_op_fusion=True, disable_single_launch_moe=True)
        try:
            g = M.Graph()
            T = M.TensorDesc
            xi, nwt = g.input(T([1, ne], DType.F32)), g.weight(T([ne], DType.F32))
            rt = g.weight(T([E, ne], DType.F32))
            gt, ut = g.weight(T([E, nff, ne], DType.Q4K)), g.weight(T([E, nff, ne], DType.Q4K))
            dt = g.weight(T([E, ne, nff], DType.Q6K))
            xn = g.output(T([1, ne], DType.F32))      # declared an output: the normalised row has to be materialised
            moe = g.internal(T([1, ne], DType.F32))
            yi = g.output(T([1, ne], DType.F32))
            g.rms_norm(x=xi, weight=nwt, dst=xn, rows=1, dim=ne, eps=eps)
            g.moe_ffn(x=xn, router=rt, gate_exps=gt, up_exps=ut, down_exps=dt, dst=moe, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff)
            bound = [(xi, x), (nwt, nw), (rt, router), (gt, gate), (ut, up), (dt, down)]
            sub = moe
            if shared:
                wg, wu, wd = g.weight(T([nff, ne], DType.Q4K)), g.weight(T([nff, ne], DType.Q4K)), g.weight(T([ne, nff], DType.Q6K))
                tg, tu, ta = (g.internal(T([1, nff], DType.F32)) for _ in range(3))
                ts, sub = g.internal(T([1, ne], DType.F32)), g.internal(T([1, ne], DType.F32))
                g.linear(x=xn, weight=wg, dst=tg, m=1, in_f=ne, out_f=nff)
                g.linear(x=xn, weight=wu, dst=tu, m=1, in_f=ne, out_f=nff)
                g.gated_act(gate=tg, up=tu, dst=ta, rows=1, nff=nff)
                g.linear(x=ta, weight=wd, dst=ts, m=1, in_f=nff, out_f=ne)
                g.add(a=moe, b=ts, dst=sub, n=ne)
                bound += [(wg, sg), (wu, su), (wd, sd)]
            g.add(a=xi, b=sub, dst=yi, n=ne)
            plan = b.compile(g)
            bufs, bind = [], M.Bindings()
            for tid, v in bound:
                bufs.append(b.buffer_from(v))
                bind.bind(tid, bufs[-1])
            o_xn, o_y = b.alloc(ne * 4), b.alloc(ne * 4)
            bind.bind(xn, o_xn)
            bind.bind(yi, o_y)
            b.prof_enable(True)
            b.execute(plan, bind)
            outs[off] = b.download(o_y, ne * 4, np.float32).copy()
            norms[off] = b.download(o_xn, ne * 4, np.float32).copy()
            names[off] = set(b.prof_read())
            b.prof_enable(False)
            for buf in bufs + [o_xn, o_y]:
                buf.free()
            plan.free()
        finally:
            if off:
                b.close()
    assert names[False] == {"moe_layer_shared" if shared else "moe_layer"}, names[False]
    assert "rms_norm" in names[True] and "add" in names[True]
    assert np.array_equal(bits(norms[False]), bits(norms[True]))
    assert np.array_equal(bits(outs[False]), bits(outs[True]))
    assert H.rel_l2(norms[False].reshape(1, ne), O.rms_norm(x, nw, eps).reshape(1, ne)) < 1e-5
