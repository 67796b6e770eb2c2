"""From a GGUF file to the device: the weight binder's upload of raw block bytes, the standalone
decode of what was uploaded (the reference's dequant probe, crates/infr-vulkan/tests/weight_dequant_parity.rs),
and the whole FFN sublayer of a qwen3moe-shaped layer built from the file's tensors and hyperparameters.
No real model file ships with the repository: the files are written by tests/gguf_writer.py with the
tensor names and metadata keys a converter writes (crates/infr-llama/src/seam/runner.rs:2519-2565)."""
import numpy as np
import pytest

import moe4all_amd as M
from moe4all_amd import gguf as G
import oracle as O

import gguf_writer as W
import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    b = M.Backend(0)
    yield b
    b.close()


def _bf16(a):
    return (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def _moe_file(path, rng, *, ne, n_ff, E, K, layers, gdt, ddt, shards=1, shexp=0, gated=False):
    """A qwen3moe-shaped file: per layer ffn_norm, ffn_gate_inp and the three expert banks; with `shexp`
    also the shared expert's three matrices and, if `gated`, its gate vector."""
    per_layer = []
    for l in range(layers):
        w = {
            "ffn_norm.weight": ((ne,), 0, (1 + 0.1 * rng.standard_normal(ne)).astype(np.float32)),
            "ffn_gate_inp.weight": ((ne, E), 0, (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)),
            "ffn_gate_exps.weight": ((ne, n_ff, E), W.GGML[gdt], H.synth_weight(getattr(H, gdt), E * n_ff * ne, 10 + l)),
            "ffn_up_exps.weight": ((ne, n_ff, E), W.GGML[gdt], H.synth_weight(getattr(H, gdt), E * n_ff * ne, 20 + l)),
            "ffn_down_exps.weight": ((n_ff, ne, E), W.GGML[ddt], H.synth_weight(getattr(H, ddt), E * ne * n_ff, 30 + l)),
        }
        if shexp:
            w["ffn_gate_shexp.weight"] = ((ne, shexp), W.GGML[gdt], H.synth_weight(getattr(H, gdt), shexp * ne, 40 + l))
            w["ffn_up_shexp.weight"] = ((ne, shexp), W.GGML[gdt], H.synth_weight(getattr(H, gdt), shexp * ne, 50 + l))
            w["ffn_down_shexp.weight"] = ((shexp, ne), W.GGML[ddt], H.synth_weight(getattr(H, ddt), ne * shexp, 60 + l))
            if gated:
                w["ffn_gate_inp_shexp.weight"] = ((ne,), 0, (rng.standard_normal(ne) * 0.05).astype(np.float32))
        per_layer.append(w)
    tensors = [(f"blk.{l}.{k}", shape, gt, np.ascontiguousarray(data).view(np.uint8).tobytes())
               for l, w in enumerate(per_layer) for k, (shape, gt, data) in w.items()]
    meta = [("general.architecture", W.STR, "qwen3moe"), ("qwen3moe.block_count", W.U32, layers),
            ("qwen3moe.embedding_length", W.U32, ne), ("qwen3moe.expert_count", W.U32, E),
            ("qwen3moe.expert_used_count", W.U32, K), ("qwen3moe.expert_feed_forward_length", W.U32, n_ff),
            ("qwen3moe.attention.layer_norm_rms_epsilon", W.F32, 1e-6),
            ("tokenizer.ggml.tokens", W.ARR, (W.STR, ["<s>", "a", "b"]))]
    if shexp:
        meta.append(("qwen3moe.expert_shared_feed_forward_length", W.U32, shexp))
    if shards == 1:
        W.write(path, meta, tensors)
        return path, per_layer
    base = str(path)[:-5]
    cut = len(tensors) // 2
    first = f"{base}-00001-of-00002.gguf"
    split = lambda i: [("split.no", W.U16, i), ("split.count", W.U16, 2), ("split.tensors.count", W.I32, len(tensors))]
    W.write(first, meta + split(0), tensors[:cut])
    W.write(f"{base}-00002-of-00002.gguf", split(1), tensors[cut:])
    return first, per_layer


_DTYPE = {"IQ4_NL": M.DType.Iq4Nl, "IQ4_XS": M.DType.Iq4Xs, "TQ1_0": M.DType.Tq1_0, "TQ2_0": M.DType.Tq2_0,
          "Q2_0": M.DType.Q2_0, "MXFP4": M.DType.Mxfp4, "NVFP4": M.DType.Nvfp4}


@pytest.mark.parametrize("dt", ["F32", "F16", "BF16", "Q8_0", "Q4K", "Q6K", "IQ4_NL", "IQ4_XS", "TQ1_0", "TQ2_0", "Q2_0", "MXFP4",
                                "NVFP4"])
def test_bound_weight_decodes_to_the_oracle_values(be, tmp_path, dt):
    """BindWeight (alloc_uninit + upload of the file's bytes) followed by the device decode of the whole
    tensor: bit-identical to the oracle's decode of the same file bytes."""
    rng = np.random.default_rng(3)
    n = 4 * 256
    if dt == "F32":
        data, code = rng.standard_normal(n).astype(np.float32), M.DType.F32
    elif dt == "F16":
        data, code = rng.standard_normal(n).astype(np.float16), M.DType.F16
    elif dt == "BF16":
        data, code = _bf16(rng.standard_normal(n)), M.DType.Bf16
    else:
        data, code = H.synth_weight(getattr(H, dt), n, 5), _DTYPE.get(dt) or getattr(M.DType, dt)
    p = tmp_path / "w.gguf"
    W.write(p, [("general.architecture", W.STR, "x")], [("pad", (3,), 0, b"\0" * 12), ("w", (256, 4), W.GGML[dt], data.tobytes())])
    with G.Gguf(p) as g:
        buf, got_dt, numel = g.bind_weight(be, "w")
        assert got_dt == int(code) and numel == n and buf.len_bytes() == g.find("w").nbytes
        assert np.array_equal(be.download(buf), g.tensor_bytes("w"))
        got = be.dequant(buf, code, n)
        buf.free()
        want = O.dequant(int(code), g.tensor_bytes("w"))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("rows,shards,gdt,ddt", [(1, 1, "Q4K", "Q6K"), (5, 2, "Q8_0", "Q8_0"), (40, 1, "Q4K", "Q6K"),
                                                 (1, 1, "MXFP4", "MXFP4"), (48, 1, "MXFP4", "MXFP4"), (3, 1, "IQ4_XS", "IQ4_NL")])
def test_ffn_sublayer_from_a_gguf_file_matches_the_oracle(be, tmp_path, rows, shards, gdt, ddt):
    ne, n_ff, E, K, layers = 512, 256, 8, 2, 2
    rng = np.random.default_rng(40 + rows)
    path, per_layer = _moe_file(tmp_path / "tiny.gguf", rng, ne=ne, n_ff=n_ff, E=E, K=K, layers=layers, gdt=gdt, ddt=ddt,
                                shards=shards)
    x = (rng.standard_normal((rows, ne)) * 2).astype(np.float32)
    with G.Gguf(path) as g:
        hp = G.moe_hyper(g)
        assert (hp.arch, hp.n_layer, hp.ne, hp.n_expert, hp.n_used, hp.n_ff_exp) == ("qwen3moe", layers, ne, E, K, n_ff)
        assert abs(hp.eps - 1e-6) < 1e-12 and g.n_shards == shards
        for l in range(layers):
            layer = G.MoeFfnLayer(be, g, l, rows, hp)
            got = layer.forward(x)
            routing = be.moe_routing(layer.plan, layer.moe_op)
            layer.free()
            w = per_layer[l]
            xn = O.rms_norm(x, w["ffn_norm.weight"][2], 1e-6).reshape(rows, ne)
            want = O.moe_ffn(xn, w["ffn_gate_inp.weight"][2], w["ffn_gate_exps.weight"][2], w["ffn_up_exps.weight"][2],
                             w["ffn_down_exps.weight"][2], ne=ne, n_expert=E, n_used=K, n_ff_exp=n_ff,
                             gate_dtype=getattr(H, gdt), down_dtype=getattr(H, ddt))
            assert np.array_equal(routing["idx"], want["idx"])
            tol = 1e-2 if rows >= 32 else 1e-3
            assert H.rel_l2(got - x, want["dst"].reshape(rows, ne)) < tol
            assert H.max_abs(got - x, want["dst"].reshape(rows, ne)) < 2e-3 * max(1.0, float(np.abs(want["dst"]).max()))


@pytest.mark.parametrize("rows,gated", [(1, False), (1, True), (4, True), (36, False)])
def test_ffn_sublayer_with_a_shared_expert_from_a_gguf_file(be, tmp_path, rows, gated):
    """The shared-expert branch as the model emits it (crates/infr-llama/src/seam/runner.rs:8089-8174):
    summed in plain, or gated by sigmoid(ffn_gate_inp_shexp . x) through Op::MoeSharedExpertAdd."""
    ne, n_ff, E, K, sff = 512, 256, 8, 2, 512
    rng = np.random.default_rng(90 + rows)
    path, per_layer = _moe_file(tmp_path / "sh.gguf", rng, ne=ne, n_ff=n_ff, E=E, K=K, layers=1, gdt="Q4K", ddt="Q6K",
                                shexp=sff, gated=gated)
    x = (rng.standard_normal((rows, ne)) * 2).astype(np.float32)
    with G.Gguf(path) as g:
        assert G.moe_hyper(g).shexp_ff == sff
        layer = G.MoeFfnLayer(be, g, 0, rows)
        assert layer.gated == gated
        got = layer.forward(x)
        layer.free()
    w = per_layer[0]
    xn = O.rms_norm(x, w["ffn_norm.weight"][2], 1e-6).reshape(rows, ne)
    moe = O.moe_ffn(xn, w["ffn_gate_inp.weight"][2], w["ffn_gate_exps.weight"][2], w["ffn_up_exps.weight"][2],
                    w["ffn_down_exps.weight"][2], ne=ne, n_expert=E, n_used=K, n_ff_exp=n_ff, gate_dtype=H.Q4K,
                    down_dtype=H.Q6K)["dst"].reshape(rows, ne)
    og = O.linear(xn, w["ffn_gate_shexp.weight"][2], H.Q4K, ne, sff)
    ou = O.linear(xn, w["ffn_up_shexp.weight"][2], H.Q4K, ne, sff)
    sh = O.linear(O.gated_act_rows(og, ou), w["ffn_down_shexp.weight"][2], H.Q6K, sff, ne)
    if gated:
        logit = O.linear(xn, w["ffn_gate_inp_shexp.weight"][2], H.F32, ne, 1)
        want = O.moe_shared_expert_add(moe, sh, logit).reshape(rows, ne)
    else:
        want = O.add(moe, sh).reshape(rows, ne)
    tol = 1e-2 if rows >= 32 else 1e-3
    assert H.rel_l2(got - x, want) < tol


def test_a_file_with_the_wrong_shapes_is_refused(be, tmp_path):
    rng = np.random.default_rng(1)
    path, _ = _moe_file(tmp_path / "tiny.gguf", rng, ne=512, n_ff=256, E=8, K=2, layers=1, gdt="Q8_0", ddt="Q8_0")
    raw = bytearray(open(path, "rb").read())
    k = raw.index(b"qwen3moe.expert_count") + len(b"qwen3moe.expert_count") + 4
    raw[k:k + 4] = (16).to_bytes(4, "little")
    open(path, "wb").write(raw)
    with G.Gguf(path) as g:
        with pytest.raises(G.LoaderError, match="hyperparameters need"):
            G.MoeFfnLayer(be, g, 0, 1)
        with pytest.raises(G.LoaderError, match="tensor not found"):
            G.MoeFfnLayer(be, g, 3, 1)
