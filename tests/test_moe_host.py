"""Routed feed-forward of the llama architecture with experts (Mixtral-shaped), on the CPU.

Restated host code under test (llama-rust_amd/csrc/llama_host.cpp): topk, router_weights, moe_ffn and
the forward pass that calls it, following langtax/src/decode.rs:9938-10116, 10148-10292, 10366-10409,
11363-11409.  The weight products come from the CPU oracle; what is pinned here is the routing and the
grouping around them: closed forms the definitions fix (ties, uniform and one-hot probabilities, the sum
of the weights, the 2^-14 clamp), and a brute-force float64 restatement that handles every token and every
selected expert on its own (tests/llama_ref.py).
"""
import importlib

import numpy as np
import pytest

import oracle
from llama_ref import numpy_forward, numpy_moe_ffn, numpy_route

TINY_MOE = dict(n_layer=2, n_embd=256, n_head=4, n_head_kv=2, n_ff=256, n_vocab=64, n_expert=4, n_expert_used=2)


@pytest.fixture(scope="module")
def llama(pkg):
    return importlib.import_module("llama-rust_amd.llama")


def oracle_matmul(ty, n_rows, n_cols, n_tokens, w, x):
    return oracle.gemm(ty, n_cols, n_tokens, w, x, n_rows)


@pytest.fixture(scope="module")
def moe_path(llama, tmp_path_factory):
    path = tmp_path_factory.mktemp("gguf") / "tiny_moe.gguf"
    llama.write_synthetic_llama(path, **TINY_MOE, seed=11)
    return path


# ------------------------------------------------------------------ routing

def test_topk_orders_descending_and_breaks_ties_towards_the_lower_index(llama):
    assert llama.topk([0.1, 0.7, 0.2], 2).tolist() == [1, 2]
    assert llama.topk([0.25, 0.25, 0.25, 0.25], 2).tolist() == [0, 1]          # all equal: the first two
    assert llama.topk([0.1, 0.4, 0.4, 0.1], 3).tolist() == [1, 2, 0]           # ties inside and at the cut
    assert llama.topk([3.0, -1.0, 3.0, 3.0, 2.0], 4).tolist() == [0, 2, 3, 4]
    assert llama.topk([-np.inf, -np.inf, -1.0], 2).tolist() == [2, 0]
    assert llama.topk([5.0], 1).tolist() == [0]
    rng = np.random.default_rng(5)
    for _ in range(50):  # against a stable sort on the negated values, which keeps the lower index first
        v = rng.integers(0, 6, 16).astype(np.float32)                           # many ties
        k = int(rng.integers(1, 17))
        assert llama.topk(v, k).tolist() == np.argsort(-v, kind="stable")[:k].tolist()
    for k in (0, 4):
        with pytest.raises(llama.LlamaError, match="expert_used_count"):
            llama.topk([0.5, 0.3, 0.2], k)


def test_topk_has_a_total_order_with_nans(llama):
    """The reference's comparator calls a NaN a tie with everything (langtax/src/decode.rs:11369-11377), which orders
    nothing once a NaN is present; here numbers come first, descending, then the NaNs, equal keys by index: the
    result is defined for every input and is the reference's on every input without NaN."""
    nan = float("nan")
    assert llama.topk([nan, 0.3, 0.9, nan, 0.3], 5).tolist() == [2, 1, 4, 0, 3]
    assert llama.topk([nan, nan, nan], 2).tolist() == [0, 1]
    assert llama.topk([nan, -np.inf, nan], 1).tolist() == [1]
    rng = np.random.default_rng(3)
    for _ in range(50):   # many NaNs among many ties: same answer as a stable sort on (is NaN, -value)
        v = rng.integers(0, 4, 64).astype(np.float32)
        v[rng.random(64) < 0.3] = np.nan
        key = np.where(np.isnan(v), np.inf, -v)
        assert llama.topk(v, 64).tolist() == np.argsort(key, kind="stable").tolist()


def test_router_weights_closed_forms(llama):
    # uniform probabilities: equal weights 1 / k
    w = llama.router_weights(np.full(8, 0.125, np.float32), [0, 1])
    assert w.tolist() == [0.5, 0.5]
    # one-hot: all weight on the chosen expert, the runner-up gets exactly zero
    w = llama.router_weights(np.array([0, 0, 1, 0], np.float32), [2, 0])
    assert w.tolist() == [1.0, 0.0]
    # the weights sum to one after renormalising whatever was selected
    rng = np.random.default_rng(9)
    for _ in range(20):
        p = rng.random(8).astype(np.float32)
        p /= p.sum()
        order = llama.topk(p, 2)
        w = llama.router_weights(p, order)
        assert abs(float(w.sum()) - 1.0) <= 2 ** -22
        assert np.allclose(w, p[order] / p[order].sum(), rtol=1e-6)
        raw = llama.router_weights(p, order, norm_w=False)
        assert raw.tolist() == p[order].tolist()
    # a selected mass below 2^-14 is divided by 2^-14, not by itself
    p = np.array([2.0 ** -20, 2.0 ** -21, 0, 0], np.float32)
    w = llama.router_weights(p, [0, 1])
    assert w.tolist() == [2.0 ** -6, 2.0 ** -7]
    # exactly at the clamp the sum itself is used
    p = np.array([2.0 ** -15, 2.0 ** -15], np.float32)
    assert llama.router_weights(p, [0, 1]).tolist() == [0.5, 0.5]


# ------------------------------------------------------------------ model

def test_model_with_experts_loads_its_parts(llama, pkg, moe_path):
    blob = np.fromfile(moe_path, dtype=np.uint8)
    by = {t[0]: t for t in llama.gguf_tensors(blob)}
    assert by["blk.0.ffn_gate_inp.weight"][1] == pkg.F32 and by["blk.0.ffn_gate_inp.weight"][2] == (256, 4)
    assert by["blk.1.ffn_gate_exps.weight"][2] == (256, 256, 4) and by["blk.1.ffn_down_exps.weight"][2] == (256, 256, 4)
    assert "blk.0.ffn_gate.weight" not in by
    m = llama.Llama(blob=blob, products=llama.CALLBACK, matmul=oracle_matmul)
    assert (m.hparams.n_expert, m.hparams.n_expert_used) == (4, 2)
    with pytest.raises(llama.LlamaError, match="dense feed-forward layers only"):
        llama.Llama(blob=blob).session(device_positions=32)
    dense = dict(TINY_MOE, n_expert=0, n_expert_used=0)
    with pytest.raises(llama.LlamaError, match="expert_used_count"):
        llama.write_synthetic_llama(moe_path.parent / "bad.gguf", **dict(TINY_MOE, n_expert_used=5))
    llama.write_synthetic_llama(moe_path.parent / "dense.gguf", **dense, seed=1)
    d = llama.Llama(path=moe_path.parent / "dense.gguf", products=llama.CALLBACK, matmul=oracle_matmul)
    assert (d.hparams.n_expert, d.hparams.n_expert_used) == (0, 0)
    with pytest.raises(llama.LlamaError, match="no routed feed-forward"):
        d.moe_ffn(0, np.zeros((1, 256), np.float32))


def _layer_weights(llama, blob, layer):
    by = {t[0]: t for t in llama.gguf_tensors(blob)}

    def parts(name):
        _, ty, shape, start, end = by[name]
        n_cols, n_rows, n_parts = shape
        return oracle.dequant(ty, n_cols, blob[start:end], n_rows * n_parts).astype(np.float64).reshape(n_parts, n_rows, n_cols)

    p = f"blk.{layer}."
    _, ty, shape, start, end = by[p + "ffn_gate_inp.weight"]
    router = oracle.dequant(ty, shape[0], blob[start:end], shape[1]).astype(np.float64)
    return router, parts(p + "ffn_gate_exps.weight"), parts(p + "ffn_up_exps.weight"), parts(p + "ffn_down_exps.weight")


def test_routed_ffn_matches_a_brute_force_float64_restatement(llama, moe_path):
    blob = np.fromfile(moe_path, dtype=np.uint8)
    m = llama.Llama(blob=blob, products=llama.CALLBACK, matmul=oracle_matmul)
    rng = np.random.default_rng(3)
    for layer, n in ((0, 1), (0, 7), (1, 33)):
        x = rng.normal(0, 1, (n, 256)).astype(np.float32)
        router, gate, up, down = _layer_weights(llama, blob, layer)
        want = numpy_moe_ffn(x.astype(np.float64), router, gate, up, down, 2)
        got = m.moe_ffn(layer, x)
        assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max(), (layer, n)
    # a token's row does not depend on which other tokens share the batch (grouping only reorders work)
    x = rng.normal(0, 1, (9, 256)).astype(np.float32)
    whole = m.moe_ffn(0, x)
    for t in range(9):
        alone = m.moe_ffn(0, x[t:t + 1])
        assert np.abs(alone[0] - whole[t]).max() <= 1e-5 * np.abs(whole).max(), t


def test_routing_edge_cases_through_the_whole_layer(llama, moe_path):
    """A zero input gives zero router logits: uniform probabilities, experts 0 and 1 (ties to the lower
    index) with weight one half each, and a zero output; experts nobody selects are skipped."""
    blob = np.fromfile(moe_path, dtype=np.uint8)
    calls = []

    def spy(ty, n_rows, n_cols, n_tokens, w, x):
        calls.append((n_rows, n_cols, n_tokens))
        return oracle.gemm(ty, n_cols, n_tokens, w, x, n_rows)

    m = llama.Llama(blob=blob, products=llama.CALLBACK, matmul=spy)
    out = m.moe_ffn(0, np.zeros((3, 256), np.float32))
    assert np.all(out == 0)
    # router, then gate for experts 0 and 1 with all three tokens each, then up, then down: 7 products, none for 2 and 3
    assert calls == [(4, 256, 3)] + [(256, 256, 3)] * 6
    # x aligned with router row e: expert e comes first for that token
    router, *_ = _layer_weights(llama, blob, 0)
    x = (8.0 * router / np.linalg.norm(router, axis=1, keepdims=True)).astype(np.float32)
    experts, _ = numpy_route(x.astype(np.float64) @ router.T, 2)
    assert experts[:, 0].tolist() == [0, 1, 2, 3]
    calls.clear()
    m.moe_ffn(0, x)
    counts = [int(np.sum(experts == e)) for e in range(4)]
    want = [(4, 256, 4)] + [(256, 256, c) for c in counts if c] * 3
    assert calls == want


def test_forward_with_experts_matches_the_float64_restatement(llama, moe_path):
    blob = np.fromfile(moe_path, dtype=np.uint8)
    m = llama.Llama(blob=blob, products=llama.CALLBACK, matmul=oracle_matmul)
    tokens = [3, 17, 12, 12, 55, 0, 41, 8, 60, 33, 2, 19, 50, 5, 28, 21, 9, 63, 30]
    want = numpy_forward(blob, llama.gguf_tensors(blob), m.hparams, tokens)
    scale = np.abs(want).max()
    got = m.session().forward(tokens)
    assert np.abs(got - want[-1]).max() <= 2e-4 * scale
    s = m.session()
    for i, t in enumerate(tokens):
        step = s.forward([t])
        assert np.abs(step - want[i]).max() <= 2e-4 * scale, i
    assert int(np.argmax(want[-1])) == llama.argmax(got)
    # greedy generation: the prompt as a batch, then single-token steps through the same routed layers
    out, _, _ = m.session().generate_greedy(tokens[:6], 8)
    s = m.session()
    tok = llama.argmax(s.forward(tokens[:6]))
    manual = [tok]
    for _ in range(7):
        tok = llama.argmax(s.forward([tok]))
        manual.append(tok)
    assert out.tolist() == manual
