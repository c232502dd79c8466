"""End-to-end greedy decode on the GPU against the same host code over the CPU checker.

The host arithmetic (norms, RoPE, attention, SwiGLU, argmax) is shared; what differs between
the two runs is only who computes the weight products: the HIP executor (resident matrices, or
the content-identified dispatch layer) or the oracle's restatement of the reference's CPU
kernels.  Identity of the generated tokens is therefore a statement about the products.
"""
import importlib

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def llama(pkg):
    return importlib.import_module("llama-rust_amd.llama")


def cpu_products(simd, threads):
    def matmul(ty, n_rows, n_cols, n_tokens, w, x):
        return oracle.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=simd, threads=threads)
    return matmul


def run_both(llama, path, prompt, n_new, simd, threads, products=None):
    gpu = llama.Llama(path=path, products=llama.RESIDENT if products is None else products)
    cpu = llama.Llama(path=path, products=llama.CALLBACK, matmul=cpu_products(simd, threads))
    sg, sc = gpu.session(), cpu.session()
    lg, lc = sg.forward(prompt), sc.forward(prompt)
    scale = float(np.abs(lc).max())
    worst = float(np.abs(lg - lc).max()) / scale
    toks_g, toks_c = [llama.argmax(lg)], [llama.argmax(lc)]
    margins = []
    for _ in range(n_new - 1):
        lg, lc = sg.forward([toks_g[-1]]), sc.forward([toks_c[-1]])
        top2 = np.sort(lc)[-2:]
        margins.append(float(top2[1] - top2[0]) / scale)
        if toks_g[-1] == toks_c[-1]:
            worst = max(worst, float(np.abs(lg - lc).max()) / scale)
        toks_g.append(llama.argmax(lg))
        toks_c.append(llama.argmax(lc))
    return toks_g, toks_c, worst, margins


@pytest.mark.parametrize("block_type,output_type", [(12, 14), (8, 8), (2, 6), (7, 1)])
def test_small_model_generates_the_same_tokens_as_the_cpu_path(pkg, llama, tmp_path, block_type, output_type):
    """Q4_K + Q6_K head (the Q4_K_M mix), Q8_0, Q4_0 + Q5_0 head, Q5_1 + F16 head."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=2048,
                                block_type=block_type, embd_type=block_type, output_type=output_type, seed=11)
    rng = np.random.default_rng(2)
    prompt = rng.integers(0, 2048, 24).tolist()
    toks_g, toks_c, worst, margins = run_both(llama, path, prompt, 24, simd=False, threads=1)
    assert toks_g == toks_c, (toks_g, toks_c, min(margins))
    assert worst <= 1e-4, worst  # logits, relative to the largest logit


def test_dispatch_route_equals_resident_route_and_hits_its_cache(pkg, llama, tmp_path):
    """The drop-in call shape (gemv_<t>_f32 / gemm_<t>_f32 behind the content-identified cache,
    langtax/src/native_gpu.rs:124-213) runs the same kernels on the same bytes."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=512, n_head=8, n_head_kv=4, n_ff=1024, n_vocab=1024, seed=5)
    prompt = list(range(100, 117))
    pkg.load_library().lnq_reset()
    a = llama.Llama(path=path, products=llama.RESIDENT)
    b = llama.Llama(path=path, products=llama.DISPATCH)
    ta, _, _ = a.session().generate_greedy(prompt, 10)
    tb, _, _ = b.session().generate_greedy(prompt, 10)
    assert ta.tolist() == tb.tolist()
    la, lb = a.session().forward(prompt), b.session().forward(prompt)
    assert la.view(np.uint32).tolist() == lb.view(np.uint32).tolist()
    st = pkg.cache_stats()
    # 15 matrices, 11 forward passes: each matrix uploaded once, found again ten times
    assert st["entries"] == 2 * 7 + 1 and st["misses"] == 15 and st["hits"] == 150


def test_prompt_as_one_batch_agrees_with_token_by_token_on_the_gpu(pkg, llama, tmp_path):
    """The batch runs the multi-token kernels, the steps the single-token ones: same values up to
    f32 summation order."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=1024, seed=9)
    m = llama.Llama(path=path)
    tokens = list(range(3, 3 + 37))
    batch = m.session().forward(tokens)
    s = m.session()
    for t in tokens:
        step = s.forward([t])
    assert np.abs(batch - step).max() <= 1e-4 * np.abs(batch).max()
    assert llama.argmax(batch) == llama.argmax(step)


def test_8b_layer_shapes_generate_the_same_tokens_as_the_simd_cpu_path(pkg, llama, tmp_path):
    """Two layers of the Llama-3-8B shape (d 4096, 32 / 8 heads, ffn 14336, vocab 128256, Q4_K with a
    Q6_K head, RoPE base 5e5, K/V block 16) against the restated AVX2 kernels with the reference's
    thread rule.  32 prompt tokens, 16 generated."""
    path = tmp_path / "l3.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=4096, n_head=32, n_head_kv=8, n_ff=14336, n_vocab=128256,
                                rope_base=5e5, rms_eps=1e-5, seed=1)
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, 128256, 32).tolist()
    toks_g, toks_c, worst, margins = run_both(llama, path, prompt, 16, simd=True, threads=0)
    assert toks_g == toks_c, (toks_g, toks_c, min(margins))
    assert worst <= 1e-4, worst


# ------------------------------------------------------------------ routed experts (llama with expert_count > 0)

@pytest.mark.parametrize("block_type", [12, 2])
def test_small_model_with_experts_generates_the_same_tokens_as_the_cpu_path(pkg, llama, tmp_path, block_type):
    """A 4-expert top-2 model (langtax/tests/native_cuda_parity.rs:198-288 runs its MoE tiny the same way):
    the host routing is shared, the router and expert products run on the GPU - as one grouped call per
    projection (resident route) and as one call per expert through the content-identified dispatch layer,
    the reference's call shape - against the CPU oracle's products."""
    path = tmp_path / "moe.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, n_ff=768, n_vocab=1024,
                                block_type=block_type, embd_type=block_type, output_type=8, seed=21,
                                weight_std=0.06, n_expert=4, n_expert_used=2)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, 1024, 21).tolist()
    toks_g, toks_c, worst, margins = run_both(llama, path, prompt, 20, simd=False, threads=1)
    assert toks_g == toks_c, (toks_g, toks_c, min(margins))
    assert worst <= 1e-4, worst
    pkg.load_library().lnq_reset()
    toks_d, _, worst_d, _ = run_both(llama, path, prompt, 20, simd=False, threads=1, products=llama.DISPATCH)
    assert toks_d == toks_c
    assert worst_d <= 1e-4, worst_d
    assert len(set(toks_c)) >= 15  # the layers matter: no fixed point, no short cycle


@pytest.mark.parametrize("kind", ["f32", "q4_0", "q4_k", "experts"])
def test_reference_session_scenario_on_every_path(pkg, llama, tmp_path, kind):
    """langtax/tests/native_cuda_parity.rs:198-249 for its four tiny models (F32, Q4_0, Q4_K weights, a model
    with experts): prefill [1, 2, 3], decode 4, 5, 1, then the divergent full prompt [1, 2, 4], which keeps the
    cached prefix [1, 2] and replaces the rest; a session with blocks of 2 positions beside one with large blocks.
    Here on three paths: host session over the HIP products, device session, host session over the CPU oracle."""
    spec = dict(n_layer=2, n_embd=256, n_head=4, n_head_kv=2, n_ff=512, n_vocab=96, seed=5, weight_std=0.06)
    if kind == "f32":
        spec.update(block_type=0, embd_type=0, output_type=0)
    elif kind == "q4_0":
        spec.update(block_type=2, embd_type=2, output_type=2)
    elif kind == "q4_k":
        spec.update(block_type=12, embd_type=12, output_type=14)
    else:
        spec.update(block_type=8, embd_type=8, output_type=8, n_expert=4, n_expert_used=2)
    path = tmp_path / "tiny.gguf"
    llama.write_synthetic_llama(path, **spec)
    gpu = llama.Llama(path=path)
    cpu = llama.Llama(path=path, products=llama.CALLBACK, matmul=cpu_products(False, 1))
    snapshots = {}
    for name, make in [("cpu", lambda kb: cpu.session(kv_block=kb)), ("host", lambda kb: gpu.session(kv_block=kb)),
                       ("device", lambda kb: gpu.session(kv_block=kb, device_positions=32))]:
        if name == "device" and kind == "experts":
            continue  # the device session is for dense models (it refuses others, tested elsewhere)
        for kb in (32, 2):
            s = make(kb)
            got = [s.forward([1, 2, 3])]
            got += [s.forward([t]) for t in (4, 5, 1)]
            reused, hit = s.prompt([1, 2, 4])
            assert hit == 2
            got.append(reused)
            fresh = make(kb).forward([1, 2, 4])
            assert np.abs(reused - fresh).max() <= 1e-5 * np.abs(fresh).max(), (name, kb)
            snapshots[(name, kb)] = np.stack(got)
    want = snapshots[("cpu", 32)]
    scale = np.abs(want).max()
    for key, got in snapshots.items():
        assert np.abs(got - want).max() <= 1e-4 * scale, key
        assert got.argmax(axis=1).tolist() == want.argmax(axis=1).tolist(), key


def test_mixtral_shaped_routed_layer_matches_the_cpu_path(pkg, llama, tmp_path, monkeypatch):
    """Benchmark configuration 5 as one checked result: 64 tokens, router logits of about unit deviation,
    softmax, top-2 of 8 experts, tokens grouped per expert, Q4_K gate / up (4096 -> 14336) and down
    (14336 -> 4096), weighted scatter-add - the whole layer on the GPU route against the same host code over
    the AVX2 restatement of the reference's CPU kernels.  Tolerance: every output within 1e-4 of
    max(|e|, rms(e) / 4), the relative criterion of the product tests applied to the layer's output."""
    path = tmp_path / "mixtral_layer.gguf"
    llama.write_synthetic_llama(path, n_layer=1, n_embd=4096, n_head=32, n_head_kv=8, n_ff=14336, n_vocab=256,
                                block_type=12, embd_type=8, output_type=8, seed=8, n_expert=8, n_expert_used=2)
    gpu = llama.Llama(path=path)
    cpu = llama.Llama(path=path, products=llama.CALLBACK, matmul=cpu_products(True, 0))
    rng = np.random.default_rng(64)
    x = rng.normal(0, 1, (64, 4096)).astype(np.float32)
    got, want = gpu.moe_ffn(0, x), cpu.moe_ffn(0, x)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert rms > 0 and np.all(np.isfinite(got))
    err = np.abs(got.astype(np.float64) - want)
    assert np.all(err <= 1e-4 * np.maximum(np.abs(want), rms / 4)), float((err / np.maximum(np.abs(want), rms / 4)).max())
    # one token alone takes the single-token kernels for its two experts: same row up to summation order
    alone = gpu.moe_ffn(0, x[5:6])
    assert np.all(np.abs(alone[0].astype(np.float64) - want[5]) <= 1e-4 * np.maximum(np.abs(want[5]), rms / 4))
    # the projections are chained on the device (rows up once, SiLU * up there, down outputs back); with
    # LLAMA_HIP_MOE_HOST_SWIGLU every projection is a call through host buffers and SiLU * up runs on the host, the
    # reference's call structure: same products, exp of the host instead of the device's
    monkeypatch.setenv("LLAMA_HIP_MOE_HOST_SWIGLU", "1")
    through_host = gpu.moe_ffn(0, x)
    monkeypatch.delenv("LLAMA_HIP_MOE_HOST_SWIGLU")
    err = np.abs(through_host.astype(np.float64) - want)
    assert np.all(err <= 1e-4 * np.maximum(np.abs(want), rms / 4))
    assert np.abs(through_host.astype(np.float64) - got).max() <= 2e-5 * rms
    assert np.array_equal(gpu.moe_ffn(0, x), got)  # and back: the same bits as before


def test_config4_full_size_greedy_decode_on_every_path(pkg, llama, tmp_path):
    """Benchmark configuration 4 at full size: a random Llama-3-8B-shaped model (32 layers, d 4096, 32 query /
    8 K/V heads of 128, ffn 14336, vocab 128256, RMSNorm eps 1e-5, RoPE base 5e5, Q4_K blocks with a Q6_K head),
    128 random prompt ids as one batch, then 128 greedy single-token steps over a paged K/V cache with blocks of
    16 positions.  The device-resident session, the host session (one GPU round trip per product, the
    reference's call structure) and the same host code over the restated AVX2 kernels of the reference's CPU
    path must produce the same 129 tokens.  The smallest gap between the two largest logits of any step,
    relative to the largest logit, says how much room rounding differences had (langtax/src/decode.rs:12104-12114
    takes the first maximum, so a flip needs two logits closer than the paths' disagreement, about 1e-5)."""
    path = tmp_path / "llama3_8b_shape.gguf"
    llama.write_synthetic_llama(path, n_layer=32, n_embd=4096, n_head=32, n_head_kv=8, n_ff=14336, n_vocab=128256,
                                rope_base=5e5, rms_eps=1e-5, weight_std=0.02, seed=20240531)
    prompt = np.random.default_rng(20240531).integers(0, 128256, 128)
    gpu = llama.Llama(path=path)
    host_toks, _, _ = gpu.session(kv_block=16).generate_greedy(prompt, 129)
    dev_toks, _, _ = gpu.session(kv_block=16, device_positions=256).generate_greedy(prompt, 129)
    gpu.close()
    cpu = llama.Llama(path=path, products=llama.CALLBACK, matmul=cpu_products(True, 0))
    s = cpu.session(kv_block=16)
    logits = s.forward(prompt)
    cpu_toks, gaps = [], []
    for step in range(129):
        top2 = np.partition(logits, -2)[-2:]
        gaps.append(float(top2[1] - top2[0]) / float(np.abs(logits).max()))
        cpu_toks.append(llama.argmax(logits))
        if step < 128:
            logits = s.forward([cpu_toks[-1]])
    print(f"\nconfig 4: 129 tokens, smallest top-2 logit gap {min(gaps):.3e} of the largest logit (step {int(np.argmin(gaps))})")
    assert host_toks.tolist() == cpu_toks, int(np.sum(np.cumprod(host_toks == np.array(cpu_toks))))
    assert dev_toks.tolist() == cpu_toks, int(np.sum(np.cumprod(dev_toks == np.array(cpu_toks))))
    assert min(gaps) > 1e-5
