"""The device-resident decode step against the host forward pass.

Both run the same model through the same resident matrices; the host session crosses the
host/device boundary once per product and does norms, RoPE, attention, SwiGLU and argmax in
the reference's operation order on the CPU, the device session does them in small kernels
between the products and replays one HIP graph per token.  They differ in the order of a few
f32 sums (RMSNorm, softmax denominator) and in the device's cos/sin/exp, so logits are
compared to 1e-4 of the largest logit and greedy tokens must be identical.
"""
import importlib

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def llama(pkg):
    return importlib.import_module("llama-rust_amd.llama")


def logits_close(a, b):
    return float(np.abs(a - b).max()) <= 1e-4 * float(np.abs(b).max())


@pytest.mark.parametrize("block_type,embd_type,output_type", [(12, 12, 14), (8, 8, 8), (2, 6, 6), (7, 1, 1), (14, 0, 2)])
def test_device_session_matches_the_host_session(pkg, llama, tmp_path, block_type, embd_type, output_type):
    """Every dtype appears as block, embedding and head type somewhere in the five mixes."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=2048,
                                block_type=block_type, embd_type=embd_type, output_type=output_type, seed=21)
    m = llama.Llama(path=path)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, 2048, 19).tolist()
    host, dev = m.session(), m.session(device_positions=64)
    lh, ld = host.forward(prompt), dev.forward(prompt)
    assert logits_close(ld, lh)
    for _ in range(12):  # teacher-forced by the host's pick, so one flip would not hide later errors
        t = llama.argmax(lh)
        assert llama.argmax(ld) == t
        lh, ld = host.forward([t]), dev.forward([t])
        assert logits_close(ld, lh)
    th, _, _ = m.session().generate_greedy(prompt, 20)
    td, _, _ = m.session(device_positions=19 + 20).generate_greedy(prompt, 20)
    assert td.tolist() == th.tolist()


@pytest.mark.parametrize("head_dim", [192, 256])
def test_device_session_with_large_heads(pkg, llama, tmp_path, head_dim):
    """Head sizes beyond 128 need more than 48 KB of LDS in both attention kernels (the single step and the
    prompt batch): the step and a 40-token prompt give the host session's tokens."""
    path = tmp_path / "wide_heads.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=2 * head_dim, n_head=2, n_head_kv=1, n_ff=1024, n_vocab=512,
                                block_type=8, embd_type=8, output_type=8, seed=31, weight_std=0.06)
    m = llama.Llama(path=path)
    assert m.hparams.head_dim == head_dim
    rng = np.random.default_rng(7)
    prompt = rng.integers(0, 512, 40).tolist()
    th, _, _ = m.session().generate_greedy(prompt, 10)
    td, _, _ = m.session(device_positions=64).generate_greedy(prompt, 10)
    assert td.tolist() == th.tolist()
    # a block table too long for the device's LDS is refused with the figures, before anything is launched
    with pytest.raises(llama.LlamaError, match="bytes of LDS"):
        m.session(kv_block=1, device_positions=1 << 16)


def test_device_session_pages_and_capacity(pkg, llama, tmp_path):
    """Any physical block order and block size gives the same tokens; running past the cache is an error
    raised before anything is launched."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=512, n_head=8, n_head_kv=4, n_ff=1024, n_vocab=1024, seed=6)
    m = llama.Llama(path=path)
    prompt = list(range(40, 40 + 21))
    ref, _, _ = m.session(kv_block=16, device_positions=48).generate_greedy(prompt, 12)
    perm = [3, 0, 5, 1, 4, 2, 6, 7, 9, 8, 11, 10]
    a, _, _ = m.session(kv_block=4, block_ids=perm, device_positions=48).generate_greedy(prompt, 12)
    assert a.tolist() == ref.tolist()
    s = m.session(kv_block=16, device_positions=32)
    s.forward(prompt)
    with pytest.raises(llama.LlamaError, match="outgrew"):
        s.forward(list(range(12)))
    assert llama.argmax(s.forward([5])) >= 0  # still usable, position 21
    with pytest.raises(llama.LlamaError, match="block ids"):
        m.session(kv_block=4, block_ids=[1, 0], device_positions=48)
    with pytest.raises(llama.LlamaError, match="resident"):
        llama.Llama(path=path, products=llama.DISPATCH).session(device_positions=16)


def test_device_session_8b_layer_shapes_against_the_simd_cpu_path(pkg, llama, tmp_path):
    """Two layers of the Llama-3-8B shape: the device session's greedy tokens equal those of the host
    code over the restated AVX2 kernels (the reference's CPU path)."""
    path = tmp_path / "l3.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=4096, n_head=32, n_head_kv=8, n_ff=14336, n_vocab=128256,
                                rope_base=5e5, rms_eps=1e-5, seed=1)
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, 128256, 24).tolist()

    def matmul(ty, n_rows, n_cols, n_tokens, w, x):
        return oracle.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=True, threads=0)
    cpu = llama.Llama(path=path, products=llama.CALLBACK, matmul=matmul)
    tc, _, _ = cpu.session().generate_greedy(prompt, 12)
    gpu = llama.Llama(path=path)
    td, _, _ = gpu.session(device_positions=64).generate_greedy(prompt, 12)
    assert td.tolist() == tc.tolist()


# ------------------------------------------------------------------ the fused prologues on their own

def _device(hip, a):
    return hip.DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.float32))


@pytest.mark.parametrize("rows,cols", [((4096, 1024, 1024), 4096), ((14336, 14336), 4096), ((4096,), 14336), ((300,), 512)])
def test_rmsnorm_prologue_equals_rmsnorm_then_product(pkg, rows, cols):
    """W (x * inv_rms(x) * g) with the norm done while the kernel stages x, against the float64 value of
    the same expression on the dequantized weights, inside the f32 summation bound of the product."""
    import cases as K
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(cols + len(rows))
    gpu = pkg.HipGemv(0)
    ws = [K.random_packed(K.Q4_K, r, cols, rng, signed=False, scale=0.02) for r in rows]
    mats = [gpu.upload_packed(K.Q4_K, r, cols, w) for r, w in zip(rows, ws)]
    x = rng.normal(0, 3.0, cols).astype(np.float32)
    g = (1 + rng.normal(0, 0.05, cols)).astype(np.float32)
    eps = 1e-5
    dx, dg = _device(hip, x), _device(hip, g)
    ys = [hip.DeviceBuffer(4 * r) for r in rows]
    for y in ys:
        y.fill_byte(0xff)
    gpu.gemv_fused_device(mats, dx.ptr, [y.ptr for y in ys], pkg.PROLOGUE_RMSNORM, dg.ptr, eps)
    gpu.synchronize()
    x64 = x.astype(np.float64)
    xn = x64 / np.sqrt(np.mean(x64 * x64) + eps) * g.astype(np.float64)
    for r, w, y in zip(rows, ws, ys):
        exact, mag = oracle.gemm_f64_mag(K.Q4_K, cols, 1, w, xn.astype(np.float32), r)
        # the f32 roundings of the normalised x (tree sum of squares, sqrt, two multiplies) on top of the product's bound
        exact64 = oracle.dequant(K.Q4_K, cols, w, r).astype(np.float64) @ xn
        got = y.to_numpy(np.float32)
        bound = K.single_kernel_bound(cols, mag.ravel()) + 16 * 2.0 ** -24 * mag.ravel()
        assert np.all(np.abs(got - exact64) <= bound), float(np.max(np.abs(got - exact64) / bound))
    # x itself is untouched
    assert dx.to_numpy(np.float32).view(np.uint32).tolist() == x.view(np.uint32).tolist()
    gpu.close()


def test_swiglu_prologue_accumulates_like_the_separate_steps(pkg):
    """x_res += W (SiLU(gate) * up), against float64 on the dequantized weights."""
    import cases as K
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(77)
    rows, cols = 4096, 14336
    gpu = pkg.HipGemv(0)
    w = K.random_packed(K.Q4_K, rows, cols, rng, signed=False, scale=0.02)
    m = gpu.upload_packed(K.Q4_K, rows, cols, w)
    gate = rng.normal(0, 2.0, cols).astype(np.float32)
    up = rng.normal(0, 1.0, cols).astype(np.float32)
    res = rng.normal(0, 1.0, rows).astype(np.float32)
    dgate, dup, dres = _device(hip, gate), _device(hip, up), _device(hip, res)
    gpu.gemv_fused_device([m], dgate.ptr, [dres.ptr], pkg.PROLOGUE_SWIGLU, dup.ptr, accumulate=True)
    gpu.synchronize()
    g64 = gate.astype(np.float64)
    h = g64 / (1 + np.exp(-g64)) * up.astype(np.float64)
    exact, mag = oracle.gemm_f64_mag(K.Q4_K, cols, 1, w, h.astype(np.float32), rows)
    exact64 = oracle.dequant(K.Q4_K, cols, w, rows).astype(np.float64) @ h + res.astype(np.float64)
    got = dres.to_numpy(np.float32)
    bound = K.single_kernel_bound(cols, mag.ravel()) + 8 * 2.0 ** -24 * (mag.ravel() + np.abs(exact64))
    assert np.all(np.abs(got - exact64) <= bound), float(np.max(np.abs(got - exact64) / bound))
    gpu.close()


def test_prologue_is_refused_where_it_is_not_built(pkg):
    """Other dtypes and rows longer than one launch: LNH_ERR_UNSUPPORTED, nothing written."""
    import cases as K
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(5)
    gpu = pkg.HipGemv(0)
    for ty, rows, cols in ((K.Q8_0, 64, 4096), (K.Q6_K, 64, 4096), (K.Q4_K, 16, 32768)):
        m = gpu.upload_packed(ty, rows, cols, K.random_packed(ty, rows, cols, rng, signed=False, scale=0.02))
        dx, dg = _device(hip, np.ones(cols)), _device(hip, np.ones(cols))
        y = hip.DeviceBuffer(4 * rows)
        y.fill_byte(0x5a)
        with pytest.raises(pkg.NativeHipError) as ei:
            gpu.gemv_fused_device([m], dx.ptr, [y.ptr], pkg.PROLOGUE_RMSNORM, dg.ptr, 1e-5)
        assert ei.value.code == pkg.ERR_UNSUPPORTED
        gpu.synchronize()
        assert set(y.to_numpy(np.uint8).tolist()) == {0x5a}
    gpu.close()


def test_fused_and_unfused_device_sessions_agree(pkg, llama, tmp_path, monkeypatch):
    """LLAMA_HIP_DECODE_UNFUSED keeps RMSNorm and SiLU*up as kernels of their own: same tokens, logits to 1e-4."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=2048, seed=33)
    m = llama.Llama(path=path)
    prompt = list(range(7, 7 + 15))
    fused = m.session(device_positions=48)
    monkeypatch.setenv("LLAMA_HIP_DECODE_UNFUSED", "1")
    plain = m.session(device_positions=48)
    monkeypatch.delenv("LLAMA_HIP_DECODE_UNFUSED")
    la, lb = fused.forward(prompt), plain.forward(prompt)
    assert logits_close(la, lb)
    ta, _, _ = m.session(device_positions=48).generate_greedy(prompt, 16)
    monkeypatch.setenv("LLAMA_HIP_DECODE_UNFUSED", "1")
    tb, _, _ = m.session(device_positions=48).generate_greedy(prompt, 16)
    assert ta.tolist() == tb.tolist()


@pytest.mark.parametrize("n_prompt", [3, 17, 140, 300])
def test_prompt_as_batches_equals_prompt_step_by_step(pkg, llama, tmp_path, monkeypatch, n_prompt):
    """All prompt tokens but the last run through the multi-token kernels in chunks of up to 128 (K and V into
    the cache, nothing else kept); LLAMA_HIP_DECODE_STEP_PREFILL runs them as single steps like decode.  Same
    tokens, logits to 1e-4, also across chunk boundaries (140: 128 + 11; 300: 128 + 128 + 43), for a prompt
    continued by a second one in the same session, and against the host session."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=2048, seed=35)
    m = llama.Llama(path=path)
    rng = np.random.default_rng(n_prompt)
    prompt = rng.integers(0, 2048, n_prompt).tolist()
    more = rng.integers(0, 2048, 9).tolist()
    cap = n_prompt + 9 + 12
    batched = m.session(device_positions=cap)
    monkeypatch.setenv("LLAMA_HIP_DECODE_STEP_PREFILL", "1")
    stepped = m.session(device_positions=cap)
    monkeypatch.delenv("LLAMA_HIP_DECODE_STEP_PREFILL")
    host = m.session()
    la, lb, lh = batched.forward(prompt), stepped.forward(prompt), host.forward(prompt)
    assert logits_close(la, lb) and logits_close(la, lh)
    la, lb, lh = batched.forward(more), stepped.forward(more), host.forward(more)  # a second chunk at past > 0
    assert logits_close(la, lb) and logits_close(la, lh)
    ta, _, _ = m.session(device_positions=cap).generate_greedy(prompt, 12)
    monkeypatch.setenv("LLAMA_HIP_DECODE_STEP_PREFILL", "1")
    tb, _, _ = m.session(device_positions=cap).generate_greedy(prompt, 12)
    assert ta.tolist() == tb.tolist()


@pytest.mark.parametrize("n_seq,block_type", [(1, 12), (2, 12), (3, 2), (8, 12), (19, 8), (5, 14)])
def test_batch_session_equals_independent_sessions(pkg, llama, tmp_path, n_seq, block_type):
    """Sequences decoded together, one token of each per step (the weight products as one multi-token product:
    single-token launches for 1 and 2 sequences, 16-token tiles up to 16, 32-token tiles above, and the 32-token
    tiles for Q6_K), against every sequence decoded on its own in a device session: the same tokens.  Prompts
    of different lengths, one of a single token, one longer than a prompt chunk."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=2048,
                                block_type=block_type, seed=41)
    m = llama.Llama(path=path)
    rng = np.random.default_rng(100 + n_seq)
    lens = [1, 150, 7, 33, 2, 64, 19, 5] + [int(v) for v in rng.integers(1, 40, 32)]
    prompts = [rng.integers(0, 2048, lens[b]).tolist() for b in range(n_seq)]
    n_new, cap = 14, 176
    bs = m.batch_session(n_seq, cap)
    together, _, _ = bs.generate_greedy(prompts, n_new)
    for b in range(n_seq):
        alone, _, _ = m.session(device_positions=cap).generate_greedy(prompts[b], n_new)
        assert together[b].tolist() == alone.tolist(), f"sequence {b} of {n_seq}"
    # A second generation in the same session starts every sequence afresh.  In between the executor's workspace
    # has grown (128-token prompt chunks above, a 300-token host batch here): the session's captured step still
    # points at the workspace it was captured with, which therefore must not have been freed.
    m.session().forward(rng.integers(0, 2048, 300).tolist())
    again, _, _ = bs.generate_greedy(prompts[::-1], n_new)
    assert again[::-1].tolist() == together.tolist()


@pytest.mark.parametrize("n_embd,n_head_kv", [(1024, 8), (4096, 8), (1024, 16), (1024, 32)])
def test_batch_step_with_more_heads_times_rows_than_large_workgroups_fit(pkg, llama, tmp_path, n_embd, n_head_kv):
    """A step whose heads x sequences exceed two 1024-thread workgroups per CU (32 heads x 20 sequences = 640 > 512
    on a 256-CU part) takes, where four query heads share a K/V head, the attention kernel with one workgroup per
    K/V head and sequence (head sizes 32 and 128), otherwise the one with 256-thread workgroups, the prompt chunks'
    instantiation with RoPE and the K/V store inside: the same tokens as every sequence decoded on its own
    (1024-thread kernel)."""
    path = tmp_path / "heads.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=n_embd, n_head=32, n_head_kv=n_head_kv, n_ff=1536, n_vocab=2048, seed=43)
    m = llama.Llama(path=path)
    rng = np.random.default_rng(77)
    n_seq, n_new, cap = 20, 10, 96
    prompts = [rng.integers(0, 2048, int(n)).tolist() for n in rng.integers(1, 70, n_seq)]
    together, _, _ = m.batch_session(n_seq, cap).generate_greedy(prompts, n_new)
    for b in range(n_seq):
        alone, _, _ = m.session(device_positions=cap).generate_greedy(prompts[b], n_new)
        assert together[b].tolist() == alone.tolist(), f"sequence {b}"


@pytest.mark.parametrize("block_type,output_type,n_seq", [(12, 1, 8), (12, 14, 20), (1, 1, 5), (2, 0, 3)])
def test_split_activation_chain_and_separate_launches_give_the_same_session(pkg, llama, tmp_path, monkeypatch, block_type,
                                                                            output_type, n_seq):
    """Multi-token steps keep their activations split between products (lnh_gemm_act_device) unless
    LLAMA_HIP_BATCH_UNFUSED is set or a layer matrix is F16 / F32: both ways the same tokens from the batch session
    and, for a prompt that runs as chunks, the same logits bit for bit from the device session (the fused launches
    sum and normalise in the order of the kernels they replace).  Heads that read plain rows (F16, F32) and heads
    that read split activations (Q6_K) both occur."""
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=1536, n_vocab=2048,
                                block_type=block_type, embd_type=block_type, output_type=output_type, seed=47)
    m = llama.Llama(path=path)
    rng = np.random.default_rng(7 + n_seq)
    prompts = [rng.integers(0, 2048, int(n)).tolist() for n in rng.integers(1, 90, n_seq)]
    long_prompt = rng.integers(0, 2048, 141).tolist()
    chained = m.batch_session(n_seq, 128).generate_greedy(prompts, 12)[0]
    logits_chained = m.session(device_positions=160).forward(long_prompt)
    monkeypatch.setenv("LLAMA_HIP_BATCH_UNFUSED", "1")
    separate = m.batch_session(n_seq, 128).generate_greedy(prompts, 12)[0]
    logits_separate = m.session(device_positions=160).forward(long_prompt)
    assert chained.tolist() == separate.tolist()
    assert logits_chained.view(np.uint32).tolist() == logits_separate.view(np.uint32).tolist()


@pytest.mark.parametrize("block_type,n_seq,n_prompt", [(12, 3, 4), (12, 8, 18), (2, 32, 33), (8, 5, 30)])
def test_split_activation_chain_where_n_ff_equals_n_embd(pkg, llama, tmp_path, monkeypatch, block_type, n_seq, n_prompt):
    """n_ff == n_embd with one block dtype: the input of the down product and the input of the next layer's q, k, v
    have the same dtype and column count, and must still be two buffers (the down product reads the one while its
    epilogue writes the other).  Steps of 3..32 rows and prompt chunks of 3..32 tokens, chained and with
    LLAMA_HIP_BATCH_UNFUSED: same tokens, same logits bit for bit."""
    path = tmp_path / "square.gguf"
    llama.write_synthetic_llama(path, n_layer=3, n_embd=512, n_head=8, n_head_kv=2, n_ff=512, n_vocab=2048,
                                block_type=block_type, embd_type=block_type, output_type=block_type, seed=53)
    m = llama.Llama(path=path)
    rng = np.random.default_rng(11 + n_seq)
    prompts = [rng.integers(0, 2048, int(n)).tolist() for n in rng.integers(1, 40, n_seq)]
    chunk_prompt = rng.integers(0, 2048, n_prompt).tolist()
    chained = m.batch_session(n_seq, 64).generate_greedy(prompts, 10)[0]
    logits_chained = m.session(device_positions=64).forward(chunk_prompt)
    monkeypatch.setenv("LLAMA_HIP_BATCH_UNFUSED", "1")
    separate = m.batch_session(n_seq, 64).generate_greedy(prompts, 10)[0]
    logits_separate = m.session(device_positions=64).forward(chunk_prompt)
    assert chained.tolist() == separate.tolist()
    assert logits_chained.view(np.uint32).tolist() == logits_separate.view(np.uint32).tolist()


def test_batch_session_refuses_what_it_cannot_do(pkg, llama, tmp_path):
    path = tmp_path / "small.gguf"
    llama.write_synthetic_llama(path, n_layer=2, n_embd=256, n_head=4, n_head_kv=2, n_ff=512, n_vocab=512, seed=43)
    m = llama.Llama(path=path)
    with pytest.raises(Exception):
        m.batch_session(129, 32)
    s = m.batch_session(2, 32)
    with pytest.raises(Exception):
        s.generate_greedy([[1, 2, 3], [4] * 40], 4)  # 40 + 4 - 1 positions > 32
    with pytest.raises(Exception):
        s.generate_greedy([[1, 2, 3], []], 4)
    with pytest.raises(Exception):
        s.generate_greedy([[1, 2, 3], [600]], 4)  # token id out of range
    out, _, _ = s.generate_greedy([[1, 2, 3], [4, 5]], 4)  # still usable
    assert out.shape == (2, 4)


@pytest.mark.parametrize("rows,cols,norm", [(14336, 4096, True), (14336, 4096, False), (1536, 2048, True), (1000, 8192, False)])
def test_paired_swiglu_epilogue_equals_the_separate_steps(pkg, rows, cols, norm):
    """h = SiLU(gate x') * (up x') from one launch against float64 on the dequantized weights: each product
    inside its own f32 summation bound, propagated through SiLU * up."""
    import cases as K
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(rows + cols)
    gpu = pkg.HipGemv(0)
    wg = K.random_packed(K.Q4_K, rows, cols, rng, signed=False, scale=0.02)
    wu = K.random_packed(K.Q4_K, rows, cols, rng, signed=False, scale=0.02)
    mg, mu = gpu.upload_packed(K.Q4_K, rows, cols, wg), gpu.upload_packed(K.Q4_K, rows, cols, wu)
    x = rng.normal(0, 1.0, cols).astype(np.float32)
    g = (1 + rng.normal(0, 0.05, cols)).astype(np.float32)
    eps = 1e-5
    dx, dg, dh = _device(hip, x), _device(hip, g), hip.DeviceBuffer(4 * rows)
    dh.fill_byte(0xff)
    if norm:
        gpu.gemv_swiglu_device(mg, mu, dx.ptr, dh.ptr, pkg.PROLOGUE_RMSNORM, dg.ptr, eps)
        x64 = x.astype(np.float64)
        xin = x64 / np.sqrt(np.mean(x64 * x64) + eps) * g.astype(np.float64)
    else:
        gpu.gemv_swiglu_device(mg, mu, dx.ptr, dh.ptr)
        xin = x.astype(np.float64)
    gpu.synchronize()
    got = dh.to_numpy(np.float32).astype(np.float64)
    a = oracle.dequant(K.Q4_K, cols, wg, rows).astype(np.float64) @ xin
    b = oracle.dequant(K.Q4_K, cols, wu, rows).astype(np.float64) @ xin
    _, mag_a = oracle.gemm_f64_mag(K.Q4_K, cols, 1, wg, xin.astype(np.float32), rows)
    _, mag_b = oracle.gemm_f64_mag(K.Q4_K, cols, 1, wu, xin.astype(np.float32), rows)
    slack = 16 * 2.0 ** -24
    ea = K.single_kernel_bound(cols, mag_a.ravel()) + slack * mag_a.ravel()
    eb = K.single_kernel_bound(cols, mag_b.ravel()) + slack * mag_b.ravel()
    with np.errstate(over="ignore"):
        sig = 1 / (1 + np.exp(-a))
    silu, dsilu = a * sig, sig * (1 + a * (1 - sig))
    want = silu * b
    # first-order propagation of the two products' bounds, second-order term, and the roundings of SiLU * up itself
    bound = np.abs(dsilu * b) * ea + np.abs(silu) * eb + 2 * ea * eb + 8 * 2.0 ** -24 * np.abs(want) + 1e-30
    assert np.all(np.abs(got - want) <= bound), float(np.max(np.abs(got - want) / bound))
    gpu.close()


def test_paired_swiglu_is_refused_where_it_is_not_built(pkg):
    import cases as K
    hip = importlib.import_module("llama-rust_amd.hiprt")
    rng = np.random.default_rng(9)
    gpu = pkg.HipGemv(0)
    # another dtype; a launch too large to give every unit its own wavefront; rows shorter than 2048 columns; unequal shapes
    for ty, rows, cols, rows2, code in ((K.Q8_0, 64, 4096, 64, pkg.ERR_UNSUPPORTED), (K.Q4_K, 65536, 4096, 65536, pkg.ERR_UNSUPPORTED),
                                        (K.Q4_K, 64, 512, 64, pkg.ERR_UNSUPPORTED), (K.Q4_K, 64, 4096, 128, pkg.ERR_INVALID)):
        a = gpu.upload_packed(ty, rows, cols, K.random_packed(ty, rows, cols, rng, signed=False, scale=0.02))
        b = gpu.upload_packed(ty, rows2, cols, K.random_packed(ty, rows2, cols, rng, signed=False, scale=0.02))
        dx, dh = _device(hip, np.ones(cols)), hip.DeviceBuffer(4 * rows)
        dh.fill_byte(0x5a)
        with pytest.raises(pkg.NativeHipError) as ei:
            gpu.gemv_swiglu_device(a, b, dx.ptr, dh.ptr)
        assert ei.value.code == code
        gpu.synchronize()
        assert set(dh.to_numpy(np.uint8).tolist()) == {0x5a}
    gpu.close()
