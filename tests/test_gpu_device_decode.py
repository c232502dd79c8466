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
