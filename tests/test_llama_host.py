"""Host side of the dense Llama decode (include/native_hip_llama.h), on the CPU.

The weight products are supplied by the test (the oracle's restatement of the
reference's scalar kernels), so everything here runs without a GPU: the GGUF
container, the row dequantizers, RMSNorm / RoPE / softmax / argmax against closed
forms, the paged K/V addressing, and the whole forward pass against an independent
float64 restatement of langtax/src/decode.rs:2710-3099 written with numpy.
"""
import importlib
import os
import struct

import numpy as np
import pytest

import oracle

TINY = dict(n_layer=2, n_embd=256, n_head=4, n_head_kv=2, n_ff=512, n_vocab=96)


@pytest.fixture(scope="module")
def llama(pkg):
    return importlib.import_module("llama-rust_amd.llama")


def oracle_matmul(ty, n_rows, n_cols, n_tokens, w, x):
    return oracle.gemm(ty, n_cols, n_tokens, w, x, n_rows)


@pytest.fixture(scope="module")
def tiny_path(llama, tmp_path_factory):
    path = tmp_path_factory.mktemp("gguf") / "tiny.gguf"
    llama.write_synthetic_llama(path, **TINY, seed=7)
    return path


# ------------------------------------------------------------------ container

def test_synthetic_model_is_a_wellformed_gguf_v3(llama, pkg, tiny_path):
    blob = np.fromfile(tiny_path, dtype=np.uint8)
    assert bytes(blob[:4]) == b"GGUF" and struct.unpack("<I", bytes(blob[4:8]))[0] == 3
    n_tensors, n_kv = struct.unpack("<qq", bytes(blob[8:24]))
    assert (n_tensors, n_kv) == (3 + 9 * TINY["n_layer"], 13)
    assert llama.gguf_inspect(blob) == (n_tensors, n_kv, 32)
    tensors = llama.gguf_tensors(blob)
    names = [t[0] for t in tensors]
    assert names[0] == "token_embd.weight" and names[-1] == "output.weight" and "blk.1.ffn_down.weight" in names
    prev_end = 0
    for name, ty, shape, start, end in tensors:
        assert start % 32 == 0 and start >= prev_end and start - prev_end < 32 + (prev_end == 0) * 10**6, name
        n_el = int(np.prod(shape))
        assert end - start == n_el // oracle.block_elems(ty) * oracle.block_bytes(ty), name
        prev_end = end
    assert prev_end == blob.size  # no padding after the last tensor (langtax/src/gguf.rs:690-701)
    by = {t[0]: t for t in tensors}
    assert by["blk.0.attn_k.weight"][2] == (256, 128)  # ggml order: columns first
    assert by["blk.0.ffn_down.weight"][2] == (512, 256)
    assert by["blk.0.attn_q.weight"][1] == pkg.Q4_K and by["output.weight"][1] == pkg.Q6_K
    assert by["output_norm.weight"][1] == pkg.F32 and by["output_norm.weight"][2] == (256,)


def test_gguf_parser_rejects_what_the_reference_rejects(llama, tiny_path):
    """langtax/src/gguf.rs:728-828: magic, version, truncation, zero dims, unknown tensor type."""
    blob = np.fromfile(tiny_path, dtype=np.uint8)
    bad = blob.copy(); bad[0] = ord("X")
    with pytest.raises(llama.LlamaError, match="bad magic"):
        llama.gguf_inspect(bad)
    bad = blob.copy(); bad[4] = 2
    with pytest.raises(llama.LlamaError, match="unsupported version 2"):
        llama.gguf_inspect(bad)
    for cut in (3, 7, 20, 200, blob.size - 1):
        with pytest.raises(llama.LlamaError, match="truncated"):
            llama.gguf_inspect(blob[:cut].copy())
    bad = blob.copy(); bad[8:16] = np.frombuffer(struct.pack("<q", -1), dtype=np.uint8)
    with pytest.raises(llama.LlamaError, match="truncated"):
        llama.gguf_inspect(bad)
    # first tensor info: name, n_dims, dims, type -- find it after the keys
    at = bytes(blob).index(b"token_embd.weight") + len(b"token_embd.weight")
    bad = blob.copy(); bad[at:at + 4] = np.frombuffer(struct.pack("<I", 5), dtype=np.uint8)
    with pytest.raises(llama.LlamaError, match="bad shape"):
        llama.gguf_inspect(bad)
    bad = blob.copy(); bad[at + 4:at + 12] = 0
    with pytest.raises(llama.LlamaError, match="bad shape"):
        llama.gguf_inspect(bad)
    bad = blob.copy(); bad[at + 20:at + 24] = np.frombuffer(struct.pack("<i", 99), dtype=np.uint8)
    with pytest.raises(llama.LlamaError, match="unsupported ggml type 99"):
        llama.gguf_inspect(bad)


def test_handwritten_gguf_with_every_metadata_type_loads(llama):
    """A file built here byte by byte (not by the library's writer): the parser is checked against the
    format itself, including arrays, 64-bit values and a non-default alignment."""
    def s(x):
        return struct.pack("<Q", len(x)) + x
    kv = [
        (b"general.alignment", 4, struct.pack("<I", 64)),
        (b"a.u8", 0, b"\x07"), (b"a.i8", 1, b"\xff"), (b"a.u16", 2, struct.pack("<H", 9)),
        (b"a.i16", 3, struct.pack("<h", -9)), (b"a.i32", 5, struct.pack("<i", -5)),
        (b"a.f32", 6, struct.pack("<f", 1.5)), (b"a.bool", 7, b"\x01"), (b"a.str", 8, s(b"hi")),
        (b"a.arr", 9, struct.pack("<iQ", 8, 2) + s(b"x") + s(b"yz")),
        (b"a.u64", 10, struct.pack("<Q", 1 << 40)), (b"a.i64", 11, struct.pack("<q", -(1 << 40))),
        (b"a.f64", 12, struct.pack("<d", 2.5)),
    ]
    head = b"GGUF" + struct.pack("<Iqq", 3, 2, len(kv))
    for k, ty, payload in kv:
        head += s(k) + struct.pack("<i", ty) + payload
    t0 = np.arange(8, dtype=np.float32).tobytes()
    t1 = np.arange(32, dtype=np.float16).tobytes()
    head += s(b"t0") + struct.pack("<Iq", 1, 8) + struct.pack("<iQ", 0, 0)
    head += s(b"t1") + struct.pack("<Iqq", 2, 16, 2) + struct.pack("<iQ", 1, 64)
    data_start = (len(head) + 63) // 64 * 64
    blob = head + b"\0" * (data_start - len(head)) + t0 + b"\0" * 32 + t1
    assert llama.gguf_inspect(blob) == (2, 13, 64)
    tensors = llama.gguf_tensors(blob)
    assert tensors[0] == ("t0", 0, (8,), data_start, data_start + 32)
    assert tensors[1] == ("t1", 1, (16, 2), data_start + 64, data_start + 128)
    with pytest.raises(llama.LlamaError, match="truncated"):
        llama.gguf_inspect(blob[:-1])


def test_gguf_parser_survives_hostile_counts_and_shapes(llama):
    """A short file must not be able to reserve memory through an array count, a shape whose byte count
    wraps 64 bits must not pass the size check, and a row that is not a whole number of blocks is refused at
    parse time (the row dequantizers and the device kernels walk rows block by block)."""
    def s(x):
        return struct.pack("<Q", len(x)) + x

    def gguf(kv_bytes, n_kv, tensor_bytes, n_tensors, data=b""):
        head = b"GGUF" + struct.pack("<Iqq", 3, n_tensors, n_kv) + kv_bytes + tensor_bytes
        pad = (len(head) + 31) // 32 * 32 - len(head)
        return np.frombuffer(head + b"\0" * pad + data, dtype=np.uint8)

    # array of 2^40 one-byte elements in a 60-byte file; and of 2^40 strings
    for elem in (0, 8):
        kv = s(b"a.arr") + struct.pack("<i", 9) + struct.pack("<iQ", elem, 1 << 40)
        with pytest.raises(llama.LlamaError, match="truncated"):
            llama.gguf_inspect(gguf(kv, 1, b"", 0))
    # a count that fits the remaining bytes but whose elements do not
    kv = s(b"a.arr") + struct.pack("<i", 9) + struct.pack("<iQ", 10, 3) + struct.pack("<Q", 1)
    with pytest.raises(llama.LlamaError, match="truncated"):
        llama.gguf_inspect(gguf(kv, 1, b"", 0))
    # F32 tensor of 2^62 elements: 2^64 bytes wraps to 0
    t = s(b"t") + struct.pack("<Iqq", 2, 1 << 31, 1 << 31) + struct.pack("<iQ", 0, 0)
    with pytest.raises(llama.LlamaError, match="bad shape|truncated"):
        llama.gguf_inspect(gguf(b"", 0, t, 1))
    # element count beyond 64 bits
    t = s(b"t") + struct.pack("<Iqqq", 3, 1 << 40, 1 << 40, 1 << 40) + struct.pack("<iQ", 0, 0)
    with pytest.raises(llama.LlamaError, match="bad shape"):
        llama.gguf_inspect(gguf(b"", 0, t, 1))
    # Q8_0 rows of 48 columns: two rows make whole blocks in total (96 = 3 x 32), one row does not
    t = s(b"t") + struct.pack("<Iqq", 2, 48, 2) + struct.pack("<iQ", 8, 0)
    with pytest.raises(llama.LlamaError, match="bad shape"):
        llama.gguf_inspect(gguf(b"", 0, t, 1, b"\0" * 102))
    t = s(b"t") + struct.pack("<Iqq", 2, 64, 2) + struct.pack("<iQ", 8, 0)
    assert llama.gguf_inspect(gguf(b"", 0, t, 1, b"\0" * 136)) == (1, 0, 32)


# ------------------------------------------------------------------ building blocks

def test_row_dequantizers_match_the_oracle_bit_for_bit(llama, pkg):
    """The embedding lookup dequantizes one row; its values are the definition every product uses."""
    rng = np.random.default_rng(5)
    for ty in pkg.ALL_TYPES:
        n_cols = 512
        rb = oracle.row_bytes(ty, n_cols)
        for _ in range(4):
            row = rng.integers(0, 256, rb, dtype=np.uint8)
            if ty in (pkg.F32, pkg.F16):  # keep floats finite
                row = (rng.standard_normal(n_cols).astype(np.float32 if ty == pkg.F32 else np.float16)
                       .view(np.uint8).copy())
            else:
                bb = oracle.block_bytes(ty)
                blocks = row.reshape(-1, bb)
                for off in {pkg.Q4_0: (0,), pkg.Q5_0: (0,), pkg.Q5_1: (0, 2), pkg.Q8_0: (0,), pkg.Q4_K: (0, 2),
                            pkg.Q6_K: (208,)}[ty]:
                    scale = rng.standard_normal(blocks.shape[0]).astype(np.float16)
                    blocks[:, off:off + 2] = scale.view(np.uint8).reshape(-1, 2)
                if ty == pkg.Q4_K:  # include a subnormal scale
                    blocks[0, 0:2] = np.array([3], dtype=np.uint16).view(np.uint8)
            got = llama.dequant_row(ty, n_cols, row)
            want = oracle.dequant_row(ty, n_cols, row)
            assert got.view(np.uint32).tolist() == want.view(np.uint32).tolist(), pkg.TYPE_NAMES[ty]
    with pytest.raises(llama.LlamaError, match="row length"):
        llama.dequant_row(pkg.Q8_0, 64, np.zeros(67, dtype=np.uint8))
    with pytest.raises(llama.LlamaError, match="unsupported ggml type"):
        llama.dequant_row(3, 64, np.zeros(64, dtype=np.uint8))


def test_rmsnorm_closed_forms(llama):
    """langtax/src/decode.rs:11498-11513."""
    x = np.full(64, 3.0, dtype=np.float32)
    w = np.arange(64, dtype=np.float32)
    out = llama.rmsnorm(x, w, 0.0)
    assert np.array_equal(out, w)  # x / rms = 1 exactly for a constant vector
    out = llama.rmsnorm(np.zeros(8, dtype=np.float32), np.ones(8, dtype=np.float32), 0.0)
    assert np.array_equal(out, np.zeros(8))  # rms 0 -> inverse 0, not a NaN
    rng = np.random.default_rng(0)
    x = rng.standard_normal(4096).astype(np.float32)
    w = rng.standard_normal(4096).astype(np.float32)
    want = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5) * w
    assert np.allclose(llama.rmsnorm(x, w, 1e-5), want, rtol=2e-6, atol=1e-7)
    # eps matters: with huge eps the output collapses
    assert np.abs(llama.rmsnorm(x, w, 1e12)).max() < 1e-4


def test_rope_rotates_adjacent_pairs(llama):
    """langtax/src/decode.rs:11578-11602: pair (2i, 2i+1) by pos * base^(-2i/n_rot); elements past n_rot stay."""
    rng = np.random.default_rng(1)
    v = rng.standard_normal(128).astype(np.float32)
    assert np.array_equal(llama.rope(v, 0, 128, 5e5), v)  # position 0: cos 1, sin 0
    for pos, n_rot, base in [(1, 128, 5e5), (17, 128, 1e4), (255, 64, 5e5)]:
        got = llama.rope(v, pos, n_rot, base)
        i = np.arange(n_rot // 2, dtype=np.float64)
        th = pos * float(base) ** (-2.0 * i / n_rot)
        z = (v[0:n_rot:2].astype(np.float64) + 1j * v[1:n_rot:2]) * np.exp(1j * th)
        want = v.astype(np.float64).copy()
        want[0:n_rot:2], want[1:n_rot:2] = z.real, z.imag
        assert np.allclose(got, want, atol=2e-4), (pos, n_rot)  # theta is accumulated in f32
        assert np.array_equal(got[n_rot:], v[n_rot:])
        pair_norm = got[0:n_rot:2] ** 2 + got[1:n_rot:2] ** 2
        assert np.allclose(pair_norm, v[0:n_rot:2] ** 2 + v[1:n_rot:2] ** 2, rtol=1e-5)
    # the relative-position property attention relies on: <R_p q, R_s k> depends on p - s only
    q, k = rng.standard_normal(64).astype(np.float32), rng.standard_normal(64).astype(np.float32)
    d1 = float(llama.rope(q, 9, 64, 1e4) @ llama.rope(k, 4, 64, 1e4))
    d2 = float(llama.rope(q, 25, 64, 1e4) @ llama.rope(k, 20, 64, 1e4))
    assert abs(d1 - d2) < 1e-3


def test_softmax_and_argmax(llama):
    """langtax/src/decode.rs:12021-12033, 12104-12114."""
    p = llama.softmax([1000.0, 1000.0, -np.inf, 999.0])
    assert abs(p.sum() - 1.0) < 1e-6 and p[2] == 0.0 and p[0] == p[1] > p[3] > 0
    e = np.exp(np.float32(-1.0))
    assert np.allclose(p[3] / p[0], e, rtol=1e-6)
    assert np.array_equal(llama.softmax([5.0]), [1.0])
    assert llama.argmax([1.0, 7.0, 7.0, -2.0]) == 1  # first maximum wins
    assert llama.argmax([-np.inf, -np.inf]) == 0
    assert llama.argmax([np.nan, 1.0]) == 1  # comparisons with NaN are false


# ------------------------------------------------------------------ forward pass

from llama_ref import numpy_forward  # noqa: E402  (independent float64 forward, shared with the routed-expert tests)


def test_model_load_reads_the_hyper_parameters(llama, pkg, tiny_path):
    m = llama.Llama(path=tiny_path, products=llama.CALLBACK, matmul=oracle_matmul)
    hp = m.hparams
    assert (hp.n_layer, hp.n_embd, hp.n_head, hp.n_head_kv, hp.n_ff, hp.n_vocab) == (2, 256, 4, 2, 512, 96)
    assert (hp.head_dim, hp.n_rot) == (64, 64)
    assert abs(hp.rope_base - 5e5) < 1 and abs(hp.rms_eps - 1e-5) < 1e-9
    assert (hp.block_type, hp.embd_type, hp.output_type) == (pkg.Q4_K, pkg.Q4_K, pkg.Q6_K)
    with pytest.raises(llama.LlamaError, match="cannot open"):
        llama.Llama(path="/nonexistent/model.gguf")
    with pytest.raises(llama.LlamaError, match="bad magic"):
        llama.Llama(blob=np.zeros(64, dtype=np.uint8))


def test_forward_matches_an_independent_float64_restatement(llama, tiny_path):
    blob = np.fromfile(tiny_path, dtype=np.uint8)
    m = llama.Llama(blob=blob, products=llama.CALLBACK, matmul=oracle_matmul)
    tokens = [3, 77, 12, 12, 95, 0, 41, 8, 60, 33, 2, 19, 70, 5, 88, 21, 9, 64, 30]  # 19: crosses a K/V block
    want = numpy_forward(blob, llama.gguf_tensors(blob), m.hparams, tokens)
    scale = np.abs(want).max()
    # the prompt as one batch: logits of the last position
    got = m.session().forward(tokens)
    assert np.abs(got - want[-1]).max() <= 2e-4 * scale
    # token by token (decode): every position's logits, and the same K/V contents
    s = m.session()
    for i, t in enumerate(tokens):
        step = s.forward([t])
        assert np.abs(step - want[i]).max() <= 2e-4 * scale, i
    # a prefix as a batch, the rest one at a time
    s = m.session()
    s.forward(tokens[:7])
    for i in range(7, len(tokens)):
        step = s.forward([tokens[i]])
    assert np.abs(step - want[-1]).max() <= 2e-4 * scale
    assert int(np.argmax(want[-1])) == llama.argmax(got)


def test_paged_kv_is_independent_of_block_size_and_placement(llama, tiny_path):
    """langtax/src/kv_page.rs:410-438: only addressing changes, so logits are bit-identical."""
    m = llama.Llama(path=tiny_path, products=llama.CALLBACK, matmul=oracle_matmul)
    tokens = list(range(40))
    ref = m.session(kv_block=16).forward(tokens)
    for kv_block, ids in [(1, None), (5, None), (64, None), (16, [2, 0, 1]), (4, list(range(9, -1, -1)))]:
        got = m.session(kv_block=kv_block, block_ids=ids).forward(tokens)
        assert got.view(np.uint32).tolist() == ref.view(np.uint32).tolist(), (kv_block, ids)
    with pytest.raises(llama.LlamaError, match="outgrew"):
        m.session(kv_block=16, block_ids=[1, 0]).forward(tokens)
    with pytest.raises(llama.LlamaError, match="permutation"):
        m.session(kv_block=16, block_ids=[0, 0])
    with pytest.raises(llama.LlamaError, match="zero K/V block"):
        m.session(kv_block=0)
    with pytest.raises(llama.LlamaError, match="token id out of range"):
        m.session().forward([96])


def test_greedy_generation_is_prefill_then_single_token_steps(llama, tiny_path):
    m = llama.Llama(path=tiny_path, products=llama.CALLBACK, matmul=oracle_matmul)
    prompt = [5, 1, 44, 90, 17, 63]
    out, tp, td = m.session().generate_greedy(prompt, 12)
    assert out.shape == (12,) and tp > 0 and td > 0
    s = m.session()
    tok = llama.argmax(s.forward(prompt))
    manual = [tok]
    for _ in range(11):
        tok = llama.argmax(s.forward([tok]))
        manual.append(tok)
    assert out.tolist() == manual
    with pytest.raises(llama.LlamaError, match="empty prompt"):
        m.session().generate_greedy([], 3)


def test_prompt_reuses_the_cached_prefix_and_replaces_the_rest(llama, tiny_path):
    """The reference's session scenario (langtax/tests/native_cuda_parity.rs:208-249): prefill [1, 2, 3], decode
    4, 5, 1, then the divergent full prompt [1, 2, 4]; reuse rule of langtax/src/decode.rs:1106-1196."""
    m = llama.Llama(path=tiny_path, products=llama.CALLBACK, matmul=oracle_matmul)
    bits = lambda a: a.view(np.uint32).tolist()
    for kv_block in (16, 2):  # its dense and its paged session (blocks of 2)
        s = m.session(kv_block=kv_block)
        s.forward([1, 2, 3])
        for t in (4, 5, 1):
            s.forward([t])
        got, hit = s.prompt([1, 2, 4])
        assert hit == 2
        want = m.session(kv_block=kv_block).forward([1, 2, 4])
        assert bits(got) == bits(want)
        # the replaced positions really hold the new sequence: going on from it equals going on from scratch
        fresh = m.session(kv_block=kv_block)
        fresh.forward([1, 2, 4])
        assert bits(s.forward([7])) == bits(fresh.forward([7]))
        # a full hit recomputes the last token and reports the whole length
        again, hit = s.prompt([1, 2, 4, 7])
        assert hit == 4 and bits(again) == bits(m.session(kv_block=kv_block).forward([1, 2, 4, 7]))
        # a longer prompt continues after the cached part; no common prefix starts over
        longer, hit = s.prompt([1, 2, 4, 7, 30, 31])
        assert hit == 4 and bits(longer) == bits(m.session(kv_block=kv_block).forward([1, 2, 4, 7, 30, 31]))
        other, hit = s.prompt([9, 2, 4])
        assert hit == 0 and bits(other) == bits(m.session(kv_block=kv_block).forward([9, 2, 4]))
    # greedy generation leaves the prompt and all picked tokens but the last in the cache
    s = m.session()
    out, _, _ = s.generate_greedy([5, 1, 44], 4)
    seq = [5, 1, 44] + out[:3].tolist()
    _, hit = s.prompt(seq + [int(out[3])])
    assert hit == len(seq)
    with pytest.raises(llama.LlamaError, match="prefill tokens"):
        s.prompt([])


def test_synthetic_weights_have_the_requested_spread_for_every_dtype(llama, pkg, tmp_path):
    """Mean 0 and the requested standard deviation (within sampling noise) for all eight dtypes, and
    the generator is deterministic in its seed."""
    for ty in pkg.ALL_TYPES:
        path = tmp_path / f"m{ty}.gguf"
        llama.write_synthetic_llama(path, n_layer=1, n_embd=256, n_head=2, n_head_kv=1, n_ff=256, n_vocab=64,
                                    block_type=ty, embd_type=ty, output_type=ty, weight_std=0.02, seed=3)
        blob = np.fromfile(path, dtype=np.uint8)
        by = {t[0]: t for t in llama.gguf_tensors(blob)}
        vals = []
        for name in ("blk.0.ffn_gate.weight", "blk.0.ffn_down.weight", "token_embd.weight"):
            _, t, (n_cols, n_rows), start, end = by[name]
            assert t == ty
            vals.append(oracle.dequant(ty, n_cols, blob[start:end], n_rows).ravel())
        v = np.concatenate(vals).astype(np.float64)
        assert abs(v.mean()) < 0.002, pkg.TYPE_NAMES[ty]
        assert 0.016 < v.std() < 0.025, (pkg.TYPE_NAMES[ty], v.std())
        again = tmp_path / "again.gguf"
        llama.write_synthetic_llama(again, n_layer=1, n_embd=256, n_head=2, n_head_kv=1, n_ff=256, n_vocab=64,
                                    block_type=ty, embd_type=ty, output_type=ty, weight_std=0.02, seed=3)
        assert np.array_equal(np.fromfile(again, dtype=np.uint8), blob)
    other = tmp_path / "other.gguf"
    llama.write_synthetic_llama(other, n_layer=1, n_embd=256, n_head=2, n_head_kv=1, n_ff=256, n_vocab=64, seed=4)
    assert os.path.getsize(other) > 0 and not np.array_equal(np.fromfile(other, dtype=np.uint8)[-4096:], blob[-4096:])
    with pytest.raises(llama.LlamaError, match="head counts"):
        llama.write_synthetic_llama(other, n_layer=1, n_embd=256, n_head=3, n_head_kv=2, n_ff=256, n_vocab=64)
    with pytest.raises(llama.LlamaError, match="whole blocks"):
        llama.write_synthetic_llama(other, n_layer=1, n_embd=96, n_head=2, n_head_kv=1, n_ff=256, n_vocab=64)
