"""Host side of a dense Llama decode over the matrix executor, seen from Python.

A ctypes view of include/native_hip_llama.h: GGUF model load, the forward pass
of langtax/src/decode.rs:2710-3099 (dense llama branch) with a paged K/V cache,
greedy generation, and the generator of random GGUF models the tests and the
benchmark use.  The weight products run on the GPU (`RESIDENT`, `DISPATCH`) or
in a function of the caller (`CALLBACK`, which is how the tests put their CPU
checker underneath the same host code).
"""
import ctypes as C
import importlib

import numpy as np

_pkg = importlib.import_module(__name__.rsplit(".", 1)[0])

RESIDENT, DISPATCH, CALLBACK = 0, 1, 2

MATMUL_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint32, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p,
                        C.c_size_t, C.c_void_p, C.c_void_p)


class HParams(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("n_layer", "n_embd", "n_head", "n_head_kv", "n_ff", "n_vocab",
                                            "head_dim", "n_rot")] + \
               [("rope_base", C.c_float), ("rms_eps", C.c_float)] + \
               [(n, C.c_uint32) for n in ("block_type", "embd_type", "output_type", "n_expert", "n_expert_used")]


class SynthSpec(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("n_layer", "n_embd", "n_head", "n_head_kv", "n_ff", "n_vocab",
                                            "block_type", "embd_type", "output_type")] + \
               [("rope_base", C.c_float), ("rms_eps", C.c_float), ("weight_std", C.c_float), ("seed", C.c_uint64),
                ("n_expert", C.c_uint32), ("n_expert_used", C.c_uint32)]


class LlamaError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise LlamaError(_pkg.load_library().lnm_last_error().decode())


def write_synthetic_llama(path, *, n_layer, n_embd, n_head, n_head_kv, n_ff, n_vocab, block_type=_pkg.Q4_K,
                          embd_type=_pkg.Q4_K, output_type=_pkg.Q6_K, rope_base=5e5, rms_eps=1e-5,
                          weight_std=0.02, seed=0, n_expert=0, n_expert_used=0):
    """n_expert > 0: every layer's feed-forward is routed over that many experts, n_expert_used per token."""
    spec = SynthSpec(n_layer, n_embd, n_head, n_head_kv, n_ff, n_vocab, block_type, embd_type, output_type,
                     rope_base, rms_eps, weight_std, seed, n_expert, n_expert_used)
    _check(_pkg.load_library().lnm_write_synthetic_llama(str(path).encode(), C.byref(spec)))


def gguf_tensors(blob):
    """[(name, ggml_type, shape, start, end)] of a GGUF blob (bytes or uint8 array)."""
    lib = _pkg.load_library()
    a = np.frombuffer(blob, dtype=np.uint8) if not isinstance(blob, np.ndarray) else blob
    n_t, n_kv, al = C.c_size_t(), C.c_size_t(), C.c_size_t()
    _check(lib.lnm_gguf_inspect(a.ctypes.data, a.size, C.byref(n_t), C.byref(n_kv), C.byref(al)))
    out = []
    for i in range(n_t.value):
        name = C.create_string_buffer(256)
        ty, nd, st, en = C.c_uint32(), C.c_uint32(), C.c_size_t(), C.c_size_t()
        shape = (C.c_uint64 * 4)()
        _check(lib.lnm_gguf_tensor(a.ctypes.data, a.size, i, name, 256, C.byref(ty), shape, C.byref(nd),
                                   C.byref(st), C.byref(en)))
        out.append((name.value.decode(), ty.value, tuple(shape[:nd.value]), st.value, en.value))
    return out


def gguf_inspect(blob):
    lib = _pkg.load_library()
    a = np.frombuffer(blob, dtype=np.uint8) if not isinstance(blob, np.ndarray) else blob
    n_t, n_kv, al = C.c_size_t(), C.c_size_t(), C.c_size_t()
    _check(lib.lnm_gguf_inspect(a.ctypes.data, a.size, C.byref(n_t), C.byref(n_kv), C.byref(al)))
    return n_t.value, n_kv.value, al.value


def dequant_row(ggml_type, n_cols, row):
    row = np.ascontiguousarray(row, dtype=np.uint8)
    y = np.empty(n_cols, dtype=np.float32)
    _check(_pkg.load_library().lnm_dequant_row(ggml_type, n_cols, row.ctypes.data, row.size, y.ctypes.data))
    return y


def rmsnorm(x, w, eps):
    x = np.array(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    _check(_pkg.load_library().lnm_rmsnorm(x.ctypes.data, w.ctypes.data, x.size, eps))
    return x


def rope(head, pos, n_rot, base):
    v = np.array(head, dtype=np.float32)
    _check(_pkg.load_library().lnm_rope(v.ctypes.data, v.size, pos, n_rot, base))
    return v


def softmax(x):
    v = np.array(x, dtype=np.float32)
    _pkg.load_library().lnm_softmax(v.ctypes.data, v.size)
    return v


def argmax(x):
    v = np.ascontiguousarray(x, dtype=np.float32)
    return _pkg.load_library().lnm_argmax(v.ctypes.data, v.size)


def topk(values, k):
    """Indices of the k largest values, descending, ties to the lower index."""
    v = np.ascontiguousarray(values, dtype=np.float32)
    order = np.empty(k, dtype=np.uint32)
    _check(_pkg.load_library().lnm_topk(v.ctypes.data, v.size, k, order.ctypes.data))
    return order


def router_weights(probs, order, norm_w=True):
    p = np.ascontiguousarray(probs, dtype=np.float32)
    o = np.ascontiguousarray(order, dtype=np.uint32)
    w = np.empty(o.size, dtype=np.float32)
    _check(_pkg.load_library().lnm_router_weights(p.ctypes.data, o.ctypes.data, o.size, int(norm_w), w.ctypes.data))
    return w


class Llama:
    """A loaded model; `products` picks the route of the weight products."""

    def __init__(self, path=None, blob=None, products=RESIDENT, matmul=None):
        lib = _pkg.load_library()
        h = C.c_void_p()
        if path is not None:
            _check(lib.lnm_load(str(path).encode(), C.byref(h)))
        else:
            a = np.frombuffer(blob, dtype=np.uint8) if not isinstance(blob, np.ndarray) else blob
            _check(lib.lnm_load_bytes(a.ctypes.data, a.size, C.byref(h)))
        self._h = h
        self._cb = None
        hp = HParams()
        _check(lib.lnm_info(h, C.byref(hp)))
        self.hparams = hp
        self.set_products(products, matmul)

    def set_products(self, route, matmul=None):
        """matmul(ggml_type, n_rows, n_cols, n_tokens, w: uint8[w_len], x: f32[n_tokens, n_cols]) -> y."""
        lib = _pkg.load_library()
        cb = None
        if route == CALLBACK:
            def thunk(_user, ty, n_rows, n_cols, n_tokens, w, w_len, x, y):
                try:
                    wa = np.ctypeslib.as_array(C.cast(w, C.POINTER(C.c_uint8)), shape=(w_len,))
                    xa = np.ctypeslib.as_array(C.cast(x, C.POINTER(C.c_float)), shape=(n_tokens, n_cols))
                    ya = np.ctypeslib.as_array(C.cast(y, C.POINTER(C.c_float)), shape=(n_tokens, n_rows))
                    ya[...] = matmul(ty, n_rows, n_cols, n_tokens, wa, xa)
                    return 0
                except Exception:  # the C side reports the failure
                    import traceback
                    traceback.print_exc()
                    return 1
            cb = MATMUL_FN(thunk)
        _check(lib.lnm_set_products(self._h, route, C.cast(cb, C.c_void_p) if cb else None, None))
        self._cb = cb  # keep the thunk alive

    def moe_ffn(self, layer, x):
        """The routed feed-forward of `layer` on the rows x [n_tokens, n_embd] (already normed)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty_like(x)
        _check(_pkg.load_library().lnm_moe_ffn(self._h, layer, x.shape[0], x.ctypes.data, out.ctypes.data))
        return out

    def session(self, kv_block=16, block_ids=None, device_positions=None):
        """device_positions: keep the whole decode step on the GPU, with a cache of that many positions."""
        return Session(self, kv_block, block_ids, device_positions)

    def batch_session(self, n_sequences, device_positions, kv_block=16):
        """A device session that decodes `n_sequences` sequences together, one token of each per step."""
        return BatchSession(self, n_sequences, device_positions, kv_block)

    def close(self):
        if self._h:
            _pkg.load_library().lnm_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class BatchSession:
    def __init__(self, model, n_sequences, device_positions, kv_block=16):
        self.model, self.n_sequences = model, n_sequences
        h = C.c_void_p()
        _check(_pkg.load_library().lnm_session_new_device_batch(model._h, kv_block, n_sequences, device_positions, C.byref(h)))
        self._h = h

    def generate_greedy(self, prompts, n_new):
        """(tokens [n_sequences, n_new], prefill seconds, decode seconds) for one prompt per sequence."""
        assert len(prompts) == self.n_sequences
        flat = np.ascontiguousarray(np.concatenate([np.asarray(p, dtype=np.uint32) for p in prompts]), dtype=np.uint32)
        lens = np.ascontiguousarray([len(p) for p in prompts], dtype=np.uintp)
        out = np.empty((self.n_sequences, n_new), dtype=np.uint32)
        tp, td = C.c_double(), C.c_double()
        _check(_pkg.load_library().lnm_batch_generate_greedy(self._h, flat.ctypes.data, lens.ctypes.data, n_new,
                                                             out.ctypes.data, C.byref(tp), C.byref(td)))
        return out, tp.value, td.value

    def close(self):
        if self._h:
            _pkg.load_library().lnm_session_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Session:
    def __init__(self, model, kv_block=16, block_ids=None, device_positions=None):
        lib = _pkg.load_library()
        self.model = model
        h = C.c_void_p()
        ids = None if block_ids is None else np.ascontiguousarray(block_ids, dtype=np.uint32)
        ids_p, ids_n = (None, 0) if ids is None else (ids.ctypes.data, ids.size)
        if device_positions is None:
            _check(lib.lnm_session_new(model._h, kv_block, ids_p, ids_n, C.byref(h)))
        else:
            _check(lib.lnm_session_new_device(model._h, kv_block, ids_p, ids_n, device_positions, C.byref(h)))
        self._h = h

    def forward(self, tokens):
        """Logits of the last of `tokens`, run as one batch after everything seen so far."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.model.hparams.n_vocab, dtype=np.float32)
        _check(_pkg.load_library().lnm_forward(self._h, t.ctypes.data, t.size, logits.ctypes.data))
        return logits

    def prompt(self, tokens):
        """(logits of the last of `tokens`, reused prefix length): `tokens` as the whole sequence, keeping the
        cached positions of the longest prefix it shares with what the session has forwarded so far
        (langtax/src/decode.rs:3956-3962)."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.model.hparams.n_vocab, dtype=np.float32)
        hit = C.c_size_t()
        _check(_pkg.load_library().lnm_prompt(self._h, t.ctypes.data, t.size, logits.ctypes.data, C.byref(hit)))
        return logits, hit.value

    def generate_greedy(self, prompt, n_new):
        """(tokens, prefill seconds, decode seconds): n_new tokens, the first from the prompt's logits."""
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.empty(n_new, dtype=np.uint32)
        tp, td = C.c_double(), C.c_double()
        _check(_pkg.load_library().lnm_generate_greedy(self._h, p.ctypes.data, p.size, n_new, out.ctypes.data,
                                                       C.byref(tp), C.byref(td)))
        return out, tp.value, td.value

    def timing(self):
        """(seconds in weight products, seconds in RoPE + attention, number of products) so far."""
        a, b, n = C.c_double(), C.c_double(), C.c_uint64()
        _check(_pkg.load_library().lnm_session_timing(self._h, C.byref(a), C.byref(b), C.byref(n)))
        return a.value, b.value, n.value

    def close(self):
        if self._h:
            _pkg.load_library().lnm_session_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
