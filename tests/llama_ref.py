"""Independent float64 restatements, written with numpy, of the host code the tests check: the llama
forward pass of langtax/src/decode.rs:2710-3099 and its routed feed-forward (decode.rs:9938-10292).
They share no code with the C++ host side: every token is handled on its own, nothing is grouped."""
import numpy as np

import oracle


def numpy_route(logits, k):
    """Per token: softmax over all experts, the k largest (ties to the lower index), weights renormalised
    with the sum clamped at 2^-14.  Returns (experts [n, k], weights [n, k])."""
    z = logits - logits.max(axis=1, keepdims=True)
    p = np.exp(z)
    p /= p.sum(axis=1, keepdims=True)
    experts = np.empty((len(p), k), dtype=np.int64)
    weights = np.empty((len(p), k))
    for t, row in enumerate(p):
        order = sorted(range(len(row)), key=lambda e: (-row[e], e))[:k]
        experts[t] = order
        weights[t] = row[order] / max(row[order].sum(), 2.0 ** -14)
    return experts, weights


def numpy_moe_ffn(h, router, gate, up, down, k):
    """Brute force: every token, every selected expert, one after the other.
    h [n, d]; router [n_expert, d]; gate, up [n_expert, ff, d]; down [n_expert, d, ff]."""
    experts, weights = numpy_route(h @ router.T, k)
    out = np.zeros_like(h)
    for t in range(len(h)):
        for e, w in zip(experts[t], weights[t]):
            g = gate[e] @ h[t]
            u = up[e] @ h[t]
            out[t] += w * (down[e] @ (g / (1 + np.exp(-g)) * u))
    return out


def numpy_forward(blob, tensors, hp, tokens, n_past_kv=None):
    """Independent float64 restatement of the llama forward over dequantized weights: logits of every
    position (causal attention, adjacent-pair RoPE, GQA, SwiGLU; routed experts when the model has them)."""
    by = {t[0]: t for t in tensors}

    def mat(name):
        _, ty, shape, start, end = by[name]
        n_cols, n_rows = shape
        return oracle.dequant(ty, n_cols, blob[start:end], n_rows).astype(np.float64)

    def parts(name):  # a 3-D tensor [n_cols, n_rows, n_parts] as [n_parts, n_rows, n_cols]
        _, ty, shape, start, end = by[name]
        n_cols, n_rows, n_parts = shape
        return oracle.dequant(ty, n_cols, blob[start:end], n_rows * n_parts).astype(np.float64).reshape(n_parts, n_rows, n_cols)

    def vec(name):
        _, _, _, start, end = by[name]
        return blob[start:end].view(np.float32).astype(np.float64)

    d, hd, n_head, n_kv = hp.n_embd, hp.head_dim, hp.n_head, hp.n_head_kv
    eps, base, n_rot = float(hp.rms_eps), float(hp.rope_base), hp.n_rot
    n = len(tokens)

    def norm(x, w):
        return x / np.sqrt((x ** 2).mean(axis=-1, keepdims=True) + eps) * w

    def rot(v):  # v: [n, heads, hd]
        i = np.arange(n_rot // 2)
        th = np.arange(n)[:, None] * base ** (-2.0 * i / n_rot)[None, :]
        z = (v[..., 0:n_rot:2] + 1j * v[..., 1:n_rot:2]) * np.exp(1j * th)[:, None, :]
        out = v.copy()
        out[..., 0:n_rot:2], out[..., 1:n_rot:2] = z.real, z.imag
        return out

    x = mat("token_embd.weight")[np.asarray(tokens)]
    for li in range(hp.n_layer):
        p = f"blk.{li}."
        h = norm(x, vec(p + "attn_norm.weight"))
        q = rot((h @ mat(p + "attn_q.weight").T).reshape(n, n_head, hd))
        k = rot((h @ mat(p + "attn_k.weight").T).reshape(n, n_kv, hd))
        v = (h @ mat(p + "attn_v.weight").T).reshape(n, n_kv, hd)
        att = np.zeros((n, n_head, hd))
        for hq in range(n_head):
            kk, vv = k[:, hq // (n_head // n_kv)], v[:, hq // (n_head // n_kv)]
            sc = q[:, hq] @ kk.T / np.sqrt(hd)
            sc[np.triu_indices(n, 1)] = -np.inf
            pr = np.exp(sc - sc.max(axis=1, keepdims=True))
            pr /= pr.sum(axis=1, keepdims=True)
            att[:, hq] = pr @ vv
        x = x + att.reshape(n, -1) @ mat(p + "attn_output.weight").T
        h = norm(x, vec(p + "ffn_norm.weight"))
        if hp.n_expert:
            x = x + numpy_moe_ffn(h, mat(p + "ffn_gate_inp.weight"), parts(p + "ffn_gate_exps.weight"),
                                  parts(p + "ffn_up_exps.weight"), parts(p + "ffn_down_exps.weight"), hp.n_expert_used)
            continue
        g = h @ mat(p + "ffn_gate.weight").T
        u = h @ mat(p + "ffn_up.weight").T
        x = x + (g / (1 + np.exp(-g)) * u) @ mat(p + "ffn_down.weight").T
    return norm(x, vec("output_norm.weight")) @ mat("output.weight").T
