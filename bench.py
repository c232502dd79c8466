#!/usr/bin/env python3
"""Benchmark of the decode GEMV hot path on one MI355X.

Workload (benchmark configuration "Llama-3-8B decode layer shapes as batch-1 GEMV"): one
step is one generated token's weight products, batch 1 - for each of 32 layers
the seven Q4_K GEMVs q, k, v, o (4096->4096/1024), gate, up (4096->14336), down
(14336->4096), then the Q6_K output head 4096->128256 - 225 products streaming
4.36 GB of distinct packed weights, so no product is served from the 256 MB
Infinity Cache.  Activations and outputs stay resident in HBM; weights are
synthetic (uniform codes, |N(0, 0.02)| f16 block scales), x ~ N(0, 1).

`value` is algorithmic bytes per step / wall time per step.  `roofline` is for the
dominant kernel (the Q4_K GEMV: 224 products in 128 launches per step, products that
share an input vector - q/k/v, gate/up - being one launch): algorithmic bytes per
launch / mean launch duration from HIP events recorded on the launch stream
around the Q4_K part of every timed step.  `cpu_baseline` times the AVX2 port of
the reference's `simd` CPU kernels on a bounded sample of the same workload.

`other_workloads` times, after the headline run and outside its timed region, the
other shapes the reference's benchmarks name: the Q8_0 4096x4096 GEMV, the
Q4_0 4096x14336 product at 8..512 tokens, and one Mixtral-shaped MoE projection
(8 Q4_K experts, 16 tokens each) as a single grouped call.  Each figure is a
mean over launches that rotate through enough distinct matrices to defeat the
256 MB Infinity Cache, from HIP events on the launch stream.

One JSON line on stdout; progress on stderr.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "Q4_K/Q8_0 GEMV HBM GB/s (% of peak); 8B-shape decode tok/s, batch 1"
HBM_PEAK_GBS = 8000.0
BF16_MFMA_PEAK_TFLOPS = 2500.0
# HBM bytes per Q4_K launch over algorithmic bytes come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script (counters scaled by a 1 GiB copy kernel), summarised in the file below; a run of this script cannot
# read the counters itself.  The summary names the kernel source it was taken with (a SHA-256 of the .inc file);
# when that no longer matches the source in the tree, the figure is stale and `traffic` is reported as null.
TRAFFIC_PROFILE = os.path.join("profiles", "decode_gemv_q4k_q6k_8b_step.txt")
KERNEL_SOURCE = os.path.join("llama-rust_amd", "csrc", "gemv_kernels.inc")


def profiled_traffic():
    """{'ratio': measured HBM bytes / algorithmic bytes of the Q4_K launches or None, 'source': where from}."""
    import hashlib
    import re
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
        ratio = float(re.search(r"^traffic_over_algorithmic_q4k:\s*([0-9.]+)", text, re.M).group(1))
        profiled = re.search(r"^kernel_source_sha256:\s*([0-9a-f]{64})", text, re.M).group(1)
        now = hashlib.sha256(open(os.path.join(ROOT, KERNEL_SOURCE), "rb").read()).hexdigest()
    except (OSError, AttributeError, ValueError) as e:
        return {"ratio": None, "source": f"{TRAFFIC_PROFILE} unreadable ({type(e).__name__})"}
    if profiled != now:
        return {"ratio": None, "source": f"{TRAFFIC_PROFILE} was taken with another {KERNEL_SOURCE} "
                                         f"(sha256 {profiled[:12]}, now {now[:12]}): stale, re-profile"}
    return {"ratio": ratio, "source": f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, {TRAFFIC_PROFILE} (kernel source sha256 {now[:12]})"}


Q4_0, Q5_0, Q5_1, Q8_0, Q4_K, Q6_K = 2, 6, 7, 8, 12, 14
F32, F16 = 0, 1
BLOCK = {Q4_0: (32, 18, 0), Q5_0: (32, 22, 0), Q5_1: (32, 24, 0), Q8_0: (32, 34, 0), Q4_K: (256, 144, 0),
         Q6_K: (256, 210, 208), F16: (1, 2, 0), F32: (1, 4, 0)}  # columns, bytes, offset of d
FP32_PEAK_TFLOPS = 157.3
N_LAYERS, D, D_KV, FF, VOCAB = 32, 4096, 1024, 14336, 128256
# (name, rows, cols, which activation buffer it reads).  Products that read the same buffer are
# independent of each other (q/k/v of the normed hidden state, gate/up of the normed residual);
# o and down read what the host computes from the earlier products, so they are launches of
# their own.  lnh_gemm_batch_device issues each run of same-input products as one launch.
LAYER = [("q", D, D, "h1"), ("k", D_KV, D, "h1"), ("v", D_KV, D, "h1"), ("o", D, D, "attn"),
         ("gate", FF, D, "h2"), ("up", FF, D, "h2"), ("down", D, FF, "act")]
LAUNCHES_PER_LAYER = 4


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def row_bytes(ty, cols):
    qk, bb, _ = BLOCK[ty]
    return cols // qk * bb


def algorithmic_bytes(ty, rows, cols, tokens=1):
    """Each weight byte once, x once, y once."""
    return rows * row_bytes(ty, cols) + 4 * tokens * cols + 4 * tokens * rows


def synth_matrix(ty, rows, cols, rng):
    """Packed GGUF bytes: uniform random codes / 6-bit scales, |N(0, 0.02)| f16 super-block scales."""
    if ty in (F16, F32):
        w = rng.normal(0, 0.02, (rows, cols)).astype(np.float16 if ty == F16 else np.float32)
        return w.view(np.uint8).reshape(-1)
    qk, bb, d_off = BLOCK[ty]
    nb = cols // qk
    blk = rng.integers(0, 256, size=(rows, nb, bb), dtype=np.uint8)
    n_scales = 2 if ty in (Q4_K, Q5_1) else 1  # Q4_K: d and dmin; Q5_1: d and m
    blk[:, :, d_off:d_off + 2 * n_scales] = (np.abs(rng.normal(0, 0.02, (rows, nb, n_scales))).astype(np.float16)
                                             .view(np.uint8).reshape(rows, nb, 2 * n_scales))
    return blk.reshape(-1)


# Layers of the step whose matrices the CPU baseline sweeps: 8 x 123 MB + a sixteenth of the head = 1.0 GB per
# sweep, beyond any last-level cache, so the figure is a memory-streaming one like the GPU's.
CPU_SAMPLE_LAYERS = 8


def host_cpu():
    """Model name, physical cores and logical CPUs of this host, and whether a Rust toolchain is present (with
    one the reference's own `--no-default-features --features simd` build could be timed instead of the port)."""
    import shutil
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name":
                model = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None and core is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    return {"cpu_model": model, "physical_cores": len(cores) or None, "logical_cpus": os.cpu_count(),
            "cargo_present": shutil.which("cargo") is not None}


def cpu_baseline(sample, x_by_cols, seconds):
    """The reference's `simd` CPU path (AVX2 port, <=10 threads, fork/join per product)
    on `sample` = [(type, rows, cols, packed bytes)], repeated for about `seconds`."""
    import oracle as O
    threads = O.load().lro_worker_count(1 << 20)
    nbytes = sum(algorithmic_bytes(ty, r, c) for ty, r, c, _, _ in sample)

    def sweep():
        for ty, r, c, w, src in sample:
            O.gemm(ty, c, 1, w, x_by_cols[src], r, simd=True, threads=0)

    sweep()  # warm-up
    t0 = time.perf_counter()
    n = 0
    while True:
        sweep()
        n += 1
        dt = time.perf_counter() - t0
        if dt >= seconds or n >= 2000:
            break
    out = {"value": nbytes * n / dt / 1e9, "unit": "GB/s", "cores": int(threads), "kind": "port",
           "sample": f"the first {CPU_SAMPLE_LAYERS} layers (7 Q4_K GEMVs each) + first {sample[-1][1]} rows of the Q6_K head, "
                     f"{nbytes / 1e6:.1f} MB per sweep, {n} sweeps in {dt:.1f} s, AVX2 port of the reference simd kernels",
           "cache_resident": False,
           "tok_per_s_equiv": n / dt * nbytes / TOKEN_BYTES}
    out.update(host_cpu())
    return out


def timed_us(hip, stream, enqueue, n_variants, reps):
    """Mean microseconds of enqueue(i), i rotating over n_variants, from HIP events on `stream`."""
    for i in range(n_variants):
        enqueue(i)
    stream.synchronize()
    a, b = hip.Event(), hip.Event()
    a.record(stream)
    for r in range(reps):
        for i in range(n_variants):
            enqueue(i)
    b.record(stream)
    stream.synchronize()
    return a.elapsed_ms(b) * 1e3 / (reps * n_variants)


def other_workloads(pkg, hip, gpu, stream, rng, cpu):
    """Shapes of the reference's other benchmark configurations (see the module docstring).
    With `cpu`, each entry also carries the AVX2 port of the reference's CPU kernels on a sample of
    the same product's rows (its threading rule, all tokens), scaled to the whole product."""
    import oracle as O
    out = {}

    def cpu_us(ty, rows, cols, tokens, w, x, sample_rows):
        """Microseconds the CPU path would take for the whole product, from `sample_rows` rows."""
        if not cpu:
            return None
        ws = w[:sample_rows * row_bytes(ty, cols)]
        O.gemm(ty, cols, tokens, ws, x, sample_rows, simd=True, threads=0)  # warm-up
        t0 = time.perf_counter()
        n = 0
        while n < 3 or time.perf_counter() - t0 < 0.3:
            O.gemm(ty, cols, tokens, ws, x, sample_rows, simd=True, threads=0)
            n += 1
        return round((time.perf_counter() - t0) / n * 1e6 * rows / sample_rows, 1)

    def check(name, ty, rows, cols, tokens, w, x, y_dev):
        got = y_dev.to_numpy(np.float32)[:tokens * rows].reshape(tokens, rows)[:, :32]
        want = O.gemm_f64(ty, cols, tokens, w[:32 * row_bytes(ty, cols)], x, 32)
        want = np.asarray(want).reshape(tokens, 32)
        if not np.allclose(got, want, rtol=1e-4, atol=1e-4 * float(np.sqrt(np.mean(want ** 2)))):
            raise RuntimeError(f"{name}: GPU output disagrees with the CPU oracle")

    # Q8_0 4096x4096, one token (the reference's demo shape)
    n = 16
    ws = [synth_matrix(Q8_0, D, D, rng) for _ in range(n)]
    ms = [gpu.upload_packed(Q8_0, D, D, w) for w in ws]
    x = rng.normal(0, 1, D).astype(np.float32)
    xd, yd = hip.DeviceBuffer.from_numpy(x), hip.DeviceBuffer(D * 4)
    us = timed_us(hip, stream, lambda i: gpu.gemm_device(ms[i], 1, xd.ptr, yd.ptr, stream.ptr), n, 20)
    gpu.gemm_device(ms[0], 1, xd.ptr, yd.ptr, stream.ptr); stream.synchronize()
    check("Q8_0 GEMV", Q8_0, D, D, 1, ws[0], x, yd)
    nbytes = algorithmic_bytes(Q8_0, D, D)
    out["gemv_q8_0_4096x4096"] = {"launch_us": round(us, 2), "achieved": round(nbytes / us / 1e3, 1), "unit": "GB/s",
                                  "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "bound": "hbm",
                                  "cpu_us": cpu_us(Q8_0, D, D, 1, ws[0], x, D)}
    for m in ms:
        m.close()

    # Q4_0 / Q5_0 / Q5_1, 4096x14336 (ffn_down) and 14336x4096 (gate/up), 1..512 tokens (continuous batching:
    # decode tokens and prefill chunks in one product); eight matrices per shape so that no call is served
    # from the 256 MB Infinity Cache
    names = {Q4_0: "q4_0", Q5_0: "q5_0", Q5_1: "q5_1"}
    for ty in (Q4_0, Q5_0, Q5_1):
        for rows, cols in ((D, FF), (FF, D)):
            n = 8
            ws = [synth_matrix(ty, rows, cols, rng) for _ in range(n)]
            ms = [gpu.upload_packed(ty, rows, cols, w) for w in ws]
            x = rng.normal(0, 1, 512 * cols).astype(np.float32)
            xd, yd = hip.DeviceBuffer.from_numpy(x), hip.DeviceBuffer(512 * rows * 4)
            for tokens in (1, 8, 32, 128, 512):
                us = timed_us(hip, stream, lambda i: gpu.gemm_device(ms[i], tokens, xd.ptr, yd.ptr, stream.ptr), n, 5)
                gpu.gemm_device(ms[0], tokens, xd.ptr, yd.ptr, stream.ptr); stream.synchronize()
                check(f"{names[ty]} GEMM {rows}x{cols} M={tokens}", ty, rows, cols, tokens, ws[0], x[:tokens * cols], yd)
                flops = 2.0 * rows * cols * tokens
                with_cpu = ty == Q4_0 and rows == D and tokens > 1
                # three bf16 MFMA products per multiply-add (the f32 activations are split in three)
                out[f"gemm_{names[ty]}_{rows}x{cols}_m{tokens}"] = {
                    "call_us": round(us, 2), "tflops": round(flops / us / 1e6, 1),
                    "mfma_frac": round(3 * flops / us / 1e6 / BF16_MFMA_PEAK_TFLOPS, 4) if tokens > 1 else None,
                    "weight_gbs": round(rows * row_bytes(ty, cols) / us / 1e3, 1),
                    "hbm_frac": round(algorithmic_bytes(ty, rows, cols, tokens) / us / 1e3 / HBM_PEAK_GBS, 4),
                    "bound": "mfma" if tokens >= 128 else "hbm",
                    "cpu_us": cpu_us(ty, rows, cols, tokens, ws[0], x[:tokens * cols], 256 if tokens >= 128 else rows)
                    if with_cpu else None}
            for m in ms:
                m.close()
            xd.free(); yd.free()

    # F16 and F32 weights, 4096x14336 (the two dtypes whose products never reach the matrix cores: one token on the
    # streaming GEMV kernel, more on a vector-ALU tile kernel)
    for ty, nm in ((F16, "f16"), (F32, "f32")):
        rows, cols, n = D, FF, 4
        ws = [synth_matrix(ty, rows, cols, rng) for _ in range(n)]
        ms = [gpu.upload_packed(ty, rows, cols, w) for w in ws]
        x = rng.normal(0, 1, 512 * cols).astype(np.float32)
        xd, yd = hip.DeviceBuffer.from_numpy(x), hip.DeviceBuffer(512 * rows * 4)
        for tokens in (1, 8, 128, 512):
            us = timed_us(hip, stream, lambda i: gpu.gemm_device(ms[i], tokens, xd.ptr, yd.ptr, stream.ptr), n, 3)
            gpu.gemm_device(ms[0], tokens, xd.ptr, yd.ptr, stream.ptr); stream.synchronize()
            check(f"{nm} GEMM {rows}x{cols} M={tokens}", ty, rows, cols, tokens, ws[0], x[:tokens * cols], yd)
            flops = 2.0 * rows * cols * tokens
            out[f"gemm_{nm}_{rows}x{cols}_m{tokens}"] = {
                "call_us": round(us, 2), "tflops": round(flops / us / 1e6, 1),
                "fp32_frac": round(flops / us / 1e6 / FP32_PEAK_TFLOPS, 4) if tokens > 1 else None,
                "weight_gbs": round(rows * row_bytes(ty, cols) / us / 1e3, 1),
                "hbm_frac": round(algorithmic_bytes(ty, rows, cols, tokens) / us / 1e3 / HBM_PEAK_GBS, 4),
                "bound": "fp32" if tokens >= 128 else "hbm", "cpu_us": None}
        for m in ms:
            m.close()
        xd.free(); yd.free()

    # one MoE projection: 8 Q4_K experts 4096 -> 14336, 16 tokens each, one grouped call
    n_exp, per = 8, 16
    sets = 2  # two sets of experts = 528 MB, so that no call is served from the Infinity Cache
    ws = [[synth_matrix(Q4_K, FF, D, rng) for _ in range(n_exp)] for _ in range(sets)]
    ms = [[gpu.upload_packed(Q4_K, FF, D, w) for w in ws_] for ws_ in ws]
    x = rng.normal(0, 1, n_exp * per * D).astype(np.float32)
    xd, yd = hip.DeviceBuffer.from_numpy(x), hip.DeviceBuffer(n_exp * per * FF * 4)
    us = timed_us(hip, stream, lambda i: gpu.gemm_grouped_device(ms[i], [per] * n_exp, xd.ptr, yd.ptr, stream.ptr), sets, 10)
    gpu.gemm_grouped_device(ms[0], [per] * n_exp, xd.ptr, yd.ptr, stream.ptr); stream.synchronize()
    check("MoE grouped GEMM", Q4_K, FF, D, per, ws[0][0], x[:per * D], yd)
    wbytes = n_exp * FF * row_bytes(Q4_K, D)
    out["moe_q4_k_8x14336x4096_m16"] = {"call_us": round(us, 2), "weight_gbs": round(wbytes / us / 1e3, 1),
                                         "frac": round(wbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                                         "tflops": round(2.0 * n_exp * per * FF * D / us / 1e6, 1), "bound": "hbm",
                                         "cpu_us": None if not cpu else round(n_exp * cpu_us(Q4_K, FF, D, per, ws[0][0], x[:per * D], 2048), 1)}
    for ms_ in ms:
        for m in ms_:
            m.close()

    # A whole MoE feed-forward, Mixtral-shaped: 8 experts, top-2 of 64 tokens by softmax of N(0,1) router
    # logits (ties to the lower index), tokens of an expert grouped; gate, up and down as one grouped call each
    n_tok = 64
    logits = rng.normal(0, 1, (n_tok, n_exp)).astype(np.float32)
    order = np.argsort(-logits, axis=1, kind="stable")[:, :2]
    counts = [int(np.sum(order == e)) for e in range(n_exp)]
    pairs = sum(counts)
    sets = 2  # 2 x 793 MB of expert weights
    wg = [[synth_matrix(Q4_K, FF, D, rng) for _ in range(n_exp)] for _ in range(sets)]
    wd = [[synth_matrix(Q4_K, D, FF, rng) for _ in range(n_exp)] for _ in range(sets)]
    mg = [[gpu.upload_packed(Q4_K, FF, D, w) for w in ws_] for ws_ in wg]
    mu = [[gpu.upload_packed(Q4_K, FF, D, w) for w in ws_] for ws_ in wg]   # same bytes, separate residency
    md = [[gpu.upload_packed(Q4_K, D, FF, w) for w in ws_] for ws_ in wd]
    x = rng.normal(0, 1, pairs * D).astype(np.float32)
    h = rng.normal(0, 1, pairs * FF).astype(np.float32)
    xd, hd_ = hip.DeviceBuffer.from_numpy(x), hip.DeviceBuffer.from_numpy(h)
    gd, ud, yd2 = hip.DeviceBuffer(pairs * FF * 4), hip.DeviceBuffer(pairs * FF * 4), hip.DeviceBuffer(pairs * D * 4)

    def layer(i):
        gpu.gemm_grouped_device(mg[i], counts, xd.ptr, gd.ptr, stream.ptr)
        gpu.gemm_grouped_device(mu[i], counts, xd.ptr, ud.ptr, stream.ptr)
        gpu.gemm_grouped_device(md[i], counts, hd_.ptr, yd2.ptr, stream.ptr)

    us = timed_us(hip, stream, layer, sets, 5)
    layer(0); stream.synchronize()
    e0 = next(e for e in range(n_exp) if counts[e] > 0)
    off = sum(counts[:e0])
    got = yd2.to_numpy(np.float32)[off * D:(off + counts[e0]) * D].reshape(counts[e0], D)[:, :32]
    want = np.asarray(O.gemm_f64(Q4_K, FF, counts[e0], wd[0][e0][:32 * row_bytes(Q4_K, FF)],
                                 h[off * FF:(off + counts[e0]) * FF], 32)).reshape(counts[e0], 32)
    if not np.allclose(got, want, rtol=1e-4, atol=1e-4 * float(np.sqrt(np.mean(want ** 2)))):
        raise RuntimeError("MoE layer: GPU output disagrees with the CPU oracle")
    wbytes = n_exp * (2 * FF * row_bytes(Q4_K, D) + D * row_bytes(Q4_K, FF))
    out["moe_layer_q4_k_8_experts_top2_64_tokens"] = {
        "call_us": round(us, 2), "calls": 3, "tokens_per_expert": counts, "weight_gbs": round(wbytes / us / 1e3, 1),
        "frac": round(wbytes / us / 1e3 / HBM_PEAK_GBS, 4), "tflops": round(2.0 * pairs * 3 * FF * D / us / 1e6, 1),
        "bound": "hbm"}
    # the same products with gate and up of all experts as ONE batch call (lnh_gemm_batch_device), the experts of
    # at most 16 tokens first: eight products of one tile size per launch, no shared columns, no launch that sums
    # shares - how the library's own routed layer issues them
    def batches(i):
        mats, toks, xs, ys = [], [], [], []
        for big in (False, True):
            ox = oh = 0
            for e in range(n_exp):
                if counts[e] and (counts[e] > 16) == big:
                    for mset, out_buf in ((mg[i], gd), (mu[i], ud)):
                        mats.append(mset[e]); toks.append(counts[e]); xs.append(xd.ptr + ox * 4); ys.append(out_buf.ptr + oh * 4)
                ox += counts[e] * D
                oh += counts[e] * FF
        return gpu.make_batch(mats, toks, xs, ys)

    pre = [batches(i) for i in range(sets)]

    def layer_batched(i):
        gpu.gemm_batch_device(pre[i], stream.ptr)
        gpu.gemm_grouped_device(md[i], counts, hd_.ptr, yd2.ptr, stream.ptr)

    # what the three grouped calls of layer(0) left, against what the batched layer leaves in the same buffers
    refs = {"gate": (gd, gd.to_numpy(np.float32).copy()), "up": (ud, ud.to_numpy(np.float32).copy()),
            "down": (yd2, yd2.to_numpy(np.float32).copy())}
    us_b = timed_us(hip, stream, layer_batched, sets, 5)
    for buf, _ in refs.values():
        buf.fill_byte(0xff)   # NaN patterns: a job that wrote to the wrong place leaves them standing
    hip.device_synchronize()  # the fill runs on the null stream, which the (non-blocking) launch stream does not wait for
    layer_batched(0); stream.synchronize()
    for name, (buf, ref) in refs.items():
        if not np.allclose(buf.to_numpy(np.float32), ref, rtol=1e-4, atol=1e-4 * float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))):
            raise RuntimeError(f"MoE layer: the batched layer's {name} products disagree with the grouped call's")
    out["moe_layer_q4_k_8_experts_top2_64_tokens"]["call_us_gate_up_as_one_batch"] = round(us_b, 2)
    for group in (mg, mu, md):
        for ms_ in group:
            for m in ms_:
                m.close()
    xd.free(); hd_.free(); gd.free(); ud.free(); yd2.free()

    # The same layer as the reference runs it, routing included (langtax/src/decode.rs:9938-10292): a Mixtral-shaped
    # layer of a synthetic GGUF, 64 tokens through the host code - the rows to the device once, the router product
    # there, its logits back for softmax, top-2 and grouping on the host, the bucket order up, then gather, the three
    # grouped expert products, SiLU * up and the weighted scatter chained on the device, the result back
    # (LLAMA_HIP_MOE_HOST_SWIGLU=1: every product a call through host buffers, SiLU * up and the scatter on the
    # host, as the reference's seam has it).
    import tempfile
    L = importlib.import_module("llama-rust_amd.llama")
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "mixtral_layer.gguf")
        L.write_synthetic_llama(path, n_layer=1, n_embd=D, n_head=32, n_head_kv=8, n_ff=FF, n_vocab=256, block_type=Q4_K,
                                embd_type=Q8_0, output_type=Q8_0, seed=8, n_expert=n_exp, n_expert_used=2)
        model = L.Llama(path=path)
        xt = rng.normal(0, 1, (n_tok, D)).astype(np.float32)
        got = model.moe_ffn(0, xt)  # uploads the experts
        t0 = time.perf_counter()
        reps = 5
        for _ in range(reps):
            got = model.moe_ffn(0, xt)
        host_us = (time.perf_counter() - t0) / reps * 1e6
        entry = {"call_us": round(host_us, 1), "tokens": n_tok, "experts": n_exp, "top_k": 2,
                 "scope": ("whole routed feed-forward, host softmax / top-k / grouping: "
                           + ("router, gate, up, down as calls through host buffers, SiLU*up and scatter on the host"
                              if os.environ.get("LLAMA_HIP_MOE_HOST_SWIGLU") else
                              "rows up once, router product, gather, gate / up / SiLU*up / down and scatter chained on the device, "
                              "logits and the result back"))}
        if cpu:
            ref = L.Llama(path=path, products=L.CALLBACK,
                          matmul=lambda ty, n_rows, n_cols, n_tokens, w, x: O.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=True, threads=0))
            t0 = time.perf_counter()
            want = ref.moe_ffn(0, xt)
            entry["cpu_us"] = round((time.perf_counter() - t0) * 1e6, 1)
            rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
            if not np.all(np.abs(got.astype(np.float64) - want) <= 1e-4 * np.maximum(np.abs(want), rms / 4)):
                raise RuntimeError("routed MoE layer: GPU route disagrees with the CPU path")
            entry["matches_cpu_path"] = True
            ref.close()
        model.close()
        out["moe_layer_routed_host_seam_q4_k_8_experts_top2_64_tokens"] = entry
    return out


def greedy_decode(pkg, layers, check_cpu, seed):
    """Benchmark configuration 4: a random Llama-3-8B-shaped Q4_K / Q6_K-head GGUF, 128 prompt ids as one
    batch, then 128 greedy single-token steps through the host decode (host attention and norms,
    every weight product on the GPU with host round trips, as the reference's executor is called).
    With check_cpu the same host code runs again over the CPU kernels and the tokens are compared."""
    import tempfile
    L = importlib.import_module("llama-rust_amd.llama")
    out = {"layers": layers, "prompt_tokens": 128, "decode_steps": 128, "kv_block": 16}
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "llama3_8b_shape.gguf")
        t0 = time.perf_counter()
        L.write_synthetic_llama(path, n_layer=layers, n_embd=D, n_head=32, n_head_kv=8, n_ff=FF, n_vocab=VOCAB,
                                rope_base=5e5, rms_eps=1e-5, weight_std=0.02, seed=seed)
        out["model_gb"] = round(os.path.getsize(path) / 1e9, 3)
        log(f"[bench] wrote {out['model_gb']} GB GGUF in {time.perf_counter() - t0:.1f} s")
        prompt = np.random.default_rng(seed).integers(0, VOCAB, 128)
        m = L.Llama(path=path, products=L.RESIDENT)
        t0 = time.perf_counter()
        m.session().forward(prompt[:2])  # uploads every matrix
        out["upload_s"] = round(time.perf_counter() - t0, 2)
        sess = m.session(kv_block=16)
        toks, prefill_s, decode_s = sess.generate_greedy(prompt, 129)
        prod_s, att_s, n_prod = sess.timing()
        out.update(products_s=round(prod_s, 3), attention_s=round(att_s, 3), products=n_prod)
        out.update(prefill_s=round(prefill_s, 3), prefill_tok_per_s=round(128 / prefill_s, 1),
                   decode_s=round(decode_s, 3), decode_tok_per_s=round(128 / decode_s, 2))
        log(f"[bench] greedy decode: prefill {prefill_s:.2f} s, 128 steps in {decode_s:.2f} s")
        # The same model with the whole step resident on the GPU (one HIP graph per token, no host round trips).
        dev = m.session(kv_block=16, device_positions=256)
        dtoks, dp, dd = dev.generate_greedy(prompt, 129)
        dsame = int(np.sum(np.cumprod(toks == dtoks)))
        out["device_session"] = {"prefill_s": round(dp, 3), "prefill_tok_per_s": round(128 / dp, 1),
                                 "decode_s": round(dd, 4), "decode_tok_per_s": round(128 / dd, 1),
                                 "ms_per_token": round(dd / 128 * 1e3, 3),
                                 "tokens_identical_to_host_session": bool(dsame == 129), "identical_prefix": dsame}
        log(f"[bench] device session: prompt (127 tokens as one batch, the last as a step) {dp:.3f} s, 128 steps in {dd:.3f} s ({128 / dd:.0f} tok/s)")
        dev.close()
        # Eight sequences decoded together (one token of each per step, the products as 8-token products): the
        # continuous-batching shape.  Sequence 0 has the prompt above, so its tokens can be compared.
        rngb = np.random.default_rng(seed + 1)
        prompts = [prompt] + [rngb.integers(0, VOCAB, 128) for _ in range(7)]
        bs = m.batch_session(8, 256, kv_block=16)
        btoks, bp, bd = bs.generate_greedy(prompts, 64)
        bsame = int(np.sum(np.cumprod(btoks[0] == dtoks[:64])))
        out["batch_session"] = {"sequences": 8, "prompt_tokens": 8 * 128, "steps": 64, "prefill_s": round(bp, 3),
                                "prefill_tok_per_s": round(8 * 127 / bp, 1), "decode_s": round(bd, 4),
                                "decode_tok_per_s_all_sequences": round(8 * 64 / bd, 1), "ms_per_step": round(bd / 64 * 1e3, 3),
                                "sequence_0_identical_prefix_to_single_session": bsame}
        log(f"[bench] batch session: 8 sequences, 64 steps in {bd:.3f} s ({8 * 64 / bd:.0f} tok/s over all sequences)")
        bs.close()
        prompts32 = prompts + [rngb.integers(0, VOCAB, 128) for _ in range(24)]
        bs = m.batch_session(32, 192, kv_block=16)
        _, bp32, bd32 = bs.generate_greedy(prompts32, 32)
        out["batch_session_32"] = {"sequences": 32, "steps": 32, "prefill_tok_per_s": round(32 * 127 / bp32, 1),
                                   "decode_tok_per_s_all_sequences": round(32 * 32 / bd32, 1), "ms_per_step": round(bd32 / 32 * 1e3, 3)}
        log(f"[bench] batch session: 32 sequences, 32 steps in {bd32:.3f} s ({32 * 32 / bd32:.0f} tok/s over all sequences)")
        bs.close()
        m.close()
        if check_cpu:
            import oracle as O
            c = L.Llama(path=path, products=L.CALLBACK,
                        matmul=lambda ty, n_rows, n_cols, n_tokens, w, x:
                        O.gemm(ty, n_cols, n_tokens, w, x, n_rows, simd=True, threads=0))
            # step by step, so that every step's logits are seen: the smallest gap between the two largest logits
            # (relative to the largest logit) is the room rounding differences between the paths had
            cs = c.session(kv_block=16)
            t0 = time.perf_counter()
            logits = cs.forward(prompt)
            cp = time.perf_counter() - t0
            ctoks, gaps = [], []
            t0 = time.perf_counter()
            for step in range(129):
                top2 = np.partition(logits, -2)[-2:]
                gaps.append(float(top2[1] - top2[0]) / float(np.abs(logits).max()))
                ctoks.append(L.argmax(logits))
                if step < 128:
                    logits = cs.forward([ctoks[-1]])
            cd = time.perf_counter() - t0
            ctoks = np.array(ctoks, dtype=toks.dtype)
            out.update(min_top2_logit_gap=float(f"{min(gaps):.3e}"), min_top2_logit_gap_step=int(np.argmin(gaps)))
            same = int(np.sum(np.cumprod(toks == ctoks)))
            out.update(cpu_prefill_s=round(cp, 2), cpu_decode_tok_per_s=round(128 / cd, 3), cpu_threads=O.load().lro_worker_count(D),
                       tokens_identical=bool(same == 129), identical_prefix=same)
            dsame_cpu = int(np.sum(np.cumprod(dtoks == ctoks)))
            out["device_session"].update(tokens_identical_to_cpu_path=bool(dsame_cpu == 129), identical_prefix_cpu=dsame_cpu)
            c.close()
    return out


TOKEN_BYTES = N_LAYERS * sum(algorithmic_bytes(Q4_K, r, c) for _, r, c, _ in LAYER) + algorithmic_bytes(Q6_K, VOCAB, D)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=N_LAYERS, help="fewer layers only for quick experiments")
    ap.add_argument("--no-graph", action="store_true", help="enqueue every product eagerly instead of replaying HIP graphs")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="0 skips the CPU baseline")
    ap.add_argument("--seed", type=int, default=20240531)
    ap.add_argument("--no-extras", action="store_true", help="skip the other_workloads section")
    ap.add_argument("--e2e-layers", type=int, default=32,
                    help="layers of the model of the end-to-end greedy decode (128 prompt + 128 steps); 32 = benchmark configuration 4, 0 skips it")
    ap.add_argument("--e2e-check", action="store_true", default=True,
                    help="repeat the greedy decode over the CPU kernels and compare tokens (default)")
    ap.add_argument("--no-e2e-check", dest="e2e_check", action="store_false")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB copy kernel three times (known traffic for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        log(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); "
            "the path shards by weight rows, which is designed but not built")
        return 2

    pkg = importlib.import_module("llama-rust_amd")
    hip = importlib.import_module("llama-rust_amd.hiprt")
    gpu = pkg.HipGemv(0)
    rng = np.random.default_rng(args.seed)

    t_setup = time.perf_counter()
    x_host = {"h1": rng.normal(0, 1, D).astype(np.float32), "attn": rng.normal(0, 1, D).astype(np.float32),
              "h2": rng.normal(0, 1, D).astype(np.float32), "act": rng.normal(0, 1, FF).astype(np.float32)}
    x_dev = {k: hip.DeviceBuffer.from_numpy(v) for k, v in x_host.items()}
    mats, xs, ys, keep = [], [], [], []
    sample = []
    y_bufs = {}
    for layer in range(args.layers):
        for name, rows, cols, src in LAYER:
            w = synth_matrix(Q4_K, rows, cols, rng)
            mats.append(gpu.upload_packed(Q4_K, rows, cols, w))
            xs.append(x_dev[src].ptr)
            slot = 0 if layer == 0 else 1 + layer % 2   # layer 0 keeps its outputs for the sanity check
            if (slot, name) not in y_bufs:
                y_bufs[(slot, name)] = hip.DeviceBuffer(rows * 4)
            ys.append(y_bufs[(slot, name)].ptr)
            if layer < CPU_SAMPLE_LAYERS:
                sample.append((Q4_K, rows, cols, w, src))
        if layer % 8 == 7:
            log(f"[bench] uploaded {layer + 1}/{args.layers} layers ({time.perf_counter() - t_setup:.1f} s)")
    head_w = synth_matrix(Q6_K, VOCAB, D, rng)
    head = gpu.upload_packed(Q6_K, VOCAB, D, head_w)
    head_rows = VOCAB // 16
    sample.append((Q6_K, head_rows, D, head_w[:head_rows * row_bytes(Q6_K, D)].copy(), "h1"))
    head_y = hip.DeviceBuffer(VOCAB * 4)
    del head_w
    n_q4k = len(mats)
    log(f"[bench] {n_q4k} Q4_K matrices + Q6_K head resident, setup {time.perf_counter() - t_setup:.1f} s")

    stream = hip.Stream()
    layers_batch = gpu.make_batch(mats, [1] * n_q4k, xs, ys)
    head_batch = gpu.make_batch([head], [1], [x_dev["h1"].ptr], [head_y.ptr])
    enqueue_layers = lambda s=stream: gpu.gemm_batch_device(layers_batch, s.ptr)
    enqueue_head = lambda s=stream: gpu.gemm_batch_device(head_batch, s.ptr)

    def enqueue_step(s=stream):
        enqueue_layers(s)
        enqueue_head(s)

    # The launches of one shape across all layers, for the per-shape figures: [q,k,v] [o] [gate,up] [down].
    shape_groups = {"[q,k,v]": ("q", "k", "v"), "[o]": ("o",), "[gate,up]": ("gate", "up"), "[down]": ("down",)}
    names = [nm for nm, _, _, _ in LAYER]
    # A launch's time is taken inside the real chain, as the difference between the whole chain and the chain
    # without that shape's launches: a chain of one shape alone would replay 0.3-0.45 GB of matrices, most of
    # which the 256 MB Infinity Cache would then serve.
    shape_batches, shape_bytes = {}, {}
    for label, members in shape_groups.items():
        idx = [layer * len(LAYER) + k for layer in range(args.layers) for k, nm in enumerate(names) if nm not in members]
        shape_batches[label] = gpu.make_batch([mats[i] for i in idx], [1] * len(idx), [xs[i] for i in idx], [ys[i] for i in idx])
        shape_bytes[label] = sum(algorithmic_bytes(Q4_K, r, c) for nm, r, c, _ in LAYER if nm in members)
    enqueue_step(); stream.synchronize()       # first launches configure the kernels
    for b in shape_batches.values():
        gpu.gemm_batch_device(b, stream.ptr)
    stream.synchronize()

    # The yardstick: a kernel that only reads, at the byte counts of the step's launches, chained the same way,
    # over memory of its own (4.4 GB, so nothing comes from the Infinity Cache either).
    read_sizes = [shape_bytes[k] // 16 * 16 for k in ("[q,k,v]", "[o]", "[gate,up]", "[down]")]
    head_bytes = algorithmic_bytes(Q6_K, VOCAB, D)
    read_buf = hip.DeviceBuffer(args.layers * sum(read_sizes) + head_bytes // 16 * 16)
    read_buf.fill_byte(0x5a)

    def enqueue_read_step(s=stream, without=None, head=True):
        at = read_buf.ptr
        for _ in range(args.layers):
            for k, nbytes in enumerate(read_sizes):
                if without != k:
                    gpu.calibration_read(at, nbytes, s.ptr)
                at += nbytes
        if head:
            gpu.calibration_read(at, head_bytes // 16 * 16, s.ptr)

    def enqueue_read_layers_merged(s=stream):
        """The same bytes with one read launch per layer instead of four: what the kernel boundaries inside a layer
        cost a reader, i.e. the most a kernel spanning a layer's products could gain on them."""
        at, per_layer = read_buf.ptr, sum(read_sizes)
        for _ in range(args.layers):
            gpu.calibration_read(at, per_layer, s.ptr)
            at += per_layer

    enqueue_read_step(); stream.synchronize()
    enqueue_read_layers_merged(); stream.synchronize()

    if not args.no_graph:
        graphs = {"step": hip.Graph(stream, enqueue_step), "layers": hip.Graph(stream, enqueue_layers),
                  "head": hip.Graph(stream, enqueue_head), "read_step": hip.Graph(stream, enqueue_read_step)}
        for label, b in shape_batches.items():
            graphs[label] = hip.Graph(stream, lambda s, b=b: gpu.gemm_batch_device(b, s.ptr))
        graphs["read layers"] = hip.Graph(stream, lambda s: enqueue_read_step(s, head=False))
        graphs["read layers merged"] = hip.Graph(stream, enqueue_read_layers_merged)
        for k, label in enumerate(shape_groups):
            graphs["read " + label] = hip.Graph(stream, lambda s, k=k: enqueue_read_step(s, without=k, head=False))
        run = {k: g.launch for k, g in graphs.items()}
    else:
        run = {"step": enqueue_step, "layers": enqueue_layers, "head": enqueue_head, "read_step": enqueue_read_step}
        for label, b in shape_batches.items():
            run[label] = lambda b=b: gpu.gemm_batch_device(b, stream.ptr)
        run["read layers"] = lambda: enqueue_read_step(stream, head=False)
        run["read layers merged"] = lambda: enqueue_read_layers_merged(stream)
        for k, label in enumerate(shape_groups):
            run["read " + label] = lambda k=k: enqueue_read_step(stream, without=k, head=False)

    # sanity: a sample of layer-0 outputs against the CPU oracle before timing anything
    import oracle as O
    run["step"](); stream.synchronize()
    for (ty, rows, cols, w, src), (name, _, _, _) in zip(sample[:len(LAYER)], LAYER):
        got = y_bufs[(0, name)].to_numpy(np.float32)[:64]
        want = O.gemm_f64(ty, cols, 1, w[:64 * row_bytes(ty, cols)], x_host[src], 64)[0]
        if not np.allclose(got, want, rtol=1e-4, atol=1e-4 * float(np.sqrt(np.mean(want ** 2)))):
            log(f"[bench] FATAL: GPU output of layer-0 {name} disagrees with the CPU oracle")
            return 1

    if args.copy_calibration:
        src, dst = hip.DeviceBuffer(1 << 30), hip.DeviceBuffer(1 << 30)
        src.fill_byte(1)
        for _ in range(3):
            gpu.calibration_copy(dst.ptr, src.ptr, 1 << 30, stream.ptr)
        stream.synchronize()
        src.free(); dst.free()

    def replay_us(key, reps):
        """Mean microseconds of one replay of run[key], from HIP events on the launch stream around `reps`
        back-to-back replays."""
        run[key](); stream.synchronize()
        a, b = hip.Event(), hip.Event()
        a.record(stream)
        for _ in range(reps):
            run[key]()
        b.record(stream)
        stream.synchronize()
        return a.elapsed_ms(b) * 1e3 / reps

    for _ in range(args.warmup):
        run["step"]()
    stream.synchronize()

    # The timed region: K steps, each one graph of all 129 launches, between two synchronisations.
    a_ev, b_ev = hip.Event(), hip.Event()
    hip.device_synchronize()
    t0 = time.perf_counter()
    a_ev.record(stream)
    for _ in range(args.steps):
        run["step"]()
    b_ev.record(stream)
    stream.synchronize()
    hip.device_synchronize()
    wall = time.perf_counter() - t0
    step_event_ms = a_ev.elapsed_ms(b_ev) / args.steps

    # The same launches again, the Q4_K part and the head on their own (HIP events on the launch stream).
    q4k_ms = replay_us("layers", args.steps) / 1e3
    head_ms = replay_us("head", args.steps) / 1e3
    q4k_bytes = (args.layers * sum(algorithmic_bytes(Q4_K, r, c) for _, r, c, _ in LAYER))
    n_launch = args.layers * LAUNCHES_PER_LAYER
    step_bytes = q4k_bytes + head_bytes
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (wall / args.steps) / 1e9
    q4k_launch_us = q4k_ms * 1e3 / n_launch
    q4k_gbs = q4k_bytes / (q4k_ms * 1e-3) / 1e9
    head_gbs = head_bytes / (head_ms * 1e-3) / 1e9

    # Per launch shape, and the read-only yardstick at the same sizes (mean over the layers' launches).
    per_shape = {}
    reps = max(3, args.steps // 2)
    layers_us, read_layers_us = replay_us("layers", reps), replay_us("read layers", reps)
    for k, label in enumerate(shape_groups):
        us = (layers_us - replay_us(label, reps)) / args.layers
        read_us = (read_layers_us - replay_us("read " + label, reps)) / args.layers
        per_shape[label] = {"bytes": shape_bytes[label], "launch_us": round(us, 2),
                            "achieved": round(shape_bytes[label] / us / 1e3, 1), "frac": round(shape_bytes[label] / us / 1e3 / HBM_PEAK_GBS, 4),
                            "plain_read_us": round(read_us, 2), "frac_of_plain_read": round(read_us / us, 3)}
    read_step_us = replay_us("read_step", max(3, args.steps // 2))
    read_merged_us = replay_us("read layers merged", reps)
    traffic = profiled_traffic()

    out = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"Llama-3-8B decode GEMV, batch 1: {args.layers} layers x 7 Q4_K products + Q6_K head 4096->128256",
                   "weights_gb": round(step_bytes / 1e9, 3), "products_per_step": n_q4k + 1, "launches_per_step": n_launch + 1,
                   "launch_grouping": "per layer [q,k,v] [o] [gate,up] [down]: products sharing an input are one launch",
                   "launch_mode": "eager" if args.no_graph else "one hip_graph per step (layers and head)"},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "tok_per_s": round(args.steps / wall, 1),
        "tok_per_s_scope": "the timed step: the weight products of one token; decode_tok_per_s_end_to_end is a whole greedy decode",
        "ms_per_step_hip_events": round(step_event_ms, 4),
        "roofline": {"bound": "hbm", "kernel": "gemv_q4k_kernel", "achieved": round(q4k_gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(q4k_gbs / HBM_PEAK_GBS, 4),
                     "traffic": round(traffic["ratio"] * q4k_bytes / n_launch) if traffic["ratio"] else None,
                     "traffic_source": traffic["source"],
                     "bytes_per_launch": round(q4k_bytes / n_launch), "launch_us": round(q4k_launch_us, 3),
                     "launches_timed": args.steps * n_launch,
                     "timing": "HIP events on the launch stream around K back-to-back replays of the graph of the 128 Q4_K launches, right after the timed region",
                     "per_shape": per_shape,
                     "per_shape_method": "time of the 128-launch chain minus the chain without that shape's 32 launches, per launch; plain_read_us the same for a kernel that only reads",
                     "plain_read_same_sizes": {
                         "what": "a kernel that only reads, launched as the same chain at the same byte counts (4 per layer + head)",
                         "step_us": round(read_step_us, 1), "gbs": round(step_bytes / read_step_us / 1e3, 1),
                         "frac_of_peak": round(step_bytes / read_step_us / 1e3 / HBM_PEAK_GBS, 4),
                         "this_step_vs_plain_read": round(read_step_us / (ms_per_step * 1e3), 3),
                         "layer_us_four_launches": round(read_layers_us / args.layers, 2),
                         "layer_us_one_launch": round(read_merged_us / args.layers, 2),
                         "layer_note": "a layer's 122.9 MB read by four dependent launches (the products' sizes) and by one: "
                                       "the difference is what the three kernel boundaries inside a layer cost a reader"}},
        "other_kernels": {"gemv_q6k_kernel (head)": {"achieved": round(head_gbs, 1), "unit": "GB/s",
                                                     "frac": round(head_gbs / HBM_PEAK_GBS, 4),
                                                     "launch_us": round(head_ms * 1e3, 2)}},
    }
    read_buf.free()
    for m in mats:
        m.close()
    head.close()
    if not args.no_extras:
        log("[bench] other workloads (Q8_0 GEMV, Q4_0 prefill GEMM, MoE grouped GEMM) ...")
        out["other_workloads"] = other_workloads(pkg, hip, gpu, stream, rng, args.cpu_seconds > 0)
    if args.e2e_layers > 0:
        log("[bench] end-to-end greedy decode ...")
        e2e = greedy_decode(pkg, args.e2e_layers, args.e2e_check, args.seed)
        out.setdefault("other_workloads", {})["llama_greedy_decode"] = e2e
        if args.e2e_layers == N_LAYERS:
            # whole tokens per second of a real greedy decode (attention, norms and sampling included): the
            # step resident on the GPU, and through the reference's host seam (one round trip per product)
            out["decode_tok_per_s_end_to_end"] = e2e["device_session"]["decode_tok_per_s"]
            out["decode_tok_per_s_host_seam"] = e2e["decode_tok_per_s"]
            # the same model with 8 and 32 sequences decoded together (not batch 1: beside the metric, not in it)
            out["decode_tok_per_s_8_sequences"] = e2e["batch_session"]["decode_tok_per_s_all_sequences"]
            out["decode_tok_per_s_32_sequences"] = e2e["batch_session_32"]["decode_tok_per_s_all_sequences"]
            out["prompt_tok_per_s_device_session"] = e2e["device_session"]["prefill_tok_per_s"]
            out["greedy_tokens_identical_to_cpu_path"] = bool(e2e.get("tokens_identical")) and bool(
                e2e["device_session"].get("tokens_identical_to_cpu_path")) if args.e2e_check else None
    if args.cpu_seconds > 0:
        log("[bench] timing the CPU baseline ...")
        out["cpu_baseline"] = cpu_baseline(sample, x_host, args.cpu_seconds)
        out["cpu_baseline"]["value"] = round(out["cpu_baseline"]["value"], 2)
        out["cpu_baseline"]["tok_per_s_equiv"] = round(out["cpu_baseline"]["tok_per_s_equiv"], 3)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
