// Host side of a dense Llama decode over the matrix executor (see include/native_hip_llama.h).
//
// Everything here is f32 host arithmetic in the reference's operation order; the only
// work that leaves the host is the weight products, which go to the executor (or to the
// caller's function).  Multiplications and additions are never contracted into FMAs, as
// in the reference's scalar Rust.
#pragma clang fp contract(off)

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>
#include <thread>
#include <map>
#include <tuple>
#include <vector>

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "../../include/native_hip.h"
#include "../../include/native_hip_llama.h"
#include "gguf.h"

namespace {

thread_local std::string t_err;
int fail(const std::string &m) {
    t_err = m;
    return 1;
}

// ------------------------------------------------------------------ numeric building blocks

float f16_to_f32(uint16_t h) {  // langtax/src/fp16.rs:4-33: exact, subnormals and specials included
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 1023u;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: man * 2^-24
            int e = 0;
            uint32_t m = man;
            while (!(m & 1024u)) {
                m <<= 1;
                e++;
            }
            bits = sign | ((uint32_t)(113 - e) << 23) | ((m & 1023u) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}
uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
uint32_t rd32(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }

// One packed row -> n_cols floats, bit for bit the value every product of the reference is
// defined on (langtax/src/quant.rs:7511-7541, 7734-7765, 7884-7950, 8046-8130, 8783-8853).
bool dequant_row(uint32_t type, size_t n_cols, const uint8_t *row, float *y) {
    size_t bb = 0, bk = 0;
    if (!nh::gguf::type_layout(type, &bb, &bk) || n_cols % bk != 0) return false;
    const size_t nb = n_cols / bk;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *w = row + b * bb;
        float *o = y + b * bk;
        switch (type) {
        case 0: std::memcpy(o, w, 4); break;
        case 1: o[0] = f16_to_f32(rd16(w)); break;
        case 8: {
            const float d = f16_to_f32(rd16(w));
            for (int j = 0; j < 32; j++) o[j] = (float)(int8_t)w[2 + j] * d;
            break;
        }
        case 2: {
            const float d = f16_to_f32(rd16(w));
            for (int j = 0; j < 16; j++) {
                o[j] = (float)((int)(w[2 + j] & 15) - 8) * d;
                o[j + 16] = (float)((int)(w[2 + j] >> 4) - 8) * d;
            }
            break;
        }
        case 6:
        case 7: {
            const bool with_min = type == 7;
            const float d = f16_to_f32(rd16(w)), m = with_min ? f16_to_f32(rd16(w + 2)) : 0.f;
            const uint32_t qh = rd32(w + (with_min ? 4 : 2));
            const uint8_t *qs = w + (with_min ? 8 : 6);
            for (int j = 0; j < 16; j++) {
                const int lo = (qs[j] & 15) | (int)(((qh >> j) & 1u) << 4);
                const int hi = (qs[j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
                if (with_min) {
                    const float a = (float)lo * d, c = (float)hi * d;
                    o[j] = a + m;
                    o[j + 16] = c + m;
                } else {
                    o[j] = (float)(lo - 16) * d;
                    o[j + 16] = (float)(hi - 16) * d;
                }
            }
            break;
        }
        case 12: {
            const float d = f16_to_f32(rd16(w)), dmin = f16_to_f32(rd16(w + 2));
            const uint8_t *s = w + 4, *qs = w + 16;
            for (int pair = 0; pair < 4; pair++) {  // 64 columns: low nibbles, then high nibbles, of 32 bytes
                for (int half = 0; half < 2; half++) {
                    const int j = 2 * pair + half;
                    uint32_t sc, mn;  // langtax/src/quant.rs:8901-8912
                    if (j < 4) {
                        sc = s[j] & 63u;
                        mn = s[j + 4] & 63u;
                    } else {
                        sc = (s[j + 4] & 15u) | ((uint32_t)(s[j - 4] >> 6) << 4);
                        mn = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
                    }
                    const float a = d * (float)sc, c = dmin * (float)mn;
                    for (int l = 0; l < 32; l++) {
                        const uint32_t q = half ? (uint32_t)(qs[32 * pair + l] >> 4) : (qs[32 * pair + l] & 15u);
                        const float p = a * (float)q;
                        o[64 * pair + 32 * half + l] = p - c;
                    }
                }
            }
            break;
        }
        case 14: {
            const uint8_t *ql = w, *qh = w + 128;
            const int8_t *sc = reinterpret_cast<const int8_t *>(w + 192);
            const float d = f16_to_f32(rd16(w + 208));
            for (int n = 0; n < 2; n++) {  // 128 columns per half
                for (int l = 0; l < 32; l++) {
                    const int is = l / 16;
                    const uint8_t h = qh[32 * n + l];
                    const int q1 = (int)((ql[64 * n + l] & 15) | ((h & 3) << 4)) - 32;
                    const int q2 = (int)((ql[64 * n + l + 32] & 15) | (((h >> 2) & 3) << 4)) - 32;
                    const int q3 = (int)((ql[64 * n + l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
                    const int q4 = (int)((ql[64 * n + l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32;
                    const float d1 = d * (float)sc[8 * n + is], d2 = d * (float)sc[8 * n + is + 2];
                    const float d3 = d * (float)sc[8 * n + is + 4], d4 = d * (float)sc[8 * n + is + 6];
                    o[128 * n + l] = d1 * (float)q1;
                    o[128 * n + l + 32] = d2 * (float)q2;
                    o[128 * n + l + 64] = d3 * (float)q3;
                    o[128 * n + l + 96] = d4 * (float)q4;
                }
            }
            break;
        }
        default: return false;
        }
    }
    return true;
}

// langtax/src/decode.rs:11498-11513.  The element count enters as the reference converts it:
// through u16, anything longer counting as 1.
void rmsnorm(float *x, const float *w, size_t n, float eps) {
    float ss = 0.f;
    for (size_t i = 0; i < n; i++) ss += x[i] * x[i];
    const float nf = n <= 65535 ? (float)n : 1.f;
    const float rms = std::sqrt(ss / nf + eps);
    const float inv = rms > 0.f ? 1.f / rms : 0.f;
    for (size_t i = 0; i < n; i++) x[i] = x[i] * inv * w[i];
}

// langtax/src/decode.rs:11578-11602: adjacent pairs, theta multiplied up pair by pair.
void rope(float *v, size_t len, size_t pos, size_t n_rot, float base) {
    const size_t n = n_rot < len ? n_rot : len;
    if (n < 2) return;
    const float n_rot_f = n_rot <= 65535 ? (float)n_rot : 2.f;
    float theta = pos <= 65535 ? (float)pos : 65535.f;
    const float theta_scale = std::pow(base, -2.0f / n_rot_f);
    for (size_t i = 0; i + 1 < n; i += 2) {
        const float c = std::cos(theta), s = std::sin(theta);
        const float x = v[i], y = v[i + 1];
        v[i] = x * c - y * s;
        v[i + 1] = x * s + y * c;
        theta *= theta_scale;
    }
}

void softmax(float *x, size_t n) {  // langtax/src/decode.rs:12021-12033
    float m = -INFINITY;
    for (size_t i = 0; i < n; i++) m = std::fmax(m, x[i]);
    float s = 0.f;
    for (size_t i = 0; i < n; i++) {
        x[i] = std::exp(x[i] - m);
        s += x[i];
    }
    if (s > 0.f)
        for (size_t i = 0; i < n; i++) x[i] /= s;
}

uint32_t argmax(const float *x, size_t n) {  // first maximum wins; langtax/src/decode.rs:12104-12114
    size_t best_i = 0;
    float best = -INFINITY;
    for (size_t i = 0; i < n; i++)
        if (x[i] > best) {
            best = x[i];
            best_i = i;
        }
    return (uint32_t)best_i;
}

// Indices of the k largest values, descending, ties to the lower index (langtax/src/decode.rs:11363-11379:
// ggml_argsort_top_k).  The reference's comparator treats a NaN as a tie with everything, which is no order
// at all once a NaN is present; here the order is total, as std::sort requires: numbers descending, then the
// NaNs, equal keys by ascending index.  On inputs without NaN both give the same result.  False when k is 0 or
// exceeds n.
bool topk(const float *v, size_t n, size_t k, std::vector<uint32_t> *order) {
    if (k == 0 || k > n) return false;
    order->resize(n);
    for (size_t i = 0; i < n; i++) (*order)[i] = (uint32_t)i;
    std::sort(order->begin(), order->end(), [&](uint32_t a, uint32_t b) {
        const float va = v[a], vb = v[b];
        const bool na = va != va, nb = vb != vb;
        if (na != nb) return nb;     // a number before a NaN
        if (!na) {
            if (vb < va) return true;    // a first: larger value
            if (vb > va) return false;
        }
        return a < b;                // equal numbers, or two NaNs: lower index first
    });
    order->resize(k);
    return true;
}

// Official build_moe_ffn norm_w clamp: the smallest normal f16 (decode.rs:321).
constexpr float MOE_NORM_W_CLAMP = 1.0f / 16384.0f;

// Router weights of the selected experts (decode.rs:11391-11409): their probabilities, renormalised to sum
// one when norm_w, with the sum clamped from below.
void router_weights(const float *probs, const uint32_t *order, size_t k, bool norm_w, float *w) {
    float wsum = 0.f;
    for (size_t j = 0; j < k; j++) {
        w[j] = probs[order[j]];
        wsum += w[j];
    }
    if (!norm_w) return;
    if (wsum < MOE_NORM_W_CLAMP) wsum = MOE_NORM_W_CLAMP;
    for (size_t j = 0; j < k; j++) w[j] /= wsum;
}

// ------------------------------------------------------------------ worker threads for the attention heads

// The reference attends head after head on one thread.  Heads are independent, so they are
// spread over a few threads here; the arithmetic of each head is untouched.
class HeadPool {
  public:
    explicit HeadPool(size_t workers) {
        for (size_t i = 0; i < workers; i++) threads_.emplace_back([this] { loop(); });
    }
    ~HeadPool() {
        {
            std::lock_guard<std::mutex> g(mu_);
            stop_ = true;
        }
        wake_.notify_all();
        for (auto &t : threads_) t.join();
    }
    // Calls fn(i) for every i < n, on the workers and on the calling thread; returns when all are done.
    void run(size_t n, const std::function<void(size_t)> &fn) {
        if (threads_.empty() || n < 2) {
            for (size_t i = 0; i < n; i++) fn(i);
            return;
        }
        {
            std::lock_guard<std::mutex> g(mu_);
            fn_ = &fn;
            n_ = n;
            next_.store(0);
            busy_ = threads_.size();
            epoch_++;
        }
        wake_.notify_all();
        drain();
        std::unique_lock<std::mutex> g(mu_);
        done_.wait(g, [this] { return busy_ == 0; });
        fn_ = nullptr;
    }

  private:
    void drain() {
        for (size_t i = next_.fetch_add(1); i < n_; i = next_.fetch_add(1)) (*fn_)(i);
    }
    void loop() {
        uint64_t seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> g(mu_);
                wake_.wait(g, [&] { return stop_ || epoch_ != seen; });
                if (stop_) return;
                seen = epoch_;
            }
            drain();
            std::lock_guard<std::mutex> g(mu_);
            if (--busy_ == 0) done_.notify_one();
        }
    }
    std::vector<std::thread> threads_;
    std::mutex mu_;
    std::condition_variable wake_, done_;
    const std::function<void(size_t)> *fn_ = nullptr;
    size_t n_ = 0, busy_ = 0;
    std::atomic<size_t> next_{0};
    uint64_t epoch_ = 0;
    bool stop_ = false;
};

// ------------------------------------------------------------------ model

struct Mat {
    std::string name;
    uint32_t type = 0;
    size_t n_rows = 0, n_cols = 0;
    const uint8_t *bytes = nullptr;
    size_t nbytes = 0;
    lnh_matrix *resident = nullptr;
};

struct Layer {
    std::vector<float> attn_norm, ffn_norm;
    Mat wq, wk, wv, wo, gate, up, down;
    // Routed feed-forward (llama.expert_count > 0, langtax/src/decode.rs:569-577, 9228-9256): the router and
    // the experts' gate / up / down matrices, expert e being part e of the 3-D *_exps tensors
    // (decode.rs:9853-9913: bytes [start + e * per, start + (e + 1) * per)).
    bool moe = false;
    Mat gate_inp;
    std::vector<Mat> gate_e, up_e, down_e;
};

// Scratch of the routed feed-forward (langtax/src/decode.rs:1530-1560, MoeScratch).
struct MoeScratch {
    std::vector<float> logits, sel_w, pack_x, g, u, y;
    std::vector<uint32_t> sel_e, order;
    std::vector<std::vector<uint32_t>> buckets;
    // Resident route (moe_ffn_on_device): grow-only device buffers, pinned staging and a stream of the scratch's own.
    // io: the n x n_embd rows in and the result out; small: logits, bucket order, weights.
    float *d_io = nullptr, *d_small = nullptr, *d_x = nullptr, *d_g = nullptr, *d_u = nullptr, *d_y = nullptr;
    float *h_io = nullptr, *h_small = nullptr;
    size_t cap_io = 0, cap_small = 0, cap_x = 0, cap_g = 0, cap_u = 0, cap_y = 0, cap_hio = 0, cap_hsmall = 0;  // floats
    hipStream_t stream = nullptr;
    MoeScratch() = default;
    MoeScratch(const MoeScratch &) = delete;
    MoeScratch &operator=(const MoeScratch &) = delete;
    ~MoeScratch() {
        for (float *p : {d_io, d_small, d_x, d_g, d_u, d_y})
            if (p) (void)hipFree(p);
        for (float *p : {h_io, h_small})
            if (p) (void)hipHostFree(p);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

}  // namespace

struct lnm_model {
    std::vector<uint8_t> owned;  // lnm_load_bytes
    void *map = nullptr;         // lnm_load
    size_t map_len = 0;
    nh::gguf::File file;
    lnm_hparams hp{};
    std::vector<Layer> layers;
    Mat token_embd, output;
    std::vector<float> output_norm;
    int route = LNM_PRODUCTS_RESIDENT;
    lnm_matmul_fn fn = nullptr;
    void *user = nullptr;
    lnh_exec *exec = nullptr;
    std::unique_ptr<MoeScratch> moe_entry;  // lnm_moe_ffn's scratch

    ~lnm_model() {
        auto drop = [](Mat &m) {
            if (m.resident) lnh_matrix_free(m.resident);
            m.resident = nullptr;
        };
        for (Layer &l : layers) {
            for (Mat *m : {&l.wq, &l.wk, &l.wv, &l.wo, &l.gate, &l.up, &l.down, &l.gate_inp}) drop(*m);
            for (auto *v : {&l.gate_e, &l.up_e, &l.down_e})
                for (Mat &m : *v) drop(m);
        }
        drop(token_embd);
        drop(output);
        if (exec) lnh_destroy(exec);
        if (map) munmap(map, map_len);
    }
};

struct DeviceDecode;  // llama_device.inc

struct lnm_session {
    lnm_model *model = nullptr;
    std::unique_ptr<DeviceDecode, void (*)(DeviceDecode *)> dev{nullptr, nullptr};  // set: the whole step runs on the GPU
    size_t kv_block = 16, past = 0;
    std::vector<uint32_t> ids;        // the tokens at positions 0 .. past-1, for lnm_prompt's prefix reuse
    std::vector<uint32_t> table;      // logical block -> physical block
    std::vector<uint32_t> preset;     // physical ids to hand out, in order (empty: 0, 1, 2, ...)
    std::vector<float> cache_k, cache_v;
    // q, k, v share one buffer (matrix after matrix), and so do gate and up: products of one
    // input can then be fetched by a single call
    std::vector<float> x, residual, qkv, attn, attn_proj, gate_up, ffn_out, xn;
    MoeScratch moe;
    double products_s = 0.0, attention_s = 0.0;  // wall time spent in weight products / in attend + RoPE
    uint64_t n_products = 0;
    std::unique_ptr<HeadPool> pool;
};

namespace {

bool read_f32s(const nh::gguf::File &f, const std::string &name, size_t n, std::vector<float> *out, std::string *err) {
    const nh::gguf::TensorInfo *t = f.tensor(name);
    if (!t) return *err = "missing tensor " + name, false;
    if (t->type != 0 || t->end - t->start != 4 * n) return *err = "tensor " + name + " is not f32[" + std::to_string(n) + "]", false;
    out->resize(n);
    std::memcpy(out->data(), f.data + t->start, 4 * n);
    return true;
}

bool read_mat(const nh::gguf::File &f, const std::string &name, size_t n_rows, size_t n_cols, Mat *out, std::string *err) {
    const nh::gguf::TensorInfo *t = f.tensor(name);
    if (!t) return *err = "missing tensor " + name, false;
    // ggml order: shape[0] = columns (contiguous), shape[1] = rows
    if (t->shape.size() != 2 || t->shape[0] != n_cols || t->shape[1] != n_rows)
        return *err = "tensor " + name + " has the wrong shape", false;
    out->name = name;
    out->type = t->type;
    out->n_rows = n_rows;
    out->n_cols = n_cols;
    out->bytes = f.data + t->start;
    out->nbytes = t->end - t->start;
    return true;
}

// A 3-D tensor [n_cols, n_rows, n_parts] (ggml order) as n_parts matrices over consecutive byte ranges
// (langtax/src/decode.rs:476-493, 9853-9913).  n_rows or n_cols given as 0 is taken from the tensor.
bool read_parts(const nh::gguf::File &f, const std::string &name, size_t n_parts, size_t n_rows, size_t n_cols,
                std::vector<Mat> *out, std::string *err) {
    const nh::gguf::TensorInfo *t = f.tensor(name);
    if (!t) return *err = "missing tensor " + name, false;
    if (t->shape.size() != 3 || t->shape[2] != n_parts || (n_cols && t->shape[0] != n_cols) ||
        (n_rows && t->shape[1] != n_rows))
        return *err = "tensor " + name + " has the wrong shape", false;
    const size_t total = t->end - t->start, per = total / n_parts;
    if (per * n_parts != total) return *err = "tensor " + name + " does not split into its parts", false;
    out->resize(n_parts);
    for (size_t e = 0; e < n_parts; e++) {
        Mat &m = (*out)[e];
        m.name = name + "[" + std::to_string(e) + "]";
        m.type = t->type;
        m.n_rows = (size_t)t->shape[1];
        m.n_cols = (size_t)t->shape[0];
        m.bytes = f.data + t->start + e * per;
        m.nbytes = per;
    }
    return true;
}

int finish_load(lnm_model *m) {
    std::string err;
    const nh::gguf::File &f = m->file;
    std::string arch;
    if (!f.kv_str("general.architecture", &arch)) return fail("missing key general.architecture");
    if (arch != "llama") return fail("unsupported architecture " + arch);
    auto need_u32 = [&](const char *field, uint32_t *out) {
        const std::string key = arch + "." + field;
        if (!f.kv_u32(key, out)) {
            err = "missing key " + key;
            return false;
        }
        return true;
    };
    lnm_hparams &hp = m->hp;
    if (!need_u32("block_count", &hp.n_layer) || !need_u32("embedding_length", &hp.n_embd) ||
        !need_u32("attention.head_count", &hp.n_head) || !need_u32("attention.head_count_kv", &hp.n_head_kv) ||
        !need_u32("feed_forward_length", &hp.n_ff))
        return fail(err);
    if (!hp.n_layer || !hp.n_embd || !hp.n_head || !hp.n_head_kv || !hp.n_ff) return fail("zero hyper-parameter");
    if (hp.n_head % hp.n_head_kv != 0 || hp.n_embd % hp.n_head != 0) return fail("head counts do not divide");
    hp.head_dim = hp.n_embd / hp.n_head;
    if (!f.kv_u32(arch + ".rope.dimension_count", &hp.n_rot)) hp.n_rot = hp.head_dim;  // decode.rs:7461-7475
    if (hp.n_rot == 0) return fail("zero rope.dimension_count");
    if (!f.kv_f32(arch + ".rope.freq_base", &hp.rope_base)) hp.rope_base = 10000.f;                  // decode.rs:2053
    if (!f.kv_f32(arch + ".attention.layer_norm_rms_epsilon", &hp.rms_eps)) hp.rms_eps = 1e-5f;      // decode.rs:1958
    const nh::gguf::TensorInfo *emb = f.tensor("token_embd.weight");
    if (!emb || emb->shape.size() != 2 || emb->shape[0] != hp.n_embd) return fail("missing or misshapen token_embd.weight");
    hp.n_vocab = (uint32_t)emb->shape[1];
    if (!read_mat(f, "token_embd.weight", hp.n_vocab, hp.n_embd, &m->token_embd, &err)) return fail(err);
    if (!read_f32s(f, "output_norm.weight", hp.n_embd, &m->output_norm, &err)) return fail(err);
    if (f.tensor("output.weight")) {
        if (!read_mat(f, "output.weight", hp.n_vocab, hp.n_embd, &m->output, &err)) return fail(err);
    } else {
        m->output = m->token_embd;  // tied head (decode.rs:2069-2072)
    }
    // decode.rs:8502-8519: a missing or zero llama.expert_count is a dense model
    hp.n_expert = hp.n_expert_used = 0;
    uint32_t n_expert = 0;
    if (f.kv_u32(arch + ".expert_count", &n_expert) && n_expert != 0) {
        if (!need_u32("expert_used_count", &hp.n_expert_used)) return fail(err);
        if (hp.n_expert_used == 0 || hp.n_expert_used > n_expert) return fail("bad " + arch + ".expert_used_count");
        hp.n_expert = n_expert;
    }
    const size_t qw = (size_t)hp.n_head * hp.head_dim, kvw = (size_t)hp.n_head_kv * hp.head_dim;
    m->layers.resize(hp.n_layer);
    for (uint32_t i = 0; i < hp.n_layer; i++) {
        Layer &l = m->layers[i];
        const std::string p = "blk." + std::to_string(i) + ".";
        if (!read_f32s(f, p + "attn_norm.weight", hp.n_embd, &l.attn_norm, &err) ||
            !read_f32s(f, p + "ffn_norm.weight", hp.n_embd, &l.ffn_norm, &err) ||
            !read_mat(f, p + "attn_q.weight", qw, hp.n_embd, &l.wq, &err) ||
            !read_mat(f, p + "attn_k.weight", kvw, hp.n_embd, &l.wk, &err) ||
            !read_mat(f, p + "attn_v.weight", kvw, hp.n_embd, &l.wv, &err) ||
            !read_mat(f, p + "attn_output.weight", hp.n_embd, qw, &l.wo, &err))
            return fail(err);
        if (hp.n_expert == 0) {
            if (!read_mat(f, p + "ffn_gate.weight", hp.n_ff, hp.n_embd, &l.gate, &err) ||
                !read_mat(f, p + "ffn_up.weight", hp.n_ff, hp.n_embd, &l.up, &err) ||
                !read_mat(f, p + "ffn_down.weight", hp.n_embd, hp.n_ff, &l.down, &err))
                return fail(err);
            continue;
        }
        // decode.rs:9228-9256: the router has one row per expert, the three expert tensors one part per expert,
        // gate and up agree on the hidden width and down takes it back to n_embd
        l.moe = true;
        if (!read_mat(f, p + "ffn_gate_inp.weight", hp.n_expert, hp.n_embd, &l.gate_inp, &err)) return fail(err);
        if (!read_parts(f, p + "ffn_gate_exps.weight", hp.n_expert, 0, hp.n_embd, &l.gate_e, &err) ||
            !read_parts(f, p + "ffn_up_exps.weight", hp.n_expert, 0, hp.n_embd, &l.up_e, &err) ||
            !read_parts(f, p + "ffn_down_exps.weight", hp.n_expert, hp.n_embd, 0, &l.down_e, &err))
            return fail(err);
        if (l.gate_e[0].n_rows != l.up_e[0].n_rows || l.down_e[0].n_cols != l.up_e[0].n_rows)
            return fail("blk." + std::to_string(i) + ".ffn_*_exps.weight disagree on the hidden width");
    }
    hp.block_type = m->layers[0].wq.type;
    hp.embd_type = m->token_embd.type;
    hp.output_type = m->output.type;
    return 0;
}

int product_routed(lnm_model *m, Mat &w, size_t n, const float *x, float *y);

using wall_clock = std::chrono::steady_clock;
double since(wall_clock::time_point t0) { return std::chrono::duration<double>(wall_clock::now() - t0).count(); }

// One weight product of a session, timed.
int product(lnm_session *s, Mat &w, size_t n, const float *x, float *y) {
    const auto t0 = wall_clock::now();
    const int rc = product_routed(s->model, w, n, x, y);
    s->products_s += since(t0);
    s->n_products++;
    return rc;
}

// Several matrices times the same input; ys[i] must lie back to back in that order.
int products_shared(lnm_session *s, std::initializer_list<Mat *> ws, size_t n, const float *x, float *y) {
    lnm_model *m = s->model;
    if (m->route != LNM_PRODUCTS_RESIDENT) {  // the reference's call shape: one product per call
        for (Mat *w : ws) {
            if (product(s, *w, n, x, y) != 0) return 1;
            y += n * w->n_rows;
        }
        return 0;
    }
    const auto t0 = wall_clock::now();
    if (!m->exec && lnh_create(0, &m->exec) != 0) return fail(std::string("executor: ") + lnh_thread_error());
    const lnh_matrix *handles[4];
    size_t k = 0, y_len = 0;
    for (Mat *w : ws) {
        if (!w->resident &&
            lnh_upload_packed(m->exec, w->type, w->n_rows, w->n_cols, w->bytes, w->nbytes, &w->resident) != 0)
            return fail(std::string(lnh_last_error(m->exec)) + " (" + w->name + ")");
        handles[k++] = w->resident;
        y_len += n * w->n_rows;
    }
    const Mat *first = *ws.begin();
    if (lnh_gemm_shared(m->exec, k, handles, n, x, n * first->n_cols, y, y_len) != 0)
        return fail(std::string(lnh_last_error(m->exec)) + " (" + first->name + ")");
    s->products_s += since(t0);
    s->n_products += k;
    return 0;
}

// One weight product, by the model's route.
int product_routed(lnm_model *m, Mat &w, size_t n, const float *x, float *y) {
    const size_t x_len = n * w.n_cols, y_len = n * w.n_rows;
    switch (m->route) {
    case LNM_PRODUCTS_CALLBACK:
        if (!m->fn) return fail("no product function set");
        if (m->fn(m->user, w.type, w.n_rows, w.n_cols, n, w.bytes, w.nbytes, x, y) != 0)
            return fail("product function failed for " + w.name);
        return 0;
    case LNM_PRODUCTS_DISPATCH: {
        const int rc = n == 1 ? lnq_gemv(w.type, w.n_cols, w.bytes, w.nbytes, x, x_len, y, y_len)
                              : lnq_gemm(w.type, w.n_cols, n, w.bytes, w.nbytes, x, x_len, y, y_len);
        return rc == 0 ? 0 : fail(std::string(lnq_last_error()) + " (" + w.name + ")");
    }
    default: {
        if (!m->exec && lnh_create(0, &m->exec) != 0) return fail(std::string("executor: ") + lnh_thread_error());
        if (!w.resident &&
            lnh_upload_packed(m->exec, w.type, w.n_rows, w.n_cols, w.bytes, w.nbytes, &w.resident) != 0)
            return fail(std::string(lnh_last_error(m->exec)) + " (" + w.name + ")");
        if (lnh_gemm(m->exec, w.resident, n, x, x_len, y, y_len) != 0)
            return fail(std::string(lnh_last_error(m->exec)) + " (" + w.name + ")");
        return 0;
    }
    }
}

// langtax/src/kv_page.rs:410-438, paged branch.
size_t kv_offset(const lnm_session *s, size_t layer, size_t head, size_t t) {
    const lnm_hparams &hp = s->model->hp;
    const size_t bs = s->kv_block, b = s->table[t / bs];
    return ((((size_t)b * hp.n_layer + layer) * hp.n_head_kv + head) * bs + t % bs) * hp.head_dim;
}

int ensure_blocks(lnm_session *s, size_t positions) {
    const lnm_hparams &hp = s->model->hp;
    const size_t need = (positions + s->kv_block - 1) / s->kv_block;
    while (s->table.size() < need) {
        uint32_t id = (uint32_t)s->table.size();
        if (!s->preset.empty()) {
            if (s->table.size() >= s->preset.size()) return fail("sequence outgrew the given block ids");
            id = s->preset[s->table.size()];
        }
        s->table.push_back(id);
        const size_t stride = (size_t)hp.n_layer * hp.n_head_kv * s->kv_block * hp.head_dim;
        const size_t floats = ((size_t)id + 1) * stride;
        if (s->cache_k.size() < floats) {
            s->cache_k.resize(floats, 0.f);
            s->cache_v.resize(floats, 0.f);
        }
    }
    return 0;
}

// Uploads w once (RESIDENT route).
int ensure_resident(lnm_model *m, Mat &w) {
    if (!m->exec && lnh_create(0, &m->exec) != 0) return fail(std::string("executor: ") + lnh_thread_error());
    if (!w.resident && lnh_upload_packed(m->exec, w.type, w.n_rows, w.n_cols, w.bytes, w.nbytes, &w.resident) != 0)
        return fail(std::string(lnh_last_error(m->exec)) + " (" + w.name + ")");
    return 0;
}

// One projection of every non-empty expert: expert e multiplies its counts[e] packed rows.  The reference
// issues one product per expert (decode.rs:10035-10058, 10148-10261: gemm_part_bytes_into, which takes the
// single-token route for one row); the RESIDENT route hands all of them to the executor in one grouped call.
int expert_products(lnm_model *m, std::vector<Mat> &parts, const std::vector<size_t> &counts, const float *x, float *y,
                    lnm_session *timed) {
    const auto t0 = wall_clock::now();
    size_t n_calls = 0;
    if (m->route == LNM_PRODUCTS_RESIDENT) {
        std::vector<const lnh_matrix *> handles;
        std::vector<size_t> toks;
        size_t x_len = 0, y_len = 0;
        for (size_t e = 0; e < parts.size(); e++) {
            if (counts[e] == 0) continue;
            if (ensure_resident(m, parts[e]) != 0) return 1;
            handles.push_back(parts[e].resident);
            toks.push_back(counts[e]);
            x_len += counts[e] * parts[e].n_cols;
            y_len += counts[e] * parts[e].n_rows;
        }
        if (!handles.empty() &&
            lnh_gemm_grouped(m->exec, handles.size(), handles.data(), toks.data(), x, x_len, y, y_len) != 0)
            return fail(std::string(lnh_last_error(m->exec)) + " (" + parts[0].name + ")");
        n_calls = handles.size();
    } else {
        for (size_t e = 0; e < parts.size(); e++) {
            if (counts[e] == 0) continue;
            if (product_routed(m, parts[e], counts[e], x, y) != 0) return 1;
            x += counts[e] * parts[e].n_cols;
            y += counts[e] * parts[e].n_rows;
            n_calls++;
        }
    }
    if (timed) {
        timed->products_s += since(t0);
        timed->n_products += n_calls;
    }
    return 0;
}

__global__ void dd_swiglu_kernel(float *gate, const float *up, uint32_t n);  // with the device session's kernels below

// packed[i] = x[row_of[i]]: the rows of every expert's bucket, contiguous (grouped_one_expert, decode.rs:10062-10116).
__global__ __launch_bounds__(256) void moe_gather_kernel(const float *x, const uint32_t *row_of, uint32_t d, float *packed) {
    const float4 *src = reinterpret_cast<const float4 *>(x + (size_t)row_of[blockIdx.x] * d);
    float4 *dst = reinterpret_cast<float4 *>(packed + (size_t)blockIdx.x * d);
    for (uint32_t i = threadIdx.x; i < d / 4; i += blockDim.x) dst[i] = src[i];
}

// out[t] = the token's expert outputs times their router weights, added in ascending expert order onto zero
// (scatter_expert_rows, decode.rs:10263-10292: ffn_out[t] += y[i] * w over the experts in ascending order).
// pair_of / w_of: per token its k selections in that order (row of y, weight).
__global__ __launch_bounds__(256) void moe_scatter_kernel(const float *y, const uint32_t *pair_of, const float *w_of, uint32_t k,
                                                          uint32_t d, float *out) {
    const uint32_t t = blockIdx.x;  // blockIdx.y: which 1024 columns (four per thread; d is a multiple of 4)
    const uint32_t i = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
    if (i >= d) return;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t j = 0; j < k; j++) {
        const float4 v = *reinterpret_cast<const float4 *>(y + (size_t)pair_of[t * k + j] * d + i);
        const float w = w_of[t * k + j];
        o.x += v.x * w;
        o.y += v.y * w;
        o.z += v.z * w;
        o.w += v.w * w;
    }
    *reinterpret_cast<float4 *>(out + (size_t)t * d + i) = o;
}

// softmax -> topk -> router weights per token, tokens bucketed per expert (route_softmax_tokens 9969-10004,
// grouped_routed_ffn 10006-10060); logits in ms->logits, overwritten by the probabilities.
int moe_route(const lnm_hparams &hp, size_t n, MoeScratch *ms, std::vector<size_t> *counts, size_t *pairs) {
    const size_t ne = hp.n_expert, k = hp.n_expert_used;
    ms->sel_e.resize(n * k);
    ms->sel_w.resize(n * k);
    for (size_t t = 0; t < n; t++) {
        float *row = &ms->logits[t * ne];
        softmax(row, ne);
        if (!topk(row, ne, k, &ms->order)) return fail("expert_used_count");
        std::copy(ms->order.begin(), ms->order.end(), &ms->sel_e[t * k]);
        router_weights(row, ms->order.data(), k, true, &ms->sel_w[t * k]);
    }
    ms->buckets.resize(ne);
    for (auto &b : ms->buckets) b.clear();
    for (size_t t = 0; t < n; t++)
        for (size_t j = 0; j < k; j++) ms->buckets[ms->sel_e[t * k + j]].push_back((uint32_t)t);
    counts->assign(ne, 0);
    *pairs = 0;
    for (size_t e = 0; e < ne; e++) *pairs += (*counts)[e] = ms->buckets[e].size();
    return 0;
}

// token_expert_weight: the first selection of expert e by token t
float moe_weight(const MoeScratch *ms, size_t k, uint32_t t, size_t e) {
    for (size_t j = 0; j < k; j++)
        if (ms->sel_e[(size_t)t * k + j] == e) return ms->sel_w[(size_t)t * k + j];
    return 0.f;
}

// The routed feed-forward with the resident products chained on the device: the rows go up once (pinned staging),
// the router product runs there and only its n x n_expert logits come back for the host's routing; then the
// bucket order goes up (a few KB), the rows are gathered, gate and up are grouped launches, SiLU(gate) * up an
// element-wise kernel, down a grouped launch, the scatter a kernel, and the n x n_embd result comes back: two host
// synchronisations, no expert output ever on the host.  Same products and the same order of additions as moe_ffn's
// host form; SiLU with the device's expf.
int moe_ffn_on_device(lnm_model *m, Layer &l, size_t n, const float *x, float *ffn_out, MoeScratch *ms, lnm_session *timed) {
    const lnm_hparams &hp = m->hp;
    const size_t d = hp.n_embd, ne = hp.n_expert, k = hp.n_expert_used, ff = l.gate_e[0].n_rows;
    const auto t0 = wall_clock::now();
    auto grow = [](float **p, size_t *cap, size_t want, bool pinned) {
        if (*cap >= want) return hipSuccess;
        if (*p) (void)(pinned ? hipHostFree(*p) : hipFree(*p));
        *p = nullptr;
        *cap = 0;
        const hipError_t e = pinned ? hipHostMalloc(reinterpret_cast<void **>(p), want * sizeof(float), hipHostMallocDefault)
                                    : hipMalloc(reinterpret_cast<void **>(p), want * sizeof(float));
        if (e == hipSuccess) *cap = want;
        return e;
    };
    auto hip_fail = [](hipError_t e) { return fail(std::string("routed feed-forward: ") + hipGetErrorString(e)); };
    const size_t pairs = n * k, n_idx = pairs + n * k;  // every token selects k distinct experts
    if (pairs * ff > UINT32_MAX || n * d > UINT32_MAX) return fail("routed feed-forward: too many rows for one call");
    hipError_t e = ms->stream ? hipSuccess : hipStreamCreateWithFlags(&ms->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = grow(&ms->h_io, &ms->cap_hio, n * d, true);
    if (e == hipSuccess) e = grow(&ms->h_small, &ms->cap_hsmall, n * ne + n_idx + n * k, true);
    if (e == hipSuccess) e = grow(&ms->d_io, &ms->cap_io, n * d, false);
    if (e == hipSuccess) e = grow(&ms->d_small, &ms->cap_small, n * ne + n_idx + n * k, false);
    if (e == hipSuccess) e = grow(&ms->d_x, &ms->cap_x, pairs * d, false);
    if (e == hipSuccess) e = grow(&ms->d_g, &ms->cap_g, pairs * ff, false);
    if (e == hipSuccess) e = grow(&ms->d_u, &ms->cap_u, pairs * ff, false);
    if (e == hipSuccess) e = grow(&ms->d_y, &ms->cap_y, pairs * d, false);
    if (e != hipSuccess) return hip_fail(e);
    float *h_logits = ms->h_small, *d_logits = ms->d_small;
    uint32_t *h_idx = reinterpret_cast<uint32_t *>(ms->h_small + n * ne), *d_idx = reinterpret_cast<uint32_t *>(ms->d_small + n * ne);
    float *h_w = ms->h_small + n * ne + n_idx, *d_w = ms->d_small + n * ne + n_idx;

    // From the first enqueue on, every return that is not the normal one leaves work on the stream that still
    // reads the pinned and device buffers: it waits for the stream before it hands them back to the next call
    // (which copies into them and may free them to grow).
    struct DrainOnError {
        hipStream_t s;
        bool armed;
        ~DrainOnError() {
            if (armed) (void)hipStreamSynchronize(s);
        }
    } drain{ms->stream, true};
    // rows up, router product, logits back
    std::memcpy(ms->h_io, x, n * d * sizeof(float));
    e = hipMemcpyAsync(ms->d_io, ms->h_io, n * d * sizeof(float), hipMemcpyHostToDevice, ms->stream);
    if (e != hipSuccess) return hip_fail(e);
    if (ensure_resident(m, l.gate_inp) != 0) return 1;
    if (lnh_gemm_device(m->exec, l.gate_inp.resident, n, ms->d_io, d_logits, ms->stream) != 0)
        return fail(std::string(lnh_last_error(m->exec)) + " (" + l.gate_inp.name + ")");
    e = hipMemcpyAsync(h_logits, d_logits, n * ne * sizeof(float), hipMemcpyDeviceToHost, ms->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ms->stream);
    if (e != hipSuccess) return hip_fail(e);
    ms->logits.assign(h_logits, h_logits + n * ne);
    std::vector<size_t> counts;
    size_t routed = 0;
    if (moe_route(hp, n, ms, &counts, &routed)) return 1;
    if (routed != pairs) return fail("routed feed-forward: the buckets do not hold k selections per token");

    // bucket order: the row of every packed position; per token its selections in ascending expert order
    std::vector<uint32_t> filled(n, 0);
    size_t at = 0;
    for (size_t ex = 0; ex < ne; ex++) {
        uint32_t before = UINT32_MAX;  // tokens ascend inside a bucket: a token twice in one would be adjacent
        for (uint32_t t : ms->buckets[ex]) {
            if (t == before || t >= n || filled[t] >= k) return fail("routed feed-forward: a token selected an expert twice");
            before = t;
            h_idx[at] = t;
            const size_t slot = (size_t)t * k + filled[t]++;
            h_idx[pairs + slot] = (uint32_t)at;
            h_w[slot] = moe_weight(ms, k, t, ex);
            at++;
        }
    }
    e = hipMemcpyAsync(d_idx, h_idx, (n_idx + n * k) * sizeof(float), hipMemcpyHostToDevice, ms->stream);  // indices and weights are adjacent
    if (e != hipSuccess) return hip_fail(e);
    std::vector<const lnh_matrix *> hg, hu, hdn;
    std::vector<size_t> toks;
    for (size_t ex = 0; ex < ne; ex++) {
        if (counts[ex] == 0) continue;
        if (ensure_resident(m, l.gate_e[ex]) != 0 || ensure_resident(m, l.up_e[ex]) != 0 || ensure_resident(m, l.down_e[ex]) != 0)
            return 1;
        hg.push_back(l.gate_e[ex].resident);
        hu.push_back(l.up_e[ex].resident);
        hdn.push_back(l.down_e[ex].resident);
        toks.push_back(counts[ex]);
    }
    hipLaunchKernelGGL(moe_gather_kernel, dim3((uint32_t)pairs), dim3(256), 0, ms->stream, ms->d_io, d_idx, (uint32_t)d, ms->d_x);
    if ((e = hipGetLastError()) != hipSuccess) return hip_fail(e);
    {
        // gate and up of every expert as one batch: the experts of at most 16 rows first, then the others, so that
        // products of one tile size lie together and share launches (up to eight each) - with eight products a
        // launch has enough tiles to fill the chip without sharing columns, and no launch sums shares
        std::vector<const lnh_matrix *> mats;
        std::vector<size_t> rows;
        std::vector<const float *> xs;
        std::vector<float *> ys;
        for (int big = 0; big < 2; big++) {
            size_t at_x = 0, at_h = 0;
            for (size_t i = 0; i < toks.size(); i++) {
                if ((toks[i] > 16) == (big == 1))
                    for (int up = 0; up < 2; up++) {
                        mats.push_back(up ? hu[i] : hg[i]);
                        rows.push_back(toks[i]);
                        xs.push_back(ms->d_x + at_x);
                        ys.push_back((up ? ms->d_u : ms->d_g) + at_h);
                    }
                at_x += toks[i] * d;
                at_h += toks[i] * ff;
            }
        }
        if (lnh_gemm_batch_device(m->exec, mats.size(), mats.data(), rows.data(), xs.data(), ys.data(), ms->stream) != 0)
            return fail(std::string(lnh_last_error(m->exec)) + " (" + l.gate_e[0].name + ")");
    }
    const uint32_t n_h = (uint32_t)(pairs * ff);
    hipLaunchKernelGGL(dd_swiglu_kernel, dim3((n_h + 1023) / 1024 < 4096 ? (n_h + 1023) / 1024 : 4096), dim3(256), 0, ms->stream,
                       ms->d_g, ms->d_u, n_h);
    if ((e = hipGetLastError()) != hipSuccess) return hip_fail(e);
    if (lnh_gemm_grouped_device(m->exec, hdn.size(), hdn.data(), toks.data(), ms->d_g, ms->d_y, ms->stream) != 0)
        return fail(std::string(lnh_last_error(m->exec)) + " (" + l.down_e[0].name + ")");
    hipLaunchKernelGGL(moe_scatter_kernel, dim3((uint32_t)n, (uint32_t)((d + 1023) / 1024)), dim3(256), 0, ms->stream, ms->d_y,
                       d_idx + pairs, d_w, (uint32_t)k, (uint32_t)d, ms->d_io);
    if ((e = hipGetLastError()) != hipSuccess) return hip_fail(e);
    e = hipMemcpyAsync(ms->h_io, ms->d_io, n * d * sizeof(float), hipMemcpyDeviceToHost, ms->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ms->stream);
    if (e != hipSuccess) return hip_fail(e);
    drain.armed = false;  // the stream is idle
    std::memcpy(ffn_out, ms->h_io, n * d * sizeof(float));
    if (timed) {
        timed->products_s += since(t0);
        timed->n_products += 1 + 3 * toks.size();
    }
    return 0;
}

// The routed feed-forward of architecture llama with experts (Mixtral-shaped), langtax/src/decode.rs:10366-10409
// (llama_moe_into: softmax over all experts, then top-k, weights renormalised with the 2^-14 clamp and applied
// after the expert, SwiGLU, no shared expert), through softmax_routed_layer 9938-9966:
//   route_softmax_tokens 9969-10004   router product, per token softmax -> topk -> router weights
//   grouped_routed_ffn 10006-10060    token indices bucketed per expert, experts in ascending order
//   grouped_one_expert 10062-10116    the bucket's rows packed contiguously
//   swiglu_expert_gemm 10148-10261    gate and up products, SiLU(gate) * up, down product
//   scatter_expert_rows 10263-10292   ffn_out[t] += y[i] * w(t, e)
// x: n x n_embd rows (already normed), ffn_out: n x n_embd, overwritten.
// Resident route: moe_ffn_on_device, unless LLAMA_HIP_MOE_HOST_SWIGLU is set (then, as in the reference's seam, every
// product is a call through host buffers and SiLU * up and the scatter run here).
int moe_ffn(lnm_model *m, Layer &l, size_t n, const float *x, float *ffn_out, MoeScratch *ms, lnm_session *timed) {
    const lnm_hparams &hp = m->hp;
    const size_t d = hp.n_embd, ne = hp.n_expert, k = hp.n_expert_used, ff = l.gate_e[0].n_rows;
    // (rows of whole float4: the gather and scatter kernels move them that way; the variable is read per call, tests switch it)
    if (m->route == LNM_PRODUCTS_RESIDENT && d % 4 == 0 && std::getenv("LLAMA_HIP_MOE_HOST_SWIGLU") == nullptr)
        return moe_ffn_on_device(m, l, n, x, ffn_out, ms, timed);
    ms->logits.resize(n * ne);
    {
        const auto t0 = wall_clock::now();
        if (product_routed(m, l.gate_inp, n, x, ms->logits.data()) != 0) return 1;
        if (timed) {
            timed->products_s += since(t0);
            timed->n_products++;
        }
    }
    std::vector<size_t> counts;
    size_t pairs = 0;
    if (moe_route(hp, n, ms, &counts, &pairs)) return 1;
    // every expert's rows, expert after expert in ascending order
    ms->pack_x.resize(pairs * d);
    ms->g.resize(pairs * ff);
    ms->u.resize(pairs * ff);
    ms->y.resize(pairs * d);
    size_t at = 0;
    for (size_t e = 0; e < ne; e++)
        for (uint32_t t : ms->buckets[e]) std::memcpy(&ms->pack_x[at++ * d], x + (size_t)t * d, d * sizeof(float));
    if (expert_products(m, l.gate_e, counts, ms->pack_x.data(), ms->g.data(), timed)) return 1;
    if (expert_products(m, l.up_e, counts, ms->pack_x.data(), ms->u.data(), timed)) return 1;
    for (size_t i = 0; i < pairs * ff; i++) {  // silu_inplace then the element-wise product, decode.rs:10244-10248
        const float g = ms->g[i];
        ms->g[i] = g / (1.f + std::exp(-g));
        ms->g[i] *= ms->u[i];
    }
    if (expert_products(m, l.down_e, counts, ms->g.data(), ms->y.data(), timed)) return 1;
    std::fill(ffn_out, ffn_out + n * d, 0.f);  // fit() zero-fills (decode.rs:1816-1819, 10381)
    at = 0;
    for (size_t e = 0; e < ne; e++) {
        for (uint32_t t : ms->buckets[e]) {
            const float w = moe_weight(ms, k, t, e);
            const float *src = &ms->y[at++ * d];
            float *dst = ffn_out + (size_t)t * d;
            const float scale = 1.f;  // no ffn_down_exps.scale tensor on this architecture (expert_part_scale)
            for (size_t i = 0; i < d; i++) dst[i] += src[i] * w * scale;
        }
    }
    return 0;
}

// langtax/src/decode.rs:2710-3099, llama branch (dense or routed feed-forward), LogitsKind::Last.
int forward(lnm_session *s, const uint32_t *tokens, size_t n, float *logits) {
    lnm_model *m = s->model;
    const lnm_hparams &hp = m->hp;
    if (n == 0) return fail("empty batch");
    const size_t d = hp.n_embd, hd = hp.head_dim, qw = (size_t)hp.n_head * hd, kvw = (size_t)hp.n_head_kv * hd;
    const size_t gqa = hp.n_head / hp.n_head_kv;
    if (ensure_blocks(s, s->past + n) != 0) return 1;
    if (!s->pool) {
        const unsigned hw = std::thread::hardware_concurrency();
        const size_t threads = hw < 2 ? 1 : (hw > 16 ? 16 : hw);
        s->pool.reset(new HeadPool(threads - 1));
    }
    s->x.resize(n * d);
    const size_t emb_row = m->token_embd.nbytes / m->token_embd.n_rows;
    for (size_t t = 0; t < n; t++) {
        if (tokens[t] >= hp.n_vocab) return fail("token id out of range");
        if (!dequant_row(m->token_embd.type, d, m->token_embd.bytes + (size_t)tokens[t] * emb_row, &s->x[t * d]))
            return fail("cannot dequantize token_embd.weight");
    }
    s->qkv.resize(n * (qw + 2 * kvw));
    s->gate_up.resize(2 * n * hp.n_ff);
    float *const q = s->qkv.data(), *const k = q + n * qw, *const v = k + n * kvw;
    float *const gate = s->gate_up.data(), *const up = gate + n * hp.n_ff;
    s->attn.resize(n * qw);
    s->attn_proj.resize(n * d);
    s->ffn_out.resize(n * d);
    const float hd_f = hd <= 65535 ? (float)hd : 1.f;
    const float root = std::sqrt(hd_f);
    const float score_scale = root > 0.f ? 1.f / root : 0.f;

    for (size_t li = 0; li < hp.n_layer; li++) {
        Layer &l = m->layers[li];
        s->residual = s->x;
        for (size_t t = 0; t < n; t++) rmsnorm(&s->x[t * d], l.attn_norm.data(), d, hp.rms_eps);
        if (products_shared(s, {&l.wq, &l.wk, &l.wv}, n, s->x.data(), q)) return 1;
        const auto t_att = wall_clock::now();
        for (size_t t = 0; t < n; t++) {  // rotate and store K, store V
            const size_t p = s->past + t;
            float *kt = k + t * kvw;
            for (size_t h = 0; h < hp.n_head_kv; h++) {
                rope(kt + h * hd, hd, p, hp.n_rot, hp.rope_base);
                std::memcpy(&s->cache_k[kv_offset(s, li, h, p)], kt + h * hd, hd * sizeof(float));
                std::memcpy(&s->cache_v[kv_offset(s, li, h, p)], v + t * kvw + h * hd, hd * sizeof(float));
            }
        }
        // decode.rs:11126-11197, one (token, query head) pair per work item
        const std::function<void(size_t)> attend = [&](size_t item) {
            static thread_local std::vector<float> scores;
            const size_t t = item / hp.n_head, hq = item % hp.n_head;
            const size_t p = s->past + t, seq = p + 1;
            scores.resize(seq);
            float *qv = q + t * qw + hq * hd;
            rope(qv, hd, p, hp.n_rot, hp.rope_base);
            const size_t hkv = hq / gqa;
            for (size_t u = 0; u < seq; u++) {
                const float *kv = &s->cache_k[kv_offset(s, li, hkv, u)];
                float dot = 0.f;
                for (size_t i = 0; i < hd; i++) dot += qv[i] * kv[i];
                scores[u] = dot * score_scale;
            }
            softmax(scores.data(), seq);
            float *dst = &s->attn[t * qw + hq * hd];
            for (size_t i = 0; i < hd; i++) dst[i] = 0.f;
            for (size_t u = 0; u < seq; u++) {
                const float *vv = &s->cache_v[kv_offset(s, li, hkv, u)];
                const float st = scores[u];
                for (size_t i = 0; i < hd; i++) dst[i] += st * vv[i];
            }
        };
        s->pool->run(n * hp.n_head, attend);
        s->attention_s += since(t_att);
        if (product(s, l.wo, n, s->attn.data(), s->attn_proj.data())) return 1;
        for (size_t i = 0; i < n * d; i++) s->x[i] = s->attn_proj[i] + s->residual[i];
        s->residual = s->x;
        for (size_t t = 0; t < n; t++) rmsnorm(&s->x[t * d], l.ffn_norm.data(), d, hp.rms_eps);
        if (l.moe) {
            if (moe_ffn(m, l, n, s->x.data(), s->ffn_out.data(), &s->moe, s)) return 1;
        } else {
            if (products_shared(s, {&l.gate, &l.up}, n, s->x.data(), gate)) return 1;
            for (size_t i = 0; i < n * hp.n_ff; i++) {  // SiLU(gate) * up, decode.rs:11826-11830 and 2981-2984
                const float g = gate[i];
                gate[i] = g / (1.f + std::exp(-g));
                gate[i] *= up[i];
            }
            if (product(s, l.down, n, gate, s->ffn_out.data())) return 1;
        }
        for (size_t i = 0; i < n * d; i++) s->x[i] = s->ffn_out[i] + s->residual[i];
    }
    s->xn.assign(s->x.begin() + (n - 1) * d, s->x.begin() + n * d);
    rmsnorm(s->xn.data(), m->output_norm.data(), d, hp.rms_eps);
    if (product(s, m->output, 1, s->xn.data(), logits)) return 1;
    s->past += n;
    return 0;
}

// ------------------------------------------------------------------ synthetic model

uint64_t splitmix(uint64_t &st) {  // langtax/src/sample.rs SplitMix64
    st += 0x9e3779b97f4a7c15ull;
    uint64_t z = st;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
struct Rng {
    uint64_t st;
    uint64_t next() { return splitmix(st); }
    float uniform() { return (float)(next() >> 40) * (1.0f / 16777216.0f); }  // top 24 bits -> [0, 1)
    float normal() {
        const float u1 = 1.0f - uniform(), u2 = uniform();
        return std::sqrt(-2.0f * std::log(u1)) * std::cos(6.28318530717958647692f * u2);
    }
};

uint16_t f32_to_f16(float f) {  // round to nearest even; enough for scales this generator draws
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const int32_t e = (int32_t)((x >> 23) & 255u) - 127 + 15;
    uint32_t man = x & 0x7fffffu;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        const int shift = 14 - e;
        uint32_t h = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}
void wr16(uint8_t *p, uint16_t v) {
    p[0] = (uint8_t)v;
    p[1] = (uint8_t)(v >> 8);
}

// Random packed rows whose dequantized values have mean 0 and standard deviation sigma.
void random_rows(uint32_t type, size_t n_cols, size_t n_rows, float sigma, uint64_t seed, uint8_t *dst) {
    size_t bb = 0, bk = 0;
    nh::gguf::type_layout(type, &bb, &bk);
    const size_t row_bytes = n_cols / bk * bb, chunk = 64;  // rows per independent random stream
    const size_t n_chunks = (n_rows + chunk - 1) / chunk;
    unsigned hw = std::thread::hardware_concurrency();
    const size_t n_threads = hw < 1 ? 1 : (hw > 16 ? 16 : hw);
    auto work = [&](size_t tid) {
        for (size_t c = tid; c < n_chunks; c += n_threads) {
            Rng r{seed ^ (0x51ed270b0a1f3c5dull * (c + 1))};
            const size_t r0 = c * chunk, r1 = r0 + chunk < n_rows ? r0 + chunk : n_rows;
            for (uint8_t *w = dst + r0 * row_bytes; w < dst + r1 * row_bytes; w += bb) {
                switch (type) {
                case 0: {
                    const float v = sigma * r.normal();
                    std::memcpy(w, &v, 4);
                    break;
                }
                case 1: wr16(w, f32_to_f16(sigma * r.normal())); break;
                case 8:  // codes uniform in [-127, 127]: rms 73.3
                    wr16(w, f32_to_f16(std::fabs(r.normal()) * sigma / 73.3f));
                    for (int j = 0; j < 32; j++) w[2 + j] = (uint8_t)(int8_t)((int)(r.next() % 255u) - 127);
                    break;
                case 2:  // nibble - 8: rms 4.64
                    wr16(w, f32_to_f16(r.normal() * sigma / 4.64f));
                    for (int j = 0; j < 16; j += 8) {
                        const uint64_t v = r.next();
                        std::memcpy(w + 2 + j, &v, 8);
                    }
                    break;
                case 6:  // code - 16: rms 9.25
                    wr16(w, f32_to_f16(r.normal() * sigma / 9.25f));
                    for (int j = 0; j < 20; j += 4) {
                        const uint32_t v = (uint32_t)r.next();
                        std::memcpy(w + 2 + j, &v, 4);
                    }
                    break;
                case 7: {  // code * d + m with m = -15.5 d: standard deviation 9.23 |d|
                    const float d = r.normal() * sigma / 9.23f;
                    wr16(w, f32_to_f16(d));
                    wr16(w + 2, f32_to_f16(-15.5f * d));
                    for (int j = 0; j < 20; j += 4) {
                        const uint32_t v = (uint32_t)r.next();
                        std::memcpy(w + 4 + j, &v, 4);
                    }
                    break;
                }
                case 12: {  // d sc q - dmin m, all codes uniform: mean 0 for dmin = 7.5 d, deviation 258 d
                    const float d = std::fabs(r.normal()) * sigma / 258.f;
                    wr16(w, f32_to_f16(d));
                    wr16(w + 2, f32_to_f16(7.5f * d));
                    for (int j = 0; j < 140; j += 4) {
                        const uint32_t v = (uint32_t)r.next();
                        std::memcpy(w + 4 + j, &v, 4);
                    }
                    break;
                }
                default: {  // Q6_K: d sc (q - 32), sc uniform in [-32, 31]: deviation 341 d
                    for (int j = 0; j < 192; j += 8) {
                        const uint64_t v = r.next();
                        std::memcpy(w + j, &v, 8);
                    }
                    for (int j = 0; j < 16; j++) w[192 + j] = (uint8_t)(int8_t)((int)(r.next() & 63u) - 32);
                    wr16(w + 208, f32_to_f16(std::fabs(r.normal()) * sigma / 341.f));
                    break;
                }
                }
            }
        }
    };
    std::vector<std::thread> pool;
    for (size_t t = 1; t < n_threads; t++) pool.emplace_back(work, t);
    work(0);
    for (auto &t : pool) t.join();
}

}  // namespace

#include "llama_device.inc"

// ------------------------------------------------------------------ C ABI

extern "C" {

const char *lnm_last_error(void) { return t_err.c_str(); }

int lnm_load_bytes(const uint8_t *bytes, size_t len, lnm_model **out) {
    if (!bytes || !out) return fail("null argument");
    std::unique_ptr<lnm_model> m(new lnm_model);
    try {
        m->owned.assign(bytes, bytes + len);
        std::string err;
        if (!nh::gguf::parse(m->owned.data(), m->owned.size(), &m->file, &err)) return fail("gguf: " + err);
        if (finish_load(m.get()) != 0) return 1;
    } catch (const std::exception &e) {  // allocation failure on a hostile file must not cross the C boundary
        return fail(std::string("gguf: ") + e.what());
    }
    *out = m.release();
    return 0;
}

int lnm_load(const char *path, lnm_model **out) {
    if (!path || !out) return fail("null argument");
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return fail(std::string("cannot open ") + path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        close(fd);
        return fail(std::string("cannot stat ") + path);
    }
    void *p = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (p == MAP_FAILED) return fail(std::string("cannot map ") + path);
    std::unique_ptr<lnm_model> m(new lnm_model);
    m->map = p;
    m->map_len = (size_t)st.st_size;
    try {
        std::string err;
        if (!nh::gguf::parse(static_cast<const uint8_t *>(p), m->map_len, &m->file, &err)) return fail("gguf: " + err);
        if (finish_load(m.get()) != 0) return 1;
    } catch (const std::exception &e) {
        return fail(std::string("gguf: ") + e.what());
    }
    *out = m.release();
    return 0;
}

void lnm_free(lnm_model *model) { delete model; }

int lnm_info(const lnm_model *model, lnm_hparams *out) {
    if (!model || !out) return fail("null argument");
    *out = model->hp;
    return 0;
}

int lnm_set_products(lnm_model *model, int route, lnm_matmul_fn fn, void *user) {
    if (!model) return fail("null argument");
    if (route < LNM_PRODUCTS_RESIDENT || route > LNM_PRODUCTS_CALLBACK) return fail("unknown product route");
    if (route == LNM_PRODUCTS_CALLBACK && !fn) return fail("callback route without a function");
    model->route = route;
    model->fn = fn;
    model->user = user;
    return 0;
}

int lnm_session_new(lnm_model *model, size_t kv_block, const uint32_t *block_ids, size_t n_block_ids,
                    lnm_session **out) {
    if (!model || !out) return fail("null argument");
    if (kv_block == 0) return fail("zero K/V block size");
    std::unique_ptr<lnm_session> s(new lnm_session);
    s->model = model;
    s->kv_block = kv_block;
    if (block_ids) {
        std::vector<bool> seen(n_block_ids, false);
        for (size_t i = 0; i < n_block_ids; i++) {
            if (block_ids[i] >= n_block_ids || seen[block_ids[i]]) return fail("block ids are not a permutation");
            seen[block_ids[i]] = true;
        }
        s->preset.assign(block_ids, block_ids + n_block_ids);
    }
    *out = s.release();
    return 0;
}

int lnm_session_new_device(lnm_model *model, size_t kv_block, const uint32_t *block_ids, size_t n_block_ids,
                           size_t max_positions, lnm_session **out) {
    lnm_session *s = nullptr;
    if (lnm_session_new(model, kv_block, block_ids, n_block_ids, &s) != 0) return 1;
    if (device_decode_create(s, max_positions) != 0) {
        delete s;
        *out = nullptr;
        return 1;
    }
    *out = s;
    return 0;
}

int lnm_session_new_device_batch(lnm_model *model, size_t kv_block, size_t n_sequences, size_t max_positions,
                                 lnm_session **out) {
    lnm_session *s = nullptr;
    if (lnm_session_new(model, kv_block, nullptr, 0, &s) != 0) return 1;
    if (device_batch_create(s, n_sequences, max_positions) != 0) {
        delete s;
        *out = nullptr;
        return 1;
    }
    *out = s;
    return 0;
}

int lnm_batch_generate_greedy(lnm_session *session, const uint32_t *prompts, const size_t *prompt_lens, size_t n_new,
                              uint32_t *out, double *prefill_seconds, double *decode_seconds) {
    if (!session || !prompts || !prompt_lens || !out) return fail("null argument");
    if (!session->dev || session->dev->n_seq == 0) return fail("not a batch session");
    return device_batch_generate(session, prompts, prompt_lens, n_new, out, prefill_seconds, decode_seconds);
}

void lnm_session_free(lnm_session *session) { delete session; }

int lnm_forward(lnm_session *session, const uint32_t *tokens, size_t n, float *logits) {
    if (!session || !tokens || !logits) return fail("null argument");
    if (session->dev && session->dev->n_seq) return fail("a batch session takes lnm_batch_generate_greedy");
    const int rc = session->dev ? device_forward(session, tokens, n, logits) : forward(session, tokens, n, logits);
    if (rc == 0) session->ids.insert(session->ids.end(), tokens, tokens + n);
    return rc;
}

// langtax/src/decode.rs:1106-1196 (reuse_prefix, rewind, prompt_suffix) and 3931-3962 (prompt_logits).
int lnm_prompt(lnm_session *session, const uint32_t *tokens, size_t n, float *logits, size_t *prefix_hit) {
    if (!session || !tokens || !logits) return fail("null argument");
    if (n == 0) return fail("prefill tokens");
    if (session->dev && session->dev->n_seq) return fail("a batch session takes lnm_batch_generate_greedy");
    size_t lcp = 0;
    if (session->ids.size() == session->past)  // ids that do not cover the cache are no basis for reuse
        while (lcp < session->ids.size() && lcp < n && session->ids[lcp] == tokens[lcp]) lcp++;
    if (prefix_hit) *prefix_hit = lcp;
    if (lcp == n) lcp = n - 1;  // a full hit recomputes the last token: the logits returned are that token's
    // positions 0 .. lcp-1 stay as they are; everything after them is written again as the sequence grows
    session->past = lcp;
    session->ids.resize(lcp);
    return lnm_forward(session, tokens + lcp, n - lcp, logits);
}

int lnm_generate_greedy(lnm_session *session, const uint32_t *prompt, size_t n_prompt, size_t n_new,
                        uint32_t *out, double *prefill_seconds, double *decode_seconds) {
    if (!session || !prompt || !out) return fail("null argument");
    if (n_prompt == 0 || n_new == 0) return fail("empty prompt or nothing to generate");
    if (session->dev && session->dev->n_seq) return fail("a batch session takes lnm_batch_generate_greedy");
    struct Remember {  // on success the cache holds the prompt and every picked token but the last
        lnm_session *s; const uint32_t *prompt; size_t n_prompt, n_new; const uint32_t *out; size_t past0; bool ok = false;
        ~Remember() {
            if (!ok || s->past != past0 + n_prompt + n_new - 1) {
                s->ids.clear();
                return;
            }
            s->ids.insert(s->ids.end(), prompt, prompt + n_prompt);
            s->ids.insert(s->ids.end(), out, out + n_new - 1);
        }
    } remember{session, prompt, n_prompt, n_new, out, session->past};
    if (session->dev) {
        const int rc = device_generate(session, prompt, n_prompt, n_new, out, prefill_seconds, decode_seconds);
        remember.ok = rc == 0;
        return rc;
    }
    std::vector<float> logits(session->model->hp.n_vocab);
    using clock = std::chrono::steady_clock;
    const auto t0 = clock::now();
    if (forward(session, prompt, n_prompt, logits.data()) != 0) return 1;
    out[0] = argmax(logits.data(), logits.size());
    const auto t1 = clock::now();
    for (size_t i = 1; i < n_new; i++) {
        if (forward(session, &out[i - 1], 1, logits.data()) != 0) return 1;
        out[i] = argmax(logits.data(), logits.size());
    }
    const auto t2 = clock::now();
    if (prefill_seconds) *prefill_seconds = std::chrono::duration<double>(t1 - t0).count();
    if (decode_seconds) *decode_seconds = std::chrono::duration<double>(t2 - t1).count();
    remember.ok = true;
    return 0;
}

int lnm_session_timing(const lnm_session *session, double *products_seconds, double *attention_seconds,
                       uint64_t *n_products) {
    if (!session) return fail("null argument");
    if (products_seconds) *products_seconds = session->products_s;
    if (attention_seconds) *attention_seconds = session->attention_s;
    if (n_products) *n_products = session->n_products;
    return 0;
}

int lnm_dequant_row(uint32_t ggml_type, size_t n_cols, const uint8_t *row, size_t row_len, float *y) {
    size_t bb = 0, bk = 0;
    if (!row || !y) return fail("null argument");
    if (!nh::gguf::type_layout(ggml_type, &bb, &bk)) return fail("unsupported ggml type " + std::to_string(ggml_type));
    if (n_cols % bk != 0 || row_len != n_cols / bk * bb) return fail("row length does not match the column count");
    return dequant_row(ggml_type, n_cols, row, y) ? 0 : fail("cannot dequantize");
}

int lnm_rmsnorm(float *x, const float *w, size_t n, float eps) {
    if (!x || !w) return fail("null argument");
    rmsnorm(x, w, n, eps);
    return 0;
}

int lnm_rope(float *head, size_t head_len, size_t pos, size_t n_rot, float base) {
    if (!head) return fail("null argument");
    rope(head, head_len, pos, n_rot, base);
    return 0;
}

void lnm_softmax(float *x, size_t n) {
    if (x) softmax(x, n);
}

uint32_t lnm_argmax(const float *x, size_t n) { return x ? argmax(x, n) : 0; }

int lnm_topk(const float *values, size_t n, size_t k, uint32_t *order) {
    if (!values || !order) return fail("null argument");
    std::vector<uint32_t> o;
    if (!topk(values, n, k, &o)) return fail("expert_used_count");
    std::copy(o.begin(), o.end(), order);
    return 0;
}

int lnm_router_weights(const float *probs, const uint32_t *order, size_t k, int norm_w, float *weights) {
    if (!probs || !order || !weights) return fail("null argument");
    router_weights(probs, order, k, norm_w != 0, weights);
    return 0;
}

int lnm_moe_ffn(lnm_model *model, size_t layer, size_t n_tokens, const float *x, float *ffn_out) {
    if (!model || !x || !ffn_out) return fail("null argument");
    if (layer >= model->layers.size() || !model->layers[layer].moe) return fail("layer has no routed feed-forward");
    if (n_tokens == 0) return fail("empty batch");
    try {
        if (!model->moe_entry) model->moe_entry = std::make_unique<MoeScratch>();  // kept: its device buffers are grow-only
        return moe_ffn(model, model->layers[layer], n_tokens, x, ffn_out, model->moe_entry.get(), nullptr);
    } catch (const std::exception &e) {
        return fail(std::string("routed feed-forward: ") + e.what());
    }
}

int lnm_write_synthetic_llama(const char *path, const lnm_synth_spec *sp) {
    if (!path || !sp) return fail("null argument");
    if (!sp->n_layer || !sp->n_embd || !sp->n_head || !sp->n_head_kv || !sp->n_ff || !sp->n_vocab)
        return fail("zero hyper-parameter");
    if (sp->n_head % sp->n_head_kv != 0 || sp->n_embd % sp->n_head != 0) return fail("head counts do not divide");
    size_t bb, bk;
    for (uint32_t t : {sp->block_type, sp->embd_type, sp->output_type}) {
        if (!nh::gguf::type_layout(t, &bb, &bk)) return fail("unsupported ggml type " + std::to_string(t));
        if (sp->n_embd % bk != 0 || sp->n_ff % bk != 0) return fail("row lengths are not whole blocks");
    }
    using nh::gguf::Kv;
    const size_t d = sp->n_embd, hd = d / sp->n_head, qw = (size_t)sp->n_head * hd, kvw = (size_t)sp->n_head_kv * hd;
    std::vector<std::pair<std::string, Kv>> kv = {
        {"general.alignment", Kv::u32(32)},
        {"general.name", Kv::str("native-hip synthetic llama")},
        {"general.architecture", Kv::str("llama")},
        {"llama.block_count", Kv::u32(sp->n_layer)},
        {"llama.context_length", Kv::u32(8192)},
        {"llama.embedding_length", Kv::u32(sp->n_embd)},
        {"llama.feed_forward_length", Kv::u32(sp->n_ff)},
        {"llama.attention.head_count", Kv::u32(sp->n_head)},
        {"llama.attention.head_count_kv", Kv::u32(sp->n_head_kv)},
        {"llama.rope.dimension_count", Kv::u32((uint32_t)hd)},
        {"llama.rope.freq_base", Kv::f32(sp->rope_base)},
        {"llama.attention.layer_norm_rms_epsilon", Kv::f32(sp->rms_eps)},
        {"llama.vocab_size", Kv::u32(sp->n_vocab)},
    };
    if (sp->n_expert) {
        if (sp->n_expert_used == 0 || sp->n_expert_used > sp->n_expert) return fail("bad expert_used_count");
        kv.push_back({"llama.expert_count", Kv::u32(sp->n_expert)});
        kv.push_back({"llama.expert_used_count", Kv::u32(sp->n_expert_used)});
    }
    std::vector<nh::gguf::TensorWrite> tensors;
    uint64_t serial = 0;
    const uint64_t seed = sp->seed;
    const float sigma = sp->weight_std;
    // n_parts > 1: a 3-D tensor [n_cols, n_rows, n_parts], part after part; sd: deviation of the weights
    auto mat = [&](const std::string &name, uint32_t type, size_t n_rows, size_t n_cols, size_t n_parts = 1, float sd = -1.f) {
        nh::gguf::TensorWrite t;
        t.name = name;
        t.type = type;
        t.shape = {n_cols, n_rows};
        if (n_parts > 1) t.shape.push_back(n_parts);
        size_t b = 0, k = 0;
        nh::gguf::type_layout(type, &b, &k);
        const size_t all_rows = n_rows * n_parts;
        t.nbytes = all_rows * (n_cols / k * b);
        uint64_t st = seed + 0x9e3779b97f4a7c15ull * ++serial;
        const uint64_t tensor_seed = splitmix(st);
        const float dev = sd < 0.f ? sigma : sd;
        t.fill = [=](uint8_t *dst) { random_rows(type, n_cols, all_rows, dev, tensor_seed, dst); };
        tensors.push_back(std::move(t));
    };
    auto norm = [&](const std::string &name) {
        nh::gguf::TensorWrite t;
        t.name = name;
        t.type = 0;
        t.shape = {d};
        t.nbytes = 4 * d;
        uint64_t st = seed + 0x9e3779b97f4a7c15ull * ++serial;
        const uint64_t tensor_seed = splitmix(st);
        t.fill = [=](uint8_t *dst) {
            Rng r{tensor_seed};
            for (size_t i = 0; i < d; i++) {
                const float v = 1.0f + 0.05f * r.normal();
                std::memcpy(dst + 4 * i, &v, 4);
            }
        };
        tensors.push_back(std::move(t));
    };
    mat("token_embd.weight", sp->embd_type, sp->n_vocab, d);
    for (uint32_t i = 0; i < sp->n_layer; i++) {
        const std::string p = "blk." + std::to_string(i) + ".";
        norm(p + "attn_norm.weight");
        mat(p + "attn_q.weight", sp->block_type, qw, d);
        mat(p + "attn_k.weight", sp->block_type, kvw, d);
        mat(p + "attn_v.weight", sp->block_type, kvw, d);
        mat(p + "attn_output.weight", sp->block_type, d, qw);
        norm(p + "ffn_norm.weight");
        if (sp->n_expert) {
            // router rows of deviation 1 / sqrt(n_embd): logits of about unit deviation on normed activations
            mat(p + "ffn_gate_inp.weight", 0, sp->n_expert, d, 1, 1.0f / std::sqrt((float)d));
            mat(p + "ffn_gate_exps.weight", sp->block_type, sp->n_ff, d, sp->n_expert);
            mat(p + "ffn_up_exps.weight", sp->block_type, sp->n_ff, d, sp->n_expert);
            mat(p + "ffn_down_exps.weight", sp->block_type, d, sp->n_ff, sp->n_expert);
        } else {
            mat(p + "ffn_gate.weight", sp->block_type, sp->n_ff, d);
            mat(p + "ffn_up.weight", sp->block_type, sp->n_ff, d);
            mat(p + "ffn_down.weight", sp->block_type, d, sp->n_ff);
        }
    }
    norm("output_norm.weight");
    mat("output.weight", sp->output_type, sp->n_vocab, d);
    FILE *f = std::fopen(path, "wb");
    if (!f) return fail(std::string("cannot create ") + path);
    std::string err;
    const bool ok = nh::gguf::write(f, kv, tensors, &err);
    if (std::fclose(f) != 0 && ok) return fail("write failed");
    return ok ? 0 : fail("gguf: " + err);
}

int lnm_gguf_inspect(const uint8_t *bytes, size_t len, size_t *n_tensors, size_t *n_kv, size_t *alignment) {
    if (!bytes) return fail("null argument");
    nh::gguf::File f;
    std::string err;
    if (!nh::gguf::parse(bytes, len, &f, &err)) return fail("gguf: " + err);
    if (n_tensors) *n_tensors = f.tensors.size();
    if (n_kv) *n_kv = f.kv.size();
    if (alignment) *alignment = f.alignment;
    return 0;
}

int lnm_gguf_tensor(const uint8_t *bytes, size_t len, size_t index, char *name, size_t name_cap, uint32_t *ggml_type,
                    uint64_t shape[4], uint32_t *n_dims, size_t *start, size_t *end) {
    if (!bytes) return fail("null argument");
    nh::gguf::File f;
    std::string err;
    if (!nh::gguf::parse(bytes, len, &f, &err)) return fail("gguf: " + err);
    if (index >= f.tensors.size()) return fail("tensor index out of range");
    const nh::gguf::TensorInfo &t = f.tensors[index];
    if (name && name_cap) {
        const size_t k = t.name.size() < name_cap - 1 ? t.name.size() : name_cap - 1;
        std::memcpy(name, t.name.data(), k);
        name[k] = 0;
    }
    if (ggml_type) *ggml_type = t.type;
    if (n_dims) *n_dims = (uint32_t)t.shape.size();
    if (shape)
        for (size_t i = 0; i < 4; i++) shape[i] = i < t.shape.size() ? t.shape[i] : 1;
    if (start) *start = t.start;
    if (end) *end = t.end;
    return 0;
}

}  // extern "C"
