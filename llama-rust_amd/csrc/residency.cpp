// Dispatch + bounded device-weight residency: the twin of
// langtax/src/native_gpu.rs and of quant::native_matmul
// (langtax/src/quant.rs:6683-6758), one executor and one cache per host thread.
//
// Identity of a weight is its dtype, shape and complete bytes; a 32-byte edge
// sample is only a shortlist (native_gpu.rs:56-99).  What is kept per entry is
// the packed matrix in HBM plus a host copy of the bytes for that identity
// check, so an entry is charged device bytes + packed length.  Budget rules,
// LRU order, eviction and the over-budget "run once, do not keep" rule follow
// native_gpu.rs:124-213; the environment variable is LLAMA_HIP_CACHE_BYTES
// ("auto" or a decimal byte count, 0 = no residency).
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <string>
#include <vector>

#include "../../include/native_hip.h"
#include "matview.h"

namespace {

constexpr size_t MIN_HEADROOM_BYTES = 512ull * 1024 * 1024;  // native_gpu.rs:16
const char *CACHE_BYTES_ENV = "LLAMA_HIP_CACHE_BYTES";

thread_local std::string q_error;

int qfail(int code, const std::string &msg) {
    q_error = "native HIP: " + msg;  // Display of QuantError::NativeCuda, quant.rs:4179
    return code;
}
int qfail_plain(int code, const std::string &msg) {
    q_error = msg;
    return code;
}
// QuantError::Size display, quant.rs:4183-4187
int size_error(const char *what, size_t actual, size_t expected) {
    return qfail_plain(LNH_ERR_INVALID, std::string(what) + " size " + std::to_string(actual) + " != " + std::to_string(expected));
}

// native_gpu.rs:20-32.  Returns 0 and fills (is_auto, bytes), or -1 (message) / -2 (too large).
int parse_cache_bytes(const char *value, bool *is_auto, size_t *bytes) {
    *is_auto = false;
    *bytes = 0;
    if (!value || std::strcmp(value, "auto") == 0) {
        *is_auto = true;
        return 0;
    }
    if (*value == '\0') return -1;
    size_t v = 0;
    for (const char *p = value; *p; ++p) {
        if (*p < '0' || *p > '9') return -1;
        size_t d = (size_t)(*p - '0');
        if (v > (SIZE_MAX - d) / 10) return -2;
        v = v * 10 + d;
    }
    *bytes = v;
    return 0;
}

// native_gpu.rs:34-39
size_t automatic_cache_bytes(size_t free_b, size_t total_b) {
    size_t available = free_b < total_b ? free_b : total_b;
    size_t reserve = available / 4 > MIN_HEADROOM_BYTES ? available / 4 : MIN_HEADROOM_BYTES;
    return available > reserve ? available - reserve : 0;
}

// native_gpu.rs:41-43
bool admission_requires_eviction(size_t used, size_t incoming, size_t limit) {
    return incoming > limit || used > limit - incoming;
}

struct WeightKey {  // native_gpu.rs:60-88
    uint32_t dtype;
    size_t rows, cols, len;
    uint8_t first[32], last[32];
    bool operator==(const WeightKey &o) const {
        return dtype == o.dtype && rows == o.rows && cols == o.cols && len == o.len &&
               std::memcmp(first, o.first, 32) == 0 && std::memcmp(last, o.last, 32) == 0;
    }
};

WeightKey make_key(uint32_t dtype, size_t rows, size_t cols, const uint8_t *p, size_t len) {
    WeightKey k{};
    k.dtype = dtype;
    k.rows = rows;
    k.cols = cols;
    k.len = len;
    size_t n = len < 32 ? len : 32;
    for (size_t i = 0; i < n; i++) {
        k.first[i] = p[i];
        k.last[i] = p[len - 1 - i];
    }
    return k;
}

struct Holder {  // keeps a device matrix alive while a call uses it, even if evicted meanwhile
    lnh_matrix *m = nullptr;
    ~Holder() { lnh_matrix_free(m); }
};

struct Entry {
    WeightKey key;
    std::vector<uint8_t> packed;
    std::shared_ptr<Holder> matrix;
    size_t bytes;
};

struct State {
    lnh_exec *gpu = nullptr;
    std::deque<Entry> cache;
    size_t bytes = 0, limit = 0, hits = 0, misses = 0;
    bool busy = false;
    ~State() {
        cache.clear();
        lnh_destroy(gpu);
    }
};

thread_local std::unique_ptr<State> t_state;

struct BusyGuard {
    State *s;
    explicit BusyGuard(State *st) : s(st) { s->busy = true; }
    ~BusyGuard() { s->busy = false; }
};

// First use on this thread: read the budget, then bring up the device (native_gpu.rs:138-159).
int ensure_state() {
    if (t_state) return LNH_OK;
    bool is_auto;
    size_t configured;
    int p = parse_cache_bytes(std::getenv(CACHE_BYTES_ENV), &is_auto, &configured);
    if (p == -1) return qfail(LNH_ERR_INVALID, std::string(CACHE_BYTES_ENV) + " must be auto or a nonnegative decimal byte count");
    if (p == -2) return qfail(LNH_ERR_INVALID, std::string(CACHE_BYTES_ENV) + " exceeds addressable memory");
    auto st = std::make_unique<State>();
    int rc = lnh_create(0, &st->gpu);
    if (rc != LNH_OK) return qfail(rc, lnh_thread_error());
    if (is_auto) {
        size_t f = 0, t = 0;
        rc = lnh_memory_info(st->gpu, &f, &t);
        if (rc != LNH_OK) return qfail(rc, lnh_last_error(st->gpu));
        st->limit = automatic_cache_bytes(f, t);
    } else {
        st->limit = configured;
    }
    t_state = std::move(st);
    return LNH_OK;
}

// A freshly uploaded matrix that enters the cache once the product that needed it has succeeded
// (native_gpu.rs:190-211 pushes the entry after gemm_resident returns Ok): a failed product leaves no
// charged entry behind.
struct Pending {
    bool keep = false;
    Entry entry;
};

void commit(State &s, Pending &p) {
    if (!p.keep) return;
    s.bytes += p.entry.bytes;
    s.cache.push_back(std::move(p.entry));
    p.keep = false;
}

// After a product: a cached matrix that made its multi-token layout in this product (matview.h) is charged for
// it from now on; what then exceeds the budget leaves from the front, the matrix just used last of all.
void recharge(State &s, const lnh_matrix *m) {
    for (Entry &en : s.cache) {
        if (en.matrix->m != m) continue;
        size_t dev = 0;
        if (lnh_matrix_info(m, nullptr, nullptr, nullptr, &dev) != LNH_OK) return;
        const size_t now = dev + en.packed.size();
        if (now > en.bytes) {
            s.bytes += now - en.bytes;
            en.bytes = now;
        }
        break;
    }
    while (!s.cache.empty() && s.bytes > s.limit) {
        s.bytes = s.bytes > s.cache.front().bytes ? s.bytes - s.cache.front().bytes : 0;
        s.cache.pop_front();
    }
}

// Resident matrix for these bytes: hit -> move to back, miss -> evict from the
// front until it fits, upload packed; `pending` then holds the entry to keep if within budget.
int resident(State &s, uint32_t type, size_t rows, size_t cols, size_t n_tokens, const uint8_t *w, size_t w_len,
             std::shared_ptr<Holder> *out, Pending *pending) {
    WeightKey key = make_key(type, rows, cols, w, w_len);
    for (size_t i = 0; i < s.cache.size(); i++) {
        Entry &en = s.cache[i];
        if (en.key == key && en.packed.size() == w_len && std::memcmp(en.packed.data(), w, w_len) == 0) {
            Entry moved = std::move(en);
            s.cache.erase(s.cache.begin() + (long)i);
            *out = moved.matrix;
            s.cache.push_back(std::move(moved));
            s.hits++;
            return LNH_OK;
        }
    }
    s.misses++;
    // what the matrix will hold on the device after this product (the single-token layout, plus the multi-token
    // layout when this product makes it: matview.h) and the host copy kept for the identity check
    size_t bytes = nh::plane_spec(type, rows, cols).total + w_len;
    if (bytes < w_len) return qfail(LNH_ERR_INVALID, "resident matrix size overflow");
    if (nh::product_reads_tiled(type, n_tokens > UINT32_MAX ? UINT32_MAX : (uint32_t)n_tokens)) {
        const size_t more = nh::tiled_spec(type, rows, cols).total;
        if (bytes + more < bytes) return qfail(LNH_ERR_INVALID, "resident matrix size overflow");
        bytes += more;
    }
    while (!s.cache.empty() && admission_requires_eviction(s.bytes, bytes, s.limit)) {
        s.bytes = s.bytes > s.cache.front().bytes ? s.bytes - s.cache.front().bytes : 0;
        s.cache.pop_front();
    }
    auto holder = std::make_shared<Holder>();
    int rc = lnh_upload_packed(s.gpu, type, rows, cols, w, w_len, &holder->m);
    if (rc != LNH_OK) return qfail(rc, lnh_last_error(s.gpu));
    *out = holder;
    if (bytes <= s.limit) {
        pending->keep = true;
        pending->entry.key = key;
        pending->entry.packed.assign(w, w + w_len);
        pending->entry.matrix = holder;
        pending->entry.bytes = bytes;
    }
    return LNH_OK;
}

// quant::native_matmul's checks, in its order (quant.rs:6698-6745).
// Returns LNH_OK with *n_rows set; n_rows == 0 means "succeed without work".
int check_matmul(uint32_t type, size_t n_cols, size_t n_tokens, size_t w_len, size_t x_len, size_t y_len,
                 size_t *n_rows) {
    if (!nh::type_supported(type)) return qfail(LNH_ERR_UNSUPPORTED, "unsupported GGUF dtype " + std::to_string(type));
    if (n_tokens == 0 || n_cols == 0 || y_len % n_tokens != 0)
        return qfail(LNH_ERR_INVALID, "matrix dimensions must be positive and token-aligned");
    if (n_cols > SIZE_MAX / n_tokens) return qfail(LNH_ERR_INVALID, "input shape overflow");
    if (x_len != n_tokens * n_cols) return size_error("X F32 elems", x_len, n_tokens * n_cols);
    *n_rows = y_len / n_tokens;
    size_t qk = nh::block_elems(type);
    if (n_cols % qk != 0)
        return qfail_plain(LNH_ERR_INVALID, "n_cols " + std::to_string(n_cols) + " is not a multiple of " + std::to_string(qk));
    size_t rb = nh::gguf_row_bytes(type, n_cols);
    if (rb == 0) return qfail(LNH_ERR_INVALID, "weight shape overflow");
    if (*n_rows != 0 && rb > SIZE_MAX / *n_rows) return qfail(LNH_ERR_INVALID, "weight shape overflow");
    if (w_len != rb * *n_rows) return size_error("W bytes", w_len, rb * *n_rows);
    return LNH_OK;
}

}  // namespace

extern "C" {

int lnq_gemm(uint32_t type, size_t n_cols, size_t n_tokens, const uint8_t *w, size_t w_len, const float *x,
             size_t x_len, float *y, size_t y_len) {
    size_t n_rows = 0;
    int rc = check_matmul(type, n_cols, n_tokens, w_len, x_len, y_len, &n_rows);
    if (rc != LNH_OK) return rc;
    if (n_rows == 0) return LNH_OK;
    if (!w || !x || !y) return qfail(LNH_ERR_INVALID, "buffer pointer is null");
    if (t_state && t_state->busy) return qfail(LNH_ERR_INVALID, "recursive GPU execution is unsupported");
    rc = ensure_state();
    if (rc != LNH_OK) return rc;
    State &s = *t_state;
    BusyGuard guard(&s);
    std::shared_ptr<Holder> mat;
    Pending pending;
    rc = resident(s, type, n_rows, n_cols, n_tokens, w, w_len, &mat, &pending);
    if (rc != LNH_OK) return rc;
    rc = lnh_gemm(s.gpu, mat->m, n_tokens, x, x_len, y, y_len);
    if (rc != LNH_OK) return qfail(rc, lnh_last_error(s.gpu));
    commit(s, pending);
    recharge(s, mat->m);
    return LNH_OK;
}

int lnq_gemv(uint32_t type, size_t n_cols, const uint8_t *w, size_t w_len, const float *x, size_t x_len, float *y,
             size_t y_len) {
    return lnq_gemm(type, n_cols, 1, w, w_len, x, x_len, y, y_len);
}

int lnq_gemm_grouped(uint32_t type, size_t n_cols, size_t n_rows, size_t n_groups, const uint8_t *const *parts,
                     size_t part_len, const size_t *tokens, const float *x, size_t x_len, float *y, size_t y_len) {
    if (!nh::type_supported(type)) return qfail(LNH_ERR_UNSUPPORTED, "unsupported GGUF dtype " + std::to_string(type));
    if (n_cols == 0 || n_rows == 0) return qfail(LNH_ERR_INVALID, "matrix dimensions must be positive and token-aligned");
    size_t qk = nh::block_elems(type);
    if (n_cols % qk != 0)
        return qfail_plain(LNH_ERR_INVALID, "n_cols " + std::to_string(n_cols) + " is not a multiple of " + std::to_string(qk));
    size_t rb = nh::gguf_row_bytes(type, n_cols);
    if (rb == 0 || rb > SIZE_MAX / n_rows) return qfail(LNH_ERR_INVALID, "weight shape overflow");
    if (part_len != rb * n_rows) return size_error("W bytes", part_len, rb * n_rows);
    if (n_groups != 0 && (!parts || !tokens)) return qfail(LNH_ERR_INVALID, "group arrays are null");
    size_t total = 0;
    for (size_t g = 0; g < n_groups; g++) {
        if (total + tokens[g] < total) return qfail(LNH_ERR_INVALID, "input shape overflow");
        total += tokens[g];
    }
    if (total != 0 && (n_cols > SIZE_MAX / total || n_rows > SIZE_MAX / total))
        return qfail(LNH_ERR_INVALID, "input shape overflow");
    if (x_len != total * n_cols) return size_error("X F32 elems", x_len, total * n_cols);
    if (y_len != total * n_rows) return size_error("Y F32 elems", y_len, total * n_rows);
    if (total == 0) return LNH_OK;
    if (!x || !y) return qfail(LNH_ERR_INVALID, "buffer pointer is null");
    for (size_t g = 0; g < n_groups; g++)
        if (tokens[g] != 0 && !parts[g]) return qfail(LNH_ERR_INVALID, "buffer pointer is null");
    if (t_state && t_state->busy) return qfail(LNH_ERR_INVALID, "recursive GPU execution is unsupported");
    int rc = ensure_state();
    if (rc != LNH_OK) return rc;
    State &s = *t_state;
    BusyGuard guard(&s);
    std::vector<std::shared_ptr<Holder>> holders(n_groups);
    std::vector<Pending> pending(n_groups);
    std::vector<const lnh_matrix *> mats(n_groups, nullptr);
    std::vector<size_t> toks(tokens, tokens + n_groups);
    // Experts without tokens are skipped before their weights are touched
    // (langtax/src/decode.rs:10043-10047).
    const lnh_matrix *any = nullptr;
    for (size_t g = 0; g < n_groups; g++) {
        if (toks[g] == 0) continue;
        // parts uploaded earlier in this call are not in the cache yet: a part that repeats is uploaded again,
        // which costs time, never correctness
        rc = resident(s, type, n_rows, n_cols, toks[g], parts[g], part_len, &holders[g], &pending[g]);
        if (rc != LNH_OK) return rc;
        mats[g] = holders[g]->m;
        any = mats[g];
    }
    for (size_t g = 0; g < n_groups; g++)
        if (!mats[g]) mats[g] = any;  // placeholder for skipped groups (tokens == 0)
    rc = lnh_gemm_grouped(s.gpu, n_groups, mats.data(), toks.data(), x, x_len, y, y_len);
    if (rc != LNH_OK) return qfail(rc, lnh_last_error(s.gpu));
    for (size_t g = 0; g < n_groups; g++) {
        // the budget may have been consumed by the parts committed before this one
        if (pending[g].keep && admission_requires_eviction(s.bytes, pending[g].entry.bytes, s.limit)) {
            while (!s.cache.empty() && admission_requires_eviction(s.bytes, pending[g].entry.bytes, s.limit)) {
                s.bytes = s.bytes > s.cache.front().bytes ? s.bytes - s.cache.front().bytes : 0;
                s.cache.pop_front();
            }
            if (admission_requires_eviction(s.bytes, pending[g].entry.bytes, s.limit)) pending[g].keep = false;
        }
        commit(s, pending[g]);
    }
    for (size_t g = 0; g < n_groups; g++)
        if (holders[g]) recharge(s, holders[g]->m);
    return LNH_OK;
}

const char *lnq_last_error(void) { return q_error.c_str(); }

int lnq_parse_cache_bytes(const char *value, int *is_auto, size_t *bytes) {
    bool a;
    size_t b;
    int p = parse_cache_bytes(value, &a, &b);
    if (p == -1) return qfail(LNH_ERR_INVALID, std::string(CACHE_BYTES_ENV) + " must be auto or a nonnegative decimal byte count");
    if (p == -2) return qfail(LNH_ERR_INVALID, std::string(CACHE_BYTES_ENV) + " exceeds addressable memory");
    if (is_auto) *is_auto = a ? 1 : 0;
    if (bytes) *bytes = b;
    return LNH_OK;
}

size_t lnq_automatic_cache_bytes(size_t free_bytes, size_t total_bytes) {
    return automatic_cache_bytes(free_bytes, total_bytes);
}

int lnq_admission_requires_eviction(size_t used, size_t incoming, size_t limit) {
    return admission_requires_eviction(used, incoming, limit) ? 1 : 0;
}

void lnq_cache_stats(size_t *entries, size_t *bytes, size_t *limit, size_t *hits, size_t *misses) {
    State *s = t_state.get();
    if (entries) *entries = s ? s->cache.size() : 0;
    if (bytes) *bytes = s ? s->bytes : 0;
    if (limit) *limit = s ? s->limit : 0;
    if (hits) *hits = s ? s->hits : 0;
    if (misses) *misses = s ? s->misses : 0;
}

void lnq_reset(void) { t_state.reset(); }

}  // extern "C"
