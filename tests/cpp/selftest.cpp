// Executor self-test through the C++ mirror (include/native_hip.hpp): the scenario of the
// reference's validation runner (native-cuda/src/main.rs:8-67) - shapes revisited after
// resizing, single-token and batched launches alternating, every reuse of a buffer size with new
// inputs, every output checked; then bad calls, which must leave the output and the executor
// intact - plus one packed (Q8_0) matrix against the same numbers uploaded as F32.
// Prints "OK" and returns 0, or says what failed and returns 1.  Needs a gfx950 device.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../include/native_hip.hpp"

using native_hip::Error;
using native_hip::HipGemv;
using native_hip::HipMatrix;

static std::vector<double> exact_product(const std::vector<float> &w, const std::vector<float> &x, size_t rows, size_t cols,
                                         size_t tokens) {
    std::vector<double> e(rows * tokens);
    for (size_t t = 0; t < tokens; t++)
        for (size_t r = 0; r < rows; r++) {
            double s = 0.0;
            for (size_t c = 0; c < cols; c++) s += (double)w[r * cols + c] * (double)x[t * cols + c];
            e[t * rows + r] = s;
        }
    return e;
}

template <typename F> static bool rejected(F &&call) {
    try {
        call();
    } catch (const Error &) {
        return true;
    }
    return false;
}

static uint16_t f16_bits_of_small_dyadic(float v) {  // v = k / 256 with 1/256 <= v < 2: exact in binary16
    int e;
    const float m = std::frexp(v, &e);  // v = m * 2^e, 0.5 <= m < 1
    const uint32_t mant = (uint32_t)std::lround((m * 2.0f - 1.0f) * 1024.0f);
    return (uint16_t)(((e - 1 + 15) << 10) | mant);
}

int main() {
    try {
        HipGemv gpu(0);
        const auto mem = gpu.memory_info();
        if (mem.first == 0 || mem.first > mem.second) throw std::runtime_error("memory_info is not (free <= total)");

        std::vector<std::pair<size_t, size_t>> shapes;
        for (size_t rows : {1, 7, 9, 257})
            for (size_t cols : {63, 64, 65, 129, 1025}) shapes.emplace_back(rows, cols);
        for (auto extra : {std::pair<size_t, size_t>{17, 33}, {1, 1}, {257, 129}, {17, 33}}) shapes.push_back(extra);
        const size_t token_rounds[] = {1, 1, 3, 3, 1, 7, 1};
        size_t checked = 0;
        for (auto [rows, cols] : shapes) {
            std::vector<float> w(rows * cols);
            for (size_t i = 0; i < w.size(); i++) w[i] = ((float)(i % 23) - 11.0f) / 16.0f;
            HipMatrix m = gpu.upload(rows, cols, w);
            if (m.rows() != rows || m.cols() != cols) throw std::runtime_error("matrix reports a wrong shape");
            for (size_t round = 0; round < 7; round++) {
                const size_t tokens = token_rounds[round];
                std::vector<float> x(tokens * cols);
                for (size_t i = 0; i < x.size(); i++) x[i] = ((float)((i * 5 + round * 7) % 29) - 14.0f) / 16.0f;
                std::vector<float> y(rows * tokens, NAN);
                if (tokens == 1)
                    gpu.gemv_resident(m, x, y);
                else
                    gpu.gemm_resident(m, tokens, x, y);
                native_hip::validate(y, exact_product(w, x, rows, cols, tokens));
                checked += y.size();
            }
        }

        // bad calls: rejected before any device work, output untouched, executor still good
        HipMatrix m = gpu.upload(2, 3, {1.0f, -2.0f, 3.0f, 4.0f, 5.0f, -6.0f});
        std::vector<float> out = {123.5f, -456.0f};
        const std::vector<float> untouched = out;
        if (!rejected([&] { gpu.gemv_resident(m, {1.0f, 2.0f}, out); }) || out != untouched)
            throw std::runtime_error("a GEMV with a short input was accepted or changed the output");
        if (!rejected([&] { gpu.gemm_resident(m, 0, {}, out); }) || out != untouched)
            throw std::runtime_error("a zero-token GEMM was accepted or changed the output");
        {
            HipGemv other(0);
            if (!rejected([&] { other.gemv_resident(m, {1.0f, 2.0f, 3.0f}, out); }) || out != untouched)
                throw std::runtime_error("a matrix of another executor was accepted or changed the output");
        }
        if (!rejected([&] { gpu.upload(0, 3, {}); }) || !rejected([&] { gpu.upload(2, 3, {1.0f}); }))
            throw std::runtime_error("an upload with a bad shape was accepted");
        gpu.gemv_resident(m, {1.0f, 2.0f, 3.0f}, out);
        native_hip::validate(out, {6.0, -4.0});
        gpu.gemv({1.0f, -2.0f, 3.0f, 4.0f, 5.0f, -6.0f}, {1.0f, 2.0f, 3.0f}, out);  // upload + run
        native_hip::validate(out, {6.0, -4.0});

        // a packed Q8_0 matrix (34-byte blocks: f16 scale, 32 int8 codes) against the same values as F32
        const size_t rows = 70, cols = 256, nb = cols / 32;
        std::vector<uint8_t> packed(rows * nb * 34);
        std::vector<float> dense(rows * cols);
        for (size_t r = 0; r < rows; r++)
            for (size_t b = 0; b < nb; b++) {
                const float d = (float)(1 + (r * 7 + b * 3) % 200) / 256.0f;
                const uint16_t bits = f16_bits_of_small_dyadic(d);
                uint8_t *blk = &packed[(r * nb + b) * 34];
                std::memcpy(blk, &bits, 2);
                for (size_t i = 0; i < 32; i++) {
                    const int q = (int)((r * 31 + b * 17 + i * 13) % 255) - 127;
                    blk[2 + i] = (uint8_t)(int8_t)q;
                    dense[r * cols + b * 32 + i] = d * (float)q;  // exact: 8 x 8 significant bits
                }
            }
        HipMatrix q8 = gpu.upload_packed(LNH_TYPE_Q8_0, rows, cols, packed);
        for (size_t tokens : {1, 5, 40}) {
            std::vector<float> x(tokens * cols);
            for (size_t i = 0; i < x.size(); i++) x[i] = ((float)((i * 11) % 37) - 18.0f) / 32.0f;
            std::vector<float> y(rows * tokens, NAN);
            if (tokens == 1)
                gpu.gemv_resident(q8, x, y);
            else
                gpu.gemm_resident(q8, tokens, x, y);
            native_hip::validate(y, exact_product(dense, x, rows, cols, tokens));
            checked += y.size();
        }
        if (q8.device_bytes() < packed.size()) throw std::runtime_error("packed matrix reports fewer device bytes than it has");
        std::printf("OK %zu outputs checked\n", checked);
        return 0;
    } catch (const std::exception &e) {
        std::printf("FAILED: %s\n", e.what());
        return 1;
    }
}
