// native-hip: C++ mirror of the reference's executor interface over the C ABI of
// native_hip.h.  Same names, argument meaning and error behaviour as
// llama_native_cuda::{CudaGemv, CudaMatrix, Shape, validate}
// (native-cuda/src/lib.rs:8-53, native-cuda/src/gpu.rs:125-418): every fallible
// operation that returns Result<_, String> there throws native_hip::Error
// (a std::runtime_error carrying that string) here; nothing falls back to the CPU.
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "native_hip.h"

namespace native_hip {

struct Error : std::runtime_error {
    int code;
    Error(int code_, const std::string &message) : std::runtime_error(message), code(code_) {}
};

// native-cuda/src/lib.rs:8-34
struct Shape {
    uint32_t rows = 0, cols = 0;
    static Shape checked(size_t rows, size_t cols, size_t weights, size_t input) {
        Shape s;
        const int rc = lnh_shape_checked(rows, cols, weights, input, &s.rows, &s.cols);
        if (rc != LNH_OK) throw Error(rc, lnh_thread_error());
        return s;
    }
    size_t elements() const { return (size_t)rows * cols; }
};

// native-cuda/src/lib.rs:36-53: |actual - expected| <= 1e-4 + 1e-4 |expected|, all finite
inline void validate(const std::vector<float> &actual, const std::vector<double> &expected) {
    const int rc = lnh_validate(actual.data(), actual.size(), expected.data(), expected.size());
    if (rc != LNH_OK) throw Error(rc, lnh_thread_error());
}

class HipGemv;

// CudaMatrix (native-cuda/src/gpu.rs:125-130): immutable, owns its device allocation.
class HipMatrix {
public:
    HipMatrix() = default;
    HipMatrix(HipMatrix &&o) noexcept : raw_(std::exchange(o.raw_, nullptr)) {}
    HipMatrix &operator=(HipMatrix &&o) noexcept {
        if (this != &o) {
            reset();
            raw_ = std::exchange(o.raw_, nullptr);
        }
        return *this;
    }
    HipMatrix(const HipMatrix &) = delete;
    HipMatrix &operator=(const HipMatrix &) = delete;
    ~HipMatrix() { reset(); }
    size_t rows() const { return info().rows; }
    size_t cols() const { return info().cols; }
    size_t device_bytes() const { return info().bytes; }

private:
    friend class HipGemv;
    struct Info {
        uint32_t type;
        size_t rows, cols, bytes;
    };
    Info info() const {
        Info i{};
        lnh_matrix_info(raw_, &i.type, &i.rows, &i.cols, &i.bytes);
        return i;
    }
    void reset() {
        if (raw_) lnh_matrix_free(raw_);
        raw_ = nullptr;
    }
    lnh_matrix *raw_ = nullptr;
};

// CudaGemv (native-cuda/src/gpu.rs:132-418).
class HipGemv {
public:
    explicit HipGemv(size_t device_ordinal) {
        const int rc = lnh_create((int)device_ordinal, &raw_);
        if (rc != LNH_OK) throw Error(rc, lnh_thread_error());
    }
    HipGemv(const HipGemv &) = delete;
    HipGemv &operator=(const HipGemv &) = delete;
    ~HipGemv() { lnh_destroy(raw_); }

    std::pair<size_t, size_t> memory_info() {  // (free, total)
        size_t f = 0, t = 0;
        check(lnh_memory_info(raw_, &f, &t));
        return {f, t};
    }
    HipMatrix upload(size_t rows, size_t cols, const std::vector<float> &weights) {
        HipMatrix m;
        check(lnh_upload_f32(raw_, rows, cols, weights.data(), weights.size(), &m.raw_));
        return m;
    }
    // Not in the reference: the GGUF bytes stay packed on the device.
    HipMatrix upload_packed(uint32_t ggml_type, size_t rows, size_t cols, const std::vector<uint8_t> &packed) {
        HipMatrix m;
        check(lnh_upload_packed(raw_, ggml_type, rows, cols, packed.data(), packed.size(), &m.raw_));
        return m;
    }
    void gemv_resident(const HipMatrix &m, const std::vector<float> &input, std::vector<float> &output) {
        check(lnh_gemv(raw_, m.raw_, input.data(), input.size(), output.data(), output.size()));
    }
    void gemm_resident(const HipMatrix &m, size_t tokens, const std::vector<float> &input, std::vector<float> &output) {
        check(lnh_gemm(raw_, m.raw_, tokens, input.data(), input.size(), output.data(), output.size()));
    }
    // upload + run, the matrix is not kept (gpu.rs:290-299)
    void gemv(const std::vector<float> &weights, const std::vector<float> &input, std::vector<float> &output) {
        check(lnh_gemv_once(raw_, weights.data(), weights.size(), input.data(), input.size(), output.data(), output.size()));
    }
    // Not in the reference: the per-expert products of one MoE projection in one call.
    void gemm_grouped(const std::vector<const HipMatrix *> &mats, const std::vector<size_t> &tokens,
                      const std::vector<float> &input, std::vector<float> &output) {
        std::vector<const lnh_matrix *> raws;
        for (const HipMatrix *m : mats) raws.push_back(m->raw_);
        check(lnh_gemm_grouped(raw_, raws.size(), raws.data(), tokens.data(), input.data(), input.size(), output.data(),
                               output.size()));
    }

private:
    void check(int rc) {
        if (rc != LNH_OK) throw Error(rc, lnh_last_error(raw_));
    }
    lnh_exec *raw_ = nullptr;
};

}  // namespace native_hip
