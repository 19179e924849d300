// Host-side C++ mirror of the ToRSh types the quantized path touches: the error
// type, Result, DType, a dense f32/i8 host Tensor, and the device runtime that
// carries host buffers through the torsh_hipq C-ABI.
//
// The reference is Rust; `Result<T>` here reproduces the call-site vocabulary of
// `TorshResult<T>` (`is_ok`, `is_err`, `unwrap`, `unwrap_err`) so code and tests
// written against crates/torsh-quantization read the same way in C++.
//
// Mirrors: TorshError            crates/torsh-core/src/error (InvalidArgument, BackendError, NotImplemented ...)
//          TorshErrorCode        crates/torsh-core/src/ffi.rs:196-220 (numeric codes of the C-ABI)
//          Tensor::data/shape    crates/torsh-tensor (owned copies: crates/torsh-tensor/src/advanced_ops.rs:624-629)
//          tensor_1d / tensor_2d crates/torsh-tensor/src/creation.rs
#pragma once

#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <utility>
#include <variant>
#include <vector>

#include "torsh_hipq.h"

namespace torsh {

enum class DType { F32, I8, U8, I16, I32, F16 };  // F16 only names a precision (mixed-precision configs)

struct TorshError {
    enum Kind { InvalidArgument, ShapeError, DimensionMismatch, BackendError, AllocationError, NotImplemented };
    Kind kind;
    std::string message;

    static TorshError invalid_argument(std::string m) { return {InvalidArgument, std::move(m)}; }
    static TorshError backend(std::string m) { return {BackendError, std::move(m)}; }
    static TorshError not_implemented(std::string m) { return {NotImplemented, std::move(m)}; }

    // Status code of the C-ABI -> error kind (codes follow TorshErrorCode, ffi.rs:196-220).
    static TorshError from_status(int32_t status) {
        const char *msg = hipq_get_last_error();
        std::string m = (msg && *msg) ? msg : "torsh_hipq call failed";
        switch (status) {
        case HIPQ_INVALID_ARGUMENT: return {InvalidArgument, m};
        case HIPQ_SHAPE_ERROR: return {ShapeError, m};
        case HIPQ_DIMENSION_MISMATCH: return {DimensionMismatch, m};
        case HIPQ_ALLOCATION_ERROR: return {AllocationError, m};
        default: return {BackendError, m};
        }
    }
};

struct Unit {};

// Result<T>: either a value or a TorshError.
template <typename T>
class Result {
  public:
    Result(T v) : v_(std::move(v)) {}
    Result(TorshError e) : v_(std::move(e)) {}
    bool is_ok() const { return v_.index() == 0; }
    bool is_err() const { return v_.index() == 1; }
    T &unwrap() & {
        if (is_err()) throw std::runtime_error("unwrap on Err: " + std::get<1>(v_).message);
        return std::get<0>(v_);
    }
    const T &unwrap() const & {
        if (is_err()) throw std::runtime_error("unwrap on Err: " + std::get<1>(v_).message);
        return std::get<0>(v_);
    }
    T unwrap() && {  // on a temporary: the value is moved out, as Rust's unwrap consumes the Result
        if (is_err()) throw std::runtime_error("unwrap on Err: " + std::get<1>(v_).message);
        return std::move(std::get<0>(v_));
    }
    const TorshError &unwrap_err() const {
        if (is_ok()) throw std::runtime_error("unwrap_err on Ok");
        return std::get<1>(v_);
    }

  private:
    std::variant<T, TorshError> v_;
};

template <typename T>
using TorshResult = Result<T>;

// Early return of an error from an expression that yields Result<...> (Rust's `?`).
#define TORSH_TRY(var, expr)                       \
    auto var##_result = (expr);                    \
    if (var##_result.is_err()) return var##_result.unwrap_err(); \
    auto &var = var##_result.unwrap()

#define TORSH_CHECK(expr)                                                \
    do {                                                                 \
        auto _r = (expr);                                                \
        if (_r.is_err()) return _r.unwrap_err();                         \
    } while (0)

class Shape {
  public:
    Shape() = default;
    explicit Shape(std::vector<size_t> d) : dims_(std::move(d)) {}
    const std::vector<size_t> &dims() const { return dims_; }
    size_t ndim() const { return dims_.size(); }
    size_t numel() const {
        size_t n = 1;
        for (size_t d : dims_) n *= d;
        return n;
    }

  private:
    std::vector<size_t> dims_;
};

// Dense row-major host tensor.  Quantized values travel in an f32 carrier exactly as
// in the reference (crates/torsh-quantization/src/algorithms.rs:277-315 returns Tensor<f32>).
template <typename T>
class TensorT {
  public:
    TensorT() = default;
    static Result<TensorT> from_data(std::vector<T> data, std::vector<size_t> dims) {
        size_t n = 1;
        for (size_t d : dims) n *= d;
        if (n != data.size())
            return TorshError::invalid_argument("Data length " + std::to_string(data.size()) +
                                                " does not match shape with " + std::to_string(n) + " elements");
        TensorT t;
        t.data_ = std::move(data);
        t.shape_ = Shape(std::move(dims));
        return t;
    }
    const Shape &shape() const { return shape_; }
    // Owned copy, like Tensor::data() in the reference.
    Result<std::vector<T>> data() const { return data_; }
    const std::vector<T> &as_slice() const { return data_; }
    size_t numel() const { return data_.size(); }

  private:
    std::vector<T> data_;
    Shape shape_;
};

using Tensor = TensorT<float>;
using TensorI8 = TensorT<int8_t>;

inline Result<Tensor> tensor_1d(const std::vector<float> &v) { return Tensor::from_data(v, {v.size()}); }
inline Result<Tensor> tensor_2d(const std::vector<float> &v, size_t rows, size_t cols) {
    return Tensor::from_data(v, {rows, cols});
}

namespace hip {

// One context (device 0, its own stream) per process, created on first use.  Every
// host-level call below is synchronous: upload, launch, download.
class Runtime {
  public:
    static Result<hipq_ctx *> ctx() {
        static Runtime rt;
        std::lock_guard<std::mutex> lock(rt.mu_);
        if (!rt.ctx_) {
            int32_t rc = hipq_ctx_create(0, &rt.ctx_);
            if (rc != HIPQ_SUCCESS) {
                rt.ctx_ = nullptr;
                return TorshError::from_status(rc);
            }
        }
        return rt.ctx_;
    }

  private:
    Runtime() = default;
    ~Runtime() {
        if (ctx_) hipq_ctx_destroy(ctx_);
    }
    std::mutex mu_;
    hipq_ctx *ctx_ = nullptr;
};

// Device allocation owned by the host object that holds it.
class DeviceBuffer {
  public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept { *this = std::move(o); }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        if (this != &o) {
            release();
            ctx_ = o.ctx_;
            ptr_ = o.ptr_;
            bytes_ = o.bytes_;
            o.ptr_ = nullptr;
            o.bytes_ = 0;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    static Result<DeviceBuffer> alloc(hipq_ctx *ctx, size_t bytes) {
        DeviceBuffer b;
        b.ctx_ = ctx;
        b.bytes_ = bytes;
        int32_t rc = hipq_device_malloc(ctx, bytes, &b.ptr_);
        if (rc != HIPQ_SUCCESS) return TorshError::from_status(rc);
        return b;
    }
    template <typename T>
    static Result<DeviceBuffer> from_host(hipq_ctx *ctx, const T *src, size_t count) {
        auto r = alloc(ctx, count * sizeof(T));
        if (r.is_err()) return r.unwrap_err();
        if (count) {
            int32_t rc = hipq_memcpy_h2d(ctx, r.unwrap().ptr_, src, count * sizeof(T));
            if (rc != HIPQ_SUCCESS) return TorshError::from_status(rc);
        }
        return std::move(r.unwrap());
    }
    template <typename T>
    Result<std::vector<T>> to_host(size_t count) const {
        std::vector<T> out(count);
        if (count) {
            int32_t rc = hipq_memcpy_d2h(ctx_, out.data(), ptr_, count * sizeof(T));
            if (rc != HIPQ_SUCCESS) return TorshError::from_status(rc);
        }
        return out;
    }
    template <typename T>
    T *as() const { return static_cast<T *>(ptr_); }
    size_t bytes() const { return bytes_; }

  private:
    void release() {
        if (ptr_) hipq_device_free(ctx_, ptr_);
        ptr_ = nullptr;
    }
    hipq_ctx *ctx_ = nullptr;
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
};

inline Result<Unit> check(int32_t rc) {
    if (rc != HIPQ_SUCCESS) return TorshError::from_status(rc);
    return Unit{};
}

}  // namespace hip
}  // namespace torsh
