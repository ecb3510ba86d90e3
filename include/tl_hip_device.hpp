// tl_hip_device.hpp : C++ adaptor that gives the C ABI of tensorlib_amd.h the shape of the
// reference's `Device<dtype>` backend interface (tensorLib/include/device/Device.hpp:5-110), so
// that it can be registered next to `CPU<dtype>` and `CUDA<dtype>` as a third backend
// (tensorLib/src/Tensor.cpp:46-52) and be called, unchanged, by Tensor / ops::matmul / nn /
// the Llama2 model.
//
// Inside the reference tree: compile with -DTL_HAVE_TENSORLIB_DEVICE_HPP so that the class
// derives from Device<dtype> and every method is an override.  Stand-alone (as in this
// repository's own Llama2 driver) the class is used directly and has no base.
//
// Method names, parameter order and meaning are exactly those of Device.hpp:13-101:
// elementwise/unary/reduction methods read `this` buffer as the (left) input and write to
// `result`; matmul2d and apply_rotary_emb take explicit pointers.  Runtime failures throw
// std::runtime_error carrying tl_last_error() (the reference prints and exits,
// tensorLib/include/device/cuda/CUDA.cuh:131-151); methods outside the matmul hot path
// (the generic unary/reduction zoo) throw std::logic_error.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "tensorlib_amd.h"

#ifdef TL_HAVE_TENSORLIB_DEVICE_HPP
#include "device/Device.hpp"
#define TL_DEVICE_BASE(dtype) : public Device<dtype>
#define TL_OVERRIDE override
#else
#define TL_DEVICE_BASE(dtype)
#define TL_OVERRIDE
#endif

namespace tl {

#if defined(__clang__) || defined(__FLT16_MANT_DIG__)
typedef _Float16 half;  // IEEE binary16 on the host; same bits as the reference's `half`
#endif

inline void throw_on_error(int status, const char* what) {
    if (status != TL_OK) throw std::runtime_error(std::string(what) + ": " + tl_last_error());
}

template <typename T>
inline uint16_t half_bits_of(T v) {
    static_assert(sizeof(T) == 2, "half_bits_of expects a 16-bit type");
    uint16_t b;
    std::memcpy(&b, &v, 2);
    return b;
}

}  // namespace tl

template <typename dtype>
class HIP TL_DEVICE_BASE(dtype) {
    static constexpr bool kIsHalf = (sizeof(dtype) == 2) && !std::is_integral<dtype>::value;

    [[noreturn]] static void outside(const char* op) {
        throw std::logic_error(std::string("tensorlib_amd HIP backend: ") + op +
                               " is outside the matmul hot path and not provided");
    }
    static void need_half(const char* op) {
        if (!kIsHalf) outside(op);
    }

public:
    // CUDA<dtype>::CUDA() / CUDA(size, ptr) / CUDA(size) / ~CUDA(): tensorLib/include/device/cuda/CUDA.cuh:14-17,
    // tensorLib/src/device/cuda/CUDA.cu:16-32.  A device object owns one allocation unless it
    // adopted an external pointer.
    HIP()
#ifdef TL_HAVE_TENSORLIB_DEVICE_HPP
        : Device<dtype>(0)
#endif
    {}
    HIP(size_t num_elements, dtype* ptr)
#ifdef TL_HAVE_TENSORLIB_DEVICE_HPP
        : Device<dtype>(num_elements),
#else
        : size(num_elements),
#endif
          data_(ptr), owns_(false) {}
    explicit HIP(size_t num_elements)
#ifdef TL_HAVE_TENSORLIB_DEVICE_HPP
        : Device<dtype>(num_elements)
#else
        : size(num_elements)
#endif
    {
        void* p = nullptr;
        tl::throw_on_error(tl_malloc(&p, num_elements * sizeof(dtype)), "HIP<dtype>::HIP");
        data_ = static_cast<dtype*>(p);
        owns_ = true;
    }
    HIP(const HIP&) = delete;
    HIP& operator=(const HIP&) = delete;
    virtual ~HIP() {
        if (owns_ && data_) tl_free(data_);
    }

    // ---- the boundary of the hot path (Device.hpp:22) ----
    void matmul2d(const dtype* A, const dtype* B, dtype* C, size_t M, size_t N, size_t K) TL_OVERRIDE {
        if constexpr (kIsHalf)
            tl::throw_on_error(tl_matmul2d_f16(A, B, C, M, N, K), "matmul2d");
        else if constexpr (std::is_same<dtype, float>::value)
            tl::throw_on_error(tl_matmul2d_f32(A, B, C, M, N, K), "matmul2d");
        else
            outside("matmul2d for this dtype");
    }

    // Old strided batched entry (Device.hpp:13-20); dead code in the reference
    // (tensorLib/src/Tensor.cpp:153-154 routes everything through call2 -> matmul2d).
    void matmul(const dtype*, const dtype*, dtype*, const std::vector<int>&, const std::vector<int>&, size_t, size_t,
                const std::vector<int>&, size_t, size_t) TL_OVERRIDE {
        outside("matmul (strided batched form; Tensor::matmul uses matmul2d)");
    }

    dtype* getDataPtr() TL_OVERRIDE { return data_; }

    void full(size_t num_elements, dtype fill_value) TL_OVERRIDE {
        if constexpr (kIsHalf) {
            tl::throw_on_error(tl_full_f16(data_, tl::half_bits_of(fill_value), num_elements), "full");
        } else {
            std::vector<dtype> host(num_elements, fill_value);
            tl::throw_on_error(tl_memcpy_h2d(data_, host.data(), num_elements * sizeof(dtype)), "full");
        }
    }
    void randn(size_t) TL_OVERRIDE { outside("randn (unseeded in the reference; use seeded inputs)"); }

    // 1-element synchronous copies, like tensorLib/src/device/cuda/CUDA.cu:71-81
    dtype getDataLinear(size_t linear_index) const TL_OVERRIDE {
        dtype v;
        tl::throw_on_error(tl_memcpy_d2h(&v, data_ + linear_index, sizeof(dtype)), "getDataLinear");
        return v;
    }
    void setDataLinear(size_t linear_index, dtype value) TL_OVERRIDE {
        tl::throw_on_error(tl_memcpy_h2d(data_ + linear_index, &value, sizeof(dtype)), "setDataLinear");
    }

    void contiguous(dtype* result, const std::vector<int>& shape, const std::vector<int>& stride, size_t offset,
                    size_t num_elements) TL_OVERRIDE {
        need_half("contiguous");
        tl::throw_on_error(tl_contiguous_f16(result, data_, shape.data(), stride.data(), (int)shape.size(), offset,
                                             num_elements), "contiguous");
    }
    void setItemEwise(dtype* src, const std::vector<int>& shape, const std::vector<int>& stride, size_t offset,
                      size_t num_elements) TL_OVERRIDE {
        need_half("setItemEwise");
        tl::throw_on_error(tl_set_item_ewise_f16(data_, src, shape.data(), stride.data(), (int)shape.size(), offset,
                                                 num_elements), "setItemEwise");
    }
    void setItemScalar(dtype, const std::vector<int>&, const std::vector<int>&, size_t, size_t) TL_OVERRIDE {
        outside("setItemScalar");
    }

    // ---- unary (Device.hpp:49-59): only silu is in the decode loop ----
    void neg(dtype*, size_t) TL_OVERRIDE { outside("neg"); }
    void sin(dtype*, size_t) TL_OVERRIDE { outside("sin"); }
    void cos(dtype*, size_t) TL_OVERRIDE { outside("cos"); }
    void exp(dtype*, size_t) TL_OVERRIDE { outside("exp"); }
    void log(dtype*, size_t) TL_OVERRIDE { outside("log"); }
    void abs(dtype*, size_t) TL_OVERRIDE { outside("abs"); }
    void tanh(dtype*, size_t) TL_OVERRIDE { outside("tanh"); }
    void sqrt(dtype*, size_t) TL_OVERRIDE { outside("sqrt"); }
    void rsqrt(dtype*, size_t) TL_OVERRIDE { outside("rsqrt"); }
    void silu(dtype* result, size_t num_elements) TL_OVERRIDE {
        need_half("silu");
        tl::throw_on_error(tl_silu_f16(result, data_, num_elements), "silu");
    }

    // ---- binary (Device.hpp:62-70) ----
    void add(dtype* result, dtype* other, size_t n) const TL_OVERRIDE { binary(result, other, n, 0, "add"); }
    void sub(dtype* result, dtype* other, size_t n) const TL_OVERRIDE { binary(result, other, n, 1, "sub"); }
    void mul(dtype* result, dtype* other, size_t n) const TL_OVERRIDE { binary(result, other, n, 2, "mul"); }
    void div(dtype* result, dtype* other, size_t n) const TL_OVERRIDE { binary(result, other, n, 3, "div"); }
    void add(dtype* result, dtype scalar, size_t n) const TL_OVERRIDE { binary_scalar(result, scalar, n, 0, "add"); }
    void sub(dtype* result, dtype scalar, size_t n) const TL_OVERRIDE { binary_scalar(result, scalar, n, 1, "sub"); }
    void mul(dtype* result, dtype scalar, size_t n) const TL_OVERRIDE { binary_scalar(result, scalar, n, 2, "mul"); }
    void div(dtype* result, dtype scalar, size_t n) const TL_OVERRIDE { binary_scalar(result, scalar, n, 3, "div"); }
    void pow(dtype*, dtype, size_t) const TL_OVERRIDE { outside("pow"); }

    // ---- reductions (Device.hpp:73-79): argmax and softmax are in the decode loop ----
    void max(dtype*, size_t, size_t) const TL_OVERRIDE { outside("max"); }
    void min(dtype*, size_t, size_t) const TL_OVERRIDE { outside("min"); }
    void sum(dtype*, size_t, size_t) const TL_OVERRIDE { outside("sum"); }
    void mean(dtype*, size_t, size_t) const TL_OVERRIDE { outside("mean"); }
    void argmin(int*, size_t, size_t) const TL_OVERRIDE { outside("argmin"); }
    void argmax(int* result, size_t reduce_size, size_t num_elements) const TL_OVERRIDE {
        need_half("argmax");
        tl::throw_on_error(tl_argmax_f16(result, data_, reduce_size, num_elements), "argmax");
    }
    void softmax(dtype* output, size_t rows, size_t cols) const TL_OVERRIDE {
        need_half("softmax");
        tl::throw_on_error(tl_softmax_f16(output, data_, rows, cols), "softmax");
    }

    void apply_rotary_emb(const dtype* input, dtype* result, int start_pos, int B, int T, int n_heads,
                          int head_dim) const TL_OVERRIDE {
        need_half("apply_rotary_emb");
        tl::throw_on_error(tl_apply_rotary_emb_f16(input, result, start_pos, B, T, n_heads, head_dim),
                           "apply_rotary_emb");
    }

    // Not a Device virtual in the reference either: reached through a dynamic_pointer_cast
    // (tensorLib/src/nn/rmsNorm.cpp:85-91, tensorLib/include/device/cuda/CUDA.cuh:108).
    void rms_norm(dtype* output, dtype* input, dtype* weight, float epsilon, int hidden_size, int num_tokens) {
        need_half("rms_norm");
        tl::throw_on_error(tl_rms_norm_f16(output, input, weight, epsilon, hidden_size, num_tokens), "rms_norm");
    }

#ifndef TL_HAVE_TENSORLIB_DEVICE_HPP
    size_t size = 0;  // element count (Device.hpp:109)
#endif

private:
    void binary(dtype* result, dtype* other, size_t n, int op, const char* name) const {
        need_half(name);
        tl::throw_on_error(tl_binary_f16(result, data_, other, n, op), name);
    }
    void binary_scalar(dtype* result, dtype scalar, size_t n, int op, const char* name) const {
        need_half(name);
        if constexpr (sizeof(dtype) == 2)
            tl::throw_on_error(tl_binary_scalar_f16(result, data_, tl::half_bits_of(scalar), n, op), name);
    }

    dtype* data_ = nullptr;
    bool owns_ = false;
};
