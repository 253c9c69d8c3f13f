// -*-c++-*-
// Internal helpers of the front end: element codecs per data type and the host buffer
// behind CPU tensors.  Backends do not include this header.
#pragma once

#include <immintrin.h>
#include <stdint.h>
#include <string.h>

#include "saga.hpp"

namespace saga {

static inline float half_bits_to_float(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t float_to_half_bits(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }

// reads element `index` of a buffer of type dt as double
static inline double load_element(const void *base, Tensor::DataType dt, size_t index)
{
    switch(dt) {
    case Tensor::DataType::U8: return ((const uint8_t *)base)[index];
    case Tensor::DataType::HALF: return half_bits_to_float(((const uint16_t *)base)[index]);
    case Tensor::DataType::FLOAT: return ((const float *)base)[index];
    case Tensor::DataType::INT64: return (double)((const int64_t *)base)[index];
    case Tensor::DataType::I32: return ((const int32_t *)base)[index];
    case Tensor::DataType::I16: return ((const int16_t *)base)[index];
    }
    return 0;
}

static inline void store_element(void *base, Tensor::DataType dt, size_t index, double v)
{
    switch(dt) {
    case Tensor::DataType::U8: ((uint8_t *)base)[index] = (uint8_t)v; break;
    case Tensor::DataType::HALF: ((uint16_t *)base)[index] = float_to_half_bits((float)v); break;
    case Tensor::DataType::FLOAT: ((float *)base)[index] = (float)v; break;
    case Tensor::DataType::INT64: ((int64_t *)base)[index] = (int64_t)v; break;
    case Tensor::DataType::I32: ((int32_t *)base)[index] = (int32_t)v; break;
    case Tensor::DataType::I16: ((int16_t *)base)[index] = (int16_t)v; break;
    }
}

// Walks every logical coordinate of `dims` in row-major order.
template <typename F> static inline void for_each_coordinate(const Dims &dims, F &&fn)
{
    const size_t rank = dims.size();
    std::vector<int64_t> ext = dims.i64();
    size_t total = 1;
    for(auto e : ext)
        total *= (size_t)e;
    Dims c(rank, (int64_t)0);
    std::vector<int64_t> cur(rank, 0);
    for(size_t i = 0; i < total; i++) {
        fn(c, i);
        for(ssize_t j = (ssize_t)rank - 1; j >= 0; j--) {
            if(++cur[j] == ext[j]) {
                cur[j] = 0;
                c[j] = (int64_t)0;
            } else {
                c[j] = cur[j];
                break;
            }
        }
    }
}

}  // namespace saga
