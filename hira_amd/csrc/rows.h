// Element-wise access to key / centre / value rows in either storage type.
#pragma once

#include "search.h"

namespace hira {

template <typename T>
__device__ __forceinline__ float load_elem(const void* base, size_t i);
template <>
__device__ __forceinline__ float load_elem<float>(const void* base, size_t i) {
    return reinterpret_cast<const float*>(base)[i];
}
template <>
__device__ __forceinline__ float load_elem<bf16_t>(const void* base, size_t i) {
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(base)[i]);
}
template <typename T>
__device__ __forceinline__ void store_elem(void* base, size_t i, float v);
template <>
__device__ __forceinline__ void store_elem<float>(void* base, size_t i, float v) {
    reinterpret_cast<float*>(base)[i] = v;
}
template <>
__device__ __forceinline__ void store_elem<bf16_t>(void* base, size_t i, float v) {
    reinterpret_cast<uint16_t*>(base)[i] = f32_to_bf16_bits(v);
}
template <typename T>
__device__ __forceinline__ float round_to(float v);
template <>
__device__ __forceinline__ float round_to<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ float round_to<bf16_t>(float v) {
    return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

}  // namespace hira
