// Shared device helpers for the gfx950 kernels: 16-byte row chunks, wave64 cross-lane
// reductions, error reporting for the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/hira_hip.h"

namespace hira {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---- error text (thread local, returned by hira_last_error) -------------------------
char* error_buffer();
int fail(int code, const char* fmt, ...);

#define HIRA_CHECK_ARG(cond, ...)                              \
    do {                                                       \
        if (!(cond)) return ::hira::fail(HIRA_EINVAL, __VA_ARGS__); \
    } while (0)

#define HIRA_CHECK_LAUNCH(what)                                                        \
    do {                                                                               \
        hipError_t e_ = hipGetLastError();                                             \
        if (e_ != hipSuccess)                                                          \
            return ::hira::fail(HIRA_ELAUNCH, "%s: %s", what, hipGetErrorString(e_));  \
    } while (0)

// ---- storage types -------------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};

template <typename T>
struct Elem;
template <>
struct Elem<float> {
    static constexpr int kPerChunk = 4;  // elements in one 16-byte chunk
};
template <>
struct Elem<bf16_t> {
    static constexpr int kPerChunk = 8;
};

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// round-to-nearest-even fp32 -> bf16 (NaN kept quiet)
__device__ __host__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    union {
        float f;
        uint32_t u;
    } v;
    v.f = f;
    uint32_t u = v.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __host__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    union {
        float f;
        uint32_t u;
    } v;
    v.u = ((uint32_t)b) << 16;
    return v.f;
}

// Unpack one 16-byte chunk into fp32 lanes.
template <typename T>
__device__ __forceinline__ void unpack(const uint4& raw, float (&f)[Elem<T>::kPerChunk]);
template <>
__device__ __forceinline__ void unpack<float>(const uint4& raw, float (&f)[4]) {
    f[0] = __uint_as_float(raw.x);
    f[1] = __uint_as_float(raw.y);
    f[2] = __uint_as_float(raw.z);
    f[3] = __uint_as_float(raw.w);
}
template <>
__device__ __forceinline__ void unpack<bf16_t>(const uint4& raw, float (&f)[8]) {
    f[0] = bf16_lo(raw.x);
    f[1] = bf16_hi(raw.x);
    f[2] = bf16_lo(raw.y);
    f[3] = bf16_hi(raw.y);
    f[4] = bf16_lo(raw.z);
    f[5] = bf16_hi(raw.z);
    f[6] = bf16_lo(raw.w);
    f[7] = bf16_hi(raw.w);
}

// 16-byte load of chunk `ch` of the row that starts at element `row_elems` of `base`.
template <typename T>
__device__ __forceinline__ uint4 load_chunk(const void* base, size_t row_elems, int ch) {
    const T* p = reinterpret_cast<const T*>(base) + row_elems + (size_t)ch * Elem<T>::kPerChunk;
    return *reinterpret_cast<const uint4*>(p);
}

// ---- cross-lane ----------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over each aligned group of LANES consecutive lanes; every lane gets the group sum.
// Lanes 1,2: quad permutes; 4: mirror inside 8; 8: mirror inside 16; 16, 32: lane swaps.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    if (LANES >= 2) v += dpp_move<0xB1>(v);
    if (LANES >= 4) v += dpp_move<0x4E>(v);
    if (LANES >= 8) v += dpp_move<0x141>(v);
    if (LANES >= 16) v += dpp_move<0x140>(v);
    if (LANES >= 32) v += __shfl_xor(v, 16, 64);
    if (LANES >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// Reductions ACROSS the 64/LANES groups of a wave (lanes with equal lane % LANES).
template <int LANES>
__device__ __forceinline__ float cross_group_max(float v) {
#pragma unroll
    for (int off = LANES; off < 64; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
template <int LANES>
__device__ __forceinline__ float cross_group_sum(float v) {
#pragma unroll
    for (int off = LANES; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

}  // namespace hira
