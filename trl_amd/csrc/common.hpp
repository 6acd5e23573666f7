// Shared host/device helpers of the trlk kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "trlk.h"

namespace trlk {

// ---- host side: thread-local error text + status helper -------------------------------
int fail(int code, const char* fmt, ...);  // records the text, returns `code`
void clear_error();
int launch_status(const char* what);  // hipGetLastError() -> 0 or positive hipError_t (text recorded)
int grpo_fused_reserve_lds();          // grpo_fused.hip: LDS of the single-pass kernel's wide builds, current device

#define TRLK_REQUIRE(cond, code, ...)                    \
    do {                                                 \
        if (!(cond)) return ::trlk::fail((code), __VA_ARGS__); \
    } while (0)

// ---- device side ----------------------------------------------------------------------
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// Block-wide sum with a fixed combination order (bit-reproducible).  `scratch` holds at
// least NT/64 floats; every thread gets the result.  Contains two barriers.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    constexpr int NW = NT / kWave;
    v = wave_sum(v);
    __syncthreads();  // protects scratch against the previous use
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) r += scratch[w];
    return r;
}

// Storage-dtype traits: EPV = elements in one 16-byte vector.
template <int DT>
struct Elem;

template <>
struct Elem<TRLK_F32> {
    typedef float type;
    static constexpr int EPV = 4;
    static __device__ __forceinline__ void unpack(u32x4 q, float* x) {
        x[0] = __uint_as_float(q.x);
        x[1] = __uint_as_float(q.y);
        x[2] = __uint_as_float(q.z);
        x[3] = __uint_as_float(q.w);
    }
    static __device__ __forceinline__ u32x4 pack(const float* x) {
        u32x4 q = {__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
        return q;
    }
    static __device__ __forceinline__ float to_float(type v) { return v; }
    static __device__ __forceinline__ float load1(const type* p) { return *p; }
    static __device__ __forceinline__ void store1(type* p, float v) { *p = v; }
};

template <>
struct Elem<TRLK_BF16> {
    typedef uint16_t type;
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack2(uint32_t w, float* x) {
        x[0] = __uint_as_float(w << 16);
        x[1] = __uint_as_float(w & 0xffff0000u);
    }
    static __device__ __forceinline__ void unpack(u32x4 q, float* x) {
        unpack2(q.x, x);
        unpack2(q.y, x + 2);
        unpack2(q.z, x + 4);
        unpack2(q.w, x + 6);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {  // round-to-nearest-even
        f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ u32x4 pack(const float* x) {
        u32x4 q = {pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
        return q;
    }
    static __device__ __forceinline__ float to_float(type v) { return __uint_as_float(uint32_t(v) << 16); }
    static __device__ __forceinline__ float load1(const type* p) { return to_float(*p); }
    static __device__ __forceinline__ void store1(type* p, float v) { *p = uint16_t(pack2(v, 0.f) & 0xffffu); }
};

template <>
struct Elem<TRLK_F16> {
    typedef uint16_t type;
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack2(uint32_t w, float* x) {
        f16x2 h = __builtin_bit_cast(f16x2, w);
        x[0] = float(h.x);
        x[1] = float(h.y);
    }
    static __device__ __forceinline__ void unpack(u32x4 q, float* x) {
        unpack2(q.x, x);
        unpack2(q.y, x + 2);
        unpack2(q.z, x + 4);
        unpack2(q.w, x + 6);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f16x2 h = {_Float16(a), _Float16(b)};
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ u32x4 pack(const float* x) {
        u32x4 q = {pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
        return q;
    }
    static __device__ __forceinline__ float to_float(type v) { return float(__builtin_bit_cast(_Float16, v)); }
    static __device__ __forceinline__ float load1(const type* p) { return to_float(*p); }
    static __device__ __forceinline__ void store1(type* p, float v) {
        *p = __builtin_bit_cast(uint16_t, _Float16(v));
    }
};

inline size_t elem_size(int dtype) { return dtype == TRLK_F32 ? 4 : 2; }

}  // namespace trlk
