// Shared host/device helpers of libcome_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/come_hip.h"

namespace come {

// ---- host: per-thread error message -------------------------------------------------
void set_error(const char *fmt, ...);
void clear_error();

#define COME_REQUIRE(cond, code, ...)          \
    do {                                       \
        if (!(cond)) {                         \
            ::come::set_error(__VA_ARGS__);    \
            return (code);                     \
        }                                      \
    } while (0)

// Checks the launch that was just enqueued.
#define COME_CHECK_LAUNCH(what)                                                         \
    do {                                                                                \
        hipError_t e_ = hipGetLastError();                                              \
        if (e_ != hipSuccess) {                                                         \
            ::come::set_error("%s: launch failed: %s", what, hipGetErrorString(e_));    \
            return COME_ERR_HIP;                                                        \
        }                                                                               \
    } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device: 16-byte vectors of the three token dtypes ------------------------------
// Vec16<DT>::N elements per 16-byte chunk; unpack to / pack from fp32.
template <int DT> struct Vec16;

template <> struct Vec16<COME_F32> {
    static constexpr int N = 4;
    static constexpr int ELEM_BYTES = 4;
    __device__ static inline void unpack(const uint4 &r, float *f) {
        f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y);
        f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
    }
    __device__ static inline uint4 pack(const float *f) {
        return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]),
                          __float_as_uint(f[2]), __float_as_uint(f[3]));
    }
    __device__ static inline float load1(const void *p, int64_t i) { return static_cast<const float *>(p)[i]; }
    __device__ static inline void store1(void *p, int64_t i, float v) { static_cast<float *>(p)[i] = v; }
};

typedef float come_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 come_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 come_f16x2 __attribute__((ext_vector_type(2)));

// round-to-nearest-even of two floats into one packed word (one v_cvt_pk_bf16_f32)
__device__ inline uint32_t pack2_bf16(float lo, float hi) {
    const come_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, come_bf16x2));
}

template <> struct Vec16<COME_BF16> {
    static constexpr int N = 8;
    static constexpr int ELEM_BYTES = 2;
    __device__ static inline void unpack(const uint4 &r, float *f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ static inline uint4 pack(const float *f) {
        return make_uint4(pack2_bf16(f[0], f[1]), pack2_bf16(f[2], f[3]),
                          pack2_bf16(f[4], f[5]), pack2_bf16(f[6], f[7]));
    }
    __device__ static inline float load1(const void *p, int64_t i) {
        return __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t *>(p)[i]) << 16);
    }
    __device__ static inline void store1(void *p, int64_t i, float v) {
        static_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(pack2_bf16(v, 0.f) & 0xffffu);
    }
};

__device__ inline uint32_t pack2_f16(float lo, float hi) {
    const come_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, come_f16x2));
}

template <> struct Vec16<COME_F16> {
    static constexpr int N = 8;
    static constexpr int ELEM_BYTES = 2;
    __device__ static inline void unpack(const uint4 &r, float *f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __half2 h = *reinterpret_cast<const __half2 *>(&w[i]);
            float2 t = __half22float2(h);
            f[2 * i] = t.x;
            f[2 * i + 1] = t.y;
        }
    }
    __device__ static inline uint4 pack(const float *f) {
        return make_uint4(pack2_f16(f[0], f[1]), pack2_f16(f[2], f[3]),
                          pack2_f16(f[4], f[5]), pack2_f16(f[6], f[7]));
    }
    __device__ static inline float load1(const void *p, int64_t i) {
        return __half2float(static_cast<const __half *>(p)[i]);
    }
    __device__ static inline void store1(void *p, int64_t i, float v) {
        static_cast<__half *>(p)[i] = __float2half_rn(v);
    }
};

// 16-byte global accesses; the streamed variants carry the non-temporal hint (data used once)
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ inline uint4 ld16(const uint4 *p) { return *p; }
__device__ inline uint4 ld16_stream(const uint4 *p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ inline void st16_stream(uint4 *p, const uint4 &v) {
    const u32x4_t w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t *>(p));
}

inline int dtype_bytes(int dtype) { return dtype == COME_F32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype == COME_F32 || dtype == COME_F16 || dtype == COME_BF16; }

}  // namespace come
