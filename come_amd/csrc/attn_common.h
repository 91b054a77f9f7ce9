// Pieces shared by the attention kernels of libcome_hip.so: argument block, 16-bit element traits,
// cross-half exchanges, the transposing LDS read and the direct global -> LDS loads.
#pragma once

#include "come_common.h"

namespace come {

struct AttnArgs {
    const uint16_t *q, *k, *v;
    const uint16_t *bias;            // may be null
    uint16_t *out;
    float *lse;                      // may be null
    const int32_t *cu;
    int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;
    int64_t total;
    int n_heads, n_mblocks, n_units;
    int rotate;                      // unit u starts its query blocks at position u (even block counts, see locate_block)
    int out_wide;                    // out rows allow 16-byte stores (pointer and strides multiples of 16 bytes)
    float scale_log2;
    // key-split tail: the last nb_tail query blocks of every (segment, head) unit are computed by `splits`
    // workgroups each, every one over its share of the keys, into `work`; a second kernel combines them
    int nb_tail, splits;
    int64_t n_full_wg;               // workgroups in front of the split ones
    float *work;
    // work queue of a launch of resident workgroups: 8 claim counters (one per class of workgroups, blockIdx.x % 8),
    // 8 item counts, then 8 lists of queue_cap entries (unit << 8 | query block)
    uint32_t *queue;
    int queue_cap;
    // optional prologue on the query rows, applied as the kernel loads them: LayerNorm over the head (qp_norm; gain
    // and shift [64] in the tensor dtype, either may be null) and the 2-D rotary embedding (qp_pos [total, 2] (y, x),
    // null: none; tables [qp_n_pos, 16] in the tensor dtype).  q in memory is then the raw projection.
    int qp_on, qp_norm;
    const void *qp_gamma, *qp_beta;
    float qp_eps;
    const int64_t *qp_pos;
    const void *qp_cos, *qp_sin;
    int64_t qp_n_pos;
};

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kBlockN = 64;          // keys per tile

template <int DT> struct Elem;
template <> struct Elem<COME_BF16> {
    static constexpr uint32_t kOne = 0x3F80u;
    __device__ static inline float to_f32(uint16_t x) { return __uint_as_float(static_cast<uint32_t>(x) << 16); }
    __device__ static inline uint16_t from_f32(float x) { return static_cast<uint16_t>(pack2_bf16(x, 0.f) & 0xffffu); }
    __device__ static inline uint32_t pack2(float lo, float hi) { return pack2_bf16(lo, hi); }
    __device__ static inline uint32_t pack2_prob(float lo, float hi) { return pack2_bf16(lo, hi); }
    // acc + lo(w) + hi(w) with fp32 accumulation (v_dot2c_f32_bf16 against packed ones)
    __device__ static inline float dot2_ones(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(come_bf16x2, w),
                                               __builtin_bit_cast(come_bf16x2, kOne | (kOne << 16)), acc, false);
    }
    __device__ static inline f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    __device__ static inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Elem<COME_F16> {
    static constexpr uint32_t kOne = 0x3C00u;
    __device__ static inline float to_f32(uint16_t x) { return __half2float(__builtin_bit_cast(__half, x)); }
    __device__ static inline uint16_t from_f32(float x) { return __builtin_bit_cast(uint16_t, __float2half_rn(x)); }
    __device__ static inline uint32_t pack2(float lo, float hi) { return pack2_f16(lo, hi); }
    // probabilities: round toward zero, so that a value beyond the fp16 range saturates at 65504 instead of
    // becoming infinite (row sums are taken from the converted values, so numerator and denominator agree)
    __device__ static inline uint32_t pack2_prob(float lo, float hi) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
    }
    __device__ static inline float dot2_ones(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(come_f16x2, w),
                                      __builtin_bit_cast(come_f16x2, kOne | (kOne << 16)), acc, false);
    }
    __device__ static inline f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    __device__ static inline f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};

__device__ inline u32x4 zero4() { return u32x4{0u, 0u, 0u, 0u}; }

// exchange between lane l and lane l ^ 32: returns {value of the lower half lane, value of the upper half lane}
__device__ inline float max_across_halves(float x) {
    const uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ inline float sum_across_halves(float x) {
    const uint32_t u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ inline s16x4 lds_read_tr(const uint16_t *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)(p));
}

// Offsets come from device memory that the host cannot check: a segment is clamped into [0, total], so that
// inconsistent offsets give wrong results for their rows instead of accesses outside the tensors.
__device__ inline void segment_of(const AttnArgs &a, int seq, int &seq_start, int &L) {
    const int total = static_cast<int>(a.total);
    seq_start = min(max(a.cu[seq], 0), total);
    L = min(max(a.cu[seq + 1], seq_start), total) - seq_start;
}

// Direct global -> LDS loads (lane l of the wavefront lands at lds_addr + 16 l, resp. + 4 l), written as
// asm so that the compiler does not order them against LDS reads it cannot tell apart: completion is
// awaited explicitly with s_waitcnt vmcnt before the barrier that publishes the tile.  m0 carries the LDS address;
// it is a register the compiler reserves and never keeps a value in across statements (it cannot be named as a
// clobber: the compiler rejects reserved registers there).
__device__ inline void dma_b128(const char *base, uint32_t lane_offset, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_offset), "s"(base), "s"(lds_addr) : "memory");
}
__device__ inline void dma_b32(const char *base, uint32_t lane_offset, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 :: "v"(lane_offset), "s"(base), "s"(lds_addr) : "memory");
}
__device__ inline uint32_t lds_address(const void *p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void *)(p)));
}

}  // namespace

// Attention for head dimensions 32 and 128 (attn_fwd_hd.hip): one 32-query tile per wavefront, the same
// arguments as the 64-wide kernel (the key-split fields are not used).
int launch_attn_hd(const AttnArgs &a, int dtype, int head_dim, int64_t max_seqlen, hipStream_t stream);

}  // namespace come
