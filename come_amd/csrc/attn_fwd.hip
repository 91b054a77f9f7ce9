// Forward attention over packed variable-length sequences with an additive per-key
// bias, head_dim 64, for gfx950 (wave64, v_mfma_f32_32x32x16 bf16/f16).
//
// Work decomposition
//   One workgroup (4 wavefronts) owns kBlockM = 128 * QT consecutive queries of one
//   (segment, head); every wavefront owns QT tiles of 32 queries and walks all keys of
//   the segment in tiles of 64.  K and V tiles are staged once per workgroup in LDS
//   (double buffered, one barrier per tile); Q stays in registers.
//
// Orientation
//   Scores are produced transposed, S^T = K' Q'^T, so that in the MFMA accumulator
//   layout a lane holds ONE query (lane % 32) and 16 keys per 32x32 tile: the row max
//   and row sum of the online softmax are in-lane reductions plus one exchange between
//   lane l and lane l ^ 32.  The same registers, rounded to 16 bit, are the B operand
//   of O^T += V^T P^T without any data movement; V^T fragments come out of the
//   row-major V tile with the transposing LDS read ds_read_b64_tr_b16.
//
// Bias and tail masking without vector ALU work
//   K' = [K | t_hi t_mid t_lo 0...] (80 columns) and Q' = [Q | 1 1 1 0...] where
//   t = float(bias) / softmax_scale split exactly into three 16-bit terms, so the
//   fifth k-step of the score MFMA adds bias / scale to every score (the reference
//   adds the same quantity, flash_fwd_kernel.h:30-55).  Keys beyond the end of the
//   segment get t_hi = -inf, which makes their scores -inf and their probabilities 0.
#include "come_common.h"

#include <cstdlib>

namespace come {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kHeadDim = 64;
constexpr int kBlockN = 64;          // keys per tile
constexpr int kKPitch = 88;          // elements per K' row in LDS (64 + 16 bias/zero + 8 pad): 176 B, odd multiple of 16 B
constexpr int kVPitch = 96;          // elements per V row in LDS: 192 B = 48 banks, 4 rows tile the 64 banks
constexpr int kThreads = 256;

struct AttnArgs {
    const uint16_t *q, *k, *v;
    const uint16_t *bias;            // may be null
    uint16_t *out;
    float *lse;                      // may be null
    const int32_t *cu;
    int64_t q_rs, q_hs, k_rs, k_hs, v_rs, v_hs, o_rs, o_hs;
    int64_t total;
    int n_heads, n_mblocks;
    float scale, scale_log2, inv_scale;
};

template <int DT> struct Elem;
template <> struct Elem<COME_BF16> {
    static constexpr uint32_t kOne = 0x3F80u, kNegInf = 0xFF80u;
    __device__ static inline float to_f32(uint16_t x) { return __uint_as_float(static_cast<uint32_t>(x) << 16); }
    __device__ static inline uint16_t from_f32(float x) { return static_cast<uint16_t>(pack2_bf16(x, 0.f) & 0xffffu); }
    __device__ static inline uint32_t pack2(float lo, float hi) { return pack2_bf16(lo, hi); }
    // acc + lo(w) + hi(w) with fp32 accumulation (v_dot2c_f32_bf16 against packed ones)
    __device__ static inline float dot2_ones(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(come_bf16x2, w),
                                               __builtin_bit_cast(come_bf16x2, kOne | (kOne << 16)), acc, false);
    }
    __device__ static inline f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Elem<COME_F16> {
    static constexpr uint32_t kOne = 0x3C00u, kNegInf = 0xFC00u;
    __device__ static inline float to_f32(uint16_t x) { return __half2float(__builtin_bit_cast(__half, x)); }
    __device__ static inline uint16_t from_f32(float x) { return __builtin_bit_cast(uint16_t, __float2half_rn(x)); }
    __device__ static inline uint32_t pack2(float lo, float hi) { return pack2_f16(lo, hi); }
    __device__ static inline float dot2_ones(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(come_f16x2, w),
                                      __builtin_bit_cast(come_f16x2, kOne | (kOne << 16)), acc, false);
    }
    __device__ static inline f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
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

template <int DT, int QT>
__global__ __launch_bounds__(kThreads) void attn_fwd_kernel(const AttnArgs a) {
    using E = Elem<DT>;
    constexpr int kBlockM = 128 * QT;
    __shared__ __attribute__((aligned(16))) uint16_t lds_k[2][kBlockN * kKPitch];
    __shared__ __attribute__((aligned(16))) uint16_t lds_v[2][kBlockN * kVPitch];

    // ---- which (segment, head, query block): consecutive blocks of one (segment, head)
    //      run on the same XCD (workgroup i is dispatched to XCD i % 8) and share K/V in its L2
    const int n_wg = gridDim.x;
    int wid = blockIdx.x;
    const int per_xcd = n_wg >> 3;
    if (wid < (per_xcd << 3)) wid = (wid & 7) * per_xcd + (wid >> 3);
    const int mblk = wid % a.n_mblocks;
    const int rest = wid / a.n_mblocks;
    const int head = rest % a.n_heads;
    const int seq = rest / a.n_heads;
    const int seq_start = a.cu[seq];
    const int L = a.cu[seq + 1] - seq_start;
    const int q0 = mblk * kBlockM;
    if (q0 >= L) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5;          // which half of the wavefront
    const int r = lane & 31;          // query column / key row inside a 32x32 tile

    // ---- Q fragments (B operand: n = query r, k = head-dim 16 * ks + 8 * h .. + 7)
    u32x4 qf[QT][4];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int row = q0 + (wave * QT + qt) * 32 + r;
        const uint16_t *qp = a.q + static_cast<int64_t>(seq_start + min(row, L - 1)) * a.q_rs + head * a.q_hs + 8 * h;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qf[qt][ks] = *reinterpret_cast<const u32x4 *>(qp + 16 * ks);
    }
    // fifth k-step of Q': ones against the three bias terms (lower half), zeros elsewhere
    const u32x4 q_ext = h == 0 ? u32x4{E::kOne | (E::kOne << 16), E::kOne, 0u, 0u} : zero4();

    // ---- staging of one K'/V tile: thread -> (row sr and sr + 32, 16-byte chunk sc)
    const int sc = tid & 7;
    const int sr = tid >> 3;
    const uint16_t *k_base = a.k + static_cast<int64_t>(seq_start) * a.k_rs + head * a.k_hs + sc * 8;
    const uint16_t *v_base = a.v + static_cast<int64_t>(seq_start) * a.v_rs + head * a.v_hs + sc * 8;
    const uint16_t *b_base = a.bias ? a.bias + seq_start : nullptr;

    u32x4 k_stage[2], v_stage[2], b_stage;
    auto fetch = [&](int n0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int key = n0 + sr + 32 * i;
            const bool ok = key < L;
            k_stage[i] = ok ? *reinterpret_cast<const u32x4 *>(k_base + static_cast<int64_t>(key) * a.k_rs) : zero4();
            v_stage[i] = ok ? *reinterpret_cast<const u32x4 *>(v_base + static_cast<int64_t>(key) * a.v_rs) : zero4();
        }
        if (tid < kBlockN) {
            const int key = n0 + tid;
            uint32_t t_hi = E::kNegInf, t_mid = 0, t_lo = 0;
            if (key < L) {
                const float t = b_base ? E::to_f32(b_base[key]) * a.inv_scale : 0.f;
                t_hi = E::from_f32(t);
                const float hi_f = E::to_f32(static_cast<uint16_t>(t_hi));
                if (fabsf(hi_f) != INFINITY) {                               // an infinite bias stays a single term
                    const float r1 = t - hi_f;
                    t_mid = E::from_f32(r1);
                    t_lo = E::from_f32(r1 - E::to_f32(static_cast<uint16_t>(t_mid)));
                }
            }
            b_stage = u32x4{t_hi | (t_mid << 16), t_lo, 0u, 0u};
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<u32x4 *>(&lds_k[buf][(sr + 32 * i) * kKPitch + sc * 8]) = k_stage[i];
            *reinterpret_cast<u32x4 *>(&lds_v[buf][(sr + 32 * i) * kVPitch + sc * 8]) = v_stage[i];
        }
        if (tid < kBlockN) {
            *reinterpret_cast<u32x4 *>(&lds_k[buf][tid * kKPitch + 64]) = b_stage;
            *reinterpret_cast<u32x4 *>(&lds_k[buf][tid * kKPitch + 72]) = zero4();
        }
    };

    // ---- running state per query tile
    f32x16 o_acc[QT][2];
    float m_run[QT], l_run[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[qt][dt][i] = 0.f;
        m_run[qt] = -INFINITY;
        l_run[qt] = 0.f;
    }

    const int n_tiles = (L + kBlockN - 1) / kBlockN;
    fetch(0);
    commit(0);
    __syncthreads();

    // LDS read offsets of this lane
    const int k_off = r * kKPitch + 8 * h;                                   // + 32*mt*pitch + 16*ks
    const int v_off = (4 * h + ((lane & 15) >> 2)) * kVPitch + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    for (int j = 0; j < n_tiles; ++j) {
        const int buf = j & 1;
        const bool more = j + 1 < n_tiles;
        if (more) fetch((j + 1) * kBlockN);

        // ---- S^T = K' Q'^T : [64 keys] x [32 * QT queries]
        f32x16 s_acc[QT][2];
        const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 5; ++ks) {
            const u32x4 kf0 = *reinterpret_cast<const u32x4 *>(&lds_k[buf][k_off + 16 * ks]);
            const u32x4 kf1 = *reinterpret_cast<const u32x4 *>(&lds_k[buf][k_off + 32 * kKPitch + 16 * ks]);
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
                const u32x4 qb = ks < 4 ? qf[qt][ks < 4 ? ks : 0] : q_ext;
                s_acc[qt][0] = E::mfma(kf0, qb, ks == 0 ? zero16 : s_acc[qt][0]);
                s_acc[qt][1] = E::mfma(kf1, qb, ks == 0 ? zero16 : s_acc[qt][1]);
            }
        }

        // ---- online softmax, in the exp2 domain
        u32x4 p_frag[QT][4];                                                  // P^T as B operand, one per 16-key step
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            float mx = s_acc[qt][0][0];
#pragma unroll
            for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s_acc[qt][0][i]);
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s_acc[qt][1][i]);
            mx = max_across_halves(mx);
            const float m_new = fmaxf(m_run[qt], mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;            // row fully masked so far
            const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_use) * a.scale_log2);
            const float mc = m_use * a.scale_log2;
            float sum = 0.f;
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[qt][mt][i], a.scale_log2, -mc));
                    s_acc[qt][mt][i] = p;
                    sum += p;
                }
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    u32x4 f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) f[w] = E::pack2(s_acc[qt][mt][8 * t + 2 * w], s_acc[qt][mt][8 * t + 2 * w + 1]);
                    p_frag[qt][2 * mt + t] = f;
                }
            }
            l_run[qt] = l_run[qt] * alpha + sum;
            if (__any(m_new != m_run[qt])) {                                  // rescale O only when some row max moved
#pragma unroll
                for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o_acc[qt][dt][i] *= alpha;
            }
            m_run[qt] = m_new;
        }

        // ---- O^T += V^T P^T
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const uint16_t *vp = &lds_v[buf][v_off + (16 * u) * kVPitch + 32 * dt];
                const s16x4 lo = lds_read_tr(vp);
                const s16x4 hi = lds_read_tr(vp + 8 * kVPitch);
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lo);
                const u32x2 hi2 = __builtin_bit_cast(u32x2, hi);
                const u32x4 vf = u32x4{lo2[0], lo2[1], hi2[0], hi2[1]};
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) o_acc[qt][dt] = E::mfma(vf, p_frag[qt][u], o_acc[qt][dt]);
            }
        }

        if (more) commit(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: normalise, write O (and LSE)
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const float l_tot = sum_across_halves(l_run[qt]);
        const float inv = 1.0f / l_tot;
        const int row = q0 + (wave * QT + qt) * 32 + r;
        if (row < L) {
            uint16_t *op = a.out + static_cast<int64_t>(seq_start + row) * a.o_rs + head * a.o_hs + 4 * h;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = E::pack2(o_acc[qt][dt][4 * g] * inv, o_acc[qt][dt][4 * g + 1] * inv);
                    w[1] = E::pack2(o_acc[qt][dt][4 * g + 2] * inv, o_acc[qt][dt][4 * g + 3] * inv);
                    *reinterpret_cast<u32x2 *>(op + 32 * dt + 8 * g) = w;
                }
            if (h == 0 && a.lse)
                a.lse[static_cast<int64_t>(head) * a.total + seq_start + row] = m_run[qt] * a.scale + __logf(l_tot);
        }
    }
}


// -------------------------------------------------------------------------------------
// Software-pipelined variant: kBlockM = 256 queries per workgroup, two query tiles per
// wavefront that alternate roles.  While the vector ALU runs the softmax of one query
// tile, the matrix pipe runs the score MFMAs (next key tile) and the P V MFMAs (current
// key tile) of the other one:
//
//   slot a(j): VALU softmax(S0(j)) -> P0      MFMA S1(j) = K'(j) Q1'^T ; O1 += V(j-1)^T P1(j-1)
//   slot b(j): VALU softmax(S1(j)) -> P1      MFMA S0(j+1) = K'(j+1) Q0'^T ; O0 += V(j)^T P0(j)
//
// K' tiles j, j+1 and V tiles j-1, j are live in one iteration, so LDS holds three tiles
// of each and one barrier per iteration suffices.
// -------------------------------------------------------------------------------------
constexpr int kStages = 3;

template <int DT>
__global__ __launch_bounds__(kThreads) void attn_fwd_pipe_kernel(const AttnArgs a) {
    using E = Elem<DT>;
    constexpr int kBlockM = 256;
    __shared__ __attribute__((aligned(16))) uint16_t lds_k[kStages][kBlockN * kKPitch];
    __shared__ __attribute__((aligned(16))) uint16_t lds_v[kStages][kBlockN * kVPitch];

    const int n_wg = gridDim.x;
    int wid = blockIdx.x;
    const int per_xcd = n_wg >> 3;
    if (wid < (per_xcd << 3)) wid = (wid & 7) * per_xcd + (wid >> 3);
    const int mblk = wid % a.n_mblocks;
    const int rest = wid / a.n_mblocks;
    const int head = rest % a.n_heads;
    const int seq = rest / a.n_heads;
    const int seq_start = a.cu[seq];
    const int L = a.cu[seq + 1] - seq_start;
    const int q0 = mblk * kBlockM;
    if (q0 >= L) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5;
    const int r = lane & 31;

    u32x4 qf[2][4];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const int row = q0 + (wave * 2 + qt) * 32 + r;
        const uint16_t *qp = a.q + static_cast<int64_t>(seq_start + min(row, L - 1)) * a.q_rs + head * a.q_hs + 8 * h;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qf[qt][ks] = *reinterpret_cast<const u32x4 *>(qp + 16 * ks);
    }
    const u32x4 q_ext = h == 0 ? u32x4{E::kOne | (E::kOne << 16), E::kOne, 0u, 0u} : zero4();

    const int sc = tid & 7;
    const int sr = tid >> 3;
    const uint16_t *k_base = a.k + static_cast<int64_t>(seq_start) * a.k_rs + head * a.k_hs + sc * 8;
    const uint16_t *v_base = a.v + static_cast<int64_t>(seq_start) * a.v_rs + head * a.v_hs + sc * 8;
    const uint16_t *b_base = a.bias ? a.bias + seq_start : nullptr;

    // Global -> register staging.  Loads are unconditional: a key index beyond the segment is clamped to
    // its last key (finite data); such keys get a bias term of -inf at commit time, so their
    // probabilities are exactly 0 and neither their K nor their V row can reach the output.
    u32x4 k_stage[2], v_stage[2];
    uint16_t b_raw = 0;
    int b_key = 0;
    // per-thread row pointers of key tile 0; a tile step is a wave-uniform offset
    const uint16_t *k_row[2], *v_row[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        k_row[i] = k_base + static_cast<int64_t>(sr + 32 * i) * a.k_rs;
        v_row[i] = v_base + static_cast<int64_t>(sr + 32 * i) * a.v_rs;
    }
    const uint16_t *k_last = k_base + static_cast<int64_t>(L - 1) * a.k_rs;
    const uint16_t *v_last = v_base + static_cast<int64_t>(L - 1) * a.v_rs;
    const int64_t k_tile_step = static_cast<int64_t>(kBlockN) * a.k_rs;
    const int64_t v_tile_step = static_cast<int64_t>(kBlockN) * a.v_rs;
    auto fetch_k = [&](int tile) {
        const int n0 = tile * kBlockN;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint16_t *p = n0 + sr + 32 * i < L ? k_row[i] + tile * k_tile_step : k_last;
            k_stage[i] = *reinterpret_cast<const u32x4 *>(p);
        }
        if (tid < kBlockN) {
            b_key = n0 + tid;
            if (b_base) b_raw = b_base[min(b_key, L - 1)];
        }
    };
    auto fetch_v = [&](int tile) {
        const int n0 = tile * kBlockN;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint16_t *p = n0 + sr + 32 * i < L ? v_row[i] + tile * v_tile_step : v_last;
            v_stage[i] = *reinterpret_cast<const u32x4 *>(p);
        }
    };
    auto commit_k = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
            *reinterpret_cast<u32x4 *>(&lds_k[buf][(sr + 32 * i) * kKPitch + sc * 8]) = k_stage[i];
        if (tid < kBlockN) {
            // t = bias / scale split exactly into three 16-bit terms; -inf beyond the segment
            const float t = b_base ? E::to_f32(b_raw) * a.inv_scale : 0.f;
            uint32_t t_hi = E::from_f32(t), t_mid = 0, t_lo = 0;
            const float hi_f = E::to_f32(static_cast<uint16_t>(t_hi));
            if (fabsf(hi_f) != INFINITY) {
                const float r1 = t - hi_f;
                t_mid = E::from_f32(r1);
                t_lo = E::from_f32(r1 - E::to_f32(static_cast<uint16_t>(t_mid)));
            }
            if (b_key >= L) {
                t_hi = E::kNegInf;
                t_mid = 0;
                t_lo = 0;
            }
            *reinterpret_cast<u32x4 *>(&lds_k[buf][tid * kKPitch + 64]) = u32x4{t_hi | (t_mid << 16), t_lo, 0u, 0u};
            *reinterpret_cast<u32x4 *>(&lds_k[buf][tid * kKPitch + 72]) = zero4();
        }
    };
    auto commit_v = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
            *reinterpret_cast<u32x4 *>(&lds_v[buf][(sr + 32 * i) * kVPitch + sc * 8]) = v_stage[i];
    };

    const int k_off = r * kKPitch + 8 * h;
    const int v_off = (4 * h + ((lane & 15) >> 2)) * kVPitch + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    f32x16 s_acc[2][2];          // scores of the two query tiles (two 32-key halves each)
    f32x16 o_acc[2][2];
    u32x4 p_frag[2][4];
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        o_acc[qt][0] = zero16;
        o_acc[qt][1] = zero16;
#pragma unroll
        for (int u = 0; u < 4; ++u) p_frag[qt][u] = zero4();
    }

    // scores of query tile `qt` against the K' tile in `buf`
    auto score_mfma = [&](int qt, int buf) {
#pragma unroll
        for (int ks = 0; ks < 5; ++ks) {
#ifdef COME_EXP_NO_LDSREAD
            const u32x4 kf0 = qf[qt ^ 1][ks & 3], kf1 = qf[qt ^ 1][(ks + 1) & 3];
#else
            const u32x4 kf0 = *reinterpret_cast<const u32x4 *>(&lds_k[buf][k_off + 16 * ks]);
            const u32x4 kf1 = *reinterpret_cast<const u32x4 *>(&lds_k[buf][k_off + 32 * kKPitch + 16 * ks]);
#endif
            const u32x4 qb = ks < 4 ? qf[qt][ks < 4 ? ks : 0] : q_ext;
            s_acc[qt][0] = E::mfma(kf0, qb, ks == 0 ? zero16 : s_acc[qt][0]);
            s_acc[qt][1] = E::mfma(kf1, qb, ks == 0 ? zero16 : s_acc[qt][1]);
        }
    };
    // O^T += V^T P^T of query tile `qt` with the V tile in `buf`
    auto pv_mfma = [&](int qt, int buf) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const uint16_t *vp = &lds_v[buf][v_off + (16 * u) * kVPitch + 32 * dt];
#ifdef COME_EXP_NO_LDSREAD
                (void)vp;
                const u32x2 lo2 = {qf[qt][u][0], qf[qt][u][1]}, hi2 = {qf[qt][u][2], qf[qt][u][3]};
#else
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lds_read_tr(vp));
                const u32x2 hi2 = __builtin_bit_cast(u32x2, lds_read_tr(vp + 8 * kVPitch));
#endif
                o_acc[qt][dt] = E::mfma(u32x4{lo2[0], lo2[1], hi2[0], hi2[1]}, p_frag[qt][u], o_acc[qt][dt]);
            }
        }
    };
    // online softmax of query tile `qt`: S -> P (16-bit B operands), updates m, l; returns the O rescale factor
    auto softmax = [&](int qt) -> float {
        float mx0 = fmaxf(s_acc[qt][0][0], s_acc[qt][0][1]);
        float mx1 = fmaxf(s_acc[qt][0][8], s_acc[qt][0][9]);
        float mx2 = fmaxf(s_acc[qt][1][0], s_acc[qt][1][1]);
        float mx3 = fmaxf(s_acc[qt][1][8], s_acc[qt][1][9]);
#pragma unroll
        for (int i = 2; i < 8; i += 2) {
            mx0 = fmaxf(fmaxf(mx0, s_acc[qt][0][i]), s_acc[qt][0][i + 1]);
            mx1 = fmaxf(fmaxf(mx1, s_acc[qt][0][8 + i]), s_acc[qt][0][9 + i]);
            mx2 = fmaxf(fmaxf(mx2, s_acc[qt][1][i]), s_acc[qt][1][i + 1]);
            mx3 = fmaxf(fmaxf(mx3, s_acc[qt][1][8 + i]), s_acc[qt][1][9 + i]);
        }
        float mx = fmaxf(fmaxf(mx0, mx1), fmaxf(mx2, mx3));
        mx = max_across_halves(mx);
        const float m_new = fmaxf(m_run[qt], mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_use) * a.scale_log2);
        const float mc = m_use * a.scale_log2;
        float sum = 0.f;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                u32x4 f;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
#ifdef COME_EXP_NO_SOFTMAX
                    const float p0 = s_acc[qt][mt][8 * t + 2 * w], p1 = s_acc[qt][mt][8 * t + 2 * w + 1];
                    f[w] = __float_as_uint(p0) ^ __float_as_uint(p1);
#else
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[qt][mt][8 * t + 2 * w], a.scale_log2, -mc));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[qt][mt][8 * t + 2 * w + 1], a.scale_log2, -mc));
                    f[w] = E::pack2(p0, p1);
                    sum = E::dot2_ones(f[w], sum);
#endif
                }
                p_frag[qt][2 * mt + t] = f;
            }
        }
        l_run[qt] = l_run[qt] * alpha + sum;
        m_run[qt] = m_new;
        // ties the rescale decision to the end of the softmax, so the branch that follows cannot be
        // hoisted into the middle of it and the whole slot stays one scheduling region
        float alpha_late = alpha;
        asm volatile("" : "+v"(alpha_late) : "v"(sum), "v"(p_frag[qt][3][3]));
        return alpha_late;
    };
    // One slot in explicit issue order.  The matrix pipe works on query tile Y: 10 score MFMAs against
    // the K' tile in `kbuf` (S[Y] is rebuilt), then 8 P V MFMAs with the V tile in `vbuf` (P[Y] from
    // the previous slot).  The vector ALU runs the softmax of query tile X in between: MFMA i is
    // followed by a chunk of softmax work, and the LDS reads of MFMA i + 2 are requested before it,
    // so an in-order wavefront always has independent vector work behind every MFMA.
    // sched_barrier keeps the compiler from regrouping the chunks.
    auto slot = [&](int X, int Y, int kbuf, int vbuf) -> float {
        u32x4 frag[18];
        auto request = [&](int i) {
            if (i < 10) {
                const int ks = i >> 1, mt = i & 1;
                frag[i] = *reinterpret_cast<const u32x4 *>(&lds_k[kbuf][k_off + 32 * mt * kKPitch + 16 * ks]);
            } else if (i < 18) {
                const int u = (i - 10) >> 1, dt = (i - 10) & 1;
                const uint16_t *vp = &lds_v[vbuf][v_off + (16 * u) * kVPitch + 32 * dt];
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lds_read_tr(vp));
                const u32x2 hi2 = __builtin_bit_cast(u32x2, lds_read_tr(vp + 8 * kVPitch));
                frag[i] = u32x4{lo2[0], lo2[1], hi2[0], hi2[1]};
            }
        };
        auto issue = [&](int i) {
            if (i < 10) {
                const int ks = i >> 1, mt = i & 1;
                const u32x4 qb = ks < 4 ? qf[Y][ks < 4 ? ks : 0] : q_ext;
                s_acc[Y][mt] = E::mfma(frag[i], qb, ks == 0 ? zero16 : s_acc[Y][mt]);
            } else {
                const int u = (i - 10) >> 1, dt = (i - 10) & 1;
                o_acc[Y][dt] = E::mfma(frag[i], p_frag[Y][u], o_acc[Y][dt]);
            }
        };
        request(0);
        request(1);
        // -- chunk 0: four partial maxima
        issue(0);
        request(2);
        float mx0 = fmaxf(s_acc[X][0][0], s_acc[X][0][1]);
        float mx1 = fmaxf(s_acc[X][0][8], s_acc[X][0][9]);
        float mx2 = fmaxf(s_acc[X][1][0], s_acc[X][1][1]);
        float mx3 = fmaxf(s_acc[X][1][8], s_acc[X][1][9]);
#pragma unroll
        for (int e = 2; e < 8; e += 2) {
            mx0 = fmaxf(fmaxf(mx0, s_acc[X][0][e]), s_acc[X][0][e + 1]);
            mx1 = fmaxf(fmaxf(mx1, s_acc[X][0][8 + e]), s_acc[X][0][9 + e]);
            mx2 = fmaxf(fmaxf(mx2, s_acc[X][1][e]), s_acc[X][1][e + 1]);
            mx3 = fmaxf(fmaxf(mx3, s_acc[X][1][8 + e]), s_acc[X][1][9 + e]);
        }
        __builtin_amdgcn_sched_barrier(0);
        // -- chunk 1: row max across the two half-waves, new running max, rescale factor
        issue(1);
        request(3);
        float mx = fmaxf(fmaxf(mx0, mx1), fmaxf(mx2, mx3));
        mx = max_across_halves(mx);
        const float m_new = fmaxf(m_run[X], mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f((m_run[X] - m_use) * a.scale_log2);
        const float mc = m_use * a.scale_log2;
        float sum = 0.f;
        __builtin_amdgcn_sched_barrier(0);
        // -- chunks 2..17: one pair of probabilities each
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            issue(2 + c);
            request(4 + c);
            const int mt = c >> 3, t = (c >> 2) & 1, w = c & 3;
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[X][mt][8 * t + 2 * w], a.scale_log2, -mc));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[X][mt][8 * t + 2 * w + 1], a.scale_log2, -mc));
            const uint32_t pw = E::pack2(p0, p1);
            p_frag[X][2 * mt + t][w] = pw;
            sum = E::dot2_ones(pw, sum);
            __builtin_amdgcn_sched_barrier(0);
        }
        l_run[X] = l_run[X] * alpha + sum;
        m_run[X] = m_new;
        // the rescale decision is tied to the end of the slot so that the branch which follows cannot be
        // moved above the probability chunks
        float alpha_late = alpha;
        asm volatile("" : "+v"(alpha_late) : "v"(sum), "v"(p_frag[X][3][3]));
        return alpha_late;
    };

    auto rescale = [&](int qt, float alpha) {
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) o_acc[qt][dt][i] *= alpha;
        }
    };

    // asks the scheduler to issue one slot as: LDS reads ahead, then 18 x {1 MFMA, LDS reads, ~7 VALU}
    auto interleave_hint = [&]() {
        // operand fragments are requested two MFMAs ahead of their use: 10 score MFMAs take one
        // ds_read_b128 each, 8 P V MFMAs two transposing reads each
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x402, 7, 0);
        }
#pragma unroll
        for (int i = 8; i < 16; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x402, 7, 0);
        }
#pragma unroll
        for (int i = 16; i < 18; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x402, 7, 0);
        }
    };

    // ---- prologue
    const int n_tiles = (L + kBlockN - 1) / kBlockN;
    {   // V stage 2 stands in for "tile -1": zeros (P1 is zero there as well)
        u32x4 *z = reinterpret_cast<u32x4 *>(&lds_v[2][0]);
        for (int i = tid; i < kBlockN * kVPitch / 8; i += kThreads) z[i] = zero4();
    }
    fetch_k(0);
    fetch_v(0);
    commit_k(0);
    commit_v(0);
    fetch_k(1);
    commit_k(1);
    __syncthreads();
    score_mfma(0, 0);

    int kb = 0;                  // stage of K'(j) and V(j); K'(j+1) is in kb + 1, V(j-1) in kb + 2 (mod 3)
    for (int j = 0; j < n_tiles; ++j) {
        const int kb1 = kb == 2 ? 0 : kb + 1;
        const int kb2 = kb1 == 2 ? 0 : kb1 + 1;
#ifndef COME_EXP_NO_STAGE
        fetch_k(j + 2);
        fetch_v(j + 1);
#endif

        const float alpha0 = slot(0, 1, kb, kb2);      // slot a
        rescale(0, alpha0);
        const float alpha1 = slot(1, 0, kb1, kb);      // slot b
        rescale(1, alpha1);

#ifndef COME_EXP_NO_STAGE
        commit_k(kb2);
        commit_v(kb1);
#endif
#ifndef COME_EXP_NO_BARRIER
        __syncthreads();
#endif
        kb = kb1;
    }
    // V(n-1) now sits in stage kb + 2 (mod 3)
    pv_mfma(1, kb == 0 ? 2 : kb - 1);

#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const float l_tot = sum_across_halves(l_run[qt]);
        const float inv = 1.0f / l_tot;
        const int row = q0 + (wave * 2 + qt) * 32 + r;
        if (row < L) {
            uint16_t *op = a.out + static_cast<int64_t>(seq_start + row) * a.o_rs + head * a.o_hs + 4 * h;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = E::pack2(o_acc[qt][dt][4 * g] * inv, o_acc[qt][dt][4 * g + 1] * inv);
                    w[1] = E::pack2(o_acc[qt][dt][4 * g + 2] * inv, o_acc[qt][dt][4 * g + 3] * inv);
                    *reinterpret_cast<u32x2 *>(op + 32 * dt + 8 * g) = w;
                }
            if (h == 0 && a.lse)
                a.lse[static_cast<int64_t>(head) * a.total + seq_start + row] = m_run[qt] * a.scale + __logf(l_tot);
        }
    }
}

}  // namespace
}  // namespace come

using namespace come;

extern "C" int come_attn_varlen_fwd(const void *q, const void *k, const void *v, int dtype, int64_t q_row_stride,
                                    int64_t q_head_stride, int64_t k_row_stride, int64_t k_head_stride,
                                    int64_t v_row_stride, int64_t v_head_stride, const int32_t *cu_seqlens,
                                    int64_t n_seq, int64_t total, int64_t n_heads, int64_t head_dim,
                                    const void *perkey_bias, int64_t max_seqlen, float softmax_scale, void *out,
                                    int64_t o_row_stride, int64_t o_head_stride, float *lse, void *stream) {
    clear_error();
    COME_REQUIRE(dtype == COME_BF16 || dtype == COME_F16, COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: only fp16 and bf16 are supported");
    COME_REQUIRE(head_dim == kHeadDim, COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: only head_dim == 64 is implemented (got %lld)", (long long)head_dim);
    COME_REQUIRE(n_seq > 0, COME_ERR_INVALID, "come_attn_varlen_fwd: batch size must be positive");
    COME_REQUIRE(total >= 0 && n_heads > 0 && max_seqlen >= 0, COME_ERR_INVALID,
                 "come_attn_varlen_fwd: negative size");
    COME_REQUIRE(total < (1ll << 31) && n_heads < 65536 && n_seq < (1ll << 24), COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: problem too large");
    COME_REQUIRE(softmax_scale > 0.f && softmax_scale < INFINITY, COME_ERR_INVALID,
                 "come_attn_varlen_fwd: softmax_scale must be positive and finite");
    if (total == 0 || max_seqlen == 0) return COME_OK;
    COME_REQUIRE(q && k && v && out && cu_seqlens, COME_ERR_INVALID, "come_attn_varlen_fwd: NULL tensor");
    const int64_t strides[8] = {q_row_stride, q_head_stride, k_row_stride, k_head_stride,
                                v_row_stride, v_head_stride, o_row_stride, o_head_stride};
    for (int i = 0; i < 8; ++i)
        COME_REQUIRE(strides[i] >= kHeadDim || (i % 2 == 1 && n_heads == 1), COME_ERR_INVALID,
                     "come_attn_varlen_fwd: stride %d is smaller than head_dim", i);
    for (int i = 0; i < 6; ++i)
        COME_REQUIRE(strides[i] % 8 == 0, COME_ERR_UNSUPPORTED,
                     "come_attn_varlen_fwd: q/k/v strides must be multiples of 8 elements (16-byte loads)");
    COME_REQUIRE(o_row_stride % 4 == 0 && o_head_stride % 4 == 0, COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: out strides must be multiples of 4 elements");
    COME_REQUIRE((reinterpret_cast<uintptr_t>(q) & 15) == 0 && (reinterpret_cast<uintptr_t>(k) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(v) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0,
                 COME_ERR_UNSUPPORTED, "come_attn_varlen_fwd: q/k/v must be 16-byte aligned, out 8-byte aligned");

    static const int QT = getenv("COME_ATTN_QT") ? atoi(getenv("COME_ATTN_QT")) : 2;
    static const bool kPipe = getenv("COME_ATTN_PIPE") ? atoi(getenv("COME_ATTN_PIPE")) != 0 : true;
    const int kBlockM = kPipe ? 256 : 128 * QT;
    AttnArgs a{};
    a.q = static_cast<const uint16_t *>(q);
    a.k = static_cast<const uint16_t *>(k);
    a.v = static_cast<const uint16_t *>(v);
    a.bias = static_cast<const uint16_t *>(perkey_bias);
    a.out = static_cast<uint16_t *>(out);
    a.lse = lse;
    a.cu = cu_seqlens;
    a.q_rs = q_row_stride; a.q_hs = q_head_stride;
    a.k_rs = k_row_stride; a.k_hs = k_head_stride;
    a.v_rs = v_row_stride; a.v_hs = v_head_stride;
    a.o_rs = o_row_stride; a.o_hs = o_head_stride;
    a.total = total;
    a.n_heads = static_cast<int>(n_heads);
    a.n_mblocks = static_cast<int>(ceil_div(max_seqlen, kBlockM));
    a.scale = softmax_scale;
    a.scale_log2 = softmax_scale * 1.4426950408889634f;
    a.inv_scale = 1.0f / softmax_scale;
    const int64_t n_wg = n_seq * n_heads * a.n_mblocks;
    COME_REQUIRE(n_wg < (1ll << 31), COME_ERR_UNSUPPORTED, "come_attn_varlen_fwd: grid too large");
    const dim3 grid(static_cast<unsigned>(n_wg)), block(kThreads);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (kPipe) {
        if (dtype == COME_BF16) hipLaunchKernelGGL((attn_fwd_pipe_kernel<COME_BF16>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((attn_fwd_pipe_kernel<COME_F16>), grid, block, 0, s, a);
    } else if (dtype == COME_BF16) {
        if (QT == 1) hipLaunchKernelGGL((attn_fwd_kernel<COME_BF16, 1>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((attn_fwd_kernel<COME_BF16, 2>), grid, block, 0, s, a);
    } else {
        hipLaunchKernelGGL((attn_fwd_kernel<COME_F16, 2>), grid, block, 0, s, a);
    }
    COME_CHECK_LAUNCH("come_attn_varlen_fwd");
    return COME_OK;
}
