// Window confidence means and lowest-confidence window selection for gfx950.
//
// One workgroup per batch element: it reduces every full window of that element's
// frames to its mean (kept in registers), finds the lower of the two order statistics
// that torch.quantile's linear interpolation needs with an exact 4 x 8-bit radix select
// over the float bit patterns and its upper neighbour with one more reduction, forms the
// threshold in fp32 and writes the strict "mean < threshold" mask.  The data is tiny (thousands of means), so the kernel is latency bound; it
// exists to keep the selection on the device and bit-exact.
#include "come_common.h"

#include <cmath>

namespace come {
namespace {

constexpr int kSelectThreads = 1024;

__device__ inline uint32_t ordered_key(float x) {           // monotone float -> uint32
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ inline float key_to_float(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

constexpr int kKeysPerThread = 8;      // means kept in registers up to 8 * 1024 per batch element

// k-th smallest (0-based) of the n values the workgroup holds: thread t owns values t, t + 1024, ...
// either in mine[] (n <= 8192) or in vals[] (global).  All threads call it and all receive the answer.
// hist: 256 counters, ctl: 2 words, red: 34 words of LDS.
// The leading bits that the smallest and the largest key share are decided up front, so the first 8-bit digit
// already spreads the keys over the histogram (confidence means sit in a narrow range: without this step they
// would all hit the same few counters) and narrow ranges need fewer passes.
__device__ float radix_select(const float *vals, const float *mine, bool in_regs, int n, int k, uint32_t *hist,
                              uint32_t *ctl, uint32_t *red) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    uint32_t kmin = 0xffffffffu, kmax = 0u;
    if (in_regs) {
#pragma unroll
        for (int r = 0; r < kKeysPerThread; ++r) {
            if (static_cast<int>(threadIdx.x) + r * kSelectThreads < n) {
                const uint32_t key = ordered_key(mine[r]);
                kmin = min(kmin, key);
                kmax = max(kmax, key);
            }
        }
    } else {
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const uint32_t key = ordered_key(vals[i]);
            kmin = min(kmin, key);
            kmax = max(kmax, key);
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        kmin = min(kmin, static_cast<uint32_t>(__shfl_xor(static_cast<int>(kmin), d)));
        kmax = max(kmax, static_cast<uint32_t>(__shfl_xor(static_cast<int>(kmax), d)));
    }
    if (lane == 0) {
        red[wave] = kmin;
        red[16 + wave] = kmax;
    }
    __syncthreads();
    kmin = red[0];
    kmax = red[16];
#pragma unroll
    for (int w = 1; w < kSelectThreads / 64; ++w) {
        kmin = min(kmin, red[w]);
        kmax = max(kmax, red[16 + w]);
    }
    int open_bits = 32 - __clz(static_cast<int>(kmin ^ kmax));        // low bits in which keys differ (0: all equal)
    if (kmin == kmax) open_bits = 0;
    uint32_t fixed = open_bits >= 32 ? 0u : ~((1u << open_bits) - 1u);
    uint32_t prefix = kmin & fixed;
    int shift = open_bits;
    while (shift > 0) {
        shift = shift > 8 ? shift - 8 : 0;
        if (threadIdx.x < 256) hist[threadIdx.x] = 0;
        __syncthreads();
        if (in_regs) {
#pragma unroll
            for (int r = 0; r < kKeysPerThread; ++r) {
                if (static_cast<int>(threadIdx.x) + r * kSelectThreads < n) {
                    const uint32_t key = ordered_key(mine[r]);
                    if ((key & fixed) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
                }
            }
        } else {
            for (int i = threadIdx.x; i < n; i += blockDim.x) {
                const uint32_t key = ordered_key(vals[i]);
                if ((key & fixed) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
            }
        }
        __syncthreads();
        if (wave == 0) {
            uint32_t c[4];
            uint32_t s = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                c[j] = hist[lane * 4 + j];
                s += c[j];
            }
            uint32_t incl = s;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t t = __shfl_up(incl, d);
                if (lane >= d) incl += t;
            }
            const uint32_t excl = incl - s;
            const uint32_t kk = static_cast<uint32_t>(k);
            if (kk >= excl && kk < incl) {
                uint32_t r = kk - excl;
                int j = 0;
                while (j < 3 && r >= c[j]) {
                    r -= c[j];
                    ++j;
                }
                ctl[0] = static_cast<uint32_t>(lane * 4 + j);
                ctl[1] = r;
            }
        }
        __syncthreads();
        // a digit may overlap bits that are already decided (last pass): they agree by construction
        prefix |= ctl[0] << shift;
        fixed |= 255u << shift;
        k = static_cast<int>(ctl[1]);
    }
    __syncthreads();                       // ctl, hist and red are free again
    return key_to_float(prefix);
}

// Workgroup-wide sum (every thread receives it).  red: 17 floats of LDS.
__device__ float block_sum(float v, float *red) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    if (wave == 0) {
        float t = lane < kSelectThreads / 64 ? red[lane] : 0.f;
#pragma unroll
        for (int d = 8; d >= 1; d >>= 1) t += __shfl_xor(t, d);
        if (lane == 0) red[16] = t;
    }
    __syncthreads();
    return red[16];
}

template <int DT> __device__ inline float round_dt(float x) {
    if (DT == COME_BF16) return __uint_as_float(pack2_bf16(x, 0.f) << 16);
    return x;
}

template <int DT>
__global__ __launch_bounds__(kSelectThreads) void select_windows_kernel(
    const void *__restrict__ conf, int frames, int H, int W, int gh, int gw, int mode, float threshold,
    int rank_lo, int rank_hi, float frac, float *__restrict__ means, uint8_t *__restrict__ mask) {
    using V = Vec16<DT>;
    __shared__ uint32_t hist[256];
    __shared__ uint32_t ctl[2];
    __shared__ float red[34];

    const int mh = H / gh, mw = W / gw;
    const int M = mh * mw;
    const int n = frames * M;
    const int64_t batch_first = static_cast<int64_t>(blockIdx.x) * n;
    float *my_means = means + batch_first;
    uint8_t *my_mask = mask + batch_first;
    const bool in_regs = n <= kKeysPerThread * kSelectThreads;

    // 0. normalised-score mode: z = (x - mean) / (std + 1e-3) over all positions of the batch element,
    //    every tensor operation of that chain rounded to the confidence dtype (unbiased std)
    float z_mean = 0.f, z_denom = 1.f;
    if (mode == 2) {
        const int64_t T = static_cast<int64_t>(frames) * H * W;
        const int64_t first = static_cast<int64_t>(blockIdx.x) * T;
        float acc = 0.f;
        for (int64_t i = threadIdx.x; i < T; i += blockDim.x) acc += V::load1(conf, first + i);
        const float mean32 = block_sum(acc, red) / static_cast<float>(T);
        acc = 0.f;
        for (int64_t i = threadIdx.x; i < T; i += blockDim.x) {
            const float d = V::load1(conf, first + i) - mean32;
            acc += d * d;
        }
        const float var = block_sum(acc, red) / static_cast<float>(T > 1 ? T - 1 : 1);
        z_mean = round_dt<DT>(mean32);
        z_denom = round_dt<DT>(round_dt<DT>(sqrtf(var)) + 1e-3f);
    }

    // 1. window means: fp32 running sum in window row-major order, one division,
    //    rounded to the confidence dtype and widened back to fp32
    float mine[kKeysPerThread];
#pragma unroll
    for (int r = 0; r < kKeysPerThread; ++r) mine[r] = 0.f;
    auto window_mean = [&](int i) {
        const int f = i / M;
        const int m = i - f * M;
        const int wy = m / mw;
        const int wx = m - wy * mw;
        const int64_t base = (static_cast<int64_t>(blockIdx.x) * frames + f) * H * W +
                             static_cast<int64_t>(wy * gh) * W + wx * gw;
        float acc = 0.f;
        for (int dy = 0; dy < gh; ++dy)
            for (int dx = 0; dx < gw; ++dx) {
                float x = V::load1(conf, base + static_cast<int64_t>(dy) * W + dx);
                if (mode == 2) x = round_dt<DT>(__fdiv_rn(round_dt<DT>(__fsub_rn(x, z_mean)), z_denom));
                acc = __fadd_rn(acc, x);
            }
        return round_dt<DT>(__fdiv_rn(acc, static_cast<float>(gh * gw)));
    };
    if (in_regs) {
#pragma unroll
        for (int r = 0; r < kKeysPerThread; ++r) {
            const int i = static_cast<int>(threadIdx.x) + r * kSelectThreads;
            if (i < n) {
                mine[r] = window_mean(i);
                my_means[i] = mine[r];
            }
        }
    } else {
        for (int i = threadIdx.x; i < n; i += blockDim.x) my_means[i] = window_mean(i);
        __syncthreads();
    }

    // 2. threshold.  Ranking: the two neighbouring order statistics of torch.quantile's linear interpolation;
    //    the upper one is either the same value again (duplicates) or the smallest value above the lower one.
    //    Absolute and normalised score compare a tensor of the confidence dtype with a scalar: the scalar is
    //    rounded to that dtype first, as the tensor library does (a bf16 mean of 0.44921875 is not below 0.45).
    float cut = round_dt<DT>(threshold);
    if (mode == 0) {
        const float a = radix_select(my_means, mine, in_regs, n, rank_lo, hist, ctl, reinterpret_cast<uint32_t *>(red));
        float b = a;
        if (rank_hi != rank_lo) {
            float le = 0.f;                                   // exact in fp32: n < 2^24 (checked by the host)
            uint32_t above = 0xffffffffu;                     // ordered key of the smallest value > a
            const uint32_t key_a = ordered_key(a);
            auto visit = [&](float x) {
                const uint32_t key = ordered_key(x);
                if (key <= key_a) le += 1.f;
                else above = min(above, key);
            };
            if (in_regs) {
#pragma unroll
                for (int r = 0; r < kKeysPerThread; ++r)
                    if (static_cast<int>(threadIdx.x) + r * kSelectThreads < n) visit(mine[r]);
            } else {
                for (int i = threadIdx.x; i < n; i += blockDim.x) visit(my_means[i]);
            }
            if (threadIdx.x == 0) ctl[0] = 0xffffffffu;
            const float count_le = block_sum(le, red);       // its barriers also publish ctl[0]
            atomicMin(&ctl[0], above);
            __syncthreads();
            if (count_le <= static_cast<float>(rank_hi)) b = key_to_float(ctl[0]);
        }
        const float diff = __fsub_rn(b, a);
        cut = frac < 0.5f ? __fadd_rn(a, __fmul_rn(frac, diff))
                          : __fsub_rn(b, __fmul_rn(diff, __fsub_rn(1.0f, frac)));
    }

    // 3. strict comparison
    if (in_regs) {
#pragma unroll
        for (int r = 0; r < kKeysPerThread; ++r) {
            const int i = static_cast<int>(threadIdx.x) + r * kSelectThreads;
            if (i < n) my_mask[i] = mine[r] < cut ? 1 : 0;
        }
    } else {
        for (int i = threadIdx.x; i < n; i += blockDim.x) my_mask[i] = my_means[i] < cut ? 1 : 0;
    }
}

}  // namespace
}  // namespace come

using namespace come;

extern "C" int64_t come_select_work_bytes(int64_t batch, int64_t frames, int64_t grid_h, int64_t grid_w,
                                          int64_t group_h, int64_t group_w) {
    if (batch < 0 || frames < 0 || grid_h < 0 || grid_w < 0 || group_h <= 0 || group_w <= 0) return -1;
    const int64_t windows = (grid_h / group_h) * (grid_w / group_w);
    return batch * frames * windows * static_cast<int64_t>(sizeof(float)) + 16;
}

extern "C" int come_select_windows(const void *conf, int dtype, int64_t batch, int64_t frames, int64_t grid_h,
                                   int64_t grid_w, int64_t group_h, int64_t group_w, int mode, float threshold,
                                   float *means_f32, uint8_t *merge_mask, void *work, int64_t work_bytes,
                                   void *stream) {
    clear_error();
    COME_REQUIRE(dtype == COME_BF16 || dtype == COME_F32, COME_ERR_UNSUPPORTED,
                 "come_select_windows: confidence must be bf16 or fp32");
    COME_REQUIRE(batch >= 0 && frames >= 0 && grid_h >= 0 && grid_w >= 0, COME_ERR_INVALID,
                 "come_select_windows: negative size");
    COME_REQUIRE(group_h > 0 && group_w > 0, COME_ERR_INVALID,
                 "come_select_windows: group_h and group_w must be > 0");
    COME_REQUIRE(mode >= 0 && mode <= 2, COME_ERR_UNSUPPORTED, "come_select_windows: unknown mode %d", mode);
    if (mode == 0)
        COME_REQUIRE(threshold >= 0.f && threshold <= 1.f, COME_ERR_INVALID,
                     "come_select_windows: ranking mode requires threshold in [0, 1], got %g", (double)threshold);
    const int64_t windows = (grid_h / group_h) * (grid_w / group_w);
    const int64_t n = frames * windows;
    if (batch == 0 || n == 0) return COME_OK;
    // n < 2^24: ranks and counts of windows are exact in fp32, which is also what the quantile's fp32 rank needs
    COME_REQUIRE(n < (1ll << 24) && batch < (1ll << 31) && batch * frames * grid_h * grid_w < (1ll << 40),
                 COME_ERR_UNSUPPORTED, "come_select_windows: problem too large");
    COME_REQUIRE(conf && merge_mask, COME_ERR_INVALID, "come_select_windows: conf / merge_mask is NULL");
    float *means = means_f32;
    if (!means) {
        COME_REQUIRE(work != nullptr && work_bytes >= batch * n * (int64_t)sizeof(float), COME_ERR_INVALID,
                     "come_select_windows: work buffer too small (%lld bytes given)", (long long)work_bytes);
        means = static_cast<float *>(work);
    }
    // rank = float(threshold) * (n - 1) in fp32, as torch.quantile computes it
    const float rank = threshold * static_cast<float>(n - 1);
    int lo = static_cast<int>(std::floor(rank));
    int hi = static_cast<int>(std::ceil(rank));
    lo = lo < 0 ? 0 : (lo > n - 1 ? static_cast<int>(n - 1) : lo);
    hi = hi < 0 ? 0 : (hi > n - 1 ? static_cast<int>(n - 1) : hi);
    const float frac = rank - static_cast<float>(lo);
    const dim3 grid(static_cast<unsigned>(batch)), block(kSelectThreads);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == COME_BF16)
        hipLaunchKernelGGL(select_windows_kernel<COME_BF16>, grid, block, 0, s, conf, static_cast<int>(frames),
                           static_cast<int>(grid_h), static_cast<int>(grid_w), static_cast<int>(group_h),
                           static_cast<int>(group_w), mode, threshold, lo, hi, frac, means, merge_mask);
    else
        hipLaunchKernelGGL(select_windows_kernel<COME_F32>, grid, block, 0, s, conf, static_cast<int>(frames),
                           static_cast<int>(grid_h), static_cast<int>(grid_w), static_cast<int>(group_h),
                           static_cast<int>(group_w), mode, threshold, lo, hi, frac, means, merge_mask);
    COME_CHECK_LAUNCH("come_select_windows");
    return COME_OK;
}
