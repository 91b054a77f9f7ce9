// Window confidence means and lowest-confidence window selection for gfx950.
//
// One workgroup per batch element: it reduces every full window of that element's
// frames to its mean, finds the two order statistics that torch.quantile's linear
// interpolation needs with an exact 4 x 8-bit radix select over the float bit
// patterns, forms the threshold in fp32 and writes the strict "mean < threshold"
// mask.  The data is tiny (thousands of means), so the kernel is latency bound; it
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

// k-th smallest (0-based) of vals[0..n); all threads of the workgroup call it and
// all receive the answer.  hist: 256 counters, ctl: 2 words of LDS.
__device__ float radix_select(const float *vals, int n, int k, uint32_t *hist, uint32_t *ctl) {
    uint32_t prefix = 0, fixed = 0;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (threadIdx.x < 256) hist[threadIdx.x] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const uint32_t key = ordered_key(vals[i]);
            if ((key & fixed) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
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
        prefix |= ctl[0] << shift;
        fixed |= 255u << shift;
        k = static_cast<int>(ctl[1]);
        __syncthreads();
    }
    return key_to_float(prefix);
}

template <int DT>
__global__ __launch_bounds__(kSelectThreads) void select_windows_kernel(
    const void *__restrict__ conf, int frames, int H, int W, int gh, int gw, int mode, float threshold,
    int rank_lo, int rank_hi, float frac, float *__restrict__ means, uint8_t *__restrict__ mask) {
    using V = Vec16<DT>;
    __shared__ uint32_t hist[256];
    __shared__ uint32_t ctl[2];

    const int mh = H / gh, mw = W / gw;
    const int M = mh * mw;
    const int n = frames * M;
    const int64_t batch_first = static_cast<int64_t>(blockIdx.x) * n;
    float *my_means = means + batch_first;
    uint8_t *my_mask = mask + batch_first;

    // 1. window means: fp32 running sum in window row-major order, one division,
    //    rounded to the confidence dtype and widened back to fp32
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int f = i / M;
        const int m = i - f * M;
        const int wy = m / mw;
        const int wx = m - wy * mw;
        const int64_t base = (static_cast<int64_t>(blockIdx.x) * frames + f) * H * W +
                             static_cast<int64_t>(wy * gh) * W + wx * gw;
        float acc = 0.f;
        for (int dy = 0; dy < gh; ++dy)
            for (int dx = 0; dx < gw; ++dx) acc = __fadd_rn(acc, V::load1(conf, base + static_cast<int64_t>(dy) * W + dx));
        float mean = __fdiv_rn(acc, static_cast<float>(gh * gw));
        if (DT == COME_BF16) mean = __uint_as_float(pack2_bf16(mean, 0.f) << 16);
        my_means[i] = mean;
    }
    __syncthreads();

    // 2. threshold
    float cut = threshold;
    if (mode == 0) {
        const float a = radix_select(my_means, n, rank_lo, hist, ctl);
        const float b = rank_hi == rank_lo ? a : radix_select(my_means, n, rank_hi, hist, ctl);
        const float diff = __fsub_rn(b, a);
        cut = frac < 0.5f ? __fadd_rn(a, __fmul_rn(frac, diff))
                          : __fsub_rn(b, __fmul_rn(diff, __fsub_rn(1.0f, frac)));
    }

    // 3. strict comparison
    for (int i = threadIdx.x; i < n; i += blockDim.x) my_mask[i] = my_means[i] < cut ? 1 : 0;
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
    COME_REQUIRE(mode == 0 || mode == 1, COME_ERR_UNSUPPORTED, "come_select_windows: unknown mode %d", mode);
    if (mode == 0)
        COME_REQUIRE(threshold >= 0.f && threshold <= 1.f, COME_ERR_INVALID,
                     "come_select_windows: ranking mode requires threshold in [0, 1], got %g", (double)threshold);
    const int64_t windows = (grid_h / group_h) * (grid_w / group_w);
    const int64_t n = frames * windows;
    if (batch == 0 || n == 0) return COME_OK;
    COME_REQUIRE(n < (1ll << 30) && batch < (1ll << 31) && batch * frames * grid_h * grid_w < (1ll << 40),
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
