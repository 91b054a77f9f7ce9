// Window confidence means, lowest-confidence window selection and the merge plan for gfx950.
//
// One workgroup per batch element: it reduces every full window of that element's frames to its mean, finds the
// lower of the two order statistics that torch.quantile's linear interpolation needs with an exact radix select,
// its upper neighbour with one more reduction, forms the threshold in fp32, writes the strict "mean < threshold"
// mask and - when asked to - turns the mask into the packed-row plan of the merge (per-window prefix, row lengths,
// row offsets) without leaving the kernel.
//
// The data is tiny (thousands of means) and lives on one CU, so the kernel is priced in issued instructions and
// dependent steps, not in bytes (an instruction of the common path costs 16 cycles of the CU: 16 wavefronts on four
// SIMDs).  Hence: the ordered keys of the means stay in LDS, cross-lane reductions and scans are DPP moves instead
// of LDS permutes, a radix pass is "count, barrier, one wavefront scans the 1024-bin histogram, barrier", the first
// digit starts at the highest bit in which the keys differ, and low key bits that all keys share (16 of them for
// bf16 means) are dropped, so that narrow value ranges need one or two passes; comparison and plan share one sweep
// in which a wavefront's ballot over 64 windows of a row gives their packed positions.  Measured for 16 frames of
// 37 x 37 (2304 windows): 7.5 us from confidence to plan (5.9 us at 576 windows, 23 us at 13 824); fewer, fatter
// wavefronts (256 or 512 threads) were slower because nothing hides their LDS and memory latencies.
#include "come_common.h"

#include <cmath>

namespace come {
namespace {

constexpr int kSelectThreads = 1024;
constexpr int kUnroll = 1;                  // keys (windows) per thread and loop iteration whose loads are issued together
                                            // (1 and 2 measure the same with 16 wavefronts to hide latencies)
constexpr int kSelectWaves = kSelectThreads / 64;
constexpr int kLdsKeys = 16384;             // windows per batch element whose keys fit in LDS (global memory beyond)
constexpr int kBinBits = 10;
constexpr int kBins = 1 << kBinBits;
constexpr int kBinsPerLane = kBins / 64;
constexpr int kMaxPasses = 4;               // 32 key bits in digits of 10

__device__ inline uint32_t ordered_key(float x) {           // monotone float -> uint32
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ inline float key_to_float(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

// x / d for 0 <= x < 2^31 as a multiply and a shift (mul = ceil(2^shift / d), shift = 31 + ceil(log2 d))
struct FastDiv {
    uint32_t mul, shift;
};
inline FastDiv make_fastdiv(int64_t d) {
    uint32_t s = 0;
    while ((int64_t{1} << s) < d) ++s;
    const uint64_t pow = uint64_t{1} << (31 + s);
    return FastDiv{static_cast<uint32_t>((pow + static_cast<uint64_t>(d) - 1) / static_cast<uint64_t>(d)), 31 + s};
}
__device__ inline uint32_t fast_div(uint32_t x, const FastDiv &f) {
    return static_cast<uint32_t>((static_cast<uint64_t>(x) * f.mul) >> f.shift);
}

// ---- cross-lane scans as data-parallel-primitive moves (no LDS traffic) -------------------------------------
// After the six steps every lane holds op over lanes 0 .. itself; lane 63 holds the wavefront's total.
// Lanes without a source in a step combine with `idle`: the identity of op, or for an idempotent op the lane's own
// value.
enum : int { kRowShr1 = 0x111, kRowShr2 = 0x112, kRowShr4 = 0x114, kRowShr8 = 0x118, kRowBcast15 = 0x142, kRowBcast31 = 0x143 };

template <int CTRL, int ROW_MASK>
__device__ inline uint32_t dpp_take(uint32_t idle, uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(idle), static_cast<int>(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ inline uint32_t wave_scan_add(uint32_t v) {
    v += dpp_take<kRowShr1, 0xf>(0u, v);
    v += dpp_take<kRowShr2, 0xf>(0u, v);
    v += dpp_take<kRowShr4, 0xf>(0u, v);
    v += dpp_take<kRowShr8, 0xf>(0u, v);
    v += dpp_take<kRowBcast15, 0xa>(0u, v);
    v += dpp_take<kRowBcast31, 0xc>(0u, v);
    return v;
}
#define COME_WAVE_REDUCE(NAME, EXPR)                                                   \
    __device__ inline uint32_t NAME(uint32_t v) {                                      \
        uint32_t t;                                                                    \
        t = dpp_take<kRowShr1, 0xf>(v, v); v = EXPR;                                   \
        t = dpp_take<kRowShr2, 0xf>(v, v); v = EXPR;                                   \
        t = dpp_take<kRowShr4, 0xf>(v, v); v = EXPR;                                   \
        t = dpp_take<kRowShr8, 0xf>(v, v); v = EXPR;                                   \
        t = dpp_take<kRowBcast15, 0xa>(v, v); v = EXPR;                                \
        t = dpp_take<kRowBcast31, 0xc>(v, v); v = EXPR;                                \
        return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63)); \
    }
COME_WAVE_REDUCE(wave_min, min(v, t))
COME_WAVE_REDUCE(wave_or, v | t)
COME_WAVE_REDUCE(wave_and, v & t)
#undef COME_WAVE_REDUCE
__device__ inline uint32_t wave_sum(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_scan_add(v)), 63));
}

struct alignas(16) SelectShared {
    uint32_t hist[kMaxPasses][kBins];       // one histogram per pass, all cleared up front
    uint32_t keys[kLdsKeys];                // ordered keys of the window means
    uint32_t red[2][kSelectWaves];          // per wavefront: OR and AND of the keys
    uint32_t found[2];                      // per pass: bin that holds rank k, keys in front of it
    uint32_t above;                         // smallest key above the lower order statistic
    float fred[kSelectWaves + 1];
};

// Workgroup-wide sum (every thread receives it).
__device__ float block_sum(float v, float *red) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < kSelectWaves; ++w) t += red[w];
    return t;
}

template <int DT> __device__ inline float round_dt(float x) {
    if (DT == COME_BF16) return __uint_as_float(pack2_bf16(x, 0.f) << 16);
    return x;
}

struct SelectArgs {
    const void *conf;
    int frames, H, W, gh, gw;
    int mode;
    float threshold;
    int rank_lo, rank_hi;
    float frac;
    float *means;
    uint8_t *mask;
    // merge plan (offsets == nullptr: selection only)
    int32_t *offsets, *prefix;
    int start, tail;
    FastDiv by_windows, by_mw;              // windows per frame, windows per grid row
};

// k-th smallest (0-based) ordered key of the keys of this workgroup; visit(f) calls f(key) for every key the
// calling thread owns.  All threads call it and all receive the key.  One barrier for the bits in which the keys
// differ, then two per pass: the keys are counted into the pass's histogram, wavefront 0 scans it and publishes the
// bin that holds rank k.
template <typename Visit>
__device__ uint32_t select_kth(SelectShared &sh, Visit visit, uint32_t k) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    uint32_t kor = 0u, kand = 0xffffffffu;
    visit([&](uint32_t key) {
        kor |= key;
        kand &= key;
    });
    kor = wave_or(kor);
    kand = wave_and(kand);
    if (lane == 0) {
        sh.red[0][wave] = kor;
        sh.red[1][wave] = kand;
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kSelectWaves; ++w) {
        kor |= sh.red[0][w];
        kand &= sh.red[1][w];
    }
    // Bits in which all keys agree carry no order.  Those below the lowest varying bit are dropped (16 of them for
    // means rounded to bf16); those above the highest one are the common start `lo` of the group of candidates.
    const uint32_t varying = kor ^ kand;
    const int drop = varying == 0 ? 0 : __builtin_ctz(varying);
    const uint32_t low_bits = kand & ((1u << drop) - 1u);
    int width = varying == 0 ? 0 : 32 - __clz(static_cast<int>(varying)) - drop;   // candidates: lo .. lo + 2^width - 1
    uint32_t lo = width >= 32 ? 0u : ((kand >> drop) >> width) << width;             // (shifted keys)
    int shift = width > kBinBits ? width - kBinBits : 0;
#pragma unroll 1
    for (int pass = 0; pass < kMaxPasses; ++pass) {
        const uint32_t limit = width >= 32 ? 0xffffffffu : (1u << width) - 1u;
        uint32_t *hist = sh.hist[pass];
        visit([&](uint32_t key) {
            const uint32_t rel = (key >> drop) - lo;
            if (rel <= limit) atomicAdd(&hist[rel >> shift], 1u);
        });
        __syncthreads();
        if (wave == 0) {            // lane l owns bins kBinsPerLane * l .. + kBinsPerLane - 1
            uint32_t c[kBinsPerLane];
            uint32_t s = 0;
#pragma unroll
            for (int j = 0; j < kBinsPerLane; j += 4) {
                const uint4 q = *reinterpret_cast<const uint4 *>(&hist[lane * kBinsPerLane + j]);
                c[j] = q.x;
                c[j + 1] = q.y;
                c[j + 2] = q.z;
                c[j + 3] = q.w;
                s += q.x + q.y + q.z + q.w;
            }
            const uint32_t incl = wave_scan_add(s);
            const uint32_t excl = incl - s;
            if (k >= excl && k < incl) {        // exactly one lane: its bin that holds rank k, the keys in front of it
                uint32_t bin = static_cast<uint32_t>(lane * kBinsPerLane), before = excl;
                uint32_t run = excl;
#pragma unroll
                for (int j = 0; j < kBinsPerLane - 1; ++j) {
                    run += c[j];
                    const bool past = k >= run;
                    bin += past ? 1u : 0u;
                    before = past ? run : before;
                }
                sh.found[0] = bin;
                sh.found[1] = before;
            }
        }
        __syncthreads();
        k -= sh.found[1];
        lo += sh.found[0] << shift;
        if (shift == 0) break;
        width = shift;
        shift = shift > kBinBits ? shift - kBinBits : 0;
    }
    return (lo << drop) | low_bits;
}

template <int DT, int GH, int GW>
__global__ __launch_bounds__(kSelectThreads) void select_windows_kernel(const SelectArgs a) {
    using V = Vec16<DT>;
    __shared__ SelectShared sh;

    const int H = a.H, W = a.W, frames = a.frames, mode = a.mode;
    const int gh = GH > 0 ? GH : a.gh, gw = GW > 0 ? GW : a.gw;
    const int mh = H / gh, mw = W / gw;
    const int M = mh * mw;
    const int n = frames * M;
    const int64_t batch_first = static_cast<int64_t>(blockIdx.x) * n;
    float *my_means = a.means + batch_first;
    uint8_t *my_mask = a.mask + batch_first;
    const bool in_lds = n <= kLdsKeys;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t conf_first = static_cast<int64_t>(blockIdx.x) * frames * H * W;

    for (int i = threadIdx.x; i < kMaxPasses * kBins; i += kSelectThreads) (&sh.hist[0][0])[i] = 0;
    if (threadIdx.x == 0) sh.above = 0xffffffffu;

    // 0. normalised-score mode: z = (x - mean) / (std + 1e-3) over all positions of the batch element,
    //    every tensor operation of that chain rounded to the confidence dtype (unbiased std)
    float z_mean = 0.f, z_denom = 1.f;
    if (mode == 2) {
        const int64_t T = static_cast<int64_t>(frames) * H * W;
        float acc = 0.f;
        for (int64_t i = threadIdx.x; i < T; i += kSelectThreads) acc += V::load1(a.conf, conf_first + i);
        const float mean32 = block_sum(acc, sh.fred) / static_cast<float>(T);
        acc = 0.f;
        for (int64_t i = threadIdx.x; i < T; i += kSelectThreads) {
            const float d = V::load1(a.conf, conf_first + i) - mean32;
            acc += d * d;
        }
        const float var = block_sum(acc, sh.fred) / static_cast<float>(T > 1 ? T - 1 : 1);
        z_mean = round_dt<DT>(mean32);
        z_denom = round_dt<DT>(round_dt<DT>(sqrtf(var)) + 1e-3f);
    }

    // 1. window means: fp32 running sum in window row-major order, one division, rounded to the confidence dtype
    //    and widened back to fp32.  With a compile-time window shape all loads of a window are issued before the
    //    first addition waits for one.
    for (int i0 = threadIdx.x; i0 < n; i0 += kUnroll * kSelectThreads) {
        constexpr int NW = GH > 0 ? GH * GW : 1;
        float x[kUnroll][NW];
        int64_t base[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int i = min(i0 + u * kSelectThreads, n - 1);       // (a window beyond the end is computed twice, stored once)
            const int f = static_cast<int>(fast_div(i, a.by_windows));
            const int m = i - f * M;
            const int wy = static_cast<int>(fast_div(m, a.by_mw));
            const int wx = m - wy * mw;
            base[u] = conf_first + static_cast<int64_t>(f) * H * W + (wy * gh) * W + wx * gw;
            if constexpr (GH > 0) {
#pragma unroll
                for (int dy = 0; dy < GH; ++dy)
#pragma unroll
                    for (int dx = 0; dx < GW; ++dx) x[u][dy * GW + dx] = V::load1(a.conf, base[u] + dy * W + dx);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int i = i0 + u * kSelectThreads;
            float acc = 0.f;
            if constexpr (GH > 0) {
#pragma unroll
                for (int t = 0; t < GH * GW; ++t) {
                    float v = x[u][t];
                    if (mode == 2) v = round_dt<DT>(__fdiv_rn(round_dt<DT>(__fsub_rn(v, z_mean)), z_denom));
                    acc = __fadd_rn(acc, v);
                }
            } else {
                for (int dy = 0; dy < gh; ++dy)
                    for (int dx = 0; dx < gw; ++dx) {
                        float v = V::load1(a.conf, base[u] + dy * W + dx);
                        if (mode == 2) v = round_dt<DT>(__fdiv_rn(round_dt<DT>(__fsub_rn(v, z_mean)), z_denom));
                        acc = __fadd_rn(acc, v);
                    }
            }
            const float mean = round_dt<DT>(__fdiv_rn(acc, static_cast<float>(gh * gw)));
            if (i < n) {
                my_means[i] = mean;
                if (in_lds) sh.keys[i] = ordered_key(mean);
            }
        }
    }
    if (!in_lds) __syncthreads();              // the means in global memory are read back by other threads
    auto visit_keys = [&](auto f) {                // kUnroll keys are read before the first one is used
        for (int i0 = threadIdx.x; i0 < n; i0 += kUnroll * kSelectThreads) {
            uint32_t key[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int i = min(i0 + u * kSelectThreads, n - 1);
                key[u] = in_lds ? sh.keys[i] : ordered_key(my_means[i]);
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                if (i0 + u * kSelectThreads < n) f(key[u]);
        }
    };

    // 2. threshold.  Ranking: the two neighbouring order statistics of torch.quantile's linear interpolation;
    //    the upper one is either the same value again (duplicates) or the smallest value above the lower one.
    //    Absolute and normalised score compare a tensor of the confidence dtype with a scalar: the scalar is
    //    rounded to that dtype first, as the tensor library does (a bf16 mean of 0.44921875 is not below 0.45).
    float cut = round_dt<DT>(a.threshold);
    if (mode == 0) {
        // (a thread only visits keys it wrote itself, so the first visit needs no barrier)
        const uint32_t key_a = select_kth(sh, visit_keys, static_cast<uint32_t>(a.rank_lo));
        const float va = key_to_float(key_a);
        float vb = va;
        if (a.rank_hi != a.rank_lo) {
            // counts are integers: exact whatever the number of windows
            uint32_t le = 0;
            uint32_t above = 0xffffffffu;
            visit_keys([&](uint32_t key) {
                if (key <= key_a) ++le;
                else above = min(above, key);
            });
            le = wave_sum(le);
            above = wave_min(above);
            if (lane == 0) {
                sh.red[0][wave] = le;          // free again: its readers passed at least two barriers since
                atomicMin(&sh.above, above);
            }
            __syncthreads();
            uint32_t count_le = 0;
#pragma unroll
            for (int w = 0; w < kSelectWaves; ++w) count_le += sh.red[0][w];
            if (count_le <= static_cast<uint32_t>(a.rank_hi)) vb = key_to_float(sh.above);
        }
        const float diff = __fsub_rn(vb, va);
        cut = a.frac < 0.5f ? __fadd_rn(va, __fmul_rn(a.frac, diff))
                            : __fsub_rn(vb, __fmul_rn(diff, __fsub_rn(1.0f, a.frac)));
    }

    // 3. strict comparison (on the float values: -0 and +0 differ as keys, not as numbers)
    if (a.offsets == nullptr) {
        for (int i0 = threadIdx.x; i0 < n; i0 += kUnroll * kSelectThreads) {
            float mean[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int i = min(i0 + u * kSelectThreads, n - 1);
                mean[u] = in_lds ? key_to_float(sh.keys[i]) : my_means[i];
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                if (i0 + u * kSelectThreads < n) my_mask[i0 + u * kSelectThreads] = mean[u] < cut ? 1 : 0;
        }
        return;
    }

    // 3 + 4. with a merge plan: a wavefront takes whole rows (frames), 64 windows at a time, so the comparison
    //    bits of a step are one ballot and give the packed position of every window inside its row
    //    (start_index + G * kept before + merged before) and the row length; with a single batch element the row
    //    offsets follow (otherwise a second small kernel scans the lengths)
    __syncthreads();                                        // keys written by other threads (no barrier yet in modes 1, 2)
    const int G = gh * gw;
    const int row_first = blockIdx.x * frames;
    const uint64_t below = (1ull << lane) - 1ull;
    for (int f = wave; f < frames; f += kSelectWaves) {
        int running = 0;                                    // wave-uniform
        for (int m0 = 0; m0 < M; m0 += 64) {
            const int m = m0 + lane;
            const bool valid = m < M;
            const int i = f * M + min(m, M - 1);
            const float mean = in_lds ? key_to_float(sh.keys[i]) : my_means[i];
            const bool merged = valid && mean < cut;
            if (valid) my_mask[i] = merged ? 1 : 0;
            const uint64_t merged_bits = __ballot(merged);
            const int merged_before = __popcll(merged_bits & below);
            if (valid)
                a.prefix[static_cast<int64_t>(row_first + f) * M + m] =
                    running + merged_before + (lane - merged_before) * G;
            const int n_valid = min(64, M - m0);
            const int n_merged = __popcll(merged_bits);
            running += n_merged + (n_valid - n_merged) * G;
        }
        if (lane == 0) a.offsets[row_first + f + 1] = a.start + a.tail + running;
    }
    if (gridDim.x != 1) return;
    if (threadIdx.x == 0) a.offsets[0] = 0;
    __syncthreads();
    if (wave == 0) {                                        // in-place inclusive scan of the row lengths
        int carry = 0;
        for (int r0 = 0; r0 < frames; r0 += 64) {
            const int r = r0 + lane;
            const uint32_t len = r < frames ? static_cast<uint32_t>(a.offsets[r + 1]) : 0u;
            const uint32_t v = wave_scan_add(len);
            if (r < frames) a.offsets[r + 1] = static_cast<int>(v) + carry;
            carry += __builtin_amdgcn_readlane(static_cast<int>(v), 63);
        }
    }
}

// offsets[0] = 0 and an in-place inclusive scan of the row lengths in offsets[1 .. rows] (one wavefront)
__global__ __launch_bounds__(64) void scan_offsets_kernel(int32_t *__restrict__ offsets, int rows) {
    const int lane = threadIdx.x;
    if (lane == 0) offsets[0] = 0;
    int carry = 0;
    for (int r0 = 0; r0 < rows; r0 += 64) {
        const int r = r0 + lane;
        const uint32_t len = r < rows ? static_cast<uint32_t>(offsets[r + 1]) : 0u;
        const uint32_t v = wave_scan_add(len);
        if (r < rows) offsets[r + 1] = static_cast<int>(v) + carry;
        carry += __builtin_amdgcn_readlane(static_cast<int>(v), 63);
    }
}

int select_impl(const char *who, const void *conf, int dtype, int64_t batch, int64_t frames, int64_t grid_h,
                int64_t grid_w, int64_t group_h, int64_t group_w, int mode, float threshold, float *means_f32,
                uint8_t *merge_mask, void *work, int64_t work_bytes, bool plan, int64_t start_index,
                int32_t *offsets, int32_t *group_prefix, void *stream) {
    COME_REQUIRE(dtype == COME_BF16 || dtype == COME_F32, COME_ERR_UNSUPPORTED, "%s: confidence must be bf16 or fp32",
                 who);
    COME_REQUIRE(batch >= 0 && frames >= 0 && grid_h >= 0 && grid_w >= 0, COME_ERR_INVALID, "%s: negative size", who);
    COME_REQUIRE(group_h > 0 && group_w > 0, COME_ERR_INVALID, "%s: group_h and group_w must be > 0", who);
    COME_REQUIRE(mode >= 0 && mode <= 2, COME_ERR_UNSUPPORTED, "%s: unknown mode %d", who, mode);
    if (mode == 0)
        COME_REQUIRE(threshold >= 0.f && threshold <= 1.f, COME_ERR_INVALID,
                     "%s: ranking mode requires threshold in [0, 1], got %g", who, (double)threshold);
    const int64_t windows = (grid_h / group_h) * (grid_w / group_w);
    const int64_t n = frames * windows;
    const int64_t rows = batch * frames;
    if (plan) {
        COME_REQUIRE(start_index >= 0, COME_ERR_INVALID, "%s: start_index must be >= 0", who);
        COME_REQUIRE(batch > 0 && n > 0, COME_ERR_UNSUPPORTED,
                     "%s: no full window to select from (plan such rows with come_merge_plan)", who);
        COME_REQUIRE(offsets != nullptr && group_prefix != nullptr, COME_ERR_INVALID,
                     "%s: offsets / group_prefix is NULL", who);
        COME_REQUIRE(rows < (1ll << 31) && rows * (start_index + grid_h * grid_w) < (1ll << 31), COME_ERR_UNSUPPORTED,
                     "%s: rows * tokens per row must stay below 2^31", who);
    }
    if (batch == 0 || n == 0) return COME_OK;
    // n < 2^24: the rank float(threshold) * (n - 1) is formed in fp32, as torch.quantile forms it
    COME_REQUIRE(n < (1ll << 24) && batch < (1ll << 31) && frames * grid_h * grid_w < (1ll << 31) &&
                     batch * frames * grid_h * grid_w < (1ll << 40),
                 COME_ERR_UNSUPPORTED, "%s: problem too large", who);
    COME_REQUIRE(conf && merge_mask, COME_ERR_INVALID, "%s: conf / merge_mask is NULL", who);
    float *means = means_f32;
    if (!means) {
        COME_REQUIRE(work != nullptr && work_bytes >= batch * n * (int64_t)sizeof(float), COME_ERR_INVALID,
                     "%s: work buffer too small (%lld bytes given)", who, (long long)work_bytes);
        means = static_cast<float *>(work);
    }
    // rank = float(threshold) * (n - 1) in fp32, as torch.quantile computes it
    const float rank = threshold * static_cast<float>(n - 1);
    int lo = static_cast<int>(std::floor(rank));
    int hi = static_cast<int>(std::ceil(rank));
    lo = lo < 0 ? 0 : (lo > n - 1 ? static_cast<int>(n - 1) : lo);
    hi = hi < 0 ? 0 : (hi > n - 1 ? static_cast<int>(n - 1) : hi);
    SelectArgs a{};
    a.conf = conf;
    a.frames = static_cast<int>(frames);
    a.H = static_cast<int>(grid_h);
    a.W = static_cast<int>(grid_w);
    a.gh = static_cast<int>(group_h);
    a.gw = static_cast<int>(group_w);
    a.mode = mode;
    a.threshold = threshold;
    a.rank_lo = lo;
    a.rank_hi = hi;
    a.frac = rank - static_cast<float>(lo);
    a.means = means;
    a.mask = merge_mask;
    a.offsets = plan ? offsets : nullptr;
    a.prefix = plan ? group_prefix : nullptr;
    a.start = static_cast<int>(start_index);
    a.tail = static_cast<int>(grid_h * grid_w - windows * group_h * group_w);
    a.by_windows = make_fastdiv(windows);
    a.by_mw = make_fastdiv(grid_w / group_w);
    const dim3 grid(static_cast<unsigned>(batch)), block(kSelectThreads);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool w33 = group_h == 3 && group_w == 3;
    if (dtype == COME_BF16) {
        if (w33) hipLaunchKernelGGL((select_windows_kernel<COME_BF16, 3, 3>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((select_windows_kernel<COME_BF16, 0, 0>), grid, block, 0, s, a);
    } else {
        if (w33) hipLaunchKernelGGL((select_windows_kernel<COME_F32, 3, 3>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((select_windows_kernel<COME_F32, 0, 0>), grid, block, 0, s, a);
    }
    COME_CHECK_LAUNCH(who);
    if (plan && batch > 1) {
        hipLaunchKernelGGL(scan_offsets_kernel, dim3(1), dim3(64), 0, s, offsets, static_cast<int>(rows));
        COME_CHECK_LAUNCH(who);
    }
    return COME_OK;
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
    return select_impl("come_select_windows", conf, dtype, batch, frames, grid_h, grid_w, group_h, group_w, mode,
                       threshold, means_f32, merge_mask, work, work_bytes, false, 0, nullptr, nullptr, stream);
}

extern "C" int come_select_plan(const void *conf, int dtype, int64_t batch, int64_t frames, int64_t grid_h,
                                int64_t grid_w, int64_t group_h, int64_t group_w, int mode, float threshold,
                                int64_t start_index, float *means_f32, uint8_t *merge_mask, int32_t *offsets,
                                int32_t *group_prefix, void *work, int64_t work_bytes, void *stream) {
    clear_error();
    return select_impl("come_select_plan", conf, dtype, batch, frames, grid_h, grid_w, group_h, group_w, mode,
                       threshold, means_f32, merge_mask, work, work_bytes, true, start_index, offsets, group_prefix,
                       stream);
}
