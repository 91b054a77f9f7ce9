// Token merge / unmerge for gfx950: HBM-bound gather-mean and gather kernels.
//
// Data movement is organised in 16-byte chunks: one thread owns one chunk column of
// one window (or of one copied token), issues all of the window's loads back to back
// (nine independent 16-byte loads for a 3x3 window) and writes either their mean
// (merged) or the rows themselves (kept).  A wavefront therefore reads 1 KiB
// contiguous per source row and writes 1 KiB contiguous per packed row.  Token data is
// touched once, so loads and stores carry the non-temporal hint; the rows an unmerge
// reads several times (merged windows) use ordinary loads and stay in L2.
#include "come_common.h"

namespace come {
namespace {

constexpr int kThreads = 256;
// the 16-byte merge kernel runs one wavefront per workgroup (measured at 64 / 128 / 256 / 512 / 1024 threads on the
// 16-frame microbenchmark: 14.2 / 14.6 / 14.8 / 16.0 / 18.1 us)
constexpr int kMergeThreads = 64;

// x / d for 0 <= x < 2^31 as one 32 x 32 -> 64 bit multiply and a shift (mul = ceil(2^shift / d),
// shift = 31 + ceil(log2 d)); the index arithmetic of the 16-byte kernels runs on these instead of the
// compiler's division sequences, which sit in front of every thread's first load
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

struct MergeGeom {
    int rows, n_tok, start, groups;
    int gh, gw, G;          // window shape, tokens per window
    int H, W, mw;           // token grid, windows per grid row
    int cov_h, cov_w;       // part of the grid covered by full windows
    int tail;               // grid positions outside the full windows
    int64_t out_rows;
};

struct MergeArgs {
    MergeGeom g;
    const void *tokens;
    void *out;
    const uint8_t *mask;
    const int32_t *offsets;
    const int32_t *prefix;
    int64_t *rev64;
    int32_t *rev32;
    float *weight;
    int32_t *count;
    int64_t group_items;     // rows * groups * chunks (or * chans in the scalar kernel)
    int64_t group_blocks;    // blocks that own group items
    int64_t single_items;    // rows * (start + tail) * chunks
    int chunks;              // 16-byte chunks per token row (vector kernel) / chans (scalar kernel)
    FastDiv by_chunks, by_groups, by_mw, by_per_row, by_side;   // 16-byte kernels only
};

__device__ inline void note_row(const MergeArgs &a, int64_t src_flat, int64_t dst) {
    if (a.rev64) a.rev64[src_flat] = dst;
    if (a.rev32) a.rev32[src_flat] = static_cast<int32_t>(dst);
}
__device__ inline void note_weight(const MergeArgs &a, int64_t dst, int n) {
    if (dst >= a.g.out_rows) return;
    if (a.weight) a.weight[dst] = static_cast<float>(n);
    if (a.count) a.count[dst] = n;
}

// position `r` (0-based) among the grid positions outside the full windows, image row-major
__device__ inline int leftover_position(const MergeGeom &g, int r) {
    const int side = g.W - g.cov_w;                 // leftover columns of a covered grid row
    const int upper = g.cov_h * side;
    if (r < upper) {
        const int y = r / side;
        return y * g.W + g.cov_w + (r - y * side);
    }
    return g.cov_h * g.W + (r - upper);
}

__device__ inline int leftover_position_fast(const MergeGeom &g, const FastDiv &by_side, int r) {
    const int side = g.W - g.cov_w;
    const int upper = g.cov_h * side;
    if (r < upper) {
        const int y = static_cast<int>(fast_div(static_cast<uint32_t>(r), by_side));
        return y * g.W + g.cov_w + (r - y * side);
    }
    return g.cov_h * g.W + (r - upper);
}

// ---------------------------------------------------------------------------------
// bookkeeping: mask -> per-window prefix, per-row length, row offsets.  A wavefront owns a row; up to
// kPlanRowsPerGroup rows run as one workgroup that also scans the lengths, more rows are spread
// over workgroups and a one-wavefront launch scans afterwards.
// ---------------------------------------------------------------------------------
constexpr int kPlanRowsPerGroup = 16;

__device__ inline void scan_row_lengths(int32_t *__restrict__ offsets, int rows) {   // one wavefront, in place
    const int lane = threadIdx.x & 63;
    int carry = 0;
    for (int r0 = 0; r0 < rows; r0 += 64) {
        const int r = r0 + lane;
        int v = r < rows ? offsets[r + 1] : 0;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int t = __shfl_up(v, d);
            if (lane >= d) v += t;
        }
        if (r < rows) offsets[r + 1] = v + carry;
        carry += __shfl(v, 63);
    }
}

__global__ __launch_bounds__(64 * kPlanRowsPerGroup) void merge_plan_kernel(const uint8_t *__restrict__ mask, int rows,
                                                                            int groups, int start, int G, int tail,
                                                                            int32_t *__restrict__ offsets,
                                                                            int32_t *__restrict__ prefix) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint64_t below = (1ull << lane) - 1ull;

    for (int b = blockIdx.x * kPlanRowsPerGroup + wave; b < rows; b += gridDim.x * kPlanRowsPerGroup) {
        int running = 0;                                    // wave-uniform
        for (int m0 = 0; m0 < groups; m0 += 64) {
            const int m = m0 + lane;
            const bool valid = m < groups;
            const bool merged = valid && mask[static_cast<int64_t>(b) * groups + m] != 0;
            const uint64_t merged_bits = __ballot(merged);
            const int merged_before = __popcll(merged_bits & below);
            if (valid) prefix[static_cast<int64_t>(b) * groups + m] = running + merged_before + (lane - merged_before) * G;
            const int n_valid = min(64, groups - m0);
            const int n_merged = __popcll(merged_bits);
            running += n_merged + (n_valid - n_merged) * G;
        }
        if (lane == 0) offsets[b + 1] = start + tail + running;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) offsets[0] = 0;
    if (gridDim.x > 1) return;                              // the scan is the next launch
    __syncthreads();
    if (wave == 0) scan_row_lengths(offsets, rows);
}

__global__ __launch_bounds__(64) void merge_plan_scan_kernel(int32_t *__restrict__ offsets, int rows) {
    scan_row_lengths(offsets, rows);
}

// ---------------------------------------------------------------------------------
// merge, 16-byte path.  GH x GW fixed at compile time (0 x 0 = run-time window shape).
// ---------------------------------------------------------------------------------
template <int DT, int GH, int GW>
__global__ __launch_bounds__(kMergeThreads) void merge_vec_kernel(const MergeArgs a) {
    using V = Vec16<DT>;
    const MergeGeom &g = a.g;
    const uint4 *__restrict__ src = static_cast<const uint4 *>(a.tokens);
    uint4 *__restrict__ dst = static_cast<uint4 *>(a.out);
    const int chunks = a.chunks;

    if (static_cast<int64_t>(blockIdx.x) < a.group_blocks) {
        const uint32_t id = blockIdx.x * kMergeThreads + threadIdx.x;     // item counts stay below 2^31 (checked by the host)
        if (id >= a.group_items) return;
        const uint32_t gm = fast_div(id, a.by_chunks);      // flat (row, window)
        const int chunk = static_cast<int>(id - gm * chunks);
        const int b = static_cast<int>(fast_div(gm, a.by_groups));
        const int m = static_cast<int>(gm) - b * g.groups;
        const int wy = static_cast<int>(fast_div(m, a.by_mw));
        const int wx = m - wy * g.mw;
        const bool merged = a.mask[gm] != 0;
        const int64_t row0 = static_cast<int64_t>(a.offsets[b]) + g.start + a.prefix[gm];
        const int64_t tok0 = static_cast<int64_t>(b) * g.n_tok + g.start + (wy * g.gh) * g.W + wx * g.gw;
        const uint4 *p = src + tok0 * chunks + chunk;

        if constexpr (GH > 0) {
            uint4 v[GH * GW];
#pragma unroll
            for (int dy = 0; dy < GH; ++dy)
#pragma unroll
                for (int dx = 0; dx < GW; ++dx)
                    v[dy * GW + dx] = ld16_stream(p + (static_cast<int64_t>(dy) * g.W + dx) * chunks);
            if (merged) {
                float acc[V::N];
#pragma unroll
                for (int e = 0; e < V::N; ++e) acc[e] = 0.f;
#pragma unroll
                for (int t = 0; t < GH * GW; ++t) {
                    float f[V::N];
                    V::unpack(v[t], f);
#pragma unroll
                    for (int e = 0; e < V::N; ++e) acc[e] += f[e];
                }
#pragma unroll
                for (int e = 0; e < V::N; ++e) acc[e] = acc[e] / static_cast<float>(GH * GW);
                if (row0 < g.out_rows) st16_stream(dst + row0 * chunks + chunk, V::pack(acc));
            } else {
#pragma unroll
                for (int t = 0; t < GH * GW; ++t)
                    if (row0 + t < g.out_rows) st16_stream(dst + (row0 + t) * chunks + chunk, v[t]);
            }
        } else {
            if (merged) {
                float acc[V::N];
#pragma unroll
                for (int e = 0; e < V::N; ++e) acc[e] = 0.f;
                for (int dy = 0; dy < g.gh; ++dy) {
#pragma unroll 4
                    for (int dx = 0; dx < g.gw; ++dx) {
                        float f[V::N];
                        V::unpack(p[(static_cast<int64_t>(dy) * g.W + dx) * chunks], f);
#pragma unroll
                        for (int e = 0; e < V::N; ++e) acc[e] += f[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < V::N; ++e) acc[e] = acc[e] / static_cast<float>(g.G);
                if (row0 < g.out_rows) dst[row0 * chunks + chunk] = V::pack(acc);
            } else {
                int64_t r = row0;
                for (int dy = 0; dy < g.gh; ++dy) {
#pragma unroll 4
                    for (int dx = 0; dx < g.gw; ++dx, ++r)
                        if (r < g.out_rows) dst[r * chunks + chunk] = p[(static_cast<int64_t>(dy) * g.W + dx) * chunks];
                }
            }
        }

        // index map and counts of this window: token t of the window is noted by the thread of chunk t, so the
        // few small stores go out side by side instead of one after the other from a single lane
        const int gw_rt = GH > 0 ? GW : g.gw;
        for (int t = chunk; t < g.G; t += chunks) {
            const int dy = t / gw_rt;
            const int dx = t - dy * gw_rt;
            note_row(a, tok0 + static_cast<int64_t>(dy) * g.W + dx, merged ? row0 : row0 + t);
            if (!merged) note_weight(a, row0 + t, 1);
        }
        if (merged && chunk == 0) note_weight(a, row0, g.G);
        return;
    }

    // copied tokens: specials in front, leftover grid positions behind the windows
    const uint32_t id = (blockIdx.x - static_cast<uint32_t>(a.group_blocks)) * kMergeThreads + threadIdx.x;
    if (id >= a.single_items) return;
    const int per_row = g.start + g.tail;
    const uint32_t t = fast_div(id, a.by_chunks);
    const int chunk = static_cast<int>(id - t * chunks);
    const int b = static_cast<int>(fast_div(t, a.by_per_row));
    const int j = static_cast<int>(t) - b * per_row;
    int tok;
    int64_t row;
    if (j < g.start) {
        tok = j;
        row = static_cast<int64_t>(a.offsets[b]) + j;
    } else {
        const int r = j - g.start;
        tok = g.start + leftover_position_fast(g, a.by_side, r);
        row = static_cast<int64_t>(a.offsets[b + 1]) - g.tail + r;
    }
    const int64_t flat = static_cast<int64_t>(b) * g.n_tok + tok;
    if (row < g.out_rows) st16_stream(dst + row * chunks + chunk, ld16_stream(src + flat * chunks + chunk));
    if (chunk == 0) {
        note_row(a, flat, row);
        note_weight(a, row, 1);
    }
}

// ---------------------------------------------------------------------------------
// merge, element path: any channel count / alignment (e.g. the 2-channel position
// tensor).  One thread per (window, channel) or (copied token, channel).
// ---------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kThreads) void merge_elem_kernel(const MergeArgs a) {
    using V = Vec16<DT>;
    const MergeGeom &g = a.g;
    const int chans = a.chunks;

    if (static_cast<int64_t>(blockIdx.x) < a.group_blocks) {
        const int64_t id = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
        if (id >= a.group_items) return;
        const int64_t gm = id / chans;
        const int c = static_cast<int>(id - gm * chans);
        const int b = static_cast<int>(gm / g.groups);
        const int m = static_cast<int>(gm - static_cast<int64_t>(b) * g.groups);
        const int wy = m / g.mw;
        const int wx = m - wy * g.mw;
        const bool merged = a.mask[gm] != 0;
        const int64_t row0 = static_cast<int64_t>(a.offsets[b]) + g.start + a.prefix[gm];
        const int64_t tok0 = static_cast<int64_t>(b) * g.n_tok + g.start + (wy * g.gh) * g.W + wx * g.gw;
        float acc = 0.f;
        int t = 0;
        for (int dy = 0; dy < g.gh; ++dy) {
            for (int dx = 0; dx < g.gw; ++dx, ++t) {
                const int64_t tok = tok0 + static_cast<int64_t>(dy) * g.W + dx;
                const float x = V::load1(a.tokens, tok * chans + c);
                if (merged) {
                    acc += x;
                } else if (row0 + t < g.out_rows) {
                    V::store1(a.out, (row0 + t) * chans + c, x);
                }
                if (c == 0) {
                    note_row(a, tok, merged ? row0 : row0 + t);
                    if (!merged) note_weight(a, row0 + t, 1);
                }
            }
        }
        if (merged) {
            if (row0 < g.out_rows) V::store1(a.out, row0 * chans + c, acc / static_cast<float>(g.G));
            if (c == 0) note_weight(a, row0, g.G);
        }
        return;
    }

    const int64_t id = (static_cast<int64_t>(blockIdx.x) - a.group_blocks) * kThreads + threadIdx.x;
    if (id >= a.single_items) return;
    const int per_row = g.start + g.tail;
    const int64_t t = id / chans;
    const int c = static_cast<int>(id - t * chans);
    const int b = static_cast<int>(t / per_row);
    const int j = static_cast<int>(t - static_cast<int64_t>(b) * per_row);
    int tok;
    int64_t row;
    if (j < g.start) {
        tok = j;
        row = static_cast<int64_t>(a.offsets[b]) + j;
    } else {
        const int r = j - g.start;
        tok = g.start + leftover_position(g, r);
        row = static_cast<int64_t>(a.offsets[b + 1]) - g.tail + r;
    }
    const int64_t flat = static_cast<int64_t>(b) * g.n_tok + tok;
    if (row < g.out_rows) V::store1(a.out, row * chans + c, V::load1(a.tokens, flat * chans + c));
    if (c == 0) {
        note_row(a, flat, row);
        note_weight(a, row, 1);
    }
}

// ---------------------------------------------------------------------------------
// unmerge: out[i, :] = merged[rev[i], :]
// ---------------------------------------------------------------------------------
constexpr int kSplitRows = 1;         // output rows per thread (measured best of 1, 2, 3, 4, 8; the host assumes 1)
constexpr int kSplitRunRows = 256;    // output rows that stay on one XCD (64 - 1024 measured: no difference)

// PAIR: two packed sources with one index map; an output row holds the row of `merged` followed by the row of
// `merged_b` (`chunks` is the width of one source row, an output row has 2 * chunks chunks).
template <typename IndexT, bool PAIR>
__global__ __launch_bounds__(kThreads) void split_vec_kernel(const uint4 *__restrict__ merged,
                                                             const uint4 *__restrict__ merged_b, int64_t merged_rows,
                                                             const IndexT *__restrict__ rev, int64_t total,
                                                             int chunks, uint4 *__restrict__ out, int64_t items,
                                                             FastDiv by_out_chunks, uint32_t run) {
    // workgroup i runs on XCD i % 8; dealing the output rows to the XCDs in runs of `run` consecutive workgroups
    // (kSplitRunRows output rows) keeps the (up to nine) consumers of a merged row on one L2
    uint32_t bid = blockIdx.x;
    if (bid < (gridDim.x / (8u * run)) * (8u * run)) {
        const uint32_t local = bid >> 3;
        bid = ((local / run) * 8u + (bid & 7u)) * run + local % run;
    }
    const uint32_t id = bid * kThreads + threadIdx.x;               // items < 2^31 (checked by the host)
    if (id >= items) return;
    const int out_chunks = PAIR ? 2 * chunks : chunks;
    const uint32_t quad = fast_div(id, by_out_chunks);
    const int out_chunk = static_cast<int>(id - quad * out_chunks);
    const bool second = PAIR && out_chunk >= chunks;
    const uint4 *__restrict__ src = second ? merged_b : merged;
    const int chunk = second ? out_chunk - chunks : out_chunk;
    const int64_t i0 = static_cast<int64_t>(quad) * kSplitRows;
    uint4 v[kSplitRows];
#pragma unroll
    for (int r = 0; r < kSplitRows; ++r) {
        v[r] = make_uint4(0, 0, 0, 0);
        if (i0 + r < total) {
            const int64_t s = static_cast<int64_t>(rev[i0 + r]);
            if (s >= 0 && s < merged_rows) v[r] = src[s * chunks + chunk];
        }
    }
#pragma unroll
    for (int r = 0; r < kSplitRows; ++r)
        if (i0 + r < total) st16_stream(out + (i0 + r) * out_chunks + out_chunk, v[r]);
}

// Wave-per-row form for rows that are a multiple of 1 KiB wide (64 chunks): a wavefront owns ROWS consecutive
// output rows x one 64-chunk (1 KiB) column segment.  The row index is wave-uniform, so the indices come through the
// scalar path (one s_load for all of the wavefront's rows, no vector load in front of the gather) and the
// wavefront's row loads are issued back to back before the first store.  Measured on 16 / 32 / 64 / 128 frames:
// one row per wavefront is best while the launch is a few rounds of wavefronts (more, shorter wavefronts drain
// evenly), two rows from about 64 k wavefronts on (+9 .. 15 %); four and eight rows are slower everywhere.
constexpr int kSplitWaves = 4;

template <typename IndexT, bool PAIR, int ROWS>
__global__ __launch_bounds__(64 * kSplitWaves) void split_wave_kernel(const uint4 *__restrict__ merged,
                                                                      const uint4 *__restrict__ merged_b,
                                                                      int64_t merged_rows,
                                                                      const IndexT *__restrict__ rev, int total,
                                                                      int chunks, uint4 *__restrict__ out,
                                                                      int segs, uint32_t n_waves, uint32_t run,
                                                                      uint32_t remapped_blocks, FastDiv by_run,
                                                                      FastDiv by_segs) {
    uint32_t bid = blockIdx.x;
    if (bid < remapped_blocks) {                            // runs of `run` workgroups stay on one XCD (one L2)
        const uint32_t local = bid >> 3;
        const uint32_t q = fast_div(local, by_run);
        bid = (q * 8u + (bid & 7u)) * run + (local - q * run);
    }
    const uint32_t wave = __builtin_amdgcn_readfirstlane(bid * kSplitWaves + (threadIdx.x >> 6));
    if (wave >= n_waves) return;
    const int lane = threadIdx.x & 63;
    const uint32_t group = fast_div(wave, by_segs);
    const int seg = static_cast<int>(wave - group * segs);
    const int row0 = static_cast<int>(group) * ROWS;
    const int out_chunks = PAIR ? 2 * chunks : chunks;
    const int out_chunk = seg * 64 + lane;
    const bool second = PAIR && seg * 64 >= chunks;          // wave-uniform: chunks is a multiple of 64
    const uint4 *__restrict__ src = second ? merged_b : merged;
    const int chunk = second ? out_chunk - chunks : out_chunk;
    uint4 *__restrict__ dst = out + static_cast<int64_t>(row0) * out_chunks + out_chunk;
    if (row0 + ROWS <= total) {
        // all indices first, then all row loads, then the stores: the wavefront's ROWS index -> row -> store
        // chains overlap instead of running one after the other
        int64_t s[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) s[r] = static_cast<int64_t>(rev[row0 + r]);
        uint4 v[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const bool ok = s[r] >= 0 && s[r] < merged_rows;
            v[r] = src[(ok ? s[r] : 0) * chunks + chunk];
            if (!ok) v[r] = make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) st16_stream(dst + static_cast<int64_t>(r) * out_chunks, v[r]);
        return;
    }
    for (int r = 0; row0 + r < total; ++r) {                 // the last, partial group of rows
        const int64_t s = static_cast<int64_t>(rev[row0 + r]);
        uint4 v = make_uint4(0, 0, 0, 0);
        if (s >= 0 && s < merged_rows) v = src[s * chunks + chunk];
        st16_stream(dst + static_cast<int64_t>(r) * out_chunks, v);
    }
}

// element-wise fallback; `pair`: output rows are [row of merged | row of merged_b]
template <typename IndexT>
__global__ __launch_bounds__(kThreads) void split_elem_kernel(const uint8_t *__restrict__ merged,
                                                              const uint8_t *__restrict__ merged_b, bool pair,
                                                              int64_t merged_rows, const IndexT *__restrict__ rev,
                                                              int64_t total, int64_t row_bytes, int elem_bytes,
                                                              uint8_t *__restrict__ out) {
    const int64_t id = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t per_row = row_bytes / elem_bytes;
    const int64_t per_out = pair ? 2 * per_row : per_row;
    if (id >= total * per_out) return;
    const int64_t i = id / per_out;
    const int64_t oc = id - i * per_out;
    const bool second = oc >= per_row;
    const uint8_t *__restrict__ src = second ? merged_b : merged;
    const int64_t c = second ? oc - per_row : oc;
    const int64_t s = static_cast<int64_t>(rev[i]);
    const bool ok = s >= 0 && s < merged_rows;
    if (elem_bytes == 4) {
        reinterpret_cast<uint32_t *>(out)[id] = ok ? reinterpret_cast<const uint32_t *>(src)[s * per_row + c] : 0u;
    } else {
        reinterpret_cast<uint16_t *>(out)[id] =
            ok ? reinterpret_cast<const uint16_t *>(src)[s * per_row + c] : uint16_t(0);
    }
}

template <int DT>
void launch_merge_vec(const MergeArgs &a, int64_t blocks, hipStream_t stream) {
    const MergeGeom &g = a.g;
    const dim3 grid(static_cast<unsigned>(blocks)), block(kMergeThreads);
#define COME_MERGE_CASE(GH_, GW_)                                                              \
    if (g.gh == GH_ && g.gw == GW_) {                                                          \
        hipLaunchKernelGGL((merge_vec_kernel<DT, GH_, GW_>), grid, block, 0, stream, a);       \
        return;                                                                                \
    }
    COME_MERGE_CASE(3, 3)
    COME_MERGE_CASE(2, 2)
    COME_MERGE_CASE(1, 2)
    COME_MERGE_CASE(1, 4)
    COME_MERGE_CASE(1, 8)
    COME_MERGE_CASE(1, 9)
#undef COME_MERGE_CASE
    hipLaunchKernelGGL((merge_vec_kernel<DT, 0, 0>), grid, block, 0, stream, a);
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace
}  // namespace come

using namespace come;

extern "C" int come_merge_plan(const uint8_t *merge_mask, int64_t rows, int64_t groups, int64_t start_index,
                               int64_t group_size, int64_t tail, int32_t *offsets, int32_t *group_prefix,
                               void *stream) {
    clear_error();
    COME_REQUIRE(rows >= 0 && groups >= 0, COME_ERR_INVALID, "come_merge_plan: rows/groups must be >= 0");
    COME_REQUIRE(start_index >= 0, COME_ERR_INVALID, "come_merge_plan: start_index must be >= 0");
    COME_REQUIRE(group_size > 0, COME_ERR_INVALID, "come_merge_plan: group_size must be > 0");
    COME_REQUIRE(tail >= 0, COME_ERR_INVALID, "come_merge_plan: tail must be >= 0");
    COME_REQUIRE(offsets != nullptr, COME_ERR_INVALID, "come_merge_plan: offsets is NULL");
    COME_REQUIRE(rows * groups == 0 || (merge_mask && group_prefix), COME_ERR_INVALID,
                 "come_merge_plan: merge_mask / group_prefix is NULL");
    const int64_t n_tok = start_index + groups * group_size + tail;
    COME_REQUIRE(rows < (1ll << 31) && groups < (1ll << 31) && rows * n_tok < (1ll << 31), COME_ERR_UNSUPPORTED,
                 "come_merge_plan: rows * tokens per row must stay below 2^31");
    const int plan_groups = static_cast<int>(std::min<int64_t>(std::max<int64_t>((rows + kPlanRowsPerGroup - 1) / kPlanRowsPerGroup, 1), 2048));
    hipLaunchKernelGGL(merge_plan_kernel, dim3(plan_groups), dim3(64 * kPlanRowsPerGroup), 0,
                       static_cast<hipStream_t>(stream), merge_mask, static_cast<int>(rows), static_cast<int>(groups),
                       static_cast<int>(start_index), static_cast<int>(group_size), static_cast<int>(tail), offsets,
                       group_prefix);
    if (plan_groups > 1)
        hipLaunchKernelGGL(merge_plan_scan_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), offsets,
                           static_cast<int>(rows));
    COME_CHECK_LAUNCH("come_merge_plan");
    return COME_OK;
}

extern "C" int come_token_merge(const void *tokens, int dtype, int64_t rows, int64_t n_tok, int64_t chans,
                                int64_t start_index, int64_t group_h, int64_t group_w, int64_t grid_h,
                                int64_t grid_w, const uint8_t *merge_mask, const int32_t *offsets,
                                const int32_t *group_prefix, void *out, int64_t out_rows, int64_t *rev_i64,
                                int32_t *rev_i32, float *weight_f32, int32_t *count_i32, void *stream) {
    clear_error();
    COME_REQUIRE(dtype_ok(dtype), COME_ERR_UNSUPPORTED, "come_token_merge: unsupported dtype %d", dtype);
    COME_REQUIRE(rows >= 0 && n_tok >= 0 && chans >= 1 && out_rows >= 0, COME_ERR_INVALID,
                 "come_token_merge: negative size or chans < 1");
    COME_REQUIRE(start_index >= 0, COME_ERR_INVALID, "come_token_merge: start_index must be >= 0");
    COME_REQUIRE(group_h > 0 && group_w > 0, COME_ERR_INVALID, "come_token_merge: group_h and group_w must be > 0");
    COME_REQUIRE(grid_h >= 0 && grid_w >= 0, COME_ERR_INVALID, "come_token_merge: grid_h / grid_w must be >= 0");
    COME_REQUIRE(n_tok == start_index + grid_h * grid_w, COME_ERR_INVALID,
                 "come_token_merge: N != start_index + grid_h * grid_w (%lld != %lld + %lld * %lld)",
                 (long long)n_tok, (long long)start_index, (long long)grid_h, (long long)grid_w);
    COME_REQUIRE(rows * n_tok < (1ll << 31) && chans < (1ll << 24), COME_ERR_UNSUPPORTED,
                 "come_token_merge: rows * tokens per row must stay below 2^31");
    if (rows == 0 || n_tok == 0) return COME_OK;
    COME_REQUIRE(tokens && out && offsets, COME_ERR_INVALID, "come_token_merge: tokens / out / offsets is NULL");

    MergeArgs a{};
    MergeGeom &g = a.g;
    g.rows = static_cast<int>(rows);
    g.n_tok = static_cast<int>(n_tok);
    g.start = static_cast<int>(start_index);
    g.gh = static_cast<int>(group_h);
    g.gw = static_cast<int>(group_w);
    g.G = g.gh * g.gw;
    g.H = static_cast<int>(grid_h);
    g.W = static_cast<int>(grid_w);
    g.mw = g.W / g.gw;
    const int mh = g.H / g.gh;
    g.groups = mh * g.mw;
    g.cov_h = mh * g.gh;
    g.cov_w = g.mw * g.gw;
    g.tail = g.H * g.W - g.cov_h * g.cov_w;
    if (g.groups == 0) {            // no full window: every grid position is a leftover, row-major
        g.cov_h = 0;
        g.cov_w = 0;
        g.mw = 1;
    }
    g.out_rows = out_rows;
    COME_REQUIRE(g.groups == 0 || (merge_mask && group_prefix), COME_ERR_INVALID,
                 "come_token_merge: merge_mask / group_prefix is NULL");
    a.tokens = tokens;
    a.out = out;
    a.mask = merge_mask;
    a.offsets = offsets;
    a.prefix = group_prefix;
    a.rev64 = rev_i64;
    a.rev32 = rev_i32;
    a.weight = weight_f32;
    a.count = count_i32;

    const int64_t row_bytes = chans * dtype_bytes(dtype);
    const bool vec = (row_bytes % 16 == 0) && aligned16(tokens) && aligned16(out);
    a.chunks = static_cast<int>(vec ? row_bytes / 16 : chans);
    const int threads = vec ? kMergeThreads : kThreads;
    a.by_chunks = make_fastdiv(a.chunks);
    a.by_groups = make_fastdiv(g.groups > 0 ? g.groups : 1);
    a.by_mw = make_fastdiv(g.mw > 0 ? g.mw : 1);
    a.by_per_row = make_fastdiv(g.start + g.tail > 0 ? g.start + g.tail : 1);
    a.by_side = make_fastdiv(g.W - g.cov_w > 0 ? g.W - g.cov_w : 1);
    // a launch of the 16-byte kernel covers fewer than 2^31 (unit, chunk) items of either kind; more rows take
    // several launches over consecutive row ranges (packed positions are absolute, so `out` stays where it is)
    const int64_t per_row_items = static_cast<int64_t>(g.groups > g.start + g.tail ? g.groups : g.start + g.tail) * a.chunks;
    int64_t rows_per_launch = rows;
    if (vec && per_row_items > 0) {
        rows_per_launch = ((1ll << 31) - 1) / per_row_items;
        COME_REQUIRE(rows_per_launch >= 1, COME_ERR_UNSUPPORTED,
                     "come_token_merge: more than 2^31 16-byte items in one row");
        if (rows_per_launch > rows) rows_per_launch = rows;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t tok_bytes = n_tok * row_bytes;
    for (int64_t f0 = 0; f0 < rows; f0 += rows_per_launch) {
        const int64_t nf = rows - f0 < rows_per_launch ? rows - f0 : rows_per_launch;
        g.rows = static_cast<int>(nf);
        a.tokens = static_cast<const char *>(tokens) + f0 * tok_bytes;
        a.mask = merge_mask ? merge_mask + f0 * g.groups : nullptr;
        a.offsets = offsets + f0;
        a.prefix = group_prefix ? group_prefix + f0 * g.groups : nullptr;
        a.rev64 = rev_i64 ? rev_i64 + f0 * n_tok : nullptr;
        a.rev32 = rev_i32 ? rev_i32 + f0 * n_tok : nullptr;
        a.group_items = nf * g.groups * a.chunks;
        a.group_blocks = ceil_div(a.group_items, threads);
        a.single_items = nf * (g.start + g.tail) * a.chunks;
        const int64_t blocks = a.group_blocks + ceil_div(a.single_items, threads);
        COME_REQUIRE(blocks < (1ll << 31), COME_ERR_UNSUPPORTED, "come_token_merge: problem too large for one launch");
        if (blocks == 0) continue;
        if (vec) {
            if (dtype == COME_BF16) launch_merge_vec<COME_BF16>(a, blocks, s);
            else if (dtype == COME_F16) launch_merge_vec<COME_F16>(a, blocks, s);
            else launch_merge_vec<COME_F32>(a, blocks, s);
        } else {
            const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
            if (dtype == COME_BF16) hipLaunchKernelGGL(merge_elem_kernel<COME_BF16>, grid, block, 0, s, a);
            else if (dtype == COME_F16) hipLaunchKernelGGL(merge_elem_kernel<COME_F16>, grid, block, 0, s, a);
            else hipLaunchKernelGGL(merge_elem_kernel<COME_F32>, grid, block, 0, s, a);
        }
        COME_CHECK_LAUNCH("come_token_merge");
    }
    return COME_OK;
}

// shared body of come_token_split (pair = false, merged_b unused) and come_token_split_pair
static int token_split_impl(const char *who, bool pair, const void *merged, const void *merged_b, int dtype,
                            int64_t merged_rows, int64_t chans, const int64_t *rev_i64, const int32_t *rev_i32,
                            int64_t total, void *out, void *stream) {
    COME_REQUIRE(dtype_ok(dtype), COME_ERR_UNSUPPORTED, "%s: unsupported dtype %d", who, dtype);
    COME_REQUIRE(merged_rows >= 0 && chans >= 1 && total >= 0, COME_ERR_INVALID,
                 "%s: negative size or chans < 1", who);
    COME_REQUIRE((rev_i64 != nullptr) != (rev_i32 != nullptr) || total == 0, COME_ERR_INVALID,
                 "%s: exactly one of rev_i64 / rev_i32 must be given", who);
    if (total == 0) return COME_OK;
    COME_REQUIRE(out != nullptr && (merged_rows == 0 || (merged != nullptr && (!pair || merged_b != nullptr))),
                 COME_ERR_INVALID, "%s: merged / out is NULL", who);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t row_bytes = chans * dtype_bytes(dtype);
    const bool vec = (row_bytes % 16 == 0) && aligned16(merged) && aligned16(merged_b) && aligned16(out);
    if (vec) {
        const int chunks = static_cast<int>(row_bytes / 16);
        const int out_chunks = pair ? 2 * chunks : chunks;
        COME_REQUIRE(out_chunks < (1 << 23), COME_ERR_UNSUPPORTED, "%s: rows wider than 128 MiB are not supported", who);
        const FastDiv by_out_chunks = make_fastdiv(out_chunks);
        const int64_t run64 = static_cast<int64_t>(kSplitRunRows) * out_chunks / kThreads;
        const uint32_t run = static_cast<uint32_t>(run64 < 1 ? 1 : (run64 > 4096 ? 4096 : run64));
        // a launch covers fewer than 2^31 (row, 16-byte chunk) items; larger outputs take several launches over
        // consecutive row ranges (whole XCD runs each)
        int64_t rows_per_launch = ((1ll << 31) - 1) / out_chunks;
        if (rows_per_launch > kSplitRunRows) rows_per_launch -= rows_per_launch % kSplitRunRows;
        for (int64_t r0 = 0; r0 < total; r0 += rows_per_launch) {
            const int64_t nr = total - r0 < rows_per_launch ? total - r0 : rows_per_launch;
            const int64_t items = nr * out_chunks;
            if (out_chunks % 64 == 0 && chunks % 64 == 0 && merged_rows > 0) {
                const int segs = out_chunks / 64;
                const int wave_rows = nr * segs > 65536 ? 2 : 1;
                const int64_t n_waves = ceil_div(nr, wave_rows) * segs;
                const int64_t wrun64 = static_cast<int64_t>(kSplitRunRows) / wave_rows * segs / kSplitWaves;
                const uint32_t wrun = static_cast<uint32_t>(wrun64 < 1 ? 1 : wrun64);
                const dim3 wgrid(static_cast<unsigned>(ceil_div(n_waves, kSplitWaves))), wblock(64 * kSplitWaves);
                const uint4 *a4 = static_cast<const uint4 *>(merged), *b4 = static_cast<const uint4 *>(merged_b);
                uint4 *o4 = static_cast<uint4 *>(out) + r0 * out_chunks;
#define COME_SPLITW_ROWS(IDX_, PAIR_, REV_, ROWS_)                                                                  \
    hipLaunchKernelGGL((split_wave_kernel<IDX_, PAIR_, ROWS_>), wgrid, wblock, 0, s, a4, b4, merged_rows,           \
                       REV_ + r0, static_cast<int>(nr), chunks, o4, segs, static_cast<uint32_t>(n_waves), wrun,     \
                       (wgrid.x / (8u * wrun)) * (8u * wrun), make_fastdiv(wrun), make_fastdiv(segs))
#define COME_SPLITW_CASE(IDX_, PAIR_, REV_)                                 \
    do {                                                                    \
        if (wave_rows == 2) COME_SPLITW_ROWS(IDX_, PAIR_, REV_, 2);         \
        else COME_SPLITW_ROWS(IDX_, PAIR_, REV_, 1);                        \
    } while (0)
                if (rev_i64 && pair) COME_SPLITW_CASE(int64_t, true, rev_i64);
                else if (rev_i64) COME_SPLITW_CASE(int64_t, false, rev_i64);
                else if (pair) COME_SPLITW_CASE(int32_t, true, rev_i32);
                else COME_SPLITW_CASE(int32_t, false, rev_i32);
#undef COME_SPLITW_CASE
#undef COME_SPLITW_ROWS
                COME_CHECK_LAUNCH(who);
                continue;
            }
            const dim3 grid(static_cast<unsigned>(ceil_div(items, kThreads))), block(kThreads);
            const uint4 *a4 = static_cast<const uint4 *>(merged), *b4 = static_cast<const uint4 *>(merged_b);
            uint4 *o4 = static_cast<uint4 *>(out) + r0 * out_chunks;
#define COME_SPLIT_CASE(IDX_, PAIR_, REV_)                                                                       \
    hipLaunchKernelGGL((split_vec_kernel<IDX_, PAIR_>), grid, block, 0, s, a4, b4, merged_rows, REV_ + r0, nr,   \
                       chunks, o4, items, by_out_chunks, run)
            if (rev_i64 && pair) COME_SPLIT_CASE(int64_t, true, rev_i64);
            else if (rev_i64) COME_SPLIT_CASE(int64_t, false, rev_i64);
            else if (pair) COME_SPLIT_CASE(int32_t, true, rev_i32);
            else COME_SPLIT_CASE(int32_t, false, rev_i32);
            COME_CHECK_LAUNCH(who);
        }
#undef COME_SPLIT_CASE
    } else {
        const int eb = dtype_bytes(dtype);
        const int64_t blocks = ceil_div(total * chans * (pair ? 2 : 1), kThreads);
        COME_REQUIRE(blocks < (1ll << 31), COME_ERR_UNSUPPORTED, "%s: problem too large for one launch", who);
        const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
        const uint8_t *a1 = static_cast<const uint8_t *>(merged), *b1 = static_cast<const uint8_t *>(merged_b);
        if (rev_i64)
            hipLaunchKernelGGL(split_elem_kernel<int64_t>, grid, block, 0, s, a1, b1, pair, merged_rows, rev_i64, total,
                               row_bytes, eb, static_cast<uint8_t *>(out));
        else
            hipLaunchKernelGGL(split_elem_kernel<int32_t>, grid, block, 0, s, a1, b1, pair, merged_rows, rev_i32, total,
                               row_bytes, eb, static_cast<uint8_t *>(out));
    }
    COME_CHECK_LAUNCH(who);
    return COME_OK;
}

extern "C" int come_token_split(const void *merged, int dtype, int64_t merged_rows, int64_t chans,
                                const int64_t *rev_i64, const int32_t *rev_i32, int64_t total, void *out,
                                void *stream) {
    clear_error();
    return token_split_impl("come_token_split", false, merged, nullptr, dtype, merged_rows, chans, rev_i64, rev_i32, total,
                            out, stream);
}

extern "C" int come_token_split_pair(const void *merged_a, const void *merged_b, int dtype, int64_t merged_rows,
                                     int64_t chans, const int64_t *rev_i64, const int32_t *rev_i32, int64_t total,
                                     void *out, void *stream) {
    clear_error();
    return token_split_impl("come_token_split_pair", true, merged_a, merged_b, dtype, merged_rows, chans, rev_i64, rev_i32,
                            total, out, stream);
}
