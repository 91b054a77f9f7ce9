// Suffix operators on packed segments: append T dense rows to every segment, or strip them again.
// Both are row copies (HBM-bound byte work): one thread per (output row, 16-byte chunk) - or per
// element when rows are not a multiple of 16 bytes - that finds its segment by bisection over the
// segment offsets and copies from the packed rows or from the dense suffix block.
#include "come_common.h"

namespace come {
namespace {

constexpr int kThreads = 256;

struct SuffixArgs {
    const uint8_t *tokens;        // [rows_in, row_bytes]
    const float *weight;          // [rows_in] or nullptr
    const int64_t *offsets;       // [n_seg + 1] boundaries of the input segments
    const uint8_t *suffix_in;     // add: [n_seg, T, row_bytes]
    uint8_t *out_tokens;          // add: [rows_in + n_seg T, ..]; strip: [rows_in - n_seg T, ..]
    float *out_weight;
    int64_t *out_offsets;         // [n_seg + 1]
    uint8_t *suffix_out;          // strip: [n_seg, T, row_bytes]
    int64_t rows_in, rows_out, n_seg, T;
    int64_t row_bytes;
    int unit;                     // bytes moved per thread: 16, 4 or 2
    int units_per_row;
    int strip;                    // 0 = append, 1 = strip
};

// largest s in [0, n_seg) with start(s) <= row, where start(s) = offsets[s] + s * step
__device__ inline int64_t find_segment(const int64_t *offsets, int64_t n_seg, int64_t step, int64_t row) {
    int64_t lo = 0, hi = n_seg - 1;
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (offsets[mid] + mid * step <= row) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

__device__ inline void copy_unit(uint8_t *dst, const uint8_t *src, int unit) {
    if (unit == 16) *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src);
    else if (unit == 4) *reinterpret_cast<uint32_t *>(dst) = *reinterpret_cast<const uint32_t *>(src);
    else *reinterpret_cast<uint16_t *>(dst) = *reinterpret_cast<const uint16_t *>(src);
}

__global__ __launch_bounds__(kThreads) void suffix_kernel(const SuffixArgs a) {
    const int64_t id = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t row = id / a.units_per_row;
    const int64_t col = (id - row * a.units_per_row) * a.unit;
    const int64_t body_rows = a.rows_out;
    const int64_t extra_rows = a.strip ? a.n_seg * a.T : 0;           // rows of the returned suffix block
    if (id <= a.n_seg && a.out_offsets != nullptr)                       // new boundaries, n_seg + 1 of them
        a.out_offsets[id] = a.offsets[id] + (a.strip ? -id : id) * a.T;
    if (row >= body_rows + extra_rows) return;

    if (row < body_rows) {
        const int64_t step = a.strip ? -a.T : a.T;
        const int64_t s = find_segment(a.offsets, a.n_seg, step, row);
        const int64_t j = row - (a.offsets[s] + s * step);               // position inside the output segment
        const int64_t len_in = a.offsets[s + 1] - a.offsets[s];
        // The offsets come from device memory that the host cannot check: indices derived from them are clamped
        // into the tensors, so that inconsistent offsets give wrong rows instead of accesses outside them.
        const uint8_t *src;
        float w = 1.f;
        if (a.rows_in > 0 && (a.strip || j < len_in)) {
            const int64_t r = min(max(a.offsets[s] + j, int64_t{0}), a.rows_in - 1);
            src = a.tokens + r * a.row_bytes;
            if (a.weight) w = a.weight[r];
        } else {
            const int64_t t = min(max(j - len_in, int64_t{0}), a.T - 1);
            src = a.suffix_in + (s * a.T + t) * a.row_bytes;
        }
        copy_unit(a.out_tokens + row * a.row_bytes + col, src + col, a.unit);
        if (col == 0 && a.out_weight) a.out_weight[row] = w;
    } else {
        const int64_t e = row - body_rows;                               // (segment, t) of the stripped block
        const int64_t s = e / a.T;
        const int64_t t = e - s * a.T;
        // a segment shorter than T (caller error) or inconsistent offsets stay in bounds
        const int64_t r = min(max(a.offsets[s + 1] - a.T + t, int64_t{0}), a.rows_in - 1);
        copy_unit(a.suffix_out + e * a.row_bytes + col, a.tokens + r * a.row_bytes + col, a.unit);
    }
}

int launch(SuffixArgs &a, int dtype, int64_t chans, const void *const *ptrs, int n_ptrs, void *stream, const char *what) {
    a.row_bytes = chans * dtype_bytes(dtype);
    bool aligned = a.row_bytes % 16 == 0;
    for (int i = 0; i < n_ptrs; ++i) aligned = aligned && (reinterpret_cast<uintptr_t>(ptrs[i]) & 15u) == 0;
    a.unit = aligned ? 16 : dtype_bytes(dtype);
    a.units_per_row = static_cast<int>(a.row_bytes / a.unit);
    const int64_t rows = a.rows_out + (a.strip ? a.n_seg * a.T : 0);
    int64_t items = rows * a.units_per_row;
    if (items < a.n_seg + 1) items = a.n_seg + 1;                        // the offsets are written in any case
    const int64_t blocks = ceil_div(items, kThreads);
    COME_REQUIRE(blocks < (1ll << 31), COME_ERR_UNSUPPORTED, "%s: problem too large for one launch", what);
    hipLaunchKernelGGL(suffix_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), a);
    COME_CHECK_LAUNCH(what);
    return COME_OK;
}

}  // namespace
}  // namespace come

using namespace come;

extern "C" int come_jagged_add_suffix(const void *tokens, const float *weight, int dtype, int64_t rows, int64_t chans,
                                      const int64_t *offsets, int64_t n_seg, const void *suffix, int64_t count,
                                      void *out_tokens, float *out_weight, int64_t *out_offsets, void *stream) {
    clear_error();
    COME_REQUIRE(dtype_ok(dtype), COME_ERR_UNSUPPORTED, "come_jagged_add_suffix: unsupported dtype %d", dtype);
    COME_REQUIRE(rows >= 0 && chans >= 1 && n_seg >= 0 && count >= 0, COME_ERR_INVALID,
                 "come_jagged_add_suffix: negative size or chans < 1");
    COME_REQUIRE(chans < (1ll << 24) && n_seg < (1ll << 31), COME_ERR_UNSUPPORTED, "come_jagged_add_suffix: too large");
    COME_REQUIRE(offsets && out_offsets, COME_ERR_INVALID, "come_jagged_add_suffix: offsets is NULL");
    COME_REQUIRE(n_seg > 0 || rows == 0, COME_ERR_INVALID, "come_jagged_add_suffix: rows without segments");
    COME_REQUIRE((rows == 0 || tokens) && (n_seg * count == 0 || suffix) && (rows + n_seg * count == 0 || out_tokens),
                 COME_ERR_INVALID, "come_jagged_add_suffix: NULL tensor");
    COME_REQUIRE((weight == nullptr) == (out_weight == nullptr) || rows == 0, COME_ERR_INVALID,
                 "come_jagged_add_suffix: weight and out_weight go together");
    SuffixArgs a{};
    a.tokens = static_cast<const uint8_t *>(tokens);
    a.weight = weight;
    a.offsets = offsets;
    a.suffix_in = static_cast<const uint8_t *>(suffix);
    a.out_tokens = static_cast<uint8_t *>(out_tokens);
    a.out_weight = out_weight;
    a.out_offsets = out_offsets;
    a.rows_in = rows;
    a.rows_out = rows + n_seg * count;
    a.n_seg = n_seg;
    a.T = count;
    a.strip = 0;
    const void *ptrs[3] = {tokens, suffix, out_tokens};
    return launch(a, dtype, chans, ptrs, 3, stream, "come_jagged_add_suffix");
}

extern "C" int come_jagged_split_suffix(const void *tokens, const float *weight, int dtype, int64_t rows,
                                        int64_t chans, const int64_t *offsets, int64_t n_seg, int64_t count,
                                        void *out_tokens, float *out_weight, int64_t *out_offsets, void *out_suffix,
                                        void *stream) {
    clear_error();
    COME_REQUIRE(dtype_ok(dtype), COME_ERR_UNSUPPORTED, "come_jagged_split_suffix: unsupported dtype %d", dtype);
    COME_REQUIRE(rows >= 0 && chans >= 1 && n_seg >= 0 && count >= 0, COME_ERR_INVALID,
                 "come_jagged_split_suffix: negative size or chans < 1");
    COME_REQUIRE(chans < (1ll << 24) && n_seg < (1ll << 31), COME_ERR_UNSUPPORTED, "come_jagged_split_suffix: too large");
    COME_REQUIRE(rows - n_seg * count >= 0, COME_ERR_INVALID,
                 "come_jagged_split_suffix: cannot strip %lld rows from each of %lld segments (%lld rows in total)",
                 (long long)count, (long long)n_seg, (long long)rows);
    COME_REQUIRE(offsets && out_offsets, COME_ERR_INVALID, "come_jagged_split_suffix: offsets is NULL");
    COME_REQUIRE(n_seg > 0 || rows == 0, COME_ERR_INVALID, "come_jagged_split_suffix: rows without segments");
    COME_REQUIRE((rows == 0 || tokens) && (rows - n_seg * count == 0 || out_tokens) && (n_seg * count == 0 || out_suffix),
                 COME_ERR_INVALID, "come_jagged_split_suffix: NULL tensor");
    COME_REQUIRE((weight == nullptr) == (out_weight == nullptr) || rows - n_seg * count == 0, COME_ERR_INVALID,
                 "come_jagged_split_suffix: weight and out_weight go together");
    SuffixArgs a{};
    a.tokens = static_cast<const uint8_t *>(tokens);
    a.weight = weight;
    a.offsets = offsets;
    a.out_tokens = static_cast<uint8_t *>(out_tokens);
    a.out_weight = out_weight;
    a.out_offsets = out_offsets;
    a.suffix_out = static_cast<uint8_t *>(out_suffix);
    a.rows_in = rows;
    a.rows_out = rows - n_seg * count;
    a.n_seg = n_seg;
    a.T = count;
    a.strip = 1;
    const void *ptrs[3] = {tokens, out_tokens, out_suffix};
    return launch(a, dtype, chans, ptrs, 3, stream, "come_jagged_split_suffix");
}
