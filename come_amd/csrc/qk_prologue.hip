// Attention prologue on the packed q / k rows, in place: LayerNorm over the head dimension
// followed by the 2-D rotary position embedding, one pass over memory.
//
// Layout: q and k are [total, n_heads, 64] views (unit stride inside a head) of the packed
// projection output.  One lane owns 8 consecutive elements (16 bytes) of one head, so the
// eight lanes of a head hold its 64 elements; reductions and the rotation partner
// (element j <-> j +- 16 inside each 32-element half) are lane exchanges inside that group of
// eight.  The first 32 elements of a head rotate with the y coordinate, the last 32 with x;
// the angle of element j of a half is position * base^(-(j mod 16) / 16), looked up in
// tables [n_pos, 16] that the caller builds in the tensor dtype.
//
// Rounding follows a chain of tensor operations in the storage dtype: the normalised value
// is rounded once, each of the two products is rounded, and their sum is rounded.
//
// The pass is bound by its in-place access pattern (4 KiB read and written out of every 6 KiB row of
// the packed projection), not by arithmetic: loads and stores carry the non-temporal hint.
#include "come_common.h"
#include "qk_math.h"

namespace come {
namespace {

struct QkArgs {
    void *ptr[2];                 // q, k
    int64_t row_stride[2];        // elements
    int64_t head_stride[2];
    const void *gamma[2];         // [64] or nullptr
    const void *beta[2];
    int64_t total;
    int n_heads;
    int apply_norm;
    float eps;
    const int64_t *positions;     // [total, 2] (y, x) or nullptr: no rotation
    const void *cos_table;        // [n_pos, 16]
    const void *sin_table;
    int64_t n_pos;
    int groups_per_wg;            // token groups that share a workgroup (1: the groups' lanes are sliced over blockIdx.y)
};

template <int DT>
__device__ inline void round_to_dtype(float *f) {
    const uint4 r = Vec16<DT>::pack(f);
    Vec16<DT>::unpack(r, f);
}

// Lane exchanges inside a group of eight lanes as data-parallel-primitive moves (no LDS traffic, no address
// arithmetic).  kSwapPairs / kSwapQuadHalves permute inside a quad of lanes (lane ^ 1, lane ^ 2);
// kMirrorEight reverses the eight lanes of a half row (lane i <-> 7 - i).
constexpr int kSwapPairs = 0xB1;           // quad_perm [1, 0, 3, 2]
constexpr int kSwapQuadHalves = 0x4E;      // quad_perm [2, 3, 0, 1]
constexpr int kMirrorEight = 0x141;        // row_half_mirror

template <int CTRL>
__device__ inline float lane_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Sum over the eight lanes of a head, the same in every lane: after the two steps inside the quads each quad
// holds its sum in all four lanes, and the mirrored lane then belongs to the other quad.
__device__ inline float group8_sum(float v) {
    v += lane_move<kSwapPairs>(v);
    v += lane_move<kSwapQuadHalves>(v);
    v += lane_move<kMirrorEight>(v);
    return v;
}

constexpr int kRowsPerThread = 4;      // consecutive rows per lane: their loads are in flight together

// Grid: x = groups of kRowsPerThread tokens, y = 256-thread slices of the (q, k) x n_heads x 8 lanes of a token
// (only the tensors that are given: a null q or k is skipped).
template <int DT>
__global__ void __launch_bounds__(256) qk_norm_rope_kernel(const QkArgs a) {
    using V = Vec16<DT>;
    using C = QkChunk<DT>;
    const int per_tensor = a.n_heads * 8;
    const int first = a.ptr[0] != nullptr ? 0 : 1, n_tensors = (a.ptr[0] != nullptr ? 1 : 0) + (a.ptr[1] != nullptr ? 1 : 0);
    const int per_group = n_tensors * per_tensor;                 // lanes that one group of tokens needs
    // a workgroup holds a.groups_per_wg token groups side by side when one of them leaves half of it or more empty
    // (few heads, or one tensor only), else one group per 256-thread slice
    const int j = a.groups_per_wg > 1 ? static_cast<int>(threadIdx.x) % per_group
                                      : static_cast<int>(blockIdx.y * 256 + threadIdx.x);       // (which, head, lane8) of this lane
    const int64_t group = a.groups_per_wg > 1
                              ? static_cast<int64_t>(blockIdx.x) * a.groups_per_wg + static_cast<int>(threadIdx.x) / per_group
                              : static_cast<int64_t>(blockIdx.x);
    const int64_t token0 = group * kRowsPerThread;
    // (the eight lanes of a head leave together: per_group is a multiple of 8)
    if (j >= per_group || token0 >= a.total) return;
    if (a.groups_per_wg > 1 && static_cast<int>(threadIdx.x) / per_group >= a.groups_per_wg) return;   // lanes beyond the last whole group
    const int which = first + (j >= per_tensor ? 1 : 0);
    const int head = (j - (which - first) * per_tensor) >> 3;
    const int lane8 = j & 7;

    char *row = static_cast<char *>(a.ptr[which]) +
                (token0 * a.row_stride[which] + head * a.head_stride[which]) * V::ELEM_BYTES + lane8 * 16;
    const int64_t row_bytes = a.row_stride[which] * V::ELEM_BYTES;
    uint4 raw[kRowsPerThread];
    int entry[kRowsPerThread];                                    // byte offset of this lane's 8 table values
    bool live[kRowsPerThread];
#pragma unroll
    for (int t = 0; t < kRowsPerThread; ++t) {
        live[t] = token0 + t < a.total;
        const int64_t token = live[t] ? token0 + t : token0;
        raw[t] = ld16_stream(reinterpret_cast<const uint4 *>(row + (live[t] ? t : 0) * row_bytes));   // read once, written once
        entry[t] = 0;
        if (a.positions != nullptr) {
            // lanes 0-3 hold the y half, lanes 4-7 the x half of a head; lanes {0,1} and {2,3} of a half are
            // rotation partners and read the same 16 angles, 8 each
            const int pc = C::table_row(a.positions[token * 2 + (lane8 >> 2)], a.n_pos);
            entry[t] = (pc * 16 + (lane8 & 1) * 8) * V::ELEM_BYTES;
        }
    }
    float g[8], b[8];
    if (a.apply_norm) {
        if (a.gamma[which] != nullptr) {
            V::unpack(static_cast<const uint4 *>(a.gamma[which])[lane8], g);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) g[i] = 1.f;
        }
        if (a.beta[which] != nullptr) {
            V::unpack(static_cast<const uint4 *>(a.beta[which])[lane8], b);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) b[i] = 0.f;
        }
    }
    // the rotated partner enters with sign -1 in the first half of each 32-element block
    const uint32_t one_and_sign = C::one_and_sign((lane8 & 2) != 0);

#pragma unroll
    for (int t = 0; t < kRowsPerThread; ++t) {
        uint4 word = raw[t];
        float f[8];
        if (a.apply_norm) {
            // mean from the packed words, then the usual two passes in registers
            const float mean = C::mean_of(group8_sum(C::sum(word)));
            V::unpack(word, f);
            const float q = C::center(f, mean);
            const float rstd = C::inv_std(group8_sum(q), a.eps);
            word = C::scale(f, rstd, g, b);                      // the normalised value is rounded once
        }
        if (a.positions != nullptr) {
            V::unpack(word, f);
            float c[8], sn[8], partner[8];
            V::unpack(*reinterpret_cast<const uint4 *>(static_cast<const char *>(a.cos_table) + entry[t]), c);
            V::unpack(*reinterpret_cast<const uint4 *>(static_cast<const char *>(a.sin_table) + entry[t]), sn);
#pragma unroll
            for (int i = 0; i < 8; ++i) partner[i] = lane_move<kSwapQuadHalves>(f[i]);
            word = C::rotate(f, partner, c, sn, one_and_sign);
        }
        if (live[t]) st16_stream(reinterpret_cast<uint4 *>(row + t * row_bytes), word);
    }
}

}  // namespace
}  // namespace come

extern "C" int come_qk_norm_rope(void *q, void *k, int dtype,
                                 int64_t q_row_stride, int64_t q_head_stride,
                                 int64_t k_row_stride, int64_t k_head_stride,
                                 int64_t total, int64_t n_heads, int64_t head_dim,
                                 int apply_norm, const void *q_weight, const void *q_bias,
                                 const void *k_weight, const void *k_bias, float eps,
                                 const int64_t *positions, const void *cos_table, const void *sin_table,
                                 int64_t n_pos, void *stream) {
    using namespace come;
    clear_error();
    COME_REQUIRE(dtype == COME_BF16 || dtype == COME_F16, COME_ERR_UNSUPPORTED,
                 "come_qk_norm_rope: dtype must be bf16 or fp16");
    COME_REQUIRE(head_dim == 64, COME_ERR_UNSUPPORTED, "come_qk_norm_rope: only head_dim 64 is implemented (got %lld)",
                 static_cast<long long>(head_dim));
    COME_REQUIRE(total >= 0 && n_heads > 0 && n_heads < (1 << 20), COME_ERR_INVALID, "come_qk_norm_rope: bad sizes");
    if (total == 0) return COME_OK;
    COME_REQUIRE(q != nullptr || k != nullptr, COME_ERR_INVALID, "come_qk_norm_rope: q and k are both null");
    const int64_t strides[4] = {q_row_stride, q_head_stride, k_row_stride, k_head_stride};
    for (int i = 0; i < 4; ++i)
        COME_REQUIRE((i < 2 ? q : k) == nullptr || (strides[i] >= 64 && strides[i] % 8 == 0), COME_ERR_INVALID,
                     "come_qk_norm_rope: strides must be multiples of 8 elements and at least 64");
    COME_REQUIRE((q == nullptr || q_row_stride >= q_head_stride * (n_heads - 1) + 64) &&
                     (k == nullptr || k_row_stride >= k_head_stride * (n_heads - 1) + 64),
                 COME_ERR_INVALID, "come_qk_norm_rope: heads of one row overlap the next row");
    const void *aligned[] = {q, k, q_weight, q_bias, k_weight, k_bias, cos_table, sin_table};
    for (const void *p : aligned)
        COME_REQUIRE((reinterpret_cast<uintptr_t>(p) & 15) == 0, COME_ERR_INVALID,
                     "come_qk_norm_rope: pointers must be 16-byte aligned");
    COME_REQUIRE(eps >= 0.f, COME_ERR_INVALID, "come_qk_norm_rope: eps must be >= 0");
    if (positions != nullptr)
        COME_REQUIRE(cos_table != nullptr && sin_table != nullptr && n_pos > 0, COME_ERR_INVALID,
                     "come_qk_norm_rope: positions need cos / sin tables with n_pos > 0");
    if (!apply_norm && positions == nullptr) return COME_OK;

    QkArgs a{};
    a.ptr[0] = q; a.ptr[1] = k;
    a.row_stride[0] = q_row_stride; a.row_stride[1] = k_row_stride;
    a.head_stride[0] = q_head_stride; a.head_stride[1] = k_head_stride;
    a.gamma[0] = q_weight; a.gamma[1] = k_weight;
    a.beta[0] = q_bias; a.beta[1] = k_bias;
    a.total = total;
    a.n_heads = static_cast<int>(n_heads);
    a.apply_norm = apply_norm;
    a.eps = eps;
    a.positions = positions;
    a.cos_table = cos_table;
    a.sin_table = sin_table;
    a.n_pos = n_pos;
    const int64_t per_group = ((q != nullptr) + (k != nullptr)) * n_heads * 8;
    a.groups_per_wg = per_group <= 128 ? static_cast<int>(256 / per_group) : 1;
    const int64_t groups = ceil_div(ceil_div(total, kRowsPerThread), a.groups_per_wg);
    const int64_t slices = a.groups_per_wg > 1 ? 1 : ceil_div(per_group, 256);
    COME_REQUIRE(groups < (int64_t{1} << 31) && slices < 65536 && n_pos < (1 << 24), COME_ERR_UNSUPPORTED,
                 "come_qk_norm_rope: too many tokens, heads or positions for one launch");
    const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(slices));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == COME_BF16) hipLaunchKernelGGL((qk_norm_rope_kernel<COME_BF16>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((qk_norm_rope_kernel<COME_F16>), grid, dim3(256), 0, s, a);
    COME_CHECK_LAUNCH("come_qk_norm_rope");
    return COME_OK;
}
