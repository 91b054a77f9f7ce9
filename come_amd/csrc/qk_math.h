// The arithmetic of the attention prologue (LayerNorm over a 64-wide head, then the 2-D rotary embedding) on one
// 8-element chunk of a head, shared by the stand-alone pass (qk_prologue.hip) and by the attention kernel, which can
// apply it to the query rows as it loads them: both produce the same bits because both run these functions and add
// the partial sums of the eight chunks of a head in the same order.
//
// A head is 8 chunks of 8 elements.  Chunks 0 - 3 rotate with the y coordinate, 4 - 7 with x; chunk c pairs with
// chunk c ^ 2 (element j <-> j +- 16 inside a 32-element half), and the angle of element i of chunk c is
// position * base^(-(8 (c & 1) + i) / 16), looked up in tables [n_pos, 16] in the storage dtype.
//
// Rounding follows a chain of tensor operations in the storage dtype: the normalised value is rounded once, each of
// the two products of the rotation is rounded, and their sum is rounded.
#pragma once

#include "come_common.h"

namespace come {
namespace {

// Packed 16-bit pairs of the storage dtype: dot products against packed constants (+-1: the products are exact), fp32
// accumulation with one rounding.  The dot instructions are written as asm blocks: as single builtins every one of them
// costs a register zeroed for its accumulator, and the kernel that streams q and k through this code feels it.  A dot
// instruction's result may be read by a different kind of vector instruction only three wait states later, and nothing
// interlocks that; the compiler pads the instructions it emits itself and cannot see into asm text, so each block ends
// with the wait states its last result needs (s_nop 2), and dependent dots inside a block feed the accumulator operand
// of the same opcode, which needs none.
#define COME_QK_PAIR(DT_, MNEMONIC_, ONE_, MINUS_ONE_, PACK_)                                                                  \
    template <> struct Pair<DT_> {                                                                                          \
        static constexpr uint32_t kOne = ONE_, kMinusOne = MINUS_ONE_;                                                      \
        /* lo + hi of all eight elements of a 16-byte chunk */                                                            \
        __device__ static inline float sum8(const uint4 &w, uint32_t ones) {                                               \
            float d;                                                                                                        \
            asm(MNEMONIC_ " %0, %1, %5, 0\n\t" MNEMONIC_ " %0, %2, %5, %0\n\t" MNEMONIC_ " %0, %3, %5, %0\n\t"            \
                MNEMONIC_ " %0, %4, %5, %0\n\ts_nop 2"                                                                     \
                : "=&v"(d) : "v"(w.x), "v"(w.y), "v"(w.z), "v"(w.w), "v"(ones));                                           \
            return d;                                                                                                       \
        }                                                                                                                   \
        /* w[i] <- lo(w[i]) * lo(k) + hi(w[i]) * hi(k), eight independent dots */                                         \
        __device__ static inline void dot8(uint32_t (&w)[8], uint32_t k) {                                                 \
            asm(MNEMONIC_ " %0, %0, %8, 0\n\t" MNEMONIC_ " %1, %1, %8, 0\n\t" MNEMONIC_ " %2, %2, %8, 0\n\t"              \
                MNEMONIC_ " %3, %3, %8, 0\n\t" MNEMONIC_ " %4, %4, %8, 0\n\t" MNEMONIC_ " %5, %5, %8, 0\n\t"              \
                MNEMONIC_ " %6, %6, %8, 0\n\t" MNEMONIC_ " %7, %7, %8, 0\n\ts_nop 2"                                      \
                : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4]), "+v"(w[5]), "+v"(w[6]), "+v"(w[7])           \
                : "v"(k));                                                                                                  \
        }                                                                                                                   \
        __device__ static inline uint32_t pack(float lo, float hi) { return PACK_(lo, hi); }                               \
    }
template <int DT> struct Pair;
COME_QK_PAIR(COME_BF16, "v_dot2_f32_bf16", 0x3F80u, 0xBF80u, pack2_bf16);
COME_QK_PAIR(COME_F16, "v_dot2_f32_f16", 0x3C00u, 0xBC00u, pack2_f16);
#undef COME_QK_PAIR

template <int DT> struct QkChunk {
    using V = Vec16<DT>;
    using W = Pair<DT>;
    static constexpr uint32_t kOnes = W::kOne | (W::kOne << 16);

    // sum of the chunk's eight elements, taken from the packed words
    __device__ static inline float sum(const uint4 &word) { return W::sum8(word, kOnes); }
    // the head's sums of all eight chunks are added pair by pair: chunks (c, c ^ 1), then the two pairs of a half,
    // then the two halves - each step is symmetric in its two terms, so every holder gets the same bits
    __device__ static inline float mean_of(float head_sum) { return head_sum * (1.0f / 64.0f); }
    // f <- f - mean; returns the chunk's sum of squares
    __device__ static inline float center(float (&f)[8], float mean) {
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            f[i] -= mean;
            q = fmaf(f[i], f[i], q);
        }
        return q;
    }
    __device__ static inline float inv_std(float head_sum_sq, float eps) { return rsqrtf(head_sum_sq * (1.0f / 64.0f) + eps); }
    // centred values -> normalised chunk, rounded to the storage dtype
    __device__ static inline uint4 scale(float (&f)[8], float rstd, const float (&g)[8], const float (&b)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = fmaf(f[i] * rstd, g[i], b[i]);
        return V::pack(f);
    }
    // rotation of a chunk: x cos and partner sin are rounded as a pair; their signed sum is one dot product and is
    // rounded by the final pack.  The partner enters with sign -1 in the first 16 elements of each half (chunks with
    // c & 2 == 0), +1 in the last 16.
    __device__ static inline uint32_t one_and_sign(bool second_half_of_block) {
        return W::kOne | ((second_half_of_block ? W::kOne : W::kMinusOne) << 16);
    }
    __device__ static inline uint4 rotate(const float (&f)[8], const float (&partner)[8], const float (&c)[8], const float (&sn)[8],
                                          uint32_t sign_word) {
        uint32_t pair[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) pair[i] = W::pack(f[i] * c[i], partner[i] * sn[i]);
        W::dot8(pair, sign_word);
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = __uint_as_float(pair[i]);
        return V::pack(o);
    }
    // table row of a position, clamped to the table
    __device__ static inline int table_row(int64_t pos, int64_t n_pos) {
        return pos < 0 ? 0 : (pos >= n_pos ? static_cast<int>(n_pos) - 1 : static_cast<int>(pos));
    }
};

}  // namespace
}  // namespace come
