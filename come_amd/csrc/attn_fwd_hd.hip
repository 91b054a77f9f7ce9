// Forward attention over packed variable-length sequences with an additive per-key bias for head
// dimensions 32 and 128 (gfx950, v_mfma_f32_32x32x16 bf16/f16).  The 64-wide heads of the shipped
// models have their own kernel (attn_fwd.hip); this one covers the other widths the reference
// instantiates up to 128 (flash_fwd_launch_template.h:174-180, 226-260; widths in between are
// zero-padded by the caller).
//
// One workgroup of 4 wavefronts owns 128 consecutive queries of one (segment, head), one 32-query
// tile per wavefront (with 128-wide heads the output accumulators of a second tile would not fit the
// register file beside Q).  K and V tiles of 64 keys go global -> LDS by direct loads, two stages,
// one barrier per tile.  Scores are computed transposed (S^T = K Q^T) so that the probabilities
// leave the accumulators as the B operand of O^T += V^T P^T, as in the 64-wide kernel.
//
// Softmax: the score accumulators start from bias / scale, so that the MFMAs deliver q . k + bias / scale as the
// reference forms it (flash_fwd_kernel.h:30-55), and one fused multiply-add per score applies the scale and
// subtracts the row's reference point in front of the exponential (softmax.h:76-88), in log2 units.  The reference point of
// a row is a running maximum that is only moved when a half-tile's maximum exceeds it by more than
// 2^8: probabilities stay below 2^8 (exact in both 16-bit types), the result is the same up to
// rounding, and the output accumulators are rescaled a few times per row instead of every 32 keys.
#include "attn_common.h"

namespace come {
namespace {

constexpr float kRefSlack = 8.f;     // log2 units a row's scores may exceed its reference point by

template <int D> struct Swizzle;
// 16-byte chunk c of row r of a staged tile sits at chunk slot c ^ k(r) (K) or c ^ v(r) (V): the 16 lanes of
// a row-fragment read (K) and the 32 lanes of a transposing read (V, four rows x 64 bytes) then cover all banks
template <> struct Swizzle<128> {
    __device__ static inline int k(int r) { return r & 15; }
    __device__ static inline int v(int r) { return (r & 3) << 2; }
};
template <> struct Swizzle<32> {
    __device__ static inline int k(int r) { return (r >> 2) & 3; }
    __device__ static inline int v(int) { return 0; }
};

template <int DT, int D>
__global__ __launch_bounds__(256) void attn_fwd_hd_kernel(const AttnArgs a) {
    using E = Elem<DT>;
    using Z = Swizzle<D>;
    constexpr int kBlockM = 128;
    constexpr int kKSteps = D / 16;            // MFMA k-steps of a score tile
    constexpr int kDTiles = D / 32;            // 32-wide tiles of the output's head dimension
    constexpr int kChunks = D / 8;             // 16-byte chunks per row
    constexpr int kRowsPerLoad = 64 / kChunks; // rows one wavefront-wide direct load covers (1 KiB)
    constexpr int kDma = kChunks / 4;          // direct loads per wavefront for one K (or V) tile
    constexpr float kLog2e = 1.4426950408889634f;
    __shared__ __attribute__((aligned(1024))) uint16_t lds_k[2][kBlockN * D];
    __shared__ __attribute__((aligned(1024))) uint16_t lds_v[2][kBlockN * D];
    __shared__ __attribute__((aligned(16))) float lds_b[2][kBlockN];     // bias / softmax_scale, -inf beyond the segment

    // workgroup i runs on XCD i % 8: the query blocks of one (segment, head) unit stay on one XCD
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int unit_on_xcd = local / a.n_mblocks;
    const int unit = xcd + 8 * unit_on_xcd;
    // the workgroups of an XCD go to its four shader engines in turn: with an even number of blocks per unit, unit u
    // starts its blocks at position u, so that the empty last blocks of short segments do not keep landing on the
    // same engines
    const int mblk = a.rotate ? (local % a.n_mblocks + unit_on_xcd) % a.n_mblocks : local % a.n_mblocks;
    if (unit >= a.n_units) return;
    const int head = unit % a.n_heads;
    const int seq = unit / a.n_heads;
    int seq_start, L;
    segment_of(a, seq, seq_start, L);
    const int q0 = mblk * kBlockM;
    if (q0 >= L) return;
    const int n_tiles = (L + kBlockN - 1) / kBlockN;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int h = lane >> 5;
    const int r = lane & 31;

    // ---- Q fragments (B operand: n = query r, k = head-dim 16 ks + 8 h ..), as they are
    u32x4 qf[kKSteps];
    {
        const int row = q0 + wave * 32 + r;
        const uint16_t *qp = a.q + static_cast<int64_t>(seq_start + min(row, L - 1)) * a.q_rs + head * a.q_hs + 8 * h;
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) qf[ks] = *reinterpret_cast<const u32x4 *>(qp + 16 * ks);
    }

    // ---- staging: load i of wavefront w fills rows kRowsPerLoad (kDma w + i) .. of a tile; lane l lands in row
    // l / kChunks of them, chunk slot l % kChunks, and fetches the chunk the swizzle puts there.  A key beyond the
    // segment is redirected to its last key (finite data; its bias is -inf, so its probability is exactly 0).
    const char *k_seg = reinterpret_cast<const char *>(a.k + static_cast<int64_t>(seq_start) * a.k_rs + head * a.k_hs);
    const char *v_seg = reinterpret_cast<const char *>(a.v + static_cast<int64_t>(seq_start) * a.v_rs + head * a.v_hs);
    const uint32_t k_rs_b = static_cast<uint32_t>(a.k_rs) * 2u, v_rs_b = static_cast<uint32_t>(a.v_rs) * 2u;
    uint32_t k_goff[kDma], v_goff[kDma], k_chunk[kDma], v_chunk[kDma];
    int st_row[kDma];
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
        st_row[i] = kRowsPerLoad * (kDma * wave + i) + lane / kChunks;
        const int slot = lane % kChunks;
        k_chunk[i] = static_cast<uint32_t>(slot ^ Z::k(st_row[i])) * 16u;
        v_chunk[i] = static_cast<uint32_t>(slot ^ Z::v(st_row[i])) * 16u;
        k_goff[i] = static_cast<uint32_t>(st_row[i]) * k_rs_b + k_chunk[i];
        v_goff[i] = static_cast<uint32_t>(st_row[i]) * v_rs_b + v_chunk[i];
    }
    const uint32_t k_last = static_cast<uint32_t>(L - 1) * k_rs_b, v_last = static_cast<uint32_t>(L - 1) * v_rs_b;
    auto stage = [&](int tile, int buf) __attribute__((always_inline)) {
        const int n0 = tile * kBlockN;
        const bool full = n0 + kBlockN <= L;                                        // wave-uniform
        const uint32_t k_tile = static_cast<uint32_t>(n0) * k_rs_b, v_tile = static_cast<uint32_t>(n0) * v_rs_b;
#pragma unroll
        for (int i = 0; i < kDma; ++i) {
            uint32_t ko = k_tile + k_goff[i], vo = v_tile + v_goff[i];
            if (!full && n0 + st_row[i] >= L) {
                ko = k_last + k_chunk[i];
                vo = v_last + v_chunk[i];
            }
            dma_b128(k_seg, ko, lds_address(&lds_k[buf][(kDma * wave_u + i) * 512]));
            dma_b128(v_seg, vo, lds_address(&lds_v[buf][(kDma * wave_u + i) * 512]));
        }
    };
    // What the scores of a tile's 64 keys start from (wavefront 0, lane = key): bias / softmax_scale, as the
    // reference adds it to the raw scores (flash_fwd_kernel.h:46-50); -inf beyond the end of the segment
    const float inv_c = 1.0f / a.scale_log2;
    auto bias_of = [&](int tile) __attribute__((always_inline)) -> float {
        const int key = tile * kBlockN + lane;
        if (key >= L) return -INFINITY;
        return a.bias ? E::to_f32(a.bias[seq_start + key]) * kLog2e * inv_c : 0.f;
    };

    // ---- LDS read offsets (in elements) of this lane
    int k_rd[kKSteps];
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) k_rd[ks] = r * D + (((2 * ks + h) ^ Z::k(r)) << 3);
    const int i16 = lane & 15;
    int v_rd[kDTiles];
    {
        const int row = 4 * h + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
            v_rd[dt] = row * D + (((4 * dt + 2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1)) ^ Z::v(row)) << 3) + 4 * (i16 & 1);
    }
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    f32x16 o_acc[kDTiles];
#pragma unroll
    for (int dt = 0; dt < kDTiles; ++dt) o_acc[dt] = zero16;
    float m_ref = -INFINITY;      // reference point of the row, log2 units
    // Row sums come from the matrix pipe: the probabilities of a 16-key step as the A operand of v_mfma_f32_16x16x32
    // (row m = lane % 16; lane group g = lane / 16 holds query m + 16 (g & 1)) against a B operand whose lane group g
    // is all ones in column g & 1: result column 0 / 1 holds the sums of queries m / m + 16.  A lane of the result
    // holds column lane % 16, rows 4 (lane / 16) .. + 3, so the running sums of queries 0 .. 15 sit in lanes 0, 16, 32,
    // 48 and those of queries 16 .. 31 in lanes 1, 17, 33, 49, four per lane; all other lanes hold zeros.
    f32x4 l_acc = {0.f, 0.f, 0.f, 0.f};
    const u32x4 ones_sel = ((lane & 15) == ((lane >> 4) & 1))
                               ? u32x4{E::kOne | (E::kOne << 16), E::kOne | (E::kOne << 16), E::kOne | (E::kOne << 16), E::kOne | (E::kOne << 16)}
                               : u32x4{0u, 0u, 0u, 0u};
    const int owner_base = (16 * (lane & 15) + 4 * (lane >> 4)) & 31;     // element j of l_acc belongs to query owner_base + j

    // k-step ks of the scores of half-tile `half` of the K tile in `buf`; the accumulator starts from the bias terms
    // of the lane's 16 keys (rows 8 g + 4 h + e of the half-tile), so that q . k + bias / scale leaves the MFMAs
    auto score_step = [&](f32x16 &s, int buf, int half, int ks) __attribute__((always_inline)) {
        const u32x4 kf = *reinterpret_cast<const u32x4 *>(&lds_k[buf][k_rd[ks] + 32 * half * D]);
        if (ks == 0) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bq = *reinterpret_cast<const f32x4 *>(&lds_b[buf][32 * half + 8 * g + 4 * h]);
#pragma unroll
                for (int e = 0; e < 4; ++e) s[4 * g + e] = bq[e];
            }
        }
        s = E::mfma(kf, qf[ks], s);
    };
    // MFMA m of O^T += V^T P^T for half-tile `half` of the V tile in `buf` (m = 16-key step x output tile)
    auto pv_step = [&](const u32x4 (&p)[2], int buf, int half, int m) __attribute__((always_inline)) {
        const int u = m / kDTiles, dt = m % kDTiles;
        const uint16_t *vp = &lds_v[buf][v_rd[dt] + (32 * half + 16 * u) * D];
        const u32x2 lo2 = __builtin_bit_cast(u32x2, lds_read_tr(vp));
        const u32x2 hi2 = __builtin_bit_cast(u32x2, lds_read_tr(vp + 8 * D));
        o_acc[dt] = E::mfma(u32x4{lo2[0], lo2[1], hi2[0], hi2[1]}, p[u], o_acc[dt]);
    };

    // Scores of one half-tile -> probabilities (B operands p[16-key step]).  `mfma(m)` issues the m-th of kKSteps
    // (= 2 kDTiles) independent MFMAs of the neighbouring half-tile, spread between the exponentials.
    auto softmax_step = [&](const f32x16 &s, int buf, int half, u32x4 (&p)[2], auto &&mfma) __attribute__((always_inline)) {
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[e]);
        mx = max_across_halves(mx) * a.scale_log2;               // the scale is positive: the maximum commutes with it
        // A reference point that moves rescales the row sum now and the output at the end of the step, behind the
        // P V MFMAs issued in between: their probabilities are relative to the old reference point.
        const bool move = mx > m_ref + kRefSlack;              // (also the first keys of a row: m_ref = -inf)
        const bool moved = __any(move);                         // wave-uniform
        float down = 1.f;
        if (moved) {
            down = move ? __builtin_amdgcn_exp2f(m_ref - mx) : 1.f;
            m_ref = move ? mx : m_ref;
#pragma unroll
            for (int j = 0; j < 4; ++j) l_acc[j] *= __shfl(down, owner_base + j);
        }
        const float neg_ref = m_ref == -INFINITY ? 0.f : -m_ref;   // (a row that has seen masked keys only: 0)
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            if (kKSteps >= 8) {
#pragma unroll
                for (int m = w * (kKSteps / 8); m < (w + 1) * (kKSteps / 8); ++m) mfma(m);
            } else if (w % (8 / kKSteps) == 0) {
                mfma(w / (8 / kKSteps));
            }
            const uint32_t pw = E::pack2_prob(__builtin_amdgcn_exp2f(__builtin_fmaf(s[2 * w], a.scale_log2, neg_ref)),
                                              __builtin_amdgcn_exp2f(__builtin_fmaf(s[2 * w + 1], a.scale_log2, neg_ref)));
            p[w >> 2][w & 3] = pw;
            if (w == 3) l_acc = E::mfma16(p[0], ones_sel, l_acc);
        }
        l_acc = E::mfma16(p[1], ones_sel, l_acc);
        if (moved) {
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) o_acc[dt][e] *= down;
        }
    };

    // ---- prologue: tile 0
    stage(0, 0);
    if (wave_u == 0) lds_b[0][lane] = bias_of(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // A wavefront whose 32 queries all lie beyond the end of the segment only helps with the staging.
    const bool idle = q0 + wave_u * 32 >= L;
    auto iteration = [&](int j, int buf) __attribute__((always_inline)) {
        float b_next = 0.f;
        if (j + 1 < n_tiles) {
            stage(j + 1, buf ^ 1);             // that stage was last read before the previous barrier
            if (wave_u == 0) b_next = bias_of(j + 1);
        }
        if (!idle) {
            f32x16 s0, s1;
            u32x4 p0[2], p1[2];
#pragma unroll
            for (int ks = 0; ks < kKSteps; ++ks) score_step(s0, buf, 0, ks);
            // keys 0..31 become probabilities while the matrix pipe builds the scores of keys 32..63
            softmax_step(s0, buf, 0, p0, [&](int m) __attribute__((always_inline)) { score_step(s1, buf, 1, m); });
            // keys 32..63 become probabilities while the matrix pipe adds P V of keys 0..31
            softmax_step(s1, buf, 1, p1, [&](int m) __attribute__((always_inline)) { pv_step(p0, buf, 0, m); });
#pragma unroll
            for (int m = 0; m < 2 * kDTiles; ++m) pv_step(p1, buf, 1, m);
        }
        if (j + 1 < n_tiles && wave_u == 0) lds_b[buf ^ 1][lane] = b_next;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };
    // two tiles per turn: the LDS stage is a constant in each copy and goes into the offset fields of the reads
    int j = 0;
    for (; j + 2 <= n_tiles; j += 2) {
        iteration(j, 0);
        iteration(j + 1, 1);
    }
    if (j < n_tiles) iteration(j, 0);
    if (idle) return;

    // ---- epilogue: normalise, write O (and LSE)
    float l_tot = 0.f;
    {
        const int sum_lane = (r >> 4) + 16 * ((r & 15) >> 2);          // where this lane's query keeps its sum (element r & 3)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float t = __shfl(l_acc[j], sum_lane);
            l_tot = (r & 3) == j ? t : l_tot;
        }
    }
    const float inv = 1.0f / l_tot;
    const int row = q0 + wave * 32 + r;
    if (row < L) {
        uint16_t *op = a.out + static_cast<int64_t>(seq_start + row) * a.o_rs + head * a.o_hs + 4 * h;
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w[0] = E::pack2(o_acc[dt][4 * g] * inv, o_acc[dt][4 * g + 1] * inv);
                w[1] = E::pack2(o_acc[dt][4 * g + 2] * inv, o_acc[dt][4 * g + 3] * inv);
                *reinterpret_cast<u32x2 *>(op + 32 * dt + 8 * g) = w;
            }
        if (h == 0 && a.lse)
            a.lse[static_cast<int64_t>(head) * a.total + seq_start + row] =
                ((m_ref == -INFINITY ? 0.f : m_ref) + __log2f(l_tot)) * 0.6931471805599453f;
    }
}

}  // namespace

int launch_attn_hd(const AttnArgs &args, int dtype, int head_dim, int64_t max_seqlen, hipStream_t stream) {
    AttnArgs a = args;
    a.n_mblocks = static_cast<int>(ceil_div(max_seqlen, 128));
    a.rotate = a.n_mblocks % 2 == 0 ? 1 : 0;
    const int64_t n_wg = ceil_div(a.n_units, 8) * 8 * a.n_mblocks;
    COME_REQUIRE(n_wg < (1ll << 31), COME_ERR_UNSUPPORTED, "come_attn_varlen_fwd: grid too large");
    const dim3 grid(static_cast<unsigned>(n_wg)), block(256);
    if (head_dim == 128) {
        if (dtype == COME_BF16) hipLaunchKernelGGL((attn_fwd_hd_kernel<COME_BF16, 128>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((attn_fwd_hd_kernel<COME_F16, 128>), grid, block, 0, stream, a);
    } else {
        if (dtype == COME_BF16) hipLaunchKernelGGL((attn_fwd_hd_kernel<COME_BF16, 32>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((attn_fwd_hd_kernel<COME_F16, 32>), grid, block, 0, stream, a);
    }
    COME_CHECK_LAUNCH("come_attn_varlen_fwd");
    return COME_OK;
}

}  // namespace come
