// Forward attention over packed variable-length sequences with an additive per-key
// bias, head_dim 64, for gfx950 (wave64, v_mfma_f32_32x32x16 bf16/f16).
//
// Work decomposition
//   One workgroup (4 wavefronts) owns 256 consecutive queries of one (segment, head);
//   every wavefront owns two tiles of 32 queries and walks all keys of the segment in
//   tiles of 64.  K and V tiles are staged once per workgroup in LDS (four stages, one
//   barrier per tile); Q stays in registers.
//
// Orientation
//   Scores are produced transposed, S^T = K (c Q)^T, so that in the MFMA accumulator
//   layout a lane holds ONE query (lane % 32) and 16 keys per 32x32 tile: the row max
//   and row sum of the online softmax are in-lane reductions plus one exchange between
//   lane l and lane l ^ 32.  The same registers, rounded to 16 bit, are the B operand
//   of O^T += V^T P^T without any data movement; V^T fragments come out of the
//   row-major V tile with the transposing LDS read ds_read_b64_tr_b16.
//
// Bias, reference point and tail masking
//   The accumulator of a score tile does not start from zero but from b_k - m_q, with
//   b = float(bias) log2(e) of the key (read from LDS, -inf beyond the end of the segment) and
//   m the reference point of the query's row, and Q is multiplied by c = softmax_scale log2(e)
//   once: after the four k-steps of the score MFMA the accumulator is the exponent of exp2.
//   (The reference adds bias / scale to the raw scores, flash_fwd_kernel.h:30-55, and
//   subtracts the scaled running maximum inside exp2, softmax.h:76-88.)  Keys beyond the end of
//   the segment get scores of -inf and probabilities of exactly 0.
//   The reference point of a row moves lazily (only when its row sum - bf16: the running one, fp16: that of a
//   half-tile - leaves the range the 16-bit probabilities keep their precision in).  A workgroup in which a stored probability left
//   the 16-bit range altogether raises a flag on the loop's last barrier and then computes its
//   query block again, tile by tile, with a running maximum per row: any finite scores are exact.
//   That is the instantiation COME_ATTN_FOLD_SCALE selects.  The default one (EXACT) keeps Q as it is: the
//   accumulator starts from (b_k - m_q) / c and every score is multiplied by c in fp32 in front of the exponential,
//   which is the reference's arithmetic (bias / scale added to the raw scores, scale applied inside exp2).
#include "attn_common.h"
#include "qk_math.h"

#include <mutex>

// Work buffer of come_attn_varlen_fwd_static: pieces of the key-split tail (unnormalised outputs, reference
// points and row sums).  Every GPU the library runs on holds its own copy of the array at its own address.
constexpr int64_t kStaticWorkBytes = 64ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticWorkBytes];

namespace come {
namespace {

constexpr int kHeadDim = 64;
constexpr int kPieceExtra = 2;       // per query row of a piece: 64 unnormalised outputs, reference point, row sum

// Which (segment, head, query block) a workgroup computes.  Workgroup i is dispatched to XCD
// i % 8, each XCD with its own L2: the query blocks of one (segment, head) unit run back to back
// on one XCD and share that unit's K/V there, and units are dealt to the XCDs round-robin so that
// segments of different lengths spread evenly.  The grid is padded to 8 * ceil(units / 8) units.
// A split workgroup (behind the n_full_wg ordinary ones) gets the index of its query block among the unit's
// tail blocks (tail >= 0) and its key share ks; the pieces of one query block are neighbours on one XCD.
__device__ inline bool locate_block(const AttnArgs &a, int &mblk, int &head, int &seq, int &tail, int &ks) {
    // one straight-line computation for both kinds of workgroup (branches that assign different outputs made the
    // compiler keep the outputs in scratch memory)
    const bool split = static_cast<int64_t>(blockIdx.x) >= a.n_full_wg;
    const int e = split ? static_cast<int>(blockIdx.x - a.n_full_wg) : static_cast<int>(blockIdx.x);
    const int xcd = e & 7;
    const int local = e >> 3;
    const int per_unit = split ? a.nb_tail * a.splits : a.n_mblocks;
    const int unit_on_xcd = local / per_unit;
    const int unit = xcd + 8 * unit_on_xcd;
    const int within = local % per_unit;
    // The workgroups of an XCD are dealt to its four shader engines in turn (position mod 4, measured: a fixed
    // assignment, also while the engines are full).  Short segments leave the same query blocks of every unit empty,
    // so with an even number of blocks per unit the empty ones would keep landing on the same engines (a launch of
    // 2 real + 2 empty blocks per unit runs 1.8 times longer than one of 2 + 1).  With `rotate`, set for even block
    // counts, unit u starts its blocks at position u: the pattern then repeats with an odd period and every engine
    // gets its share, while a unit's blocks stay neighbours in dispatch order (they share K / V in L2).
    mblk = split ? 0 : (a.rotate ? (within + unit_on_xcd) % per_unit : within);
    tail = split ? within / a.splits : -1;
    ks = split ? within % a.splits : 0;
    head = unit % a.n_heads;
    seq = unit / a.n_heads;
    return unit < a.n_units;
}

// -------------------------------------------------------------------------------------
// Software-pipelined kernel: kBlockM = 256 queries per workgroup, two query tiles per
// wavefront that alternate roles.  While the vector ALU turns the scores of one query tile
// into probabilities, the matrix pipe runs the score MFMAs (next key tile) and the P V MFMAs
// (current key tile) of the other one:
//
//   slot a(j): VALU P0 = exp2(S0(j))      MFMA S1(j) = K(j) Q1^T ; O1 += V(j-1)^T P1(j-1)
//   slot b(j): VALU P1 = exp2(S1(j))      MFMA S0(j+1) = K(j+1) Q0^T ; O0 += V(j)^T P0(j)
//
// K tiles j, j+1 and V tiles j-1, j are live in one iteration and the tiles of the next iteration
// are in flight from global memory, so LDS holds four tiles of each; one barrier per iteration.
//
// Scores leave the MFMA already in the form the exponential needs:
//   S'' = (c q) . k + bias log2(e) - m,      c = softmax_scale log2(e)
// Q is multiplied by c once (and rounded back to 16 bit); bias log2(e) - m is the initial value of the
// accumulator (one subtraction per score on the vector ALU).  m is the row maximum of the first 32 keys and
// is moved, by a power of two, only when the row sum leaves a safe range (sums and outputs are
// then rescaled as in the usual online softmax); softmax is invariant to the choice of m, and fp32 / 16-bit
// floats keep full relative precision for probabilities above 1.  Row sums are taken on the matrix pipe too
// (the rounded probabilities times a matrix of ones, v_mfma_f32_16x16x32), so the steady state spends one
// exp2 and half a pack per score on the vector ALU (plus one multiplication where the scale is applied in fp32)
// and six additions per half-tile for the range check.
// -------------------------------------------------------------------------------------
constexpr int kStages = 4;
// Launches whose segments are at most this long walk their work items in resident workgroups (PERSIST below): a few
// query blocks per (segment, head) unit, so a fixed share of the item list per workgroup is a balanced share.
constexpr int64_t kPersistMaxSeqlen = 2048;

// Range of the probabilities relative to the reference point of their row.  They are stored in the 16-bit type of
// the inputs: bf16 has the exponent range of fp32, fp16 reaches only 65504 and loses precision below 2^-14.
//   kSumLimit  a row sum above this (bf16: the running sum, fp16: the sum over a half-tile) moves the reference point
//              of the row up
//   kMaxGap    a row whose own maximum lies further below the workgroup's reference point keeps its own offset
template <int DT> struct Range;
//   kHardLimit a row sum above this may come from probabilities that left the 16-bit type's range
//              (infinite, or saturated): the workgroup then computes its block again with a running maximum
template <> struct Range<COME_BF16> {
    static constexpr float kSumLimit = 1099511627776.f;   // 2^40
    static constexpr float kMaxGap = 64.f;
    // bf16 has the exponent range of fp32, but the fp32 outputs collect p * v over the 32 keys of a step: 2^100
    // leaves 2^27 of headroom for |v| and the accumulation, and is still far above kSumLimit
    static constexpr float kHardLimit = 1.2676506e30f;     // 2^100
};
template <> struct Range<COME_F16> {
    static constexpr float kSumLimit = 32.f;               // 2^5: a probability may grow by 2^11 more before fp16 saturates
    static constexpr float kMaxGap = 4.f;
    static constexpr float kHardLimit = 32768.f;           // one probability near 65504 (where the conversion saturates)
};

//
// PERSIST (short segments, 4 wavefronts): the launch has two workgroups per CU and every workgroup walks a list of work
// items - (segment, head, 256-query block) - of its own: item g, g + G, g + 2 G, ... of the launch's G workgroups.  The
// K / V / bias ring does not stop at the end of an item: the last iterations of an item stage the first tiles of the
// next one (other segment, other head), its Q rows are requested as soon as the last scores of the current item have
// been issued, and arrive while the current item is normalised and written.  What a short segment otherwise pays per
// workgroup - the chain of dependent latencies from the segment offsets to the first staged tiles, and the launch
// of a new workgroup - is paid once per workgroup instead of once per item.
template <int DT, int NW, bool EXACT, bool PERSIST>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_fwd_pipe_kernel(const AttnArgs a) {
    using E = Elem<DT>;
    constexpr float kSumLimit = Range<DT>::kSumLimit;
    static_assert(NW == 4 || NW == 8, "4 or 8 wavefronts per workgroup");
    static_assert(!PERSIST || NW == 4, "the item loop exists for 256-query workgroups");
    constexpr int kBlockM = 64 * NW;           // queries per workgroup
    constexpr int kThreads = 64 * NW;
    constexpr int kDma = 8 / NW;               // direct loads per wavefront for one K (or V) tile
    // K and V tiles: 64 rows of 128 bytes, unpadded, filled by direct global->LDS loads (a wavefront's
    // load lands as 1 KiB in lane order); bank conflicts are avoided by permuting the 16-byte chunks
    // inside a row: K chunk c of row r sits at slot c ^ ((r >> 1) & 7), V chunk c at c ^ (((r >> 1) & 1) << 2).
    // lds_b: per key one float, bias log2(e) (-inf beyond the end of the segment): the initial value of its scores.
    __shared__ __attribute__((aligned(1024))) uint16_t lds_k[kStages][kBlockN * kHeadDim];
    __shared__ __attribute__((aligned(1024))) uint16_t lds_v[kStages][kBlockN * kHeadDim];
    __shared__ __attribute__((aligned(16))) float lds_b[kStages][kBlockN];
    __shared__ __attribute__((aligned(256))) uint32_t lds_braw[kStages][kBlockN];   // raw bias words as loaded
    __shared__ float lds_ref[NW];                                                   // prologue: reference point per wavefront

    // ---- the work item (wave-uniform): rows seq_start .. + L of the packed tensors, one head, queries q0 .. of the
    // segment; key tiles tile_base .. tile_base + n_tiles (all tiles of the segment unless the workgroup computes a
    // key share into `piece`).  nx_*: PERSIST, the item after it.
    int seq_start = 0, L = 0, head = 0, q0 = 0, tile_base = 0, n_tiles = 0;
    float *piece = nullptr;
    int nx_seq_start = 0, nx_L = 0, nx_head = 0, nx_q0 = 0;
    bool has_next = false;
    // PERSIST: the workgroups of class c = blockIdx.x % 8 (dispatched to XCD c) share list c of the queue, which
    // attn_items_kernel filled with the query blocks of the units u = c mod 8, block after block and unit after unit, so
    // that the workgroups resident on one XCD work on the blocks of the same few units at the same time and find
    // their K / V in that L2.  A workgroup's first two items are fixed by its index; every further one is claimed from
    // the class counter, two items ahead: the claim is issued at the top of an item, published to the workgroup on the
    // last barrier of its key loop, and the item it names is looked up while the current item is written.
    // (The two workgroups of a CU do not run at the same pace: the one dispatched first wins every arbitration for the
    // matrix pipe and runs its tiles about 1.4 times as fast, for the whole launch.  A fixed share per workgroup would
    // leave the CUs half empty at the end; with the queue the faster one simply takes more items.)
    __shared__ uint32_t lds_claim;
    const uint32_t cls = blockIdx.x & 7u, per_cls = gridDim.x >> 3;
    const uint32_t *item_list = PERSIST ? a.queue + 16 + static_cast<size_t>(cls) * a.queue_cap : nullptr;
    uint32_t n_items = 0;
    int aa_seq_start = 0, aa_L = 0, aa_head = 0, aa_q0 = 0;          // the item after the next one
    auto decode_item = [&](uint32_t t, int &o_start, int &o_len, int &o_head, int &o_q0) __attribute__((always_inline)) {
        const uint32_t entry = item_list[t];
        const uint32_t unit = entry >> 8;
        segment_of(a, static_cast<int>(unit / static_cast<uint32_t>(a.n_heads)), o_start, o_len);
        o_head = static_cast<int>(unit % static_cast<uint32_t>(a.n_heads));
        o_q0 = static_cast<int>(entry & 255u) * kBlockM;
    };
    if constexpr (PERSIST) {
        n_items = a.queue[8 + cls];
        const uint32_t t0 = blockIdx.x >> 3, t1 = t0 + per_cls;
        if (t0 >= n_items) return;
        decode_item(t0, seq_start, L, head, q0);
        has_next = t1 < n_items;
        if (has_next) decode_item(t1, nx_seq_start, nx_L, nx_head, nx_q0);
    } else {
        int mblk, seq, tail, ks;
        if (!locate_block(a, mblk, head, seq, tail, ks)) return;
        segment_of(a, seq, seq_start, L);
        const int n_qblocks = (L + kBlockM - 1) / kBlockM;
        if (tail >= 0) {
            mblk = n_qblocks - a.nb_tail + tail;          // split workgroup: one of the unit's last query blocks
            if (mblk < 0) return;
        } else if (a.splits > 1 && mblk >= n_qblocks - a.nb_tail) {
            return;                                       // left to the split workgroups (or beyond the segment)
        }
        q0 = mblk * kBlockM;
        if (q0 >= L) return;
        // keys of this workgroup: all tiles, or share ks of them
        const int all_tiles = (L + kBlockN - 1) / kBlockN;
        tile_base = tail >= 0 ? static_cast<int>(static_cast<int64_t>(ks) * all_tiles / a.splits) : 0;
        n_tiles = (tail >= 0 ? static_cast<int>(static_cast<int64_t>(ks + 1) * all_tiles / a.splits) : all_tiles) - tile_base;
        if (tail >= 0) {
            const int64_t index = (static_cast<int64_t>(seq * a.n_heads + head) * a.nb_tail + tail) * a.splits + ks;
            piece = a.work + index * (kBlockM * (kHeadDim + kPieceExtra));
        }
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5;
    const int r = lane & 31;
    constexpr float kLog2e = 1.4426950408889634f;

    // ---- Q fragments (B operand: n = query r, k = head-dim 16 ks + 8 h ..).  EXACT: as they are - the scores leave
    // the MFMA unscaled and c is applied in fp32 in front of the exponential, as the reference applies it
    // (softmax.h:76-88).  Otherwise scaled by c here and rounded back to 16 bit.
    u32x4 qf[2][4];
    // (tl: the thread index, passed in so that the item loop can hand over a copy the compiler knows nothing about -
    // otherwise every address term that depends on the lane alone is kept in a register across the whole loop)
    auto load_q = [&](int tl, int start, int len, int hd, int first) __attribute__((always_inline)) {
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const int row = first + ((tl >> 6) * 2 + qt) * 32 + (tl & 31);
            const uint16_t *qp = a.q + static_cast<int64_t>(start + min(row, len - 1)) * a.q_rs + hd * a.q_hs + 8 * ((tl >> 5) & 1);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qf[qt][ks] = *reinterpret_cast<const u32x4 *>(qp + 16 * ks);
        }
    };
    auto scale_q = [&]() __attribute__((always_inline)) {
        if (EXACT) return;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t raw = qf[qt][ks][w];
                    qf[qt][ks][w] = E::pack2(E::to_f32(static_cast<uint16_t>(raw & 0xffffu)) * a.scale_log2,
                                             E::to_f32(static_cast<uint16_t>(raw >> 16)) * a.scale_log2);
                }
    };
    // The prologue of the attention (q LayerNorm + 2-D rotary embedding, qkv.py:31-39 of the reference's common
    // package) on the fragments just loaded, with the arithmetic and the summation order of the stand-alone pass, so
    // that the fragments hold the bits that pass would have written to memory.  A lane holds chunks 2 ks + h of its
    // query's head (ks = 0 .. 3): the rotation partner of a chunk (c ^ 2) is in the same lane, the neighbour in the
    // sums (c ^ 1) in lane l ^ 32.
    auto prepare_q = [&](int tl, int start, int len, int first) __attribute__((always_inline)) {
        using C = QkChunk<DT>;
        using V = Vec16<DT>;
        const int hh = (tl >> 5) & 1;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            uint4 word[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) word[ks] = __builtin_bit_cast(uint4, qf[qt][ks]);
            if (a.qp_norm) {
                float part[4];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) part[ks] = sum_across_halves(C::sum(word[ks]));
                const float mean = C::mean_of((part[0] + part[1]) + (part[2] + part[3]));
                float f[4][8];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    V::unpack(word[ks], f[ks]);
                    part[ks] = sum_across_halves(C::center(f[ks], mean));
                }
                const float rstd = C::inv_std((part[0] + part[1]) + (part[2] + part[3]), a.qp_eps);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    float g[8], b[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) g[i] = 1.f, b[i] = 0.f;
                    if (a.qp_gamma != nullptr) V::unpack(static_cast<const uint4 *>(a.qp_gamma)[2 * ks + hh], g);
                    if (a.qp_beta != nullptr) V::unpack(static_cast<const uint4 *>(a.qp_beta)[2 * ks + hh], b);
                    word[ks] = C::scale(f[ks], rstd, g, b);
                }
            }
            if (a.qp_pos != nullptr) {
                const int row = first + ((tl >> 6) * 2 + qt) * 32 + (tl & 31);
                const int64_t token = start + min(row, len - 1);
#pragma unroll
                for (int half = 0; half < 2; ++half) {                 // y: chunks 0 - 3 (ks 0, 1), x: chunks 4 - 7 (ks 2, 3)
                    const int entry = (C::table_row(a.qp_pos[token * 2 + half], a.qp_n_pos) * 16 + hh * 8) * V::ELEM_BYTES;
                    float c[8], sn[8], lo[8], hi[8];
                    V::unpack(*reinterpret_cast<const uint4 *>(static_cast<const char *>(a.qp_cos) + entry), c);
                    V::unpack(*reinterpret_cast<const uint4 *>(static_cast<const char *>(a.qp_sin) + entry), sn);
                    V::unpack(word[2 * half], lo);
                    V::unpack(word[2 * half + 1], hi);
                    word[2 * half] = C::rotate(lo, hi, c, sn, C::one_and_sign(false));
                    word[2 * half + 1] = C::rotate(hi, lo, c, sn, C::one_and_sign(true));
                }
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qf[qt][ks] = __builtin_bit_cast(u32x4, word[ks]);
        }
    };
    if constexpr (!PERSIST) {
        load_q(tid, seq_start, L, head, q0);
        if (a.qp_on) prepare_q(tid, seq_start, L, q0);
        scale_q();
    }
    // ---- global -> LDS staging.  Wavefront w fills rows 16 w .. 16 w + 15 of a tile with two direct
    // loads; lane l of load i brings row 8 (2 w + i) + l / 8, slot l % 8.  A key index beyond the segment
    // is redirected to its last key (finite data); such keys get a bias term of -inf, so their
    // probabilities are exactly 0 and neither their K nor their V row can reach the output.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // K, V of the item's segment and head; its bias as bytes from a 4-byte aligned base (b_mis: the misalignment of
    // the first key).  nx_*: the same for the next item.
    const char *k_seg, *v_seg, *b_seg, *nx_k_seg = nullptr, *nx_v_seg = nullptr, *nx_b_seg = nullptr;
    uint32_t b_mis, nx_b_mis = 0;
    auto segment_pointers = [&](int start, int hd, const char *&ks, const char *&vs, const char *&bs, uint32_t &mis) __attribute__((always_inline)) {
        ks = reinterpret_cast<const char *>(a.k + static_cast<int64_t>(start) * a.k_rs + hd * a.k_hs);
        vs = reinterpret_cast<const char *>(a.v + static_cast<int64_t>(start) * a.v_rs + hd * a.v_hs);
        const uintptr_t b_addr = reinterpret_cast<uintptr_t>(a.bias) + 2u * static_cast<uintptr_t>(start);
        bs = a.bias ? reinterpret_cast<const char *>(b_addr & ~static_cast<uintptr_t>(3)) : nullptr;
        mis = static_cast<uint32_t>(b_addr & 3);
    };
    segment_pointers(seq_start, head, k_seg, v_seg, b_seg, b_mis);
    const uint32_t k_rs_b = static_cast<uint32_t>(a.k_rs) * 2u, v_rs_b = static_cast<uint32_t>(a.v_rs) * 2u;
    uint32_t k_goff[kDma], v_goff[kDma], k_chunk[kDma], v_chunk[kDma];
    int st_row[kDma];
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
        st_row[i] = 8 * (kDma * wave + i) + (lane >> 3);
        k_chunk[i] = static_cast<uint32_t>((lane & 7) ^ ((st_row[i] >> 1) & 7)) * 16u;
        v_chunk[i] = static_cast<uint32_t>((lane & 7) ^ (((st_row[i] >> 1) & 1) << 2)) * 16u;
        k_goff[i] = static_cast<uint32_t>(st_row[i]) * k_rs_b + k_chunk[i];
        v_goff[i] = static_cast<uint32_t>(st_row[i]) * v_rs_b + v_chunk[i];
    }
    const uint32_t k_tile_step = static_cast<uint32_t>(kBlockN) * k_rs_b, v_tile_step = static_cast<uint32_t>(kBlockN) * v_rs_b;

    // rel_tile counts from the item's first tile; PERSIST: tiles behind the item's last one are the first tiles of the
    // next item (the ring runs on)
    auto stage_k = [&](int rel_tile, int buf) __attribute__((always_inline)) {
        const bool own = !PERSIST || rel_tile < n_tiles;                            // wave-uniform, like all of these
        const char *base = own ? k_seg : nx_k_seg;
        const int len = own ? L : nx_L;
        const int tile = tile_base + (own ? rel_tile : rel_tile - n_tiles);
        const int n0 = tile * kBlockN;
        const uint32_t tile_off = static_cast<uint32_t>(tile) * k_tile_step;
        const uint32_t last = static_cast<uint32_t>(len - 1) * k_rs_b;
        const bool full = n0 + kBlockN <= len;
#pragma unroll
        for (int i = 0; i < kDma; ++i) {
            uint32_t off = tile_off + k_goff[i];
            if (!full) off = n0 + st_row[i] < len ? off : last + k_chunk[i];
            dma_b128(base, off, lds_address(&lds_k[buf][(kDma * wave_u + i) * 512]));
        }
    };
    // raw bias of the 64 keys of a tile: wavefront 0 brings the aligned 32-bit word that holds each key's
    // 16-bit bias; it is converted to a float two iterations later (commit_bias)
    auto load_bias = [&](int rel_tile, int buf) __attribute__((always_inline)) {
        const bool own = !PERSIST || rel_tile < n_tiles;
        const char *base = own ? b_seg : nx_b_seg;
        const int len = own ? L : nx_L;
        const uint32_t mis = own ? b_mis : nx_b_mis;
        const int tile = tile_base + (own ? rel_tile : rel_tile - n_tiles);
        if (wave_u == 0 && a.bias) {
            const uint32_t key = static_cast<uint32_t>(min(tile * kBlockN + lane, len - 1));
            dma_b32(base, ((mis + 2u * key) & ~3u), lds_address(&lds_braw[buf][0]));
        }
    };
    auto stage_v = [&](int rel_tile, int buf) __attribute__((always_inline)) {
        const bool own = !PERSIST || rel_tile < n_tiles;
        const char *base = own ? v_seg : nx_v_seg;
        const int len = own ? L : nx_L;
        const int tile = tile_base + (own ? rel_tile : rel_tile - n_tiles);
        const int n0 = tile * kBlockN;
        const uint32_t tile_off = static_cast<uint32_t>(tile) * v_tile_step;
        const uint32_t last = static_cast<uint32_t>(len - 1) * v_rs_b;
        const bool full = n0 + kBlockN <= len;
#pragma unroll
        for (int i = 0; i < kDma; ++i) {
            uint32_t off = tile_off + v_goff[i];
            if (!full) off = n0 + st_row[i] < len ? off : last + v_chunk[i];
            dma_b128(base, off, lds_address(&lds_v[buf][(kDma * wave_u + i) * 512]));
        }
    };
    // conversion of the raw bias of one tile, split in two so that the LDS read is in flight during a slot:
    // peek_bias() requests the word, commit_bias() writes bias log2(e) - m_base as a float, -inf beyond the segment
    // EXACT: what the accumulators hold is in units of the raw scores, 1 / c of the exponent of exp2
    const float c_scale = a.scale_log2;
    const float inv_c = 1.0f / a.scale_log2;
    const float unit = EXACT ? inv_c : 1.f;
    float m_base = 0.f;           // reference point shared by the rows of the workgroup (uniform), log2 units
    uint32_t b_word = 0;
    auto peek_bias = [&](int buf) __attribute__((always_inline)) {
        if (wave_u == 0 && a.bias) b_word = lds_braw[buf][lane];
    };
    // (a tile of the next item is converted against a reference point of 0: its own is not known yet)
    auto commit_bias = [&](int rel_tile, int buf) __attribute__((always_inline)) {
        if (wave_u == 0) {
            const bool own = !PERSIST || rel_tile < n_tiles;
            const int len = own ? L : nx_L;
            const uint32_t mis = own ? b_mis : nx_b_mis;
            const float base = own ? m_base : 0.f;
            const int key = (tile_base + (own ? rel_tile : rel_tile - n_tiles)) * kBlockN + lane;
            float bias = 0.f;
            if (a.bias) {
                const uint32_t at = mis + 2u * static_cast<uint32_t>(min(key, len - 1));
                bias = E::to_f32(static_cast<uint16_t>((at & 2u) ? (b_word >> 16) : (b_word & 0xffffu)));
            }
            lds_b[buf][lane] = key < len ? (bias * kLog2e - base) * unit : -INFINITY;
        }
    };
    auto staged_wait = [&](bool with_bias_load) __attribute__((always_inline)) {
        // the direct loads issued in this iteration (K, V and, on wavefront 0, the bias) may stay in flight
        if (with_bias_load && wave_u == 0 && a.bias) {
            if (NW == 4) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
        } else {
            if (NW == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        }
    };

    // LDS read offsets (in elements) of this lane
    int k_rd[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) k_rd[ks] = r * kHeadDim + (((2 * ks + h) ^ ((r >> 1) & 7)) << 3);
    const int b_rd = 4 * h;                // keys 8 g + 4 h .. + 3 of a half-tile are accumulator elements 4 g .. 4 g + 3
    const int i16 = lane & 15;
    int v_rd[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
        v_rd[dt] = (4 * h + (i16 >> 2)) * kHeadDim +
                   (((4 * dt + 2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1)) ^ (((i16 >> 3) & 1) << 2)) << 3) + 4 * (i16 & 1);
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // s_acc[b][qt]: S'' of query tile qt for one 32-key half-tile; buffer b alternates between "being
    // turned into probabilities" and "being built by the matrix pipe".  p_frag[b][qt][u]: the
    // probabilities of that half-tile as B operands (u = 16-key step).
    f32x16 s_acc[2][2];
    f32x16 o_acc[2][2];          // [query tile][head-dim half]
    u32x4 p_frag[2][2][2];
    float m_run[2] = {0.f, 0.f};  // reference point of the row, log2 units: m_base + delta
    float delta[2] = {0.f, 0.f};  // what the row's reference point differs from m_base by (0 for nearly all rows)
    bool has_delta = false;       // wave-uniform: some row of this wavefront has delta != 0
    float l_run[2] = {0.f, 0.f};  // per-lane partial row sum (outside the key loop: the block that is computed again, the epilogues)
    // Row sums in the key loop come from the matrix pipe: with the probabilities of a 16-key step as the A operand of
    // v_mfma_f32_16x16x32 (row m = lane % 16, eight keys per lane: lane group g = lane / 16 holds query m + 16 (g & 1),
    // keys 8 (g >> 1) ..) and a B operand whose lane group g is all ones in column g & 1 and zero elsewhere, the result
    // column n = 0 / 1 holds the sums of queries m / m + 16 over the step's 16 keys, whatever order the unit gives the
    // keys inside a lane.  In the 16 x 16 result a lane holds column lane % 16, rows 4 (lane / 16) .. + 3: the sums of
    // queries 0 .. 15 sit in lanes 0, 16, 32, 48, those of queries 16 .. 31 in lanes 1, 17, 33, 49, four per lane, and
    // every other lane holds zeros.  Four such MFMAs per slot (64 cycles of the matrix pipe) replace 16 v_dot2c_f32,
    // which hold the matrix pipe for as long as eight of them and the vector ALU on top.
    // bf16 (kChain): the MFMAs accumulate straight onto the running sums and the range check looks at those - a running
    // sum beyond 2^40 moves the reference point just as well as a half-tile sum beyond it.  fp16: its limit (2^5) is
    // about the size of the current probabilities, which a running sum says nothing about, so the sums of a slot are
    // formed on their own and added afterwards.
    constexpr bool kChain = DT == COME_BF16;
    f32x4 l_acc[2];               // running row sums in that layout
    const u32x4 ones_sel = ((lane & 15) == ((lane >> 4) & 1))
                               ? u32x4{E::kOne | (E::kOne << 16), E::kOne | (E::kOne << 16), E::kOne | (E::kOne << 16), E::kOne | (E::kOne << 16)}
                               : zero4();
    const int sum_lane = (r >> 4) + 16 * ((r & 15) >> 2);         // where this lane's query keeps its row sum (element r & 3)
    // row sum of this lane's query out of that layout (a few LDS permutes: rare path and loop exit only)
    auto row_value = [&](const f32x4 &v) __attribute__((always_inline)) -> float {
        float out = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float t = __shfl(v[j], sum_lane);
            out = (r & 3) == j ? t : out;
        }
        return out;
    };

    // scores of both query tiles against half-tile `half` of the K tile in `buf`, into buffer b: the accumulators
    // start from the LDS bias values of their keys and collect the four k-steps of (c Q) K^T
    auto score_mfma = [&](int b, int buf, int half) __attribute__((always_inline)) {
        f32x16 seed;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 bq = *reinterpret_cast<const f32x4 *>(&lds_b[buf][32 * half + 8 * g + b_rd]);
#pragma unroll
            for (int e = 0; e < 4; ++e) seed[4 * g + e] = bq[e];
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const u32x4 kf = *reinterpret_cast<const u32x4 *>(&lds_k[buf][k_rd[ks] + 32 * half * kHeadDim]);
#pragma unroll
            for (int qt = 0; qt < 2; ++qt)
                s_acc[b][qt] = E::mfma(kf, qf[qt][ks], ks == 0 ? seed : s_acc[b][qt]);
        }
    };
    // O^T += V^T P^T of both query tiles for half-tile `half` of the V tile in `buf`, probabilities of buffer b
    auto pv_mfma = [&](int b, int buf, int half) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const uint16_t *vp = &lds_v[buf][v_rd[dt] + (32 * half + 16 * u) * kHeadDim];
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lds_read_tr(vp));
                const u32x2 hi2 = __builtin_bit_cast(u32x2, lds_read_tr(vp + 8 * kHeadDim));
                const u32x4 vf = u32x4{lo2[0], lo2[1], hi2[0], hi2[1]};
#pragma unroll
                for (int qt = 0; qt < 2; ++qt) o_acc[qt][dt] = E::mfma(vf, p_frag[b][qt][u], o_acc[qt][dt]);
            }
        }
    };

    // One slot in explicit issue order.  The vector ALU turns the scores in buffer X (one 32-key half-tile,
    // both query tiles) into probabilities.  Meanwhile the matrix pipe builds the scores of the next
    // half-tile in buffer Y (8 MFMAs on 4 K fragments, each fragment shared by both query tiles) and
    // adds the previous half-tile's P V (8 MFMAs on 4 V fragments, probabilities of buffer Y from the
    // previous slot).  Every MFMA is followed by a chunk of vector work and fragments are requested two
    // fragments (four MFMAs) ahead, so an in-order wavefront always has independent work behind each
    // MFMA.  sched_barrier keeps the compiler from regrouping the chunks.
    // Returns through ssum[qt] the row sums of the half-tile (layout of l_acc).
    auto slot = [&](int X, int Y, int kbuf, int khalf, int vbuf, int vhalf, f32x4 (&ssum)[2]) __attribute__((always_inline)) {
        // fragments 0..3: V (u, dt) of the P V MFMAs 0..7; fragments 4..7: K k-steps of the score MFMAs 8..15.
        // P V goes first: the probabilities of buffer Y die while those of buffer X are born, and the score
        // registers of buffer Y are not needed before half of buffer X has been consumed.
        u32x4 frag[8];
        f32x16 seed;                  // (bias log2(e) - m_base) * unit of this lane's 16 keys of the half-tile being scored
        auto request = [&](int f) __attribute__((always_inline)) {
            if (f < 4) {
                const int u = f >> 1, dt = f & 1;
                const uint16_t *vp = &lds_v[vbuf][v_rd[dt] + (32 * vhalf + 16 * u) * kHeadDim];
                const u32x2 lo2 = __builtin_bit_cast(u32x2, lds_read_tr(vp));
                const u32x2 hi2 = __builtin_bit_cast(u32x2, lds_read_tr(vp + 8 * kHeadDim));
                frag[f] = u32x4{lo2[0], lo2[1], hi2[0], hi2[1]};
            } else if (f < 8) {
                frag[f] = *reinterpret_cast<const u32x4 *>(&lds_k[kbuf][k_rd[f - 4] + 32 * khalf * kHeadDim]);
            }
        };
        auto issue = [&](int m) __attribute__((always_inline)) {
            const int f = m >> 1, qt = m & 1;
            // empty asm statements are ordering pins: MFMAs and exponentials are pure operations which the
            // compiler would otherwise float out of their chunk (sched_barrier only fences what is already there)
            if (qt == 0) asm volatile("" : "+v"(frag[f]));
            if (f < 4) {
                const int u = f >> 1, dt = f & 1;
                o_acc[qt][dt] = E::mfma(frag[f], p_frag[Y][qt][u], o_acc[qt][dt]);
            } else {
                s_acc[Y][qt] = E::mfma(frag[f], qf[qt][f - 4], f == 4 ? seed : s_acc[Y][qt]);
            }
        };
        request(0);
        request(1);
        const f32x4 zero4f = {0.f, 0.f, 0.f, 0.f};
        f32x4 &dst0 = kChain ? l_acc[0] : ssum[0];
        f32x4 &dst1 = kChain ? l_acc[1] : ssum[1];
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            // one MFMA per chunk: P V MFMAs 0..7, score MFMAs 8..15; fragments are requested four chunks ahead
            issue(c);
            if ((c & 1) == 0 && c <= 10) request((c >> 1) + 2);      // chunk 0 -> fragment 2, ..., chunk 10 -> fragment 7
            if (c >= 1 && c <= 4) {                                  // initial values of the scores, needed by chunk 8
                const f32x4 bq = *reinterpret_cast<const f32x4 *>(&lds_b[kbuf][32 * khalf + 8 * (c - 1) + b_rd]);
#pragma unroll
                for (int e = 0; e < 4; ++e) seed[4 * (c - 1) + e] = bq[e];
            }
            if (c > 0) {                    // pack and add the pair whose exponentials were issued one chunk ago
                const int pc = c - 1, qt = pc >> 3, w = pc & 7;
                const uint32_t pw = E::pack2_prob(p0, p1);
                p_frag[X][qt][w >> 2][w & 3] = pw;
                // a 16-key step of a query tile is complete: its row sums
                if (pc == 3) dst0 = E::mfma16(p_frag[X][0][0], ones_sel, kChain ? l_acc[0] : zero4f);
                if (pc == 7) dst0 = E::mfma16(p_frag[X][0][1], ones_sel, dst0);
                if (pc == 11) dst1 = E::mfma16(p_frag[X][1][0], ones_sel, kChain ? l_acc[1] : zero4f);
            }
            float s0 = s_acc[X][c >> 3][2 * (c & 7)], s1 = s_acc[X][c >> 3][2 * (c & 7) + 1];
            if (EXACT) {
                s0 *= c_scale;
                s1 *= c_scale;
            }
            p0 = __builtin_amdgcn_exp2f(s0);
            p1 = __builtin_amdgcn_exp2f(s1);
            asm volatile("" : "+v"(p0), "+v"(p1));
            __builtin_amdgcn_sched_barrier(0);
        }
        {
            const uint32_t pw = E::pack2_prob(p0, p1);
            p_frag[X][1][1][3] = pw;
            dst1 = E::mfma16(p_frag[X][1][1], ones_sel, dst1);
        }
        // the decision that follows the slot is tied to its end, so that the branch cannot be moved
        // above the probability chunks
        asm volatile("" : "+v"(dst1) : "v"(p_frag[X][1][1][3]));
    };

    // O[qt] *= f, in place.  Written as asm so that the accumulator tuples keep their registers across a
    // rarely taken branch (plain arithmetic makes the register allocator copy the 16-register tuples).
    auto scale_o = [&](int qt, float f) __attribute__((always_inline)) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float t = o_acc[qt][dt][e];
                asm volatile("v_mul_f32 %0, %1, %0" : "+v"(t) : "v"(f));
                o_acc[qt][dt][e] = t;
            }
    };

    // End of a slot.  Steady state: the range check (fp16: and adding the slot's row sums).  The scores the slot built (buffer Y) are
    // relative to m_base; rows whose reference point differs from it are corrected here (rare: it takes a
    // wavefront whose rows differ by more than 2^kMaxGap in magnitude, or a row sum that left the safe range).
    // When a row sum leaves the safe range the reference point of the row moves up by a power of two, 2^shift:
    //  - the row sum is rescaled now;
    //  - O is rescaled one slot later (o_pending), after the P V MFMAs of the probabilities just made,
    //    which are relative to the old reference, have been accumulated.
    float o_pending[2] = {1.f, 1.f};
    bool any_pending = false;                  // wave-uniform
    bool overflowed = false;                   // wave-uniform: some row sum exceeded kHardLimit
    auto finish_slot = [&](int Y, const f32x4 (&ssum)[2]) __attribute__((always_inline)) {
        // sums are not negative: if the four rows of a lane together stay within the limit, each of them does
        // (written so that a NaN counts as beyond it)
        // kChain: the running sums only grow between two moves of the reference point, so one query tile is looked
        // at per slot, each of them once per key tile (whatever the other collected in between is still in its sum)
        const f32x4 &c0 = kChain ? l_acc[Y] : ssum[0];
        const f32x4 &c1 = kChain ? l_acc[Y] : ssum[1];
        const float t0 = (c0[0] + c0[1]) + (c0[2] + c0[3]);
        const float t1 = kChain ? t0 : (c1[0] + c1[1]) + (c1[2] + c1[3]);
        const bool bad = !(t0 <= kSumLimit) || !(t1 <= kSumLimit);
        if (__any(bad) || any_pending || has_delta) {
            // the asm arithmetic below reads MFMA results; the compiler cannot see that, so the wait states an
            // MFMA result needs before a vector instruction may read it are spent here explicitly
            asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
            bool again = false;
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                if (any_pending) scale_o(qt, o_pending[qt]);
                // of this lane's query: over all 32 keys of the half-tile, or (kChain) over all keys so far
                float row_sum = row_value(kChain ? l_acc[qt] : ssum[qt]);
                asm volatile("" : "+v"(row_sum));       // keeps the arithmetic of this rare path inside the branch
                overflowed = overflowed || __any(!(row_sum <= Range<DT>::kHardLimit));
                const int shift = row_sum <= kSumLimit ? 0 : max(__builtin_amdgcn_frexp_expf(row_sum) - 2, 1);
                const float down = __builtin_amdgcn_exp2f(static_cast<float>(-shift));
                delta[qt] += static_cast<float>(shift);
                m_run[qt] += static_cast<float>(shift);
                const float d = EXACT ? delta[qt] * inv_c : delta[qt];       // EXACT: the accumulators hold unscaled scores
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float t = s_acc[Y][qt][e];
                    asm volatile("v_sub_f32 %0, %0, %1" : "+v"(t) : "v"(d));
                    s_acc[Y][qt][e] = t;
                }
                // the running sums, where they live: element j of a lane belongs to query 16 (lane % 16) + 4 (lane / 16) + j
                // (lanes whose column is neither 0 nor 1 hold zeros and stay zero)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float dj = __shfl(down, (16 * (lane & 15) + 4 * (lane >> 4) + j) & 31);
                    l_acc[qt][j] = (kChain ? l_acc[qt][j] : l_acc[qt][j] + ssum[qt][j]) * dj;
                }
                o_pending[qt] = down;
                again = again || __any(shift != 0);
            }
            any_pending = again;
            has_delta = __any(delta[0] != 0.f || delta[1] != 0.f);
        } else if (!kChain) {
            l_acc[0] += ssum[0];
            l_acc[1] += ssum[1];
        }
    };

    // ---- the item loop (a single pass unless PERSIST).  ring: stage of the item's tile 0 (the K / V / bias ring runs on
    // from item to item); cold: nothing of this item has been staged yet (first item, or the one after a block that
    // had to be computed again, which uses the stages for itself).
    int ring = 0;
    bool cold = true;
    for (;;) {
    int tl = tid;                            // this item's private copy of the thread index
    if constexpr (PERSIST) asm volatile("" : "+v"(tl));
    if constexpr (PERSIST) {
        // at least kStages tiles per item, so that what an iteration stages ahead never reaches beyond the next item;
        // tiles behind the end of the segment are masked like the tail of its last tile
        n_tiles = max((L + kBlockN - 1) / kBlockN, kStages);
        if (!has_next) {                     // staging ahead then re-reads the first tiles of this item
            nx_seq_start = seq_start;
            nx_L = L;
            nx_head = head;
        }
        segment_pointers(nx_seq_start, nx_head, nx_k_seg, nx_v_seg, nx_b_seg, nx_b_mis);
    }
    uint32_t claim = 0;                      // (one lane) what the class counter hands out for the item after next
    if constexpr (PERSIST) {
        if (has_next && tl == 0)
            claim = __hip_atomic_fetch_add(a.queue + cls, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (n_tiles <= 0) {                      // a key share without tiles (segment shorter than the split count)
        for (int i = tl; i < kBlockM; i += kThreads) {
            piece[kBlockM * kHeadDim + i] = -1e30f;               // reference point
            piece[kBlockM * (kHeadDim + 1) + i] = 0.f;            // row sum
        }
        return;
    }
    m_base = 0.f;
    o_pending[0] = 1.f;
    o_pending[1] = 1.f;
    any_pending = false;
    overflowed = false;
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        o_acc[qt][0] = zero16;
        o_acc[qt][1] = zero16;
        l_run[qt] = 0.f;
        l_acc[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            p_frag[b][qt][0] = zero4();
            p_frag[b][qt][1] = zero4();
        }
    }
    if (cold) {
        ring = 0;
        if constexpr (PERSIST) {
            __syncthreads();                   // (after a block that was computed again: nobody reads the stages any more)
            load_q(tl, seq_start, L, head, q0);
        }
        {   // the last V stage stands in for "tile -1": zeros (its probabilities are zero as well)
            u32x4 *z = reinterpret_cast<u32x4 *>(&lds_v[kStages - 1][0]);
            for (int i = tl; i < kBlockN * kHeadDim / 8; i += kThreads) z[i] = zero4();
        }
        load_bias(0, 0);
        load_bias(1, 1);
        load_bias(2, 2);
        load_bias(3, 3);
        stage_k(0, 0);
        stage_v(0, 0);
        stage_k(1, 1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        peek_bias(0);
        commit_bias(0, 0);
        peek_bias(1);
        commit_bias(1, 1);
        stage_k(2, 2);                     // tiles of iteration 1 start their flight
        stage_v(1, 1);
        staged_wait(false);                // everything but this last group has landed
    } else {
        // the previous item's last iterations staged K 0 .. 2, V 0 .. 1 and the bias of tiles 0 .. 3 of this one and
        // converted the bias of tiles 0 and 1; its V tiles stand in for "tile -1" (finite, times zero probabilities);
        // Q was requested behind its last iteration
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    if constexpr (PERSIST) scale_q();
    __syncthreads();
    const int st0 = ring & 3, st1 = (ring + 1) & 3;
    // Reference points.  Every row looks at its maximum over the first 32 keys; m_base is the largest of them in
    // the workgroup and is folded into the bias values in LDS, so that in the steady state nothing is subtracted
    // per score.  A row whose own maximum is more than 2^kMaxGap below m_base keeps the difference as its delta.
    score_mfma(0, st0, 0);             // bias values in LDS are still relative to 0: plain scores
    float row_max[2];
    float wave_max = -INFINITY;
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s_acc[0][qt][e]);
        mx = max_across_halves(mx) * (EXACT ? c_scale : 1.f);       // c > 0: the maximum commutes with the scale
        row_max[qt] = (mx == -INFINITY || mx != mx) ? 0.f : mx;
        wave_max = fmaxf(wave_max, row_max[qt]);
    }
#pragma unroll
    for (int d = 16; d >= 1; d >>= 1) wave_max = fmaxf(wave_max, __shfl_xor(wave_max, d));
    if (lane == 0) lds_ref[wave] = wave_max;
    __syncthreads();                   // also: every wavefront has read the bias values of tiles 0 and 1
    m_base = lds_ref[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) m_base = fmaxf(m_base, lds_ref[w]);
    if (wave_u == 0) {                 // tiles 0 and 1 were converted against a base of 0
        lds_b[st0][lane] -= m_base * unit;
        lds_b[st1][lane] -= m_base * unit;
    }
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const float gap = row_max[qt] - m_base;
        delta[qt] = gap < -Range<DT>::kMaxGap ? floorf(gap) : 0.f;
        m_run[qt] = m_base + delta[qt];
        // the same scores, now relative to the reference
        const float back = m_run[qt] * unit;
#pragma unroll
        for (int e = 0; e < 16; ++e) s_acc[0][qt][e] -= back;
    }
    has_delta = __any(delta[0] != 0.f || delta[1] != 0.f);
    __syncthreads();                   // the rebased bias values are visible

    // A wavefront whose 64 queries all lie beyond the end of the segment (last workgroup of a segment) only
    // helps with the staging: it has nothing to compute and nothing to write.  Wavefront 0 always has queries.
    const bool idle = q0 + wave_u * 64 >= L;
    if (idle) {
        for (int j = 0; j < n_tiles; ++j) {
            stage_k(j + 3, (ring + j + 3) & 3);
            stage_v(j + 2, (ring + j + 2) & 3);
            staged_wait(true);
            if (lane == 0) lds_ref[wave] = 0.f;
            __syncthreads();
        }
    } else {
        // one key tile: `kb` is the ring stage of tile j
        auto iteration = [&](int j, int kb) __attribute__((always_inline)) {
            const int kb1 = (kb + 1) & 3, kb2 = (kb + 2) & 3, kb3 = (kb + 3) & 3;   // stage of tile j + 1, ..
            load_bias(j + 4, kb);      // raw bias runs one more tile ahead (converted between the slots of iteration j+2)
            stage_k(j + 3, kb3);       // K(j+3) replaces K(j-1), V(j+2) replaces V(j-2): both idle since the
            stage_v(j + 2, kb2);       // last barrier; they are first read two barriers from now
            f32x4 sum[2];
            peek_bias(kb2);
            // slot a: keys 0..31 of tile j become probabilities; scores of keys 32..63; P V of keys 32..63 of tile j-1
            slot(0, 1, kb, 1, kb3, 1, sum);
            finish_slot(1, sum);
            commit_bias(j + 2, kb2);   // raw bias landed before the last barrier; published by the next one
            // slot b: keys 32..63 of tile j become probabilities; scores of keys 0..31 of tile j+1; P V of keys 0..31 of tile j
            slot(1, 0, kb1, 0, kb, 0, sum);
            finish_slot(0, sum);

            staged_wait(true);         // loads issued one iteration ago have landed
            if (lane == 0) lds_ref[wave] = overflowed ? 1.f : 0.f;      // (read behind the last of these barriers)
            if constexpr (PERSIST) {
                if (j == n_tiles - 1 && tl == 0) lds_claim = claim;
            }
            __syncthreads();
        };
        if constexpr (PERSIST || NW != 8) {
            for (int j = 0; j < n_tiles; ++j) iteration(j, (ring + j) & 3);
        } else {
            // long segments (the ring starts at stage 0): four tiles per turn of the loop make every stage a constant,
            // so that the fragment reads address LDS through their offset fields instead of through six additions
            // per slot (+2.5 %).  The workgroups of short segments keep the plain loop: their few tiles do not repay
            // the registers the four copies cost there.
            int j = 0;
            for (; j + 4 <= n_tiles; j += 4) {
                iteration(j, 0);
                iteration(j + 1, 1);
                iteration(j + 2, 2);
                iteration(j + 3, 3);
            }
            if (j < n_tiles) {
                iteration(j, 0);
                if (j + 1 < n_tiles) {
                    iteration(j + 1, 1);
                    if (j + 2 < n_tiles) iteration(j + 2, 2);
                }
            }
        }
    }

    // ---- Probabilities are stored in the 16-bit type relative to a reference point that follows the scores lazily.
    // A key that beats everything its row has seen by more than that type can hold (2^127 for bf16, about 2^15 for
    // fp16) within one 32-key step leaves an infinite or saturated probability behind.  The wavefront that saw such a
    // row sum said so in front of the loop's last barrier, and the workgroup then computes its block once more with the textbook running maximum
    // (one tile at a time, no pipelining: slow, exact for any scores, and never taken by ordinary attention logits).
    if constexpr (kChain) {
        // The checks inside the loop look at one query tile per slot: what the last slot added to the other one is
        // looked at here (only a sum beyond the hard limit matters now), and the wavefront's word is said once more.
        if (!idle) {
            const float ta = (l_acc[0][0] + l_acc[0][1]) + (l_acc[0][2] + l_acc[0][3]);
            const float tb = (l_acc[1][0] + l_acc[1][1]) + (l_acc[1][2] + l_acc[1][3]);
            overflowed = overflowed || __any(!(ta <= Range<DT>::kHardLimit) || !(tb <= Range<DT>::kHardLimit));
            if (lane == 0) lds_ref[wave] = overflowed ? 1.f : 0.f;
        }
        __syncthreads();
    }
    bool again = false;
#pragma unroll
    for (int w = 0; w < NW; ++w) again = again || lds_ref[w] != 0.f;
    bool has_after = false;
    if constexpr (PERSIST) {
        if (has_next) {
            const uint32_t t2 = 2u * per_cls + static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(lds_claim)));
            has_after = t2 < n_items;
            if (has_after) decode_item(t2, aa_seq_start, aa_L, aa_head, aa_q0);
        }
        // Q of the next item: requested now, needed behind this item's epilogue (a block that is computed again
        // still needs its own Q; the next item then starts cold)
        if (!again && has_next) load_q(tl, nx_seq_start, nx_L, nx_head, nx_q0);
    }
    if (!idle) {
        if (!again) {
            // the row sums leave the layout of the key loop: the lower half-wave carries the total, the upper one nothing
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                const float total = row_value(l_acc[qt]);
                l_run[qt] = h == 0 ? total : 0.f;
            }
            pv_mfma(1, (ring + n_tiles - 1) & 3, 1);      // keys 32..63 of the last tile
#pragma unroll
            for (int qt = 0; qt < 2; ++qt)
#pragma unroll
                for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o_acc[qt][dt][e] *= o_pending[qt];
        }
    }
    if (again) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // no direct load is in flight any more
        m_base = 0.f;                                           // the seeds are absolute now
        float m_row[2] = {-INFINITY, -INFINITY};
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            o_acc[qt][0] = zero16;
            o_acc[qt][1] = zero16;
            l_run[qt] = 0.f;
        }
        for (int j = 0; j < n_tiles; ++j) {
            __syncthreads();                                    // stage 0 is free again
            load_bias(j, 0);
            stage_k(j, 0);
            stage_v(j, 0);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            peek_bias(0);
            commit_bias(j, 0);
            __syncthreads();
            if (idle) continue;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                score_mfma(0, 0, half);
#pragma unroll
                for (int qt = 0; qt < 2; ++qt) {
                    float ex[16];
                    float mx = -INFINITY;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        ex[e] = EXACT ? s_acc[0][qt][e] * c_scale : s_acc[0][qt][e];
                        mx = fmaxf(mx, ex[e]);
                    }
                    mx = fmaxf(max_across_halves(mx), m_row[qt]);
                    const float ref = mx == -INFINITY ? 0.f : mx;          // a row that has seen masked keys only
                    const float down = __builtin_amdgcn_exp2f(m_row[qt] - ref);
                    m_row[qt] = mx;
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                        for (int e = 0; e < 16; ++e) o_acc[qt][dt][e] *= down;
                    float part = 0.f;
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        const uint32_t pw = E::pack2_prob(__builtin_amdgcn_exp2f(ex[2 * w] - ref),
                                                          __builtin_amdgcn_exp2f(ex[2 * w + 1] - ref));
                        p_frag[0][qt][w >> 2][w & 3] = pw;
                        part = E::dot2_ones(pw, part);
                    }
                    l_run[qt] = l_run[qt] * down + part;
                }
                pv_mfma(0, 0, half);
            }
        }
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) m_run[qt] = m_row[qt] == -INFINITY ? 0.f : m_row[qt];
        __syncthreads();                                        // the epilogue reuses the stages
    }

    // ---- epilogue of a split workgroup: unnormalised outputs, reference point and row sum of its key share
    const int wave_e = tl >> 6, r_e = tl & 31, h_e = (tl >> 5) & 1;
    if (!idle && piece != nullptr) {
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const float l_tot = sum_across_halves(l_run[qt]);
            const int local_row = (wave_e * 2 + qt) * 32 + r_e;
            if (q0 + local_row < L) {
                float *op = piece + local_row * kHeadDim + 4 * h_e;
#pragma unroll
                for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        *reinterpret_cast<f32x4 *>(op + 32 * dt + 8 * g) =
                            f32x4{o_acc[qt][dt][4 * g], o_acc[qt][dt][4 * g + 1], o_acc[qt][dt][4 * g + 2],
                                  o_acc[qt][dt][4 * g + 3]};
                if (h_e == 0) {
                    piece[kBlockM * kHeadDim + local_row] = m_run[qt];
                    piece[kBlockM * (kHeadDim + 1) + local_row] = l_tot;
                }
            }
        }
    }

    // ---- epilogue: normalise, write O (and LSE).  In the accumulators a lane holds 8-byte pieces of one output row,
    // 32 rows per store instruction; written like that, a wavefront's 32 stores touch 32 rows each and queue up in the
    // memory pipeline for microseconds.  Each wavefront therefore passes its two 32 x 64 tiles through 4 KiB of LDS
    // (16-byte chunk c of row r at chunk c ^ (r & 7)) and stores whole 128-byte rows, eight rows per instruction.
    // The LDS comes from stages nothing reads or fills any more: K of the item's last tile and V of the one before
    // (their next loads are issued behind at least one barrier from here), for wavefronts 4 .. 7 the K stages of the
    // two tiles staged ahead of the end, which have landed.
    if (!idle && piece == nullptr) {
        const int last = ring + n_tiles - 1;
        uint16_t *slot_base = wave_u < 2   ? &lds_k[last & 3][2048 * wave_u]
                              : wave_u < 4 ? &lds_v[(last - 1) & 3][2048 * (wave_u - 2)]
                              : wave_u < 6 ? &lds_k[(last + 1) & 3][2048 * (wave_u - 4)]
                                           : &lds_k[(last + 2) & 3][2048 * (wave_u - 6)];
        const int lane_e = tl & 63;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const float l_tot = sum_across_halves(l_run[qt]);
            const float inv = 1.0f / l_tot;
            const int row = q0 + (wave_e * 2 + qt) * 32 + r_e;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = E::pack2(o_acc[qt][dt][4 * g] * inv, o_acc[qt][dt][4 * g + 1] * inv);
                    w[1] = E::pack2(o_acc[qt][dt][4 * g + 2] * inv, o_acc[qt][dt][4 * g + 3] * inv);
                    *reinterpret_cast<u32x2 *>(slot_base + r_e * 64 + (((4 * dt + g) ^ (r_e & 7)) << 3) + 4 * h_e) = w;
                }
            if (row < L && h_e == 0 && a.lse)
                a.lse[static_cast<int64_t>(head) * a.total + seq_start + row] =
                    (m_run[qt] + __log2f(l_tot)) * 0.6931471805599453f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tr = 8 * i + (lane_e >> 3);                      // row of the tile, 8 lanes per row
                const int c = (lane_e & 7) ^ (tr & 7);                     // the chunk this lane finds at position lane % 8
                const u32x4 v = *reinterpret_cast<const u32x4 *>(slot_base + tr * 64 + ((lane_e & 7) << 3));
                const int orow = q0 + (wave_e * 2 + qt) * 32 + tr;
                if (orow < L) {
                    uint16_t *op = a.out + static_cast<int64_t>(seq_start + orow) * a.o_rs + head * a.o_hs + 8 * c;
                    if (a.out_wide) {
                        *reinterpret_cast<u32x4 *>(op) = v;
                    } else {
                        *reinterpret_cast<u32x2 *>(op) = u32x2{v[0], v[1]};
                        *reinterpret_cast<u32x2 *>(op + 4) = u32x2{v[2], v[3]};
                    }
                }
            }
        }
    }
    if constexpr (!PERSIST) {
        return;
    } else {
        if (!has_next) return;
        ring = (ring + n_tiles) & 3;
        cold = again;
        seq_start = nx_seq_start;
        L = nx_L;
        head = nx_head;
        q0 = nx_q0;
        k_seg = nx_k_seg;
        v_seg = nx_v_seg;
        b_seg = nx_b_seg;
        b_mis = nx_b_mis;
        has_next = has_after;
        nx_seq_start = aa_seq_start;
        nx_L = aa_L;
        nx_head = aa_head;
        nx_q0 = aa_q0;
    }
    }   // item loop
}

// Work queue of a launch of resident workgroups (PERSIST above), built from the segment offsets on the device: one
// wavefront per class c writes list c - for every (segment, head) unit u = c mod 8 in turn the entries (u << 8 | b) of
// its query blocks b = 0 .. ceil(L / 256) - 1, full blocks first - together with the length of the list, and clears
// the class's claim counter.  No empty entries: a bound on the segment lengths that is far above them (a caller that
// does not want to read the longest segment back) costs nothing.  One launch of one workgroup in front of the
// attention kernel; 64 units per step and wavefront.
__global__ __launch_bounds__(512) void attn_items_kernel(const AttnArgs a) {
    const uint32_t lane = threadIdx.x & 63u, cls = threadIdx.x >> 6;
    uint32_t *list = a.queue + 16 + static_cast<size_t>(cls) * a.queue_cap;
    const uint32_t n_units = static_cast<uint32_t>(a.n_units);
    const uint32_t per_class = n_units > cls ? (n_units - cls + 7u) / 8u : 0u;       // units cls, cls + 8, ...
    uint32_t carry = 0;
    for (uint32_t i0 = 0; i0 < per_class; i0 += 64u) {
        const uint32_t i = i0 + lane, unit = cls + 8u * i;
        uint32_t nb = 0;
        if (i < per_class) {
            int start, len;
            segment_of(a, static_cast<int>(unit / static_cast<uint32_t>(a.n_heads)), start, len);
            nb = static_cast<uint32_t>(min((len + 255) / 256, a.n_mblocks));         // (never beyond the list)
        }
        uint32_t incl = nb;
#pragma unroll
        for (uint32_t d = 1; d < 64u; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        const uint32_t at = carry + incl - nb;
        for (uint32_t b = 0; b < nb; ++b) list[at + b] = (unit << 8) | b;
        carry += __shfl(incl, 63);
    }
    if (lane == 0) {
        a.queue[8 + cls] = carry;
        a.queue[cls] = 0;
    }
}

// Combines the key shares of the split query blocks: with m* the largest reference point of a row,
// O = sum_i 2^(m_i - m*) O_i / sum_i 2^(m_i - m*) l_i.  One thread per (row, four output elements); a workgroup
// covers 16 rows of a split query block, so the grid is (split query blocks) x block_m / 16 workgroups.
template <int DT>
__global__ __launch_bounds__(256) void attn_combine_kernel(const AttnArgs a, int block_m) {
    using E = Elem<DT>;
    const int groups = block_m / 16;
    const int group = blockIdx.x % groups;
    const int block = blockIdx.x / groups;
    const int tail = block % a.nb_tail;
    const int unit = block / a.nb_tail;
    const int head = unit % a.n_heads;
    const int seq = unit / a.n_heads;
    int seq_start, L;
    segment_of(a, seq, seq_start, L);
    const int mblk = (L + block_m - 1) / block_m - a.nb_tail + tail;
    if (mblk < 0) return;
    const int q0 = mblk * block_m;
    const int64_t piece_floats = static_cast<int64_t>(block_m) * (kHeadDim + kPieceExtra);
    const float *first = a.work + (static_cast<int64_t>(unit) * a.nb_tail + tail) * a.splits * piece_floats;
    {
        const int idx = group * 256 + threadIdx.x;
        const int local_row = idx / (kHeadDim / 4);
        const int c4 = idx % (kHeadDim / 4);
        if (q0 + local_row >= L) return;
        float m_star = -INFINITY;
        for (int i = 0; i < a.splits; ++i) {
            const float *pc = first + i * piece_floats;
            if (pc[block_m * (kHeadDim + 1) + local_row] > 0.f) m_star = fmaxf(m_star, pc[block_m * kHeadDim + local_row]);
        }
        float l_sum = 0.f;
        f32x4 o = {0.f, 0.f, 0.f, 0.f};
        for (int i = 0; i < a.splits; ++i) {
            const float *pc = first + i * piece_floats;
            const float l_i = pc[block_m * (kHeadDim + 1) + local_row];
            if (!(l_i > 0.f)) continue;
            const float w = __builtin_amdgcn_exp2f(pc[block_m * kHeadDim + local_row] - m_star);
            l_sum += w * l_i;
            const f32x4 v = *reinterpret_cast<const f32x4 *>(pc + local_row * kHeadDim + 4 * c4);
            o += v * w;
        }
        const float inv = 1.0f / l_sum;
        u32x2 packed;
        packed[0] = E::pack2(o[0] * inv, o[1] * inv);
        packed[1] = E::pack2(o[2] * inv, o[3] * inv);
        *reinterpret_cast<u32x2 *>(a.out + static_cast<int64_t>(seq_start + q0 + local_row) * a.o_rs + head * a.o_hs + 4 * c4) = packed;
        if (c4 == 0 && a.lse)
            a.lse[static_cast<int64_t>(head) * a.total + seq_start + q0 + local_row] =
                (m_star + __log2f(l_sum)) * 0.6931471805599453f;
    }
}

// How a launch is shaped.
//  - 8 wavefronts per workgroup share every staged K / V tile among 512 queries (half the L2 -> LDS traffic),
//    but such a workgroup fills a whole CU, so a partly filled last round of workgroups costs a full round.
//    Without a work buffer it is used for long segments only when the expected number of workgroups nearly
//    fills its last round; otherwise two 256-query workgroups share a CU and the last round finishes early.
//  - With a work buffer the query blocks of that last round are cut along the keys into `splits` workgroups
//    each, which fill the chip with short pieces instead; a small kernel combines the pieces.
//  - Segments of at most kPersistMaxSeqlen keys: with a work buffer the launch is two resident workgroups per CU
//    that take their query blocks from a queue in the buffer (attn_items_kernel builds it first); without one,
//    one workgroup per query block as for everything else.
struct Plan {
    bool wide = false;
    int nb_tail = 0, splits = 1;
    bool persist = false;
    int64_t queue_cap = 0;
    int64_t work_bytes = 0;
};

int cu_count() {
    static const int n_cu = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        return n;
    }();
    return n_cu;
}

// Bytes of the work queue of a launch of resident workgroups (0: the shape is not eligible).
int64_t queue_cap_of(int64_t n_seq, int64_t n_heads, int64_t max_seqlen) {
    const int64_t units = n_seq * n_heads;
    if (max_seqlen <= 0 || max_seqlen > kPersistMaxSeqlen || units <= 0 || units > 65536) return 0;
    return ceil_div(units, 8) * ceil_div(max_seqlen, 256);
}

Plan make_plan(int64_t n_seq, int64_t total, int64_t n_heads, int64_t max_seqlen, bool may_split, bool work_queue) {
    Plan p;
    const int64_t units = n_seq * n_heads;
    if (max_seqlen <= kPersistMaxSeqlen) {
        if (work_queue && may_split && queue_cap_of(n_seq, n_heads, max_seqlen) > 0) {
            p.persist = true;
            p.queue_cap = ceil_div(units, 8) * ceil_div(max_seqlen, 256);
            p.work_bytes = static_cast<int64_t>(sizeof(uint32_t)) * (16 + 8 * p.queue_cap);
        }
        return p;
    }
    if (max_seqlen < 4096) return p;
    const int n_cu = cu_count();
    // one segment: exact; several: half a block of padding per segment on average
    const int64_t expected = n_seq == 1 ? n_heads * ceil_div(total, 512) : n_heads * ceil_div(total + n_seq * 256, 512);
    const int64_t rounds = ceil_div(expected, n_cu);
    if (expected * 100 >= rounds * n_cu * 95) {
        p.wide = true;
        return p;
    }
    if (!may_split) return p;
    const int64_t full = expected / n_cu;
    const int64_t tail = expected - full * n_cu;
    if (full == 0 || tail == 0) return p;
    const int64_t nb_tail = ceil_div(tail, units);
    const int64_t tiles = ceil_div(max_seqlen, kBlockN);
    int best = 0;
    double best_cost = 0.6;                          // what the partly filled last round of 256-query workgroups costs
    for (int sp = 2; sp <= 8; ++sp) {
        if (tiles / sp < 16) break;                  // pieces of at least 16 key tiles
        const double cost = static_cast<double>(ceil_div(nb_tail * units * sp, n_cu)) / sp + 0.02 * sp;
        if (cost < best_cost) {
            best_cost = cost;
            best = sp;
        }
    }
    if (best == 0 || nb_tail > ceil_div(max_seqlen, 512)) return p;
    p.wide = true;
    p.nb_tail = static_cast<int>(nb_tail);
    p.splits = best;
    p.work_bytes = units * nb_tail * best * 512 * (kHeadDim + kPieceExtra) * static_cast<int64_t>(sizeof(float));
    return p;
}

}  // namespace
}  // namespace come

using namespace come;

extern "C" int64_t come_attn_queue_bytes(int64_t n_seq, int64_t n_heads, int64_t max_seqlen) {
    const int64_t cap = queue_cap_of(n_seq, n_heads, max_seqlen);
    return cap > 0 ? static_cast<int64_t>(sizeof(uint32_t)) * (16 + 8 * cap) : 0;
}

extern "C" int64_t come_attn_work_bytes(int64_t n_seq, int64_t total, int64_t n_heads, int64_t max_seqlen) {
    if (n_seq <= 0 || total <= 0 || n_heads <= 0 || max_seqlen <= 0) return 0;
    return make_plan(n_seq, total, n_heads, max_seqlen, true, false).work_bytes;
}

// Address of this device's copy of `scratch` (nullptr + error message on failure).  The array's name is only a
// host-side handle: the device address is asked for once per device, with that device current, and kept.
static void *static_work_pointer() {
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static void *known[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("come_attn_varlen_fwd_static: no usable current device (%s)", hipGetErrorString(e));
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(lock);
    if (known[dev] == nullptr) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            set_error("come_attn_varlen_fwd_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return nullptr;
        }
        known[dev] = p;
    }
    return known[dev];
}

// Shared body of the attention entry points.  static_work: the buffer is the library's own fixed-size array; a launch
// that needs more is an error instead of a launch without the key split.
static int attn_varlen_fwd_impl(const void *q, const void *k, const void *v, int dtype, int64_t q_row_stride,
                                int64_t q_head_stride, int64_t k_row_stride, int64_t k_head_stride,
                                int64_t v_row_stride, int64_t v_head_stride, const int32_t *cu_seqlens,
                                int64_t n_seq, int64_t total, int64_t n_heads, int64_t head_dim,
                                const void *perkey_bias, int64_t max_seqlen, float softmax_scale, void *out,
                                int64_t o_row_stride, int64_t o_head_stride, float *lse, void *work,
                                int64_t work_bytes, bool static_work, int flags, void *stream,
                                const come_q_prologue *qp = nullptr) {
    clear_error();
    COME_REQUIRE((flags & ~(COME_ATTN_FOLD_SCALE | COME_ATTN_WORK_QUEUE)) == 0, COME_ERR_INVALID,
                 "come_attn_varlen_fwd: unknown bits in flags (%d)", flags);
    COME_REQUIRE(dtype == COME_BF16 || dtype == COME_F16, COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: only fp16 and bf16 are supported");
    COME_REQUIRE(head_dim == 32 || head_dim == kHeadDim || head_dim == 128, COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: head_dim must be 32, 64 or 128 (got %lld)", (long long)head_dim);
    COME_REQUIRE(n_seq > 0, COME_ERR_INVALID, "come_attn_varlen_fwd: batch size must be positive");
    COME_REQUIRE(total >= 0 && n_heads > 0 && max_seqlen >= 0, COME_ERR_INVALID,
                 "come_attn_varlen_fwd: negative size");
    COME_REQUIRE(total < (1ll << 31) && n_heads < 65536 && n_seq < (1ll << 24), COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: problem too large");
    COME_REQUIRE(softmax_scale > 0.f && softmax_scale < INFINITY, COME_ERR_INVALID,
                 "come_attn_varlen_fwd: softmax_scale must be positive and finite");
    if (total == 0 || max_seqlen == 0) return COME_OK;
    // offsets inside a segment are 32-bit byte offsets from the segment's first row
    COME_REQUIRE(max_seqlen * (k_row_stride > v_row_stride ? k_row_stride : v_row_stride) * 2 < (1ll << 32),
                 COME_ERR_UNSUPPORTED, "come_attn_varlen_fwd: a segment may span at most 4 GiB of K or V rows");
    COME_REQUIRE(q && k && v && out && cu_seqlens, COME_ERR_INVALID, "come_attn_varlen_fwd: NULL tensor");
    const int64_t strides[8] = {q_row_stride, q_head_stride, k_row_stride, k_head_stride,
                                v_row_stride, v_head_stride, o_row_stride, o_head_stride};
    for (int i = 0; i < 8; ++i)
        COME_REQUIRE(strides[i] >= head_dim || (i % 2 == 1 && n_heads == 1), COME_ERR_INVALID,
                     "come_attn_varlen_fwd: stride %d is smaller than head_dim", i);
    for (int i = 0; i < 6; ++i)
        COME_REQUIRE(strides[i] % 8 == 0, COME_ERR_UNSUPPORTED,
                     "come_attn_varlen_fwd: q/k/v strides must be multiples of 8 elements (16-byte loads)");
    COME_REQUIRE(o_row_stride % 4 == 0 && o_head_stride % 4 == 0, COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: out strides must be multiples of 4 elements");
    COME_REQUIRE((reinterpret_cast<uintptr_t>(q) & 15) == 0 && (reinterpret_cast<uintptr_t>(k) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(v) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0,
                 COME_ERR_UNSUPPORTED, "come_attn_varlen_fwd: q/k/v must be 16-byte aligned, out 8-byte aligned");

    if (qp != nullptr) {
        COME_REQUIRE(head_dim == kHeadDim, COME_ERR_UNSUPPORTED, "come_attn_varlen_fwd_qp: head_dim must be 64");
        COME_REQUIRE((flags & COME_ATTN_WORK_QUEUE) == 0, COME_ERR_UNSUPPORTED,
                     "come_attn_varlen_fwd_qp: not available together with COME_ATTN_WORK_QUEUE");
        COME_REQUIRE(qp->eps >= 0.f, COME_ERR_INVALID, "come_attn_varlen_fwd_qp: eps must be >= 0");
        const void *aligned[] = {qp->weight, qp->bias, qp->cos_table, qp->sin_table};
        for (const void *p : aligned)
            COME_REQUIRE((reinterpret_cast<uintptr_t>(p) & 15) == 0, COME_ERR_INVALID,
                         "come_attn_varlen_fwd_qp: prologue pointers must be 16-byte aligned");
        if (qp->positions != nullptr)
            COME_REQUIRE(qp->cos_table != nullptr && qp->sin_table != nullptr && qp->n_pos > 0 && qp->n_pos < (1 << 24),
                         COME_ERR_INVALID, "come_attn_varlen_fwd_qp: positions need cos / sin tables with 0 < n_pos < 2^24");
    }
    if (head_dim != kHeadDim) {               // the other widths: one kernel, no work buffer
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
        a.n_units = static_cast<int>(n_seq * n_heads);
        a.scale_log2 = softmax_scale * 1.4426950408889634f;
        a.splits = 1;
        return launch_attn_hd(a, dtype, static_cast<int>(head_dim), max_seqlen, static_cast<hipStream_t>(stream));
    }
    const bool want_queue = (flags & COME_ATTN_WORK_QUEUE) != 0;
    Plan plan = make_plan(n_seq, total, n_heads, max_seqlen, work != nullptr || static_work, want_queue);
    if (static_work && (plan.splits > 1 || plan.persist)) {
        COME_REQUIRE(plan.work_bytes <= kStaticWorkBytes, COME_ERR_UNSUPPORTED,
                     "come_attn_varlen_fwd_static: this launch needs a work buffer of %lld bytes, the built-in one "
                     "holds %lld; use come_attn_varlen_fwd_ws with a buffer of come_attn_work_bytes() bytes",
                     (long long)plan.work_bytes, (long long)kStaticWorkBytes);
        work = static_work_pointer();
        if (work == nullptr) return COME_ERR_HIP;
        work_bytes = kStaticWorkBytes;
    }
    if ((plan.splits > 1 || plan.persist) && (work_bytes < plan.work_bytes || (reinterpret_cast<uintptr_t>(work) & 15) != 0))
        plan = make_plan(n_seq, total, n_heads, max_seqlen, false, false);  // buffer too small or misaligned: neither split nor queue
    const bool wide = plan.wide;
    const int kBlockM = wide ? 512 : 256;
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
    a.scale_log2 = softmax_scale * 1.4426950408889634f;
    a.n_units = static_cast<int>(n_seq * n_heads);
    a.rotate = (!wide && a.n_mblocks % 2 == 0) ? 1 : 0;
    a.out_wide = (o_row_stride % 8 == 0 && o_head_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) ? 1 : 0;
    a.nb_tail = plan.nb_tail;
    a.splits = plan.splits;
    a.work = static_cast<float *>(work);
    a.queue = static_cast<uint32_t *>(work);
    a.queue_cap = static_cast<int>(plan.queue_cap);
    if (qp != nullptr && (qp->apply_norm || qp->positions != nullptr)) {
        a.qp_on = 1;
        a.qp_norm = qp->apply_norm ? 1 : 0;
        a.qp_gamma = qp->weight;
        a.qp_beta = qp->bias;
        a.qp_eps = qp->eps;
        a.qp_pos = qp->positions;
        a.qp_cos = qp->cos_table;
        a.qp_sin = qp->sin_table;
        a.qp_n_pos = qp->n_pos;
    }
    a.n_full_wg = ceil_div(n_seq * n_heads, 8) * 8 * a.n_mblocks;
    const int64_t n_wg = a.n_full_wg + ceil_div(n_seq * n_heads, 8) * 8 * (plan.splits > 1 ? plan.nb_tail * plan.splits : 0);
    const int64_t n_cwg = n_seq * n_heads * plan.nb_tail * (kBlockM / 16);       // combine kernel: 16 rows each
    COME_REQUIRE(n_wg < (1ll << 31) && n_cwg < (1ll << 31), COME_ERR_UNSUPPORTED,
                 "come_attn_varlen_fwd: grid too large");
    const dim3 grid(static_cast<unsigned>(n_wg)), block(wide ? 512 : 256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool exact = (flags & COME_ATTN_FOLD_SCALE) == 0;
    // short segments with a buffer for the queue: two workgroups per CU that take their items from it
    const bool persist = plan.persist;
    if (persist) {
        hipLaunchKernelGGL(attn_items_kernel, dim3(1), dim3(512), 0, s, a);
        COME_CHECK_LAUNCH("come_attn_varlen_fwd (work queue)");
    }
    const int64_t resident = (2 * static_cast<int64_t>(cu_count())) & ~7ll;
    const dim3 pgrid(static_cast<unsigned>(n_wg < resident ? n_wg : resident));
#define COME_ATTN_LAUNCH(DT_, NW_)                                                                                 \
    do {                                                                                                           \
        if (exact) hipLaunchKernelGGL((attn_fwd_pipe_kernel<DT_, NW_, true, false>), grid, block, 0, s, a);        \
        else hipLaunchKernelGGL((attn_fwd_pipe_kernel<DT_, NW_, false, false>), grid, block, 0, s, a);             \
    } while (0)
#define COME_ATTN_LAUNCH_ITEMS(DT_)                                                                                \
    do {                                                                                                           \
        if (exact) hipLaunchKernelGGL((attn_fwd_pipe_kernel<DT_, 4, true, true>), pgrid, block, 0, s, a);          \
        else hipLaunchKernelGGL((attn_fwd_pipe_kernel<DT_, 4, false, true>), pgrid, block, 0, s, a);               \
    } while (0)
    if (persist) {
        if (dtype == COME_BF16) COME_ATTN_LAUNCH_ITEMS(COME_BF16);
        else COME_ATTN_LAUNCH_ITEMS(COME_F16);
    } else if (wide) {
        if (dtype == COME_BF16) COME_ATTN_LAUNCH(COME_BF16, 8);
        else COME_ATTN_LAUNCH(COME_F16, 8);
    } else {
        if (dtype == COME_BF16) COME_ATTN_LAUNCH(COME_BF16, 4);
        else COME_ATTN_LAUNCH(COME_F16, 4);
    }
#undef COME_ATTN_LAUNCH_ITEMS
#undef COME_ATTN_LAUNCH
    COME_CHECK_LAUNCH("come_attn_varlen_fwd");
    if (plan.splits > 1) {
        static_assert(kHeadDim / 4 == 16, "a workgroup of the combine kernel covers 16 rows of 16 four-element chunks");
        const dim3 cgrid(static_cast<unsigned>(n_cwg));
        if (dtype == COME_BF16) hipLaunchKernelGGL(attn_combine_kernel<COME_BF16>, cgrid, dim3(256), 0, s, a, kBlockM);
        else hipLaunchKernelGGL(attn_combine_kernel<COME_F16>, cgrid, dim3(256), 0, s, a, kBlockM);
        COME_CHECK_LAUNCH("come_attn_varlen_fwd (combine)");
    }
    return COME_OK;
}

extern "C" int come_attn_varlen_fwd_ws(const void *q, const void *k, const void *v, int dtype, int64_t q_row_stride,
                                       int64_t q_head_stride, int64_t k_row_stride, int64_t k_head_stride,
                                       int64_t v_row_stride, int64_t v_head_stride, const int32_t *cu_seqlens,
                                       int64_t n_seq, int64_t total, int64_t n_heads, int64_t head_dim,
                                       const void *perkey_bias, int64_t max_seqlen, float softmax_scale, void *out,
                                       int64_t o_row_stride, int64_t o_head_stride, float *lse, void *work,
                                       int64_t work_bytes, int flags, void *stream) {
    return attn_varlen_fwd_impl(q, k, v, dtype, q_row_stride, q_head_stride, k_row_stride, k_head_stride,
                                v_row_stride, v_head_stride, cu_seqlens, n_seq, total, n_heads, head_dim,
                                perkey_bias, max_seqlen, softmax_scale, out, o_row_stride, o_head_stride, lse,
                                work, work_bytes, false, flags, stream);
}

extern "C" int come_attn_varlen_fwd_qp(const void *q, const void *k, const void *v, int dtype, int64_t q_row_stride,
                                       int64_t q_head_stride, int64_t k_row_stride, int64_t k_head_stride,
                                       int64_t v_row_stride, int64_t v_head_stride, const int32_t *cu_seqlens,
                                       int64_t n_seq, int64_t total, int64_t n_heads, int64_t head_dim,
                                       const void *perkey_bias, int64_t max_seqlen, float softmax_scale, void *out,
                                       int64_t o_row_stride, int64_t o_head_stride, float *lse, void *work,
                                       int64_t work_bytes, const come_q_prologue *prologue, int flags, void *stream) {
    return attn_varlen_fwd_impl(q, k, v, dtype, q_row_stride, q_head_stride, k_row_stride, k_head_stride,
                                v_row_stride, v_head_stride, cu_seqlens, n_seq, total, n_heads, head_dim,
                                perkey_bias, max_seqlen, softmax_scale, out, o_row_stride, o_head_stride, lse,
                                work, work_bytes, false, flags, stream, prologue);
}

extern "C" int come_attn_varlen_fwd(const void *q, const void *k, const void *v, int dtype, int64_t q_row_stride,
                                    int64_t q_head_stride, int64_t k_row_stride, int64_t k_head_stride,
                                    int64_t v_row_stride, int64_t v_head_stride, const int32_t *cu_seqlens,
                                    int64_t n_seq, int64_t total, int64_t n_heads, int64_t head_dim,
                                    const void *perkey_bias, int64_t max_seqlen, float softmax_scale, void *out,
                                    int64_t o_row_stride, int64_t o_head_stride, float *lse, int flags,
                                    void *stream) {
    return attn_varlen_fwd_impl(q, k, v, dtype, q_row_stride, q_head_stride, k_row_stride, k_head_stride,
                                v_row_stride, v_head_stride, cu_seqlens, n_seq, total, n_heads, head_dim,
                                perkey_bias, max_seqlen, softmax_scale, out, o_row_stride, o_head_stride, lse,
                                nullptr, 0, false, flags, stream);
}

// Also takes the address of the current device's copy of the array, so that a caller who asks for the size before
// its first launch (as a capturing caller has to, outside the capture) leaves nothing but kernel launches to the
// entry point itself.  Returns -1 when that fails (come_last_error() says why).
extern "C" int64_t come_attn_static_work_bytes(void) {
    clear_error();
    return static_work_pointer() != nullptr ? kStaticWorkBytes : -1;
}

extern "C" int come_attn_varlen_fwd_static(const void *q, const void *k, const void *v, int dtype,
                                           int64_t q_row_stride, int64_t q_head_stride, int64_t k_row_stride,
                                           int64_t k_head_stride, int64_t v_row_stride, int64_t v_head_stride,
                                           const int32_t *cu_seqlens, int64_t n_seq, int64_t total, int64_t n_heads,
                                           int64_t head_dim, const void *perkey_bias, int64_t max_seqlen,
                                           float softmax_scale, void *out, int64_t o_row_stride,
                                           int64_t o_head_stride, float *lse, int flags, void *stream) {
    return attn_varlen_fwd_impl(q, k, v, dtype, q_row_stride, q_head_stride, k_row_stride, k_head_stride,
                                v_row_stride, v_head_stride, cu_seqlens, n_seq, total, n_heads, head_dim,
                                perkey_bias, max_seqlen, softmax_scale, out, o_row_stride, o_head_stride, lse,
                                nullptr, 0, true, flags, stream);
}
