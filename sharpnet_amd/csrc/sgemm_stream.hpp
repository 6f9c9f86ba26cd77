// fp32 GEMM for products whose time goes into moving operands and results rather than into the k loop:
// strided batches of small matrices with a short K (attention scores Q.K^T with K = head dimension, the
// probabilities-times-values product, their backward counterparts).  For such shapes one MFMA pass over the data
// takes about as long as streaming the data through HBM once, so the kernel is built to keep both busy at once:
//
//   * a workgroup is persistent: it walks through its share of the (matrix, tile, k panel) work items, and while
//     the MFMAs of one panel run out of LDS, the global loads of the next item - the next k panel of the tile or
//     the first panel of the workgroup's next tile - are already in flight into registers;
//   * k is walked in panels of BK = 32 (or 64) through a single LDS stage, with the next panel written to LDS
//     before the finished tile's results go out, so those stores are in flight during the next MFMAs;
//   * three to four workgroups share a compute unit (34 / 26 KB of LDS, <= 168 / 128 registers with BK = 32), so
//     one workgroup's loads and write-out overlap another's MFMAs;
//   * a wavefront owns 32 rows x all BN columns of the workgroup's 128 x BN tile (TM = 1, TN = BN / 32 tiles
//     interleaved by element), so a lane owns TN consecutive columns and C goes out in 16-byte (TN = 4) or
//     8-byte (TN = 2) pieces, a whole 512- or 256-byte row segment per store instruction and half wavefront.
//
// Same contract, operand layout, staging code and write-out as sgemm_mfma_kernel (all four transposes, ragged
// M / N / K in-kernel, alpha / beta / bias, beta == 0 never reads C); no split-K, single-level batch.
// Work items are assigned so that each XCD gets one contiguous range of the (matrix, tile) order: the tiles of a
// matrix share its operand panels in one L2.
#pragma once
#include "bgemm_mfma.hpp"
#include "sgemm_mfma.hpp"

namespace snhip {

// workgroups per compute unit the register budget is set for
constexpr int stream_occupancy(int tn, int bk) { return bk == 64 ? 2 : (tn == 2 ? 4 : 3); }

template <int TN_, int BK_ = 64>
struct StreamCfg {
    static constexpr int TN = TN_;
    static constexpr int BM = 128, BN = 32 * TN, BK = BK_, NT = 256;
    static constexpr int PA = BM + 4, PB = BN + 4;
    static constexpr int LDS_BYTES = BK * (PA + PB) * 4;
};

// TWO_LEVEL: entry z of the batch is matrix z % batch_inner of outer step z / batch_inner (heads addressed in place);
// a variant of its own because the extra address arithmetic does not fit the register budget of the single-level
// kernel's occupancy (it runs with one workgroup fewer per compute unit).
template <int TN, bool TA, bool TB, int BK_ = 64, bool TWO_LEVEL = false>
__global__ void __launch_bounds__(256, stream_occupancy(TN, BK_) - (TWO_LEVEL ? 1 : 0)) sgemm_stream_kernel(const GemmParams p) {
    using CFG = StreamCfg<TN, BK_>;
    constexpr int BM = CFG::BM, BN = CFG::BN, BK = CFG::BK, NT = CFG::NT, PA = CFG::PA, PB = CFG::PB;
    using StageA = TileStage<BM, BK, NT, PA, !TA, true>;
    using StageB = TileStage<BN, BK, NT, PB, TB, true>;

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const As = smem;            // [BK][PA]
    float* const Bs = smem + BK * PA;  // [BK][PB]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;

    // This workgroup's tiles: XCD x (= linear id % 8) owns the logical range [start, start + cnt); its workgroups
    // take every nwg-th tile of it, so the tiles in flight on an XCD at any time are neighbours.
    constexpr unsigned NXCD = 8;
    const unsigned ntiles = (unsigned)(p.tiles_m * p.tiles_n);
    const unsigned total = ntiles * (unsigned)p.nz;
    const unsigned xcd = blockIdx.x % NXCD, slot = blockIdx.x / NXCD;
    const unsigned nwg = (gridDim.x - xcd + NXCD - 1) / NXCD;  // workgroups on this XCD
    const unsigned q = total / NXCD, r = total % NXCD;
    const unsigned start = xcd * q + (xcd < r ? xcd : r), cnt = q + (xcd < r ? 1u : 0u);
    if (slot >= cnt) return;  // uniform over the workgroup
    const int nkp = (p.K + BK - 1) / BK;

    struct Tile {
        int z, m0, n0;
    };
    auto tile_at = [&](unsigned idx) {
        const unsigned L = start + idx;
        Tile t;
        t.z = (int)(L / ntiles);
        const int logical = (int)(L - (unsigned)t.z * ntiles);
        // tile rows fastest inside a matrix: neighbours share the B panel (the small matrices this kernel is for
        // have one to four tiles each)
        t.m0 = (logical % p.tiles_m) * BM;
        t.n0 = (logical / p.tiles_m) * BN;
        return t;
    };

    StageA sa;
    StageB sb;
    f32x4 ra[StageA::NV], rb[StageB::NV];
    auto fetch = [&](const Tile& t, int kp) {
        if constexpr (TWO_LEVEL) {
            const BatchIndex bz = split_batch(t.z, p.batch_inner);
            sa.init(p.A + batch_offset(bz, p.strideA, p.strideA2), p.lda, t.m0, kp * BK, tid);
            sb.init(p.B + batch_offset(bz, p.strideB, p.strideB2), p.ldb, t.n0, kp * BK, tid);
        } else {
            sa.init(p.A + (long long)t.z * p.strideA, p.lda, t.m0, kp * BK, tid);
            sb.init(p.B + (long long)t.z * p.strideB, p.ldb, t.n0, kp * BK, tid);
        }
        const int m_rem = p.M - t.m0, n_rem = p.N - t.n0, k_rem = p.K - kp * BK;
        if (m_rem >= BM && n_rem >= BN && k_rem >= BK) {
            sa.load_fast(ra);
            sb.load_fast(rb);
        } else {
            sa.load_safe(ra, m_rem, k_rem);
            sb.load_safe(rb, n_rem, k_rem);
        }
    };

    f32x16 acc[1][TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[0][j][e] = 0.0f;

    const float* const a_rd = As + lhi * PA + wave * 32 + l32;
    const float* const b_rd = Bs + lhi * PB + l32 * TN;

    unsigned idx = slot;
    int kp = 0;
    Tile cur = tile_at(idx);
    fetch(cur, kp);
    sa.store_lds(As, ra);
    sb.store_lds(Bs, rb);
    lds_barrier();
    for (;;) {
        // the next work item's operands start their way from memory now and land during the MFMAs below
        const bool last_panel = (kp + 1 == nkp);
        const unsigned idx_next = last_panel ? idx + nwg : idx;
        const int kp_next = last_panel ? 0 : kp + 1;
        const bool has_next = idx_next < cnt;
        Tile nxt = cur;
        if (has_next) {
            if (last_panel) nxt = tile_at(idx_next);
            fetch(nxt, kp_next);
        }

        Frag<1> fa[2];
        Frag<TN> fb[2];
        fa[0].load(a_rd);
        fb[0].load(b_rd);
#pragma unroll
        for (int s = 0; s < BK / 2; ++s) {
            if (s + 1 < BK / 2) {
                fa[(s + 1) & 1].load(a_rd + (2 * (s + 1)) * PA);
                fb[(s + 1) & 1].load(b_rd + (2 * (s + 1)) * PB);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s & 1].v[0], fb[s & 1].v[j], acc[0][j], 0, 0, 0);
        }

        // The next panel goes into LDS before this tile's results go out: the stores of the write-out are then in
        // flight during the next panel's MFMAs, and nothing waits for them until the panel after that is staged.
        lds_barrier();  // every wavefront has finished reading the current panel
        if (has_next) {
            sa.store_lds(As, ra);
            sb.store_lds(Bs, rb);
        }
        if (last_panel) {
            if constexpr (TWO_LEVEL)
                store_accumulators_plain<1, TN, false, true>(acc, p, cur.m0 + wave * 32, cur.n0 + TN * l32, lhi, cur.z, cur.z, 0,
                                                batch_offset(split_batch(cur.z, p.batch_inner), p.strideC, p.strideC2));
            else
                store_accumulators_plain<1, TN, false, true>(acc, p, cur.m0 + wave * 32, cur.n0 + TN * l32, lhi, cur.z, cur.z, 0);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[0][j][e] = 0.0f;
        }
        if (!has_next) break;
        lds_barrier();
        cur = nxt;
        idx = idx_next;
        kp = kp_next;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same persistent streaming scheme with bf16-input / fp32-accumulate arithmetic (v_mfma_f32_32x32x16_bf16,
// staging and LDS layout of bgemm_mfma.hpp: tiles kept [row][k] in bf16, rows of the TN column tiles stored
// tile-major).  TIN = float: operands are fp32 in memory and rounded on their way into LDS; TIN = __bf16: they are
// stored as bf16.  With eight times the MFMA rate of the fp32 kernel these products are plain streaming: the k
// panel is 64 wide (one panel for an attention head of 64; 128 for the 64-column tile), one LDS stage, the next work
// item's loads in flight during the MFMAs and the write-out of the current one.
// ---------------------------------------------------------------------------------------------------------------
template <int TN_>
struct BStreamCfg {
    static constexpr int TN = TN_;
    // the 64-column tile takes k panels of 128 (its operands then split evenly over the threads in every layout)
    static constexpr int BM = 128, BN = 32 * TN, BK = (TN_ == 2) ? 128 : 64, NT = 256;
    static constexpr int PITCH = BK + 8;  // bf16 elements
    static constexpr int LDS_BYTES = (BM + BN) * PITCH * 2;
};

// workgroups per compute unit the register budget is set for: fp32 storage keeps twice the bytes in flight
constexpr int bstream_occupancy(int bytes_per_element) { return bytes_per_element == 4 ? 2 : 3; }

template <int TN, bool TA, bool TB, typename TIN, bool TWO_LEVEL = false>
__global__ void __launch_bounds__(256, bstream_occupancy(sizeof(TIN)) - (TWO_LEVEL ? 1 : 0)) bgemm_stream_kernel(const GemmParams p) {
    using CFG = BStreamCfg<TN>;
    constexpr int BM = CFG::BM, BN = CFG::BN, BK = CFG::BK, NT = CFG::NT, PITCH = CFG::PITCH;
    using StageA = BStage<BM, BK, NT, PITCH, 1, !TA, TIN>;
    using StageB = BStage<BN, BK, NT, PITCH, TN, TB, TIN>;

    extern __shared__ __attribute__((aligned(16))) float smem_f[];
    __bf16* const As = reinterpret_cast<__bf16*>(smem_f);  // [BM][PITCH]
    __bf16* const Bs = As + BM * PITCH;                    // [BN][PITCH]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;

    constexpr unsigned NXCD = 8;
    const unsigned ntiles = (unsigned)(p.tiles_m * p.tiles_n);
    const unsigned total = ntiles * (unsigned)p.nz;
    const unsigned xcd = blockIdx.x % NXCD, slot = blockIdx.x / NXCD;
    const unsigned nwg = (gridDim.x - xcd + NXCD - 1) / NXCD;
    const unsigned q = total / NXCD, r = total % NXCD;
    const unsigned start = xcd * q + (xcd < r ? xcd : r), cnt = q + (xcd < r ? 1u : 0u);
    if (slot >= cnt) return;  // uniform over the workgroup
    const int nkp = (p.K + BK - 1) / BK;

    struct Tile {
        int z, m0, n0;
    };
    auto tile_at = [&](unsigned idx) {
        const unsigned L = start + idx;
        Tile t;
        t.z = (int)(L / ntiles);
        const int logical = (int)(L - (unsigned)t.z * ntiles);
        t.m0 = (logical % p.tiles_m) * BM;
        t.n0 = (logical / p.tiles_m) * BN;
        return t;
    };

    StageA sa;
    StageB sb;
    f32x4 ra[StageA::NV], rb[StageB::NV];
    auto fetch = [&](const Tile& t, int kp) {
        if constexpr (TWO_LEVEL) {
            const BatchIndex bz = split_batch(t.z, p.batch_inner);
            sa.init(reinterpret_cast<const TIN*>(p.A) + batch_offset(bz, p.strideA, p.strideA2), p.lda, t.m0, kp * BK, tid);
            sb.init(reinterpret_cast<const TIN*>(p.B) + batch_offset(bz, p.strideB, p.strideB2), p.ldb, t.n0, kp * BK, tid);
        } else {
            sa.init(reinterpret_cast<const TIN*>(p.A) + (long long)t.z * p.strideA, p.lda, t.m0, kp * BK, tid);
            sb.init(reinterpret_cast<const TIN*>(p.B) + (long long)t.z * p.strideB, p.ldb, t.n0, kp * BK, tid);
        }
        const int m_rem = p.M - t.m0, n_rem = p.N - t.n0, k_rem = p.K - kp * BK;
        if (m_rem >= BM && n_rem >= BN && k_rem >= BK) {
            sa.load_fast(ra);
            sb.load_fast(rb);
        } else {
            sa.load_safe(ra, m_rem, k_rem);
            sb.load_safe(rb, n_rem, k_rem);
        }
    };

    f32x16 acc[1][TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[0][j][e] = 0.0f;

    // physical row of this lane: the wavefront's 32 rows of A; in tile j of B row 32 j + l32
    const __bf16* const a_rd = As + (wave * 32 + l32) * PITCH + 8 * lhi;
    const __bf16* const b_rd = Bs + l32 * PITCH + 8 * lhi;

    unsigned idx = slot;
    int kp = 0;
    Tile cur = tile_at(idx);
    fetch(cur, kp);
    sa.store_lds(As, ra);
    sb.store_lds(Bs, rb);
    lds_barrier();
    for (;;) {
        const bool last_panel = (kp + 1 == nkp);
        const unsigned idx_next = last_panel ? idx + nwg : idx;
        const int kp_next = last_panel ? 0 : kp + 1;
        const bool has_next = idx_next < cnt;
        Tile nxt = cur;
        if (has_next) {
            if (last_panel) nxt = tile_at(idx_next);
            fetch(nxt, kp_next);
        }

#pragma unroll
        for (int s = 0; s < BK / 16; ++s) {
            const bf16x8 fa = *reinterpret_cast<const bf16x8*>(a_rd + 16 * s);
            bf16x8 fb[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const bf16x8*>(b_rd + (32 * j) * PITCH + 16 * s);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb[j], acc[0][j], 0, 0, 0);
        }

        lds_barrier();  // every wavefront has finished reading the current panel
        if (has_next) {
            sa.store_lds(As, ra);
            sb.store_lds(Bs, rb);
        }
        if (last_panel) {
            if constexpr (TWO_LEVEL)
                store_accumulators_plain<1, TN, false, true>(acc, p, cur.m0 + wave * 32, cur.n0 + TN * l32, lhi, cur.z, cur.z, 0,
                                                batch_offset(split_batch(cur.z, p.batch_inner), p.strideC, p.strideC2));
            else
                store_accumulators_plain<1, TN, false, true>(acc, p, cur.m0 + wave * 32, cur.n0 + TN * l32, lhi, cur.z, cur.z, 0);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[0][j][e] = 0.0f;
        }
        if (!has_next) break;
        lds_barrier();
        cur = nxt;
        idx = idx_next;
        kp = kp_next;
    }
}

}  // namespace snhip
