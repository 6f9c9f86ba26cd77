// bf16-storage GEMM for gfx950 fed by global -> LDS direct loads:
//     C[M x N] = alpha * op(A) . op(B) + beta * C + bias,   A and B stored as bf16, fp32 accumulation, fp32 C.
// Same contract as bgemm_mfma_kernel<..., __bf16> for the shapes it takes: M and N multiples of 256, K a multiple
// of 32, rows and matrices on 16-byte boundaries.  All four transpose combinations (template arguments TA, TB).
//
// What is different from bgemm_mfma.hpp is how a tile reaches LDS: global_load_lds_dwordx4 (16 bytes per lane,
// written to LDS at base + 16 * lane without passing through registers).  No staging registers, no ds_write
// instructions, and the loads of a tile can be dealt out one at a time between the MFMAs of the tile before.  That
// last point is what the schedule is built around: a vector-memory instruction holds its wavefront until the address
// unit has taken all 64 lanes, and the address unit takes one such instruction per ~18 cycles for the whole compute
// unit, so eight loads issued back to back by each of four wavefronts stall every one of them for ~600 cycles per
// tile (measured), with the matrix pipes idle; one load behind every fourth MFMA costs nothing.
//
// Tile 256 x 256 x 32, four wavefronts of 128 x 128 (4 x 4 MFMA tiles of 32 x 32 x 16: the fewest LDS bytes per flop
// a wavefront can have), four LDS stages of 32 KB.  Tile t is multiplied while tile t + 1 is resident, tile t + 2 is
// landing and tile t + 3 is being requested; one workgroup barrier per tile, placed so that the fragments of the
// next tile's first k step are already in registers when it is reached (the matrix pipes run through it).
//
// A direct load writes 1024 contiguous bytes per wavefront, so the LDS image of an operand tile is the memory image
// up to a permutation of 16-byte chunks that is applied on the global side (each lane fetches the chunk that belongs
// at its LDS position).  Two images:
//  * operand contiguous along k (A not transposed, B transposed): 256 rows of 64 bytes (32 k).  Chunk c of physical
//    row r sits at chunk position c ^ ((r >> 1) & 3); a fragment is one ds_read_b128 (8 k of one row) and the 16 lanes
//    served per cycle touch 16 distinct 16-byte slots.  Physical row 32 t + i of a wavefront's 128 rows holds logical
//    row 4 i + t (the rows of the four MFMA tiles interleaved as in the other kernels), so that a lane owns four
//    consecutive rows / columns of C.
//  * operand contiguous along m / n (A transposed, B not transposed): 32 k rows of 512 bytes (256 m).  The MFMA wants
//    8 consecutive k of one m per lane; ds_read_b64_tr_b16 delivers that from this image: in a group of 16 lanes,
//    lane 4 s + q supplies the address of k row k0 + s, columns m0 + 4 q .. + 3, and lane i receives the four k
//    values k0 .. k0 + 3 of column m0 + i.  Two such reads make one fragment.  Chunk c of k row r sits at chunk
//    position c ^ (4 (r & 3)): the 32 lanes of two groups then read 16 distinct chunks of the 512-byte row set.
//    Columns cannot be interleaved here (a 16-byte chunk is 8 consecutive m in memory), so MFMA tile t of a wavefront
//    covers columns 32 t .. 32 t + 31 and the write-out addresses C accordingly.
#pragma once
#include "bgemm_mfma.hpp"

namespace snhip {

struct BDtlCfg {
    static constexpr int BM = 256, BN = 256, BK = 32, NT = 256, TM = 4, TN = 4, WN = 2;
    static constexpr int STAGES = 4;
    static constexpr int OPND_BYTES = 256 * BK * 2, STAGE_BYTES = 2 * OPND_BYTES;
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int ROUNDS = OPND_BYTES / (4 * 1024);  // direct loads per thread, operand and tile
    static constexpr int L = 2 * ROUNDS;                    // loads per thread and tile
    static constexpr int KSTEPS = BK / 16;
};

typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

// s_waitcnt vmcnt(n) with the other counters left alone (vmcnt is split over bits 3:0 and 15:14 on gfx9)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

// One operand tile (256 rows or columns of C x 32 k) of bgemm_dtl_kernel.  KMAJOR: the operand is stored with m / n
// contiguous (k rows of 256 elements), else with k contiguous (256 rows of 32 k).
template <bool KMAJOR>
struct BDtlOperand {
    // global element offset (from the tile's origin at k = 0) and nothing else: where the 16 bytes that belong at LDS
    // position `pos` (in 16-byte chunks) of the tile image come from
    __device__ __forceinline__ static long long source_offset(int pos, long long ld) {
        if constexpr (KMAJOR) {
            const int row = pos >> 5, pc = pos & 31;  // k row, physical chunk
            const int lc = pc ^ (4 * (row & 3));
            return (long long)row * ld + 8 * lc;
        } else {
            const int pr = pos >> 2, pc = pos & 3;  // physical row, physical chunk
            const int lc = pc ^ ((pr >> 1) & 3);
            return (long long)logical_row<4>(pr) * ld + 8 * lc;
        }
    }
    // elements between consecutive k tiles
    __device__ __forceinline__ static long long tile_step(long long ld) { return KMAJOR ? 32 * ld : 32; }

    // byte offsets (inside the tile image) of the LDS reads that make fragment (MFMA tile `t` of the wavefront whose
    // block of 128 starts at `w128`, k step s): one 16-byte read, or two transposing 8-byte reads
    struct FragAddr {
        int off[KMAJOR ? 2 : 1];
    };
    __device__ __forceinline__ static FragAddr frag_addr(int w128, int t, int s, int lane) {
        FragAddr f;
        if constexpr (KMAJOR) {
            const int g = lane >> 4, j = lane & 15, sj = j >> 2, q = j & 3;
            const int m_base = w128 + 32 * t + 16 * (g & 1);
            const int c8 = (m_base >> 2) + q;  // 8-byte chunk (4 columns) this lane addresses
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int row = 16 * s + 8 * (g >> 1) + 4 * h + sj;
                f.off[h] = row * 512 + (((c8 >> 1) ^ (4 * (row & 3))) << 4) + ((c8 & 1) << 3);
            }
        } else {
            const int l32 = lane & 31, lhi = lane >> 5;
            const int row = w128 + 32 * t + l32;
            f.off[0] = row * 64 + (((2 * s + lhi) ^ ((row >> 1) & 3)) << 4);
        }
        return f;
    }
    __device__ __forceinline__ static bf16x8 read_frag(const char* tile, const FragAddr& f) {
        if constexpr (KMAJOR) {
            typedef __attribute__((address_space(3))) bf16x4_t* lds_ptr;
            const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)(tile + f.off[0]));
            const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr)(tile + f.off[1]));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
            return *reinterpret_cast<const bf16x8*>(tile + f.off[0]);
        }
    }
};

// Write-out for accumulators whose rows and / or columns are not interleaved over the MFMA tiles (an operand stored
// with m / n contiguous).  acc[i][j][r]: MFMA tile (i, j), row 8 (r / 4) + 4 lhi + r % 4 and column l32 inside it.
//   ROW_IL: tile-row index q of MFMA tile i is C row 4 q + i of the wavefront's 128, else row 32 i + q;
//   COL_IL: column l32 of MFMA tile j is C column 4 l32 + j (a lane owns four consecutive columns), else 32 j + l32.
// Whole tiles only (the kernel takes no ragged shapes).  C = alpha * acc + beta * C + bias.
template <bool ROW_IL, bool COL_IL>
__device__ __forceinline__ void bdtl_store(const f32x16 (&acc)[4][4], const GemmParams& p, float* Cb, int row_base,
                                           int col_base, int l32, int lhi) {
    const float alpha = p.alpha, beta = p.beta;
    const bool vec = COL_IL && (p.flags & GEMM_FLAG_C_VEC);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int q = 8 * (r / 4) + 4 * lhi + (r % 4);
            const int row = row_base + (ROW_IL ? 4 * q + i : 32 * i + q);
            float* crow = Cb + (long long)row * p.ldc;
            if (vec) {
                const int col = col_base + 4 * l32;
                f32x4 v = {acc_value<true>(acc[i][0][r]), acc_value<true>(acc[i][1][r]), acc_value<true>(acc[i][2][r]),
                           acc_value<true>(acc[i][3][r])};
                v *= alpha;
                if (p.ep.bias != nullptr) v += *reinterpret_cast<const f32x4*>(p.ep.bias + col);
                if (beta != 0.0f) v += beta * *reinterpret_cast<const f32x4*>(crow + col);
                *reinterpret_cast<f32x4*>(crow + col) = v;
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int col = col_base + (COL_IL ? 4 * l32 + j : 32 * j + l32);
                    float v = alpha * acc_value<true>(acc[i][j][r]);
                    if (p.ep.bias != nullptr) v += p.ep.bias[col];
                    if (beta != 0.0f) v += beta * crow[col];
                    crow[col] = v;
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // one MFMA-tile row of results at a time (see store_patch_fast)
    }
}

template <bool TA, bool TB>
__global__ void __launch_bounds__(BDtlCfg::NT) bgemm_dtl_kernel(const GemmParams p) {
    using C = BDtlCfg;
    constexpr int TM = C::TM, TN = C::TN, WN = C::WN, BK = C::BK, S = C::STAGES, L = C::L, KSTEPS = C::KSTEPS;
    using OpA = BDtlOperand<TA>;    // A transposed: stored K x M, m contiguous
    using OpB = BDtlOperand<!TB>;   // B not transposed: stored K x N, n contiguous
    extern __shared__ __attribute__((aligned(1024))) char smem_dtl[];
    char* const smem = smem_dtl;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS bases of the direct loads are scalars
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, lhi = lane >> 5;

    const WorkCoords wc = work_coords(blockIdx.x, p.tiles_m, p.tiles_n, p.nz, p.group_m);
    const int m0 = wc.tile_m * C::BM, n0 = wc.tile_n * C::BN;
    const int batch = wc.zb;  // no split-K in this kernel
    const __bf16* Ab = reinterpret_cast<const __bf16*>(p.A) + (long long)batch * p.strideA;
    const __bf16* Bb = reinterpret_cast<const __bf16*>(p.B) + (long long)batch * p.strideB;
    const int KT = p.K / BK;

    // this lane's 16 bytes of load j: LDS position (j * 4 + wave) * 64 + lane of the operand's tile image
    const __bf16* gsrc[2][C::ROUNDS];
#pragma unroll
    for (int j = 0; j < C::ROUNDS; ++j) {
        const int pos = (j * 4 + wave) * 64 + lane;
        gsrc[0][j] = Ab + (TA ? (long long)m0 : (long long)m0 * p.lda) + OpA::source_offset(pos, p.lda);
        gsrc[1][j] = Bb + (TB ? (long long)n0 * p.ldb : (long long)n0) + OpB::source_offset(pos, p.ldb);
    }
    const long long step_a = OpA::tile_step(p.lda), step_b = OpB::tile_step(p.ldb);
    // load x (0 .. L-1: operand A first, then B) of tile t.  Past the last tile the last one is requested again into
    // a stage nobody reads any more: the wait counts below stay the same in every pass of the loop.
    auto issue_one = [&](int t, int x) {
        const int st = t % S;
        const int tt = t < KT ? t : KT - 1;
        const int o = x / C::ROUNDS, j = x % C::ROUNDS;
        char* dst = smem + st * C::STAGE_BYTES + o * C::OPND_BYTES + (j * 4 + wave) * 1024;
        __builtin_amdgcn_global_load_lds(gsrc[o][j] + (long long)tt * (o == 0 ? step_a : step_b),
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    typename OpA::FragAddr a_off[TM][KSTEPS];
    typename OpB::FragAddr b_off[TN][KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
        for (int i = 0; i < TM; ++i) a_off[i][s] = OpA::frag_addr(wm * 128, i, s, lane);
#pragma unroll
        for (int j = 0; j < TN; ++j) b_off[j][s] = OpB::frag_addr(wn * 128, j, s, lane);
    }

#pragma unroll
    for (int t = 0; t < S - 1; ++t)
#pragma unroll
        for (int x = 0; x < L; ++x) issue_one(t, x);

    bf16x8 fa[2][TM], fb[2][TN];
    wait_vmcnt<(S - 2) * L>();     // tile 0 has landed (this wavefront's part) ...
    __builtin_amdgcn_s_barrier();  // ... and everybody else's
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[0][i] = OpA::read_frag(smem, a_off[i][0]);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[0][j] = OpB::read_frag(smem + C::OPND_BYTES, b_off[j][0]);

    constexpr int LP = L / KSTEPS, MT = TM * TN;
    static_assert(L % KSTEPS == 0 && KSTEPS % 2 == 0, "loads split evenly over an even number of k steps");
    for (int t = 0; t < KT; ++t) {
        // Tile t + 1 has landed - this wavefront's loads, then, behind the barrier, everyone's - and every wavefront is
        // done reading the stage of tile t - 1, which the loads issued in this pass (tile t + 3) overwrite.
        wait_vmcnt<(S - 3) * L>();
        __builtin_amdgcn_s_barrier();
        const char* base = smem + (t % S) * C::STAGE_BYTES;
        const char* next = smem + ((t + 1) % S) * C::STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const int cur = s & 1;  // KSTEPS is even: k step s of every tile uses fragment buffer s & 1
            const char* fbase = (s + 1 < KSTEPS) ? base : next;
            const int sn = (s + 1 < KSTEPS) ? s + 1 : 0;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int m = i * TN + j;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
                    // behind each of the first eight MFMAs one fragment of the next k step; behind every fourth MFMA
                    // one direct load of tile t + 3; the fences pin that order
                    __builtin_amdgcn_sched_barrier(0);
                    if (m < TM)
                        fa[cur ^ 1][m] = OpA::read_frag(fbase, a_off[m][sn]);
                    else if (m < TM + TN)
                        fb[cur ^ 1][m - TM] = OpB::read_frag(fbase + C::OPND_BYTES, b_off[m - TM][sn]);
#pragma unroll
                    for (int x = 0; x < LP; ++x)
                        if (m == (x * MT) / LP + 1) issue_one(t + S - 1, s * LP + x);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    }
    wait_vmcnt<0>();  // the trailing reloads must have landed before this workgroup's LDS is handed on

    if constexpr (!TA && TB) {
        // both operands k-contiguous: rows and columns interleaved, the write-out of the other kernels
        store_accumulators_plain<TM, TN, true>(acc, p, m0 + wm * (TM * 32), n0 + wn * (TN * 32) + TN * l32, lhi, batch,
                                               batch, wc.tile_m * p.tiles_n + wc.tile_n);
    } else {
        bdtl_store<!TA, TB>(acc, p, p.C + (long long)batch * p.strideC, m0 + wm * 128, n0 + wn * 128, l32, lhi);
    }
}

}  // namespace snhip
