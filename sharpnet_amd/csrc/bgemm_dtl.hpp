// bf16-storage GEMM in the "NT" form for gfx950: C[M x N] = alpha * A[M x K] . B[N x K]^T + beta * C + bias, both
// operands stored as bf16 with k contiguous (A not transposed, B transposed: the form the bf16-stored products are
// meant to be brought into), fp32 accumulation and fp32 C.  Same contract as bgemm_mfma_kernel<..., __bf16> for the
// shapes it takes: M and N multiples of 256, K a multiple of 32, rows 16-byte aligned.
//
// What is different from bgemm_mfma.hpp is how a tile reaches LDS: global -> LDS direct loads
// (global_load_lds_dwordx4: 16 bytes per lane, written to LDS at base + 16 * lane without passing through registers).
// No staging registers, no ds_write instructions, and the loads of a tile can be dealt out one at a time between the
// MFMAs of the tile before.  That last point is what the layout is built around: a vector-memory instruction holds
// its wavefront until the address unit has taken all 64 lanes, and the address unit takes one such instruction per
// ~18 cycles for the whole compute unit, so eight loads issued back to back by each of four wavefronts stall every
// one of them for ~600 cycles per tile (measured), with the matrix pipes idle; one load behind every fourth MFMA
// costs nothing.
//
// Tile 256 x 256 x 32, four wavefronts of 128 x 128 (4 x 4 MFMA tiles of 32 x 32 x 16: the fewest LDS bytes per
// flop a wavefront can have), four LDS stages of 32 KB.  Tile t is multiplied while tile t + 1 is resident, tile
// t + 2 is landing and tile t + 3 is being requested; one workgroup barrier per tile, placed so that the fragments of
// the next tile's first k step are already in registers when it is reached (the matrix pipes run through it).
//
// LDS image of an operand tile: 256 rows of 64 bytes (32 k), 16-byte chunk c of physical row r stored at chunk
// position c ^ ((r >> 1) & 3): the 16 lanes a ds_read_b128 serves per cycle then touch 16 distinct 16-byte slots of
// the 256 bytes the 64 banks hold.  A direct load writes 1024 contiguous bytes per wavefront (16 physical rows), so
// the swizzle and the row order are applied on the global side: lane l of the instruction that fills LDS position
// pos = 64 * n + l fetches chunk (pos % 4) ^ swizzle of logical row logical_row<4>(pos / 4).  Logical rows are
// interleaved over the four MFMA tiles of a wavefront as in the other kernels (lane i of tile t <-> row 4 i + t), so
// the write-out is the shared one (a lane owns four consecutive columns of C: 16-byte stores).
#pragma once
#include "bgemm_mfma.hpp"

namespace snhip {

// T: MFMA tiles per wavefront along each dimension.  T = 4: the 256 x 256 tile described above; T = 2: 128 x 128 (64 x 64
// per wavefront, 16 KB stages), for products with too few 256 x 256 tiles to fill the chip.
template <int T>
struct BDtlCfgT {
    static constexpr int TM = T, TN = T, WN = 2, NT = 256;
    static constexpr int ROWS = 64 * T;  // rows of an operand tile
    static constexpr int BM = ROWS, BN = ROWS, BK = 32;
    static constexpr int STAGES = 4;
    static constexpr int ROW_BYTES = BK * 2, CPR = ROW_BYTES / 16;  // chunks of 16 bytes per row
    static constexpr int OPND_BYTES = ROWS * ROW_BYTES, STAGE_BYTES = 2 * OPND_BYTES;
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int ROWS_PER_INST = 1024 / ROW_BYTES;       // physical rows one wavefront instruction fills
    static constexpr int ROUNDS = ROWS / (4 * ROWS_PER_INST);    // instructions per thread, operand and tile
    static constexpr int L = 2 * ROUNDS;                         // loads per thread and tile
    static constexpr int KSTEPS = BK / 16;
    static_assert(TM * TN >= TM + TN, "one fragment read per MFMA slot of a k step");
};
using BDtlCfg = BDtlCfgT<4>;

__device__ __forceinline__ int bdtl_swizzle(int phys_row) { return (phys_row >> 1) & (BDtlCfg::CPR - 1); }

// s_waitcnt vmcnt(n) with the other counters left alone (vmcnt is split over bits 3:0 and 15:14 on gfx9)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt has six bits");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

// 16 bytes per lane from global memory to LDS at dst + 16 * lane.  (A function of its own: with the builtin inside a lambda
// of the kernel template the host pass drops the instantiation without a word, and the library then lacks the kernel's stub.)
__device__ __forceinline__ void bdtl_load16(const __bf16* src, char* dst) {
    __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
}

template <int T>
__global__ void __launch_bounds__(256) bgemm_nt_dtl_kernel(const GemmParams p) {
    static_assert(BDtlCfgT<T>::NT == 256, "launch bounds");
    using C = BDtlCfgT<T>;
    constexpr int TM = C::TM, TN = C::TN, WN = C::WN, BK = C::BK, S = C::STAGES, L = C::L, KSTEPS = C::KSTEPS;
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

    // this lane's 16 bytes of load j: LDS position (j * 4 + wave) * 64 + lane of the operand tile
    const __bf16* gsrc[2][C::ROUNDS];
#pragma unroll
    for (int j = 0; j < C::ROUNDS; ++j) {
        const int pos = (j * 4 + wave) * 64 + lane;
        const int pr = pos / C::CPR, pc = pos % C::CPR;
        const int lc = pc ^ bdtl_swizzle(pr);
        gsrc[0][j] = Ab + (long long)(m0 + logical_row<TM>(pr)) * p.lda + 8 * lc;
        gsrc[1][j] = Bb + (long long)(n0 + logical_row<TN>(pr)) * p.ldb + 8 * lc;
    }
    // load x (0 .. L-1: operand A first, then B) of tile t.  Past the last tile the last one is requested again into
    // a stage nobody reads any more: the wait counts below stay the same in every pass of the loop.
    auto issue_one = [&](int t, int x) {
        const int st = t % S;
        const int tt = t < KT ? t : KT - 1;
        const int o = x / C::ROUNDS, j = x % C::ROUNDS;
        char* dst = smem + st * C::STAGE_BYTES + o * C::OPND_BYTES + (j * 4 + wave) * 1024;
        bdtl_load16(gsrc[o][j] + (long long)tt * BK, dst);
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // fragment addresses inside a stage: MFMA tile i of this wavefront, lane l32 <-> physical row block + 32 i + l32,
    // k step s <-> chunks 2 s (lanes 0-31) and 2 s + 1 (lanes 32-63)
    int a_off[TM][KSTEPS], b_off[TN][KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row = wm * (32 * TM) + 32 * i + l32;
            a_off[i][s] = row * C::ROW_BYTES + (((2 * s + lhi) ^ bdtl_swizzle(row)) << 4);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int row = wn * (32 * TN) + 32 * j + l32;
            b_off[j][s] = C::OPND_BYTES + row * C::ROW_BYTES + (((2 * s + lhi) ^ bdtl_swizzle(row)) << 4);
        }
    }

#pragma unroll
    for (int t = 0; t < S - 1; ++t)
#pragma unroll
        for (int x = 0; x < L; ++x) issue_one(t, x);

    bf16x8 fa[2][TM], fb[2][TN];
    wait_vmcnt<(S - 2) * L>();  // tile 0 has landed (this wavefront's part) ...
    __builtin_amdgcn_s_barrier();  // ... and everybody else's
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[0][i] = *reinterpret_cast<const bf16x8*>(smem + a_off[i][0]);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[0][j] = *reinterpret_cast<const bf16x8*>(smem + b_off[j][0]);

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
                    // behind each of the first eight MFMAs one fragment read of the next k step; behind every fourth
                    // MFMA one direct load of tile t + 3; the fences pin that order
                    __builtin_amdgcn_sched_barrier(0);
                    if (m < TM)
                        fa[cur ^ 1][m] = *reinterpret_cast<const bf16x8*>(fbase + a_off[m][sn]);
                    else if (m < TM + TN)
                        fb[cur ^ 1][m - TM] = *reinterpret_cast<const bf16x8*>(fbase + b_off[m - TM][sn]);
#pragma unroll
                    for (int x = 0; x < LP; ++x)
                        if (m == (x * MT) / LP + 1) issue_one(t + S - 1, s * LP + x);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    }
    wait_vmcnt<0>();  // the trailing reloads must have landed before this workgroup's LDS is handed on

    store_accumulators_plain<TM, TN>(acc, p, m0 + wm * (TM * 32), n0 + wn * (TN * 32) + TN * l32, lhi, batch, batch,
                                           wc.tile_m * p.tiles_n + wc.tile_n);
}

}  // namespace snhip
