// fp32 GEMM for products with few output tiles and a K of up to about a thousand (a Dense layer on a small batch:
// 128 x 256 x 784, 256 x 784 x 128; 512 x 512 x 512).  The tiled kernels of sgemm_mfma.hpp give
// such a product a handful of workgroups, each walking a long k loop behind LDS barriers: 8-16 us for 3 us of
// MFMA work, or a split-K launch plus a reduction launch.  Here a workgroup owns a 32 x 32 tile of C and splits K
// over its four wavefronts instead; a wavefront works alone - whole-line global loads of its 32 x 32 operand
// pieces, several groups of 32 k values in flight in registers, a private LDS patch to bring a group into MFMA
// operand layout, v_mfma_f32_32x32x2_f32 on four independent accumulators - and the four partial tiles meet in
// LDS once, where alpha, beta, the bias, the addend and the (leaky) ReLU are applied.  One launch, no workspace,
// deterministic.
//
// Operands: op(A) is M x K, op(B) is K x N, row-major storage with row pitch lda / ldb.  An operand whose storage
// is contiguous along k (A not transposed, B transposed) is fetched 16 bytes per lane along k; one that is
// contiguous along its rows (A transposed, B not transposed) is fetched 16 bytes per lane along the rows, kept in
// that orientation in the patch and transposed by the reads.  Both need 16-byte aligned rows (the dispatcher
// checks pointers, pitches and the contiguous extent); M, N are arbitrary, K is a multiple of 4.
// Must be included by exactly one translation unit.
#pragma once
#include <hip/hip_runtime.h>

#include "sgemm_mfma.hpp"

namespace snhip {

// GemmParams::flags bit of this kernel (next to GEMM_FLAG_C_VEC / GEMM_FLAG_WS_VEC of the tiled kernels): the
// column-tile index runs fastest in blockIdx.x
constexpr int GEMM_FLAG_TILE_N_FASTEST = 4;

// NT: 32-column tiles per workgroup (1 or 2); the NW wavefronts (4, or 8 for products with so few tiles that even
// four slices leave most of the chip idle) are NT tiles x NW / NT slices of K.
template <int NT_, int NW_ = 4>
struct KsplitCfg {
    static constexpr int NT = NT_, NW = NW_;
    static constexpr int KS = NW_ / NT_;  // K slices
    static constexpr int DEPTH = 4;     // groups of 32 k values in flight per wavefront
    static constexpr int PITCH = 36;    // floats per patch row
    // LDS (dynamic): a patch of 2 x 32 rows per wavefront during the k loop; afterwards the same memory holds the
    // KS partial tiles
    static constexpr int PATCH_FLOATS = NW_ * 2 * 32 * PITCH, PART_FLOATS = KS * NT_ * 32 * 33;
    static constexpr int LDS_BYTES = 4 * (PATCH_FLOATS > PART_FLOATS ? PATCH_FLOATS : PART_FLOATS);
};

// One operand of one wavefront: 32 rows (m or n) x the k range.
//   KMAJOR = false: storage [row][k]; instruction i of a group reads row 8 i + lane / 8, k 4 (lane % 8) .. + 3.
//   KMAJOR = true:  storage [k][row]; instruction i reads k 8 i + lane / 8, rows 4 (lane % 8) .. + 3.
template <bool KMAJOR>
struct KsplitOperand {
    const float* ptr[4];   // address of the lane's vector of group 0, per instruction
    long long step;        // floats between consecutive groups
    bool row_ok[4];        // KMAJOR: the lane's four rows exist; else unused (rows are clamped instead)
    int k_first[4];        // k of the lane's vector (element 0) within a group

    __device__ __forceinline__ void init(const float* base, long long ld, int row0, int rows, int lane) {
        const int lrow = lane >> 3, lcol = (lane & 7) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (KMAJOR) {
                row_ok[i] = row0 + lcol < rows;                       // rows % 4 == 0: all four or none
                k_first[i] = 8 * i + lrow;
                ptr[i] = base + (long long)k_first[i] * ld + (row_ok[i] ? row0 + lcol : 0);
            } else {
                const int r = (row0 + 8 * i + lrow < rows) ? row0 + 8 * i + lrow : rows - 1;
                row_ok[i] = true;
                k_first[i] = lcol;
                ptr[i] = base + (long long)r * ld + lcol;
            }
        }
        step = KMAJOR ? 32 * ld : 32;
    }
    // the vector of group m; beyond K the address falls back to group 0 (always inside the matrix) and the value
    // is discarded in `keep`
    __device__ __forceinline__ f32x4 load(int i, int m, int K) const {
        const bool ok = 32 * m + k_first[i] < K;
        return *reinterpret_cast<const f32x4*>(ptr[i] + (ok ? (long long)m * step : 0));
    }
    __device__ __forceinline__ f32x4 keep(f32x4 v, int i, int m, int K) const {
        const bool ok = (32 * m + k_first[i] < K) && row_ok[i];
        f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
        return ok ? v : z;
    }
    // registers -> patch, in the orientation of the storage: patch[row][k], or patch[k][row] for KMAJOR (either way
    // one 16-byte store per vector, eight lanes per 128-byte line)
    __device__ __forceinline__ void to_patch(float* patch, int P, int i, int lane, f32x4 v) const {
        const int lrow = lane >> 3, lcol = (lane & 7) * 4;
        *reinterpret_cast<f32x4*>(patch + (8 * i + lrow) * P + lcol) = v;
    }
    // MFMA operand piece of a lane: row lane % 32, k = 16 (lane / 32) + 4 j .. + 3.  One 16-byte read from
    // patch[row][k]; four 4-byte reads from patch[k][row] (consecutive lanes on consecutive banks).
    __device__ __forceinline__ f32x4 fragment(const float* patch, int P, int lane, int j) const {
        const int l32 = lane & 31, lhi = lane >> 5;
        if constexpr (KMAJOR) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = patch[(16 * lhi + 4 * j + e) * P + l32];
            return v;
        } else {
            return *reinterpret_cast<const f32x4*>(patch + l32 * P + 16 * lhi + 4 * j);
        }
    }
};

// One workgroup's share of the product: tile `tile_index` (of p.tiles_m * p.tiles_n) of matrix z.  `smem` is the
// workgroup's dynamic LDS (KsplitCfg<NT, NW>::LDS_BYTES).
template <bool TA, bool TB, int NT, int NW>
__device__ __forceinline__ void ksplit_tile(const GemmParams& p, int tile_index, int z, float* smem) {
    using C = KsplitCfg<NT, NW>;
    constexpr int KS = C::KS, D = C::DEPTH, P = C::PITCH;
    float(*const part)[NT][32][33] = reinterpret_cast<float(*)[NT][32][33]>(smem);  // [KS][NT][32][33], after the k loop
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int nt = wave % NT, kg = wave / NT;
    // Workgroups go to the eight XCDs round-robin by their linear index.  The index that runs fastest spreads over
    // the XCDs, the other one stays put (when the fast count is a multiple of 8): the dispatcher lets the tiles of
    // the smaller operand run fastest, so that each XCD's L2 fetches its own part of the larger operand only once.
    const bool n_fastest = (p.flags & GEMM_FLAG_TILE_N_FASTEST) != 0;
    const int tile_m = n_fastest ? tile_index / p.tiles_n : tile_index % p.tiles_m;
    const int tile_n = n_fastest ? tile_index % p.tiles_n : tile_index / p.tiles_m;
    const int m0 = tile_m * 32, n0 = tile_n * (32 * NT) + 32 * nt;
    const float* Ab = p.A + (long long)z * p.strideA;
    const float* Bb = p.B + (long long)z * p.strideB;
    float* Cb = p.C + (long long)z * p.strideC;

    // What the write-out reads from memory - bias, old C, addend - is asked for here, in front of the k loop, for all
    // of a thread's elements and from addresses clamped into the matrix: in a kernel that lasts a few microseconds the
    // way of these values from memory would otherwise come on top of the operands' (the three conditions are uniform).
    constexpr int Q = (16 * NT) / NW;
    float bval[Q], cold[Q], dold[Q];
    {
        const int nbase = tile_n * (32 * NT);
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int e = threadIdx.x + (64 * NW) * q;
            const int lr = e / (32 * NT), lc = e % (32 * NT);
            const int row = m0 + lr < p.M ? m0 + lr : p.M - 1, col = nbase + lc < p.N ? nbase + lc : p.N - 1;
            bval[q] = cold[q] = dold[q] = 0.0f;
            if (p.ep.bias != nullptr) bval[q] = p.ep.bias[col];
            if (p.beta != 0.0f) cold[q] = Cb[(long long)row * p.ldc + col];
            if (p.ep.addend != nullptr) dold[q] = p.ep.addend[(long long)z * p.ep.strideD + (long long)row * p.ep.ldd + col];
        }
    }

    KsplitOperand<TA> oa;     // A transposed: stored K x M, contiguous along m
    KsplitOperand<!TB> ob;    // B not transposed: stored K x N, contiguous along n
    oa.init(Ab, p.lda, m0, p.M, lane);
    ob.init(Bb, p.ldb, n0, p.N, lane);
    float* pa = smem + (wave * 2 + 0) * (32 * P);
    float* pb = smem + (wave * 2 + 1) * (32 * P);

    const int K = p.K;
    const int groups = (K + 31) / 32;
    const int per = (groups + KS - 1) / KS;
    const int mbeg = kg * per, mend = (mbeg + per < groups) ? mbeg + per : groups;

    f32x4 ra[D][4], rb[D][4], fa[2][4], fb[2][4];
    f32x16 acc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[e][r] = 0.0f;

    auto load = [&](int slot, int m) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[slot][i] = oa.load(i, m, K);
            rb[slot][i] = ob.load(i, m, K);
        }
    };
    // a group goes from its registers through the wavefront's LDS patch into operand layout (fragment buffer f);
    // the fences keep the compiler from moving LDS accesses across the points where lanes exchange data
    auto stage = [&](int slot, int m, int f) {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            oa.to_patch(pa, P, i, lane, oa.keep(ra[slot][i], i, m, K));
            ob.to_patch(pb, P, i, lane, ob.keep(rb[slot][i], i, m, K));
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            fa[f][j] = oa.fragment(pa, P, lane, j);
            fb[f][j] = ob.fragment(pb, P, lane, j);
        }
    };
    auto multiply = [&](int f) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[f][j][e], fb[f][j][e], acc[e], 0, 0, 0);
    };

    // blocks of D groups without a branch between a load and its use (exact s_waitcnt vmcnt(N)); the LDS round
    // trip of group i + 1 is issued before the MFMAs of group i
    const int cnt = mend > mbeg ? mend - mbeg : 0;
    const int mmain = mbeg + (cnt / D) * D;
    int m = mbeg;
    if (m < mmain) {
#pragma unroll
        for (int d = 0; d < D; ++d) load(d, m + d);
        stage(0, m, 0);
        for (; m + D < mmain; m += D) {
            load(0, m + D);
#pragma unroll
            for (int d = 0; d < D; ++d) {
                stage((d + 1) % D, m + d + 1, (d + 1) % 2);
                if (d + 1 < D) load(d + 1, m + d + 1 + D);
                multiply(d % 2);
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (d + 1 < D) stage(d + 1, m + d + 1, (d + 1) % 2);
            multiply(d % 2);
        }
    }
#pragma unroll
    for (int d = 0; d < D - 1; ++d)
        if (mmain + d < mend) load(d, mmain + d);
#pragma unroll
    for (int d = 0; d < D - 1; ++d)
        if (mmain + d < mend) {
            stage(d, mmain + d, 0);
            multiply(0);
        }

    __syncthreads();  // every wavefront is done with its patch: the memory now takes the partial tiles
    // accumulator register r holds row 8 (r / 4) + 4 lhi + r % 4, column l32 of the tile
#pragma unroll
    for (int r = 0; r < 16; ++r)
        part[kg][nt][8 * (r / 4) + 4 * lhi + (r % 4)][l32] = (acc[0][r] + acc[1][r]) + (acc[2][r] + acc[3][r]);
    __syncthreads();

    const int nbase = tile_n * (32 * NT);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int e = threadIdx.x + (64 * NW) * q;
        const int lr = e / (32 * NT), lc = e % (32 * NT);
        const int row = m0 + lr, col = nbase + lc;
        if (row >= p.M || col >= p.N) continue;
        float v = 0.0f;
#pragma unroll
        for (int k = 0; k < KS; ++k) v += part[k][lc / 32][lr][lc % 32];
        v *= p.alpha;
        v += bval[q];
        if (p.beta != 0.0f) v += p.beta * cold[q];
        if (p.ep.addend != nullptr) v += p.ep.gamma * dold[q];
        if (p.ep.act == ACT_RELU || p.ep.act == ACT_LEAKY_RELU) v = leaky_relu(v, p.ep.act_param);
        Cb[(long long)row * p.ldc + col] = v;
    }
}

template <bool TA, bool TB, int NT = 1, int NW = 4>
__global__ void __launch_bounds__(64 * NW) sgemm_ksplit_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    ksplit_tile<TA, TB, NT, NW>(p, blockIdx.x, blockIdx.y, smem);
}

// The backward pass of a Dense layer on a small batch in ONE launch (Linear.DenseBackwardPropagation,
// Prod/Layers/Linear.cs:142-191): the three results come from the same dy,
//     dW = multiplier * dy^T . x + gamma * W     (pw: transposed A = dy, plain B = x, addend W)
//     dx = dy . W                                (px: plain A = dy, plain B = W)
//     db[c] = sum over rows of dy[r][c] + bias_alpha * bias[c]     (64 columns per workgroup; the second term is
//                                                the weight decay on the bias of Linear.cs:178-181, bias may be nullptr)
// and each alone is a handful of 32 x 32 tiles that costs a launch more than its arithmetic.  The grid is the
// concatenation of the three jobs' workgroups: [0, blocks_x) tiles of dx, then blocks_w tiles of dW, then the column
// blocks of db; every workgroup runs exactly the code its job would run in a launch of its own (32 x 32 tiles with
// four K slices, or 32 x 64 tiles with two: the order of summation inside a K slice and across slices is the same
// ascending one either way).
struct DenseBackwardSmallParams {
    GemmParams pw, px;
    int blocks_w, blocks_x;
    int nt_w, nt_x;    // 32-column tiles per workgroup (1: four K slices, 2: two) of the dW / dx product: the host
                       // picks them so that the whole grid is resident at once when it can be
    const float* dy;   // rows x cols, row pitch ld; db may be nullptr (no column blocks in the grid then)
    float* db;
    const float* bias;
    float bias_alpha;
    int rows, cols;
    long long ld;
};
__global__ void __launch_bounds__(256) dense_backward_small_kernel(const DenseBackwardSmallParams q) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int b = blockIdx.x;  // uniform: the three branches never diverge inside a workgroup
    if (b < q.blocks_x) {  // the longer K first
        if (q.nt_x == 2)
            ksplit_tile<false, false, 2, 4>(q.px, b, 0, smem);
        else
            ksplit_tile<false, false, 1, 4>(q.px, b, 0, smem);
    } else if (b < q.blocks_x + q.blocks_w) {
        if (q.nt_w == 2)
            ksplit_tile<true, false, 2, 4>(q.pw, b - q.blocks_x, 0, smem);
        else
            ksplit_tile<true, false, 1, 4>(q.pw, b - q.blocks_x, 0, smem);
    } else {
        // wavefront w adds rows w, w + 4, ... of its 64 columns; the four partial sums meet in LDS in a fixed order
        float(*const part)[64] = reinterpret_cast<float(*)[64]>(smem);
        const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
        const int c = (b - q.blocks_w - q.blocks_x) * 64 + lane;
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
        if (c < q.cols) {
            int r = w;
            for (; r + 12 < q.rows; r += 16) {
                s0 += q.dy[(long long)r * q.ld + c];
                s1 += q.dy[(long long)(r + 4) * q.ld + c];
                s2 += q.dy[(long long)(r + 8) * q.ld + c];
                s3 += q.dy[(long long)(r + 12) * q.ld + c];
            }
            for (; r < q.rows; r += 4) s0 += q.dy[(long long)r * q.ld + c];
        }
        part[w][lane] = (s0 + s1) + (s2 + s3);
        __syncthreads();
        if (w == 0 && c < q.cols) {
            float v = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
            if (q.bias != nullptr) v += q.bias_alpha * q.bias[c];
            q.db[c] = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same scheme on 16 x 16 tiles (v_mfma_f32_16x16x4_f32) with K split over the eight wavefronts of a workgroup,
// for products with so few 32 x 32 tiles that most compute units would get none (the forward product of a Dense
// layer on a small batch, 128 x 256 x 784: 32 tiles of 32 x 32, 128 of 16 x 16).
// ---------------------------------------------------------------------------------------------------------------
typedef float f32x4_acc16 __attribute__((ext_vector_type(4)));

struct Ksplit16Cfg {
    static constexpr int NW = 8;        // wavefronts = K slices
    static constexpr int DEPTH = 4;     // groups of 32 k values in flight per wavefront
    static constexpr int PITCH = 36;    // floats per row of a patch[16 rows][32 k]
    static constexpr int PITCH_K = 20;  // floats per row of a patch[32 k][16 rows]
    static constexpr int PATCH_FLOATS = NW * 2 * 32 * PITCH_K;  // >= NW * 2 * 16 * PITCH
    static constexpr int PART_FLOATS = NW * 16 * 17;
    static constexpr int LDS_BYTES = 4 * (PATCH_FLOATS > PART_FLOATS ? PATCH_FLOATS : PART_FLOATS);
};

// One operand of one wavefront: 16 rows (m or n) x the k range, two 16-byte loads per lane and group of 32 k.
//   KMAJOR = false: storage [row][k]; instruction i reads row 8 i + lane / 8, k 4 (lane % 8) .. + 3.
//   KMAJOR = true:  storage [k][row]; instruction i reads k 16 i + lane / 4, rows 4 (lane % 4) .. + 3.
template <bool KMAJOR>
struct KsplitOperand16 {
    const float* ptr[2];
    long long step;
    bool row_ok[2];
    int k_first[2];

    __device__ __forceinline__ void init(const float* base, long long ld, int row0, int rows, int lane) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if constexpr (KMAJOR) {
                const int lcol = (lane & 3) * 4;
                row_ok[i] = row0 + lcol < rows;  // rows % 4 == 0: all four or none
                k_first[i] = 16 * i + (lane >> 2);
                ptr[i] = base + (long long)k_first[i] * ld + (row_ok[i] ? row0 + lcol : 0);
            } else {
                const int lrow = lane >> 3, lcol = (lane & 7) * 4;
                const int r = (row0 + 8 * i + lrow < rows) ? row0 + 8 * i + lrow : rows - 1;
                row_ok[i] = true;
                k_first[i] = lcol;
                ptr[i] = base + (long long)r * ld + lcol;
            }
        }
        step = KMAJOR ? 32 * ld : 32;
    }
    __device__ __forceinline__ f32x4 load(int i, int m, int K) const {
        const bool ok = 32 * m + k_first[i] < K;
        return *reinterpret_cast<const f32x4*>(ptr[i] + (ok ? (long long)m * step : 0));
    }
    __device__ __forceinline__ f32x4 keep(f32x4 v, int i, int m, int K) const {
        const bool ok = (32 * m + k_first[i] < K) && row_ok[i];
        f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
        return ok ? v : z;
    }
    __device__ __forceinline__ void to_patch(float* patch, int i, int lane, f32x4 v) const {
        if constexpr (KMAJOR)
            *reinterpret_cast<f32x4*>(patch + (16 * i + (lane >> 2)) * Ksplit16Cfg::PITCH_K + (lane & 3) * 4) = v;
        else
            *reinterpret_cast<f32x4*>(patch + (8 * i + (lane >> 3)) * Ksplit16Cfg::PITCH + (lane & 7) * 4) = v;
    }
    // The eight MFMAs of a group: MFMA j takes k = 8 q + j from lane group q = lane / 16 (any assignment of the 32 k
    // values to (j, q) will do as long as both operands use the same one).  f[j] = operand[row lane % 16][8 q + j].
    __device__ __forceinline__ void fragment(const float* patch, int lane, float (&f)[8]) const {
        const int r = lane & 15, q = lane >> 4;
        if constexpr (KMAJOR) {
#pragma unroll
            for (int j = 0; j < 8; ++j) f[j] = patch[(8 * q + j) * Ksplit16Cfg::PITCH_K + r];
        } else {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(patch + r * Ksplit16Cfg::PITCH + 8 * q);
            const f32x4 hi = *reinterpret_cast<const f32x4*>(patch + r * Ksplit16Cfg::PITCH + 8 * q + 4);
            f[0] = lo.x, f[1] = lo.y, f[2] = lo.z, f[3] = lo.w, f[4] = hi.x, f[5] = hi.y, f[6] = hi.z, f[7] = hi.w;
        }
    }
};

template <bool TA, bool TB>
__global__ void __launch_bounds__(512) sgemm_ksplit16_kernel(const GemmParams p) {
    using C = Ksplit16Cfg;
    constexpr int NW = C::NW, D = C::DEPTH;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float(*const part)[16][17] = reinterpret_cast<float(*)[16][17]>(smem);  // [NW][16][17], after the k loop
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool n_fastest = (p.flags & GEMM_FLAG_TILE_N_FASTEST) != 0;
    const int tile_m = n_fastest ? blockIdx.x / p.tiles_n : blockIdx.x % p.tiles_m;
    const int tile_n = n_fastest ? blockIdx.x % p.tiles_n : blockIdx.x / p.tiles_m;
    const int m0 = tile_m * 16, n0 = tile_n * 16;
    const int z = blockIdx.y;
    const float* Ab = p.A + (long long)z * p.strideA;
    const float* Bb = p.B + (long long)z * p.strideB;
    float* Cb = p.C + (long long)z * p.strideC;

    // bias, old C and addend of this thread's element, asked for in front of the k loop (see ksplit_tile)
    float bval = 0.0f, cold = 0.0f, dold = 0.0f;
    if (threadIdx.x < 256) {
        const int lr = threadIdx.x / 16, lc = threadIdx.x % 16;
        const int row = m0 + lr < p.M ? m0 + lr : p.M - 1, col = n0 + lc < p.N ? n0 + lc : p.N - 1;
        if (p.ep.bias != nullptr) bval = p.ep.bias[col];
        if (p.beta != 0.0f) cold = Cb[(long long)row * p.ldc + col];
        if (p.ep.addend != nullptr) dold = p.ep.addend[(long long)z * p.ep.strideD + (long long)row * p.ep.ldd + col];
    }

    KsplitOperand16<TA> oa;
    KsplitOperand16<!TB> ob;
    oa.init(Ab, p.lda, m0, p.M, lane);
    ob.init(Bb, p.ldb, n0, p.N, lane);
    float* pa = smem + (wave * 2 + 0) * (32 * C::PITCH_K);
    float* pb = smem + (wave * 2 + 1) * (32 * C::PITCH_K);

    const int K = p.K;
    const int groups = (K + 31) / 32;
    const int per = (groups + NW - 1) / NW;
    const int mbeg = wave * per, mend = (mbeg + per < groups) ? mbeg + per : groups;

    f32x4 ra[D][2], rb[D][2];
    float fa[8], fb[8];
    f32x4_acc16 acc[2];
#pragma unroll
    for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[e][r] = 0.0f;

    // all of a wavefront's groups are requested before the first one is used (up to D at a time)
    for (int m = mbeg; m < mend; m += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (m + d < mend) {  // uniform
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    ra[d][i] = oa.load(i, m + d, K);
                    rb[d][i] = ob.load(i, m + d, K);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (m + d < mend) {
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    oa.to_patch(pa, i, lane, oa.keep(ra[d][i], i, m + d, K));
                    ob.to_patch(pb, i, lane, ob.keep(rb[d][i], i, m + d, K));
                }
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                __builtin_amdgcn_wave_barrier();
                oa.fragment(pa, lane, fa);
                ob.fragment(pb, lane, fb);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    acc[j & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[j], fb[j], acc[j & 1], 0, 0, 0);
            }
        }
    }

    __syncthreads();  // every wavefront is done with its patch: the memory now takes the partial tiles
    // accumulator register e holds row 4 (lane / 16) + e, column lane % 16 of the tile
#pragma unroll
    for (int e = 0; e < 4; ++e) part[wave][4 * (lane >> 4) + e][lane & 15] = acc[0][e] + acc[1][e];
    __syncthreads();

    if (threadIdx.x < 256) {
        const int lr = threadIdx.x / 16, lc = threadIdx.x % 16;
        const int row = m0 + lr, col = n0 + lc;
        if (row < p.M && col < p.N) {
            float v = 0.0f;
#pragma unroll
            for (int k = 0; k < NW; ++k) v += part[k][lr][lc];
            v *= p.alpha;
            v += bval;
            if (p.beta != 0.0f) v += p.beta * cold;
            if (p.ep.addend != nullptr) v += p.ep.gamma * dold;
            if (p.ep.act == ACT_RELU || p.ep.act == ACT_LEAKY_RELU) v = leaky_relu(v, p.ep.act_param);
            Cb[(long long)row * p.ldc + col] = v;
        }
    }
}

}  // namespace snhip
