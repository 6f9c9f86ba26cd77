// fp32 GEMM for gfx950 (MI355X) built on v_mfma_f32_32x32x2_f32.
//
// Computes, for every matrix of a strided batch, the row-major product
//     C[M x N] = alpha * op(A) * op(B) + beta * C  (+ bias[n] broadcast over rows)
// which is the contract of SharpNet's Tensor.Dot / BatchMatrixMultiplication
// (reference: Prod/Data/BlasServices.cs:10-21, Prod/CPU/CpuTensor.cs:2991-3025,
// Prod/GPU/GpuTensor.cs:1163-1227).  op(X) = X or X^T; A is stored with leading
// dimension lda, i.e. element op(A)[m][k] lives at A[m*lda + k] (no transpose)
// or A[k*lda + m] (transpose); likewise for B with op(B)[k][n].
//
// Work decomposition
//   * one workgroup owns a BM x BN tile of C (and, with split-K, one K slice);
//   * the workgroup is WM x WN wavefronts of 64 lanes, each wavefront owns
//     TM x TN MFMA tiles of 32 x 32, accumulated in registers (AGPR/VGPR);
//   * K is walked in steps of BK through a double-buffered LDS stage.  Both
//     operands are kept in LDS "k-major": As[k][m] and Bs[k][n], which is the
//     order the 32x32x2 MFMA wants (lane l supplies A[l%32][l/32], B[l/32][l%32]).
//   * the TM (TN) tiles of a wavefront are interleaved at element granularity:
//     lane i of tile t covers row  TM*i + t.  One ds_read of TM consecutive
//     floats therefore feeds all TM tiles, and in the epilogue a lane owns TN
//     consecutive columns of C, so stores are 16-byte vectors when TN == 4.
//
// Operand staging.  An operand whose memory is contiguous along m/n (A with
// transposeA, B without transposeB) is copied global->LDS as 16-byte vectors.
// An operand contiguous along k is loaded as 16-byte vectors along k and
// scattered to LDS as four dwords; the row pitch (tile + 4 floats) makes the
// scatter hit 64 distinct banks.
//
// Only 4-byte alignment of A, B, C is assumed (SharpNet tensors may be views at
// any element offset, GpuTensor.cs:616,1520).  Vector loads of global memory go
// through 4-byte-aligned vector types; the 16-byte C accesses are used only when
// the host has verified pointer and pitch alignment.
//
// beta == 0 never reads C (SharpNet hands out uninitialised pool memory,
// Prod/Data/TensorMemoryPool.cs:59-64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace snhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

enum : int {
    GEMM_FLAG_C_VEC = 1,  // C (and bias) may be accessed as aligned 16-byte vectors
};

struct GemmParams {
    const float* A;
    const float* B;
    float* C;           // destination; split-K partial sums go to ws instead
    const float* bias;  // optional, length N, added after alpha/beta
    float* ws;          // split-K workspace [batch][splitk][M][N], or nullptr
    int M, N, K;
    int lda, ldb, ldc;
    long long strideA, strideB, strideC;  // in elements
    int tiles_m, tiles_n;
    int splitk;   // >= 1
    int kchunk;   // K range of one split, multiple of BK
    float alpha, beta;
    int flags;
    int group_m;  // tile rows per swizzle group
};

// ---------------------------------------------------------------------------
// Global -> register -> LDS staging of one operand tile of logical shape
// [BK (k)] x [BMN (m or n)].  KCONTIG: global memory is contiguous along k.
// ---------------------------------------------------------------------------
template <int BMN, int BK, int NT, int PITCH, bool KCONTIG>
struct TileStage {
    static constexpr int NV = (BK * BMN) / (4 * NT);  // 16-byte vectors per thread
    static_assert((BK * BMN) % (4 * NT) == 0, "tile must split evenly over threads");
    static constexpr int VEC_PER_LINE = KCONTIG ? BK / 4 : BMN / 4;
    static_assert(NT % VEC_PER_LINE == 0, "thread count must be a multiple of vectors per line");
    static constexpr int LINE_STEP = NT / VEC_PER_LINE;  // lines advanced per vector index

    // position of this thread's vector 0 inside the tile
    int k0, mn0;
    const float* gptr;  // address of vector 0 for the current k tile
    long long ld;

    __device__ __forceinline__ void init(const float* base, long long ld_, int tile_mn, int kbeg, int tid) {
        const int vec = tid % VEC_PER_LINE;
        const int line = tid / VEC_PER_LINE;
        ld = ld_;
        if (KCONTIG) {
            k0 = vec * 4;
            mn0 = line;
            gptr = base + (long long)(tile_mn + mn0) * ld + (kbeg + k0);
        } else {
            mn0 = vec * 4;
            k0 = line;
            gptr = base + (long long)(kbeg + k0) * ld + (tile_mn + mn0);
        }
    }

    __device__ __forceinline__ void advance() { gptr += KCONTIG ? (long long)BK : (long long)BK * ld; }

    // Unchecked load: every element of the tile is inside the matrix.
    __device__ __forceinline__ void load_fast(f32x4 (&r)[NV]) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const float* p = gptr + (long long)(v * LINE_STEP) * ld;
            __builtin_memcpy(&r[v], p, 16);
        }
    }

    // Checked load: elements with m/n >= mn_rem or k >= k_rem read as zero
    // (mn_rem, k_rem are counted from the tile origin).
    __device__ __forceinline__ void load_safe(f32x4 (&r)[NV], int mn_rem, int k_rem) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const float* p = gptr + (long long)(v * LINE_STEP) * ld;
            int nval;
            if (KCONTIG) {
                const int mn = mn0 + v * LINE_STEP;
                nval = (mn < mn_rem) ? (k_rem - k0) : 0;
            } else {
                const int k = k0 + v * LINE_STEP;
                nval = (k < k_rem) ? (mn_rem - mn0) : 0;
            }
            f32x4 x;
            x.x = (nval > 0) ? p[0] : 0.0f;
            x.y = (nval > 1) ? p[1] : 0.0f;
            x.z = (nval > 2) ? p[2] : 0.0f;
            x.w = (nval > 3) ? p[3] : 0.0f;
            r[v] = x;
        }
    }

    __device__ __forceinline__ void store_lds(float* s, const f32x4 (&r)[NV]) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (KCONTIG) {
                float* d = s + k0 * PITCH + (mn0 + v * LINE_STEP);
                d[0 * PITCH] = r[v].x;
                d[1 * PITCH] = r[v].y;
                d[2 * PITCH] = r[v].z;
                d[3 * PITCH] = r[v].w;
            } else {
                float* d = s + (k0 + v * LINE_STEP) * PITCH + mn0;
                *reinterpret_cast<f32x4*>(d) = r[v];
            }
        }
    }
};

template <int T>
struct Frag;
template <>
struct Frag<1> {
    float v[1];
    __device__ __forceinline__ void load(const float* p) { v[0] = p[0]; }
};
template <>
struct Frag<2> {
    float v[2];
    __device__ __forceinline__ void load(const float* p) {
        f32x2 t = *reinterpret_cast<const f32x2*>(p);
        v[0] = t.x;
        v[1] = t.y;
    }
};
template <>
struct Frag<4> {
    float v[4];
    __device__ __forceinline__ void load(const float* p) {
        f32x4 t = *reinterpret_cast<const f32x4*>(p);
        v[0] = t.x;
        v[1] = t.y;
        v[2] = t.z;
        v[3] = t.w;
    }
};

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Remap the id
// so that each XCD (which has a private L2) works on a contiguous range of
// tiles, then walk that range in groups of `group_m` tile rows so concurrently
// resident tiles share A row panels and B column panels.
__device__ __forceinline__ void tile_coords(int bid, int ntiles, int tiles_m, int tiles_n, int group_m, int& tm,
                                            int& tn) {
    constexpr int NXCD = 8;
    const int q = ntiles / NXCD, r = ntiles % NXCD;
    const int xcd = bid % NXCD, local = bid / NXCD;
    const int logical = xcd * q + (xcd < r ? xcd : r) + local;
    const int per_group = group_m * tiles_n;
    const int g = logical / per_group;
    const int first_m = g * group_m;
    const int gsz = (tiles_m - first_m < group_m) ? (tiles_m - first_m) : group_m;
    const int in_g = logical - g * per_group;
    tm = first_m + in_g % gsz;
    tn = in_g / gsz;
}

template <int TM_, int TN_, int WM_, int WN_, int BK_>
struct TileCfg {
    static constexpr int TM = TM_, TN = TN_, WM = WM_, WN = WN_, BK = BK_;
    static constexpr int BM = TM * WM * 32, BN = TN * WN * 32;
    static constexpr int NT = WM * WN * 64;
    static constexpr int PA = BM + 4, PB = BN + 4;  // LDS row pitch in floats (== 4 mod 16)
    static constexpr int LDS_BYTES = 2 * BK * (PA + PB) * 4;
};

template <class CFG, bool TA, bool TB>
__global__ void __launch_bounds__(CFG::NT) sgemm_mfma_kernel(const GemmParams p) {
    constexpr int TM = CFG::TM, TN = CFG::TN, WN = CFG::WN, BK = CFG::BK;
    constexpr int BM = CFG::BM, BN = CFG::BN, NT = CFG::NT, PA = CFG::PA, PB = CFG::PB;
    // A is contiguous along k when it is NOT transposed; B when it IS transposed.
    using StageA = TileStage<BM, BK, NT, PA, !TA>;
    using StageB = TileStage<BN, BK, NT, PB, TB>;

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* const As = smem;                // [2][BK][PA]
    float* const Bs = smem + 2 * BK * PA;  // [2][BK][PB]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, lhi = lane >> 5;

    int tile_m, tile_n;
    tile_coords(blockIdx.x, p.tiles_m * p.tiles_n, p.tiles_m, p.tiles_n, p.group_m, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int zb = blockIdx.y;  // batch * splitk + split
    const int batch = zb / p.splitk, split = zb - batch * p.splitk;

    const int kbeg = split * p.kchunk;
    const int kend = (kbeg + p.kchunk < p.K) ? (kbeg + p.kchunk) : p.K;
    const int klen = kend - kbeg;  // may be <= 0 for a trailing empty split
    const int nk = (klen + BK - 1) / BK;
    const int nk_full = klen / BK;

    const float* Ab = p.A + (long long)batch * p.strideA;
    const float* Bb = p.B + (long long)batch * p.strideB;

    const int m_rem = p.M - m0, n_rem = p.N - n0;  // > 0 by construction
    const bool full_mn = (m_rem >= BM) && (n_rem >= BN);

    StageA sa;
    StageB sb;
    sa.init(Ab, p.lda, m0, kbeg, tid);
    sb.init(Bb, p.ldb, n0, kbeg, tid);

    f32x4 ra[StageA::NV], rb[StageB::NV];
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto load_tile = [&](int kt) {
        if (full_mn && kt < nk_full) {
            sa.load_fast(ra);
            sb.load_fast(rb);
        } else {
            const int k_rem = klen - kt * BK;
            sa.load_safe(ra, m_rem, k_rem);
            sb.load_safe(rb, n_rem, k_rem);
        }
        sa.advance();
        sb.advance();
    };

    if (nk > 0) {
        load_tile(0);
        sa.store_lds(As, ra);
        sb.store_lds(Bs, rb);
        __syncthreads();
    }

    const int a_off = wm * (TM * 32) + l32 * TM;
    const int b_off = wn * (TN * 32) + l32 * TN;

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        const bool has_next = (kt + 1 < nk);
        if (has_next) load_tile(kt + 1);

        const float* as = As + cur * (BK * PA) + lhi * PA + a_off;
        const float* bs = Bs + cur * (BK * PB) + lhi * PB + b_off;

        Frag<TM> fa[2];
        Frag<TN> fb[2];
        fa[0].load(as);
        fb[0].load(bs);
#pragma unroll
        for (int s = 0; s < BK / 2; ++s) {
            // Issue the LDS reads of the next k step right behind the first MFMA of
            // this one, so their latency is covered by the remaining MFMAs.  The
            // scheduling fences keep the compiler from sinking them to the end.
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s & 1].v[i], fb[s & 1].v[j], acc[i][j], 0, 0, 0);
                    if (i == 0 && j == 0 && s + 1 < BK / 2) {
                        __builtin_amdgcn_sched_barrier(0);
                        fa[(s + 1) & 1].load(as + (2 * (s + 1)) * PA);
                        fb[(s + 1) & 1].load(bs + (2 * (s + 1)) * PB);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    // The prefetched tile goes to the other LDS buffer behind the first
                    // MFMA of the last k step; the rest of that step covers the writes.
                    if (i == 0 && j == 0 && s + 1 == BK / 2) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (has_next) {
                            sa.store_lds(As + (cur ^ 1) * (BK * PA), ra);
                            sb.store_lds(Bs + (cur ^ 1) * (BK * PB), rb);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---------------- epilogue ----------------
    // acc[i][j][r] holds C[row][col] with
    //   row = m0 + wm*TM*32 + TM*(8*(r/4) + 4*lhi + r%4) + i
    //   col = n0 + wn*TN*32 + TN*l32 + j
    const int col0 = n0 + wn * (TN * 32) + TN * l32;
    const int row_base = m0 + wm * (TM * 32);
    const bool to_ws = (p.splitk > 1);
    float* out;
    long long ldo;
    float alpha, beta;
    const float* bias;
    if (to_ws) {
        out = p.ws + (long long)zb * p.M * p.N;
        ldo = p.N;
        alpha = 1.0f;
        beta = 0.0f;
        bias = nullptr;
    } else {
        out = p.C + (long long)batch * p.strideC;
        ldo = p.ldc;
        alpha = p.alpha;
        beta = p.beta;
        bias = p.bias;
    }
    const bool vec_ok = (TN == 4) && (p.flags & GEMM_FLAG_C_VEC) && (col0 + TN <= p.N);

    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) bv[j] = (bias != nullptr && col0 + j < p.N) ? bias[col0 + j] : 0.0f;

#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = row_base + TM * (8 * (r / 4) + 4 * lhi + (r % 4)) + i;
            if (row >= p.M) continue;
            float* crow = out + (long long)row * ldo + col0;
            float v[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] = alpha * acc[i][j][r] + bv[j];
            if (vec_ok) {
                if constexpr (TN == 4) {
                    f32x4 o = {v[0], v[1], v[2], v[3]};
                    if (beta != 0.0f) {
                        const f32x4 c = *reinterpret_cast<const f32x4*>(crow);
                        o += beta * c;
                    }
                    *reinterpret_cast<f32x4*>(crow) = o;
                }
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if (col0 + j < p.N) {
                        float o = v[j];
                        if (beta != 0.0f) o += beta * crow[j];
                        crow[j] = o;
                    }
                }
            }
        }
    }
}

// C = alpha * sum_s ws[batch][s] + beta * C + bias, splits summed in index
// order so the result does not depend on scheduling.
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ ws, float* C,
                                                            const float* __restrict__ bias, int M, int N, int ldc,
                                                            long long strideC, int splitk, int batch, float alpha,
                                                            float beta) {
    const long long mn = (long long)M * N;
    const long long total = mn * batch;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const long long b = idx / mn;
        const long long e = idx - b * mn;
        const int row = (int)(e / N), col = (int)(e - (long long)row * N);
        const float* w = ws + b * splitk * mn + e;
        float s = 0.0f;
        for (int k = 0; k < splitk; ++k) s += w[(long long)k * mn];
        float o = alpha * s;
        if (bias != nullptr) o += bias[col];
        float* c = C + b * strideC + (long long)row * ldc + col;
        if (beta != 0.0f) o += beta * *c;
        *c = o;
    }
}

// C = beta * C (+ bias): the alpha == 0 or K == 0 degenerate product.
__global__ void __launch_bounds__(256) scale_c_kernel(float* C, const float* __restrict__ bias, int M, int N, int ldc,
                                                      long long strideC, int batch, float beta) {
    const long long mn = (long long)M * N;
    const long long total = mn * batch;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const long long b = idx / mn;
        const long long e = idx - b * mn;
        const int row = (int)(e / N), col = (int)(e - (long long)row * N);
        float* c = C + b * strideC + (long long)row * ldc + col;
        float o = (beta != 0.0f) ? beta * *c : 0.0f;
        if (bias != nullptr) o += bias[col];
        *c = o;
    }
}

}  // namespace snhip
