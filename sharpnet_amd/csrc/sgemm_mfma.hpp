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

#include <type_traits>

namespace snhip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

enum : int {
    GEMM_FLAG_C_VEC = 1,   // C (and the addend D, if any) rows may be accessed as aligned vectors of up to 16 bytes
                           // (pointer, pitch, batch strides)
    GEMM_FLAG_WS_VEC = 2,  // split-K workspace rows may be accessed as aligned 16-byte vectors (N % 4 == 0)
    // (4: GEMM_FLAG_TILE_N_FASTEST of sgemm_ksplit.hpp)
    GEMM_FLAG_K_FROM_M = 8,  // a hint, honoured by the extended fp32 kernels: op(A)[m][k] is zero for k < m (the
                             // transposed softmax weights of a causally masked attention layer), so the tile whose
                             // first row is m0 starts its k loop at m0 rounded down to a whole k tile
    GEMM_FLAG_LONGEST_FIRST = 16,  // with K_FROM_M: tiles are dealt out by work_coords_longest_first (group_m then
                                   // carries the number of compute units per XCD)
};

// Element-wise function applied last in the epilogue (the layer that follows a
// Linear layer in the reference's networks, Prod/CPU/CpuTensorActivationFunctions.cs:184-245).
enum : int { ACT_NONE = 0, ACT_RELU = 1, ACT_LEAKY_RELU = 2, ACT_SIGMOID = 3, ACT_TANH = 4 };

__device__ __forceinline__ float activate(float v, int act, float a) {
    switch (act) {
        case ACT_RELU:
            return v < 0.0f ? 0.0f : v;
        case ACT_LEAKY_RELU:
            return v >= 0.0f ? v : a * v;
        case ACT_SIGMOID:
            return 1.0f / (1.0f + expf(-v));
        case ACT_TANH:
            return tanhf(v);
        default:
            return v;
    }
}

// ReLU is the slope-0 member: v < 0 ? 0 : v  (a NaN stays a NaN, as in the reference's CPU path).
__device__ __forceinline__ float leaky_relu(float v, float slope) { return v < 0.0f ? slope * v : v; }

// What happens to alpha * (A.B) on its way to C:
//     C = act(alpha * A.B + bias[col] + beta * C + gamma * D[row][col])
// bias: the Linear layer's bias (Linear.cs:130-131); gamma * D: the weight-decay term
// dW += (k * batch * weight_decay) * W of Linear.cs:168-178; act: the following activation layer.
// The GEMM kernels themselves apply only the (leaky) ReLU family - one compare and one multiply per element;
// for the transcendental ones the host clears `act` for the GEMM launch and runs scale_c_kernel over C afterwards.
struct Epilogue {
    const float* bias;    // optional, length N
    const float* addend;  // optional D, M x N, row pitch ldd
    int ldd;
    long long strideD, strideD2;  // batch strides of D (inner level, outer level), in elements
    float gamma;
    int act;
    float act_param;
};

// Matrix z of a two-level strided batch is z = outer * inner_count + inner and sits at
// base + outer * stride_outer + inner * stride_inner.
struct BatchIndex {
    int outer, inner;
};
__device__ __host__ __forceinline__ BatchIndex split_batch(int z, int inner_count) {
    BatchIndex b = {0, z};
    if (z >= inner_count) {  // a single-level batch (the common case) takes no division
        b.outer = z / inner_count;
        b.inner = z - b.outer * inner_count;
    }
    return b;
}
__device__ __host__ __forceinline__ long long batch_offset(BatchIndex b, long long stride_inner, long long stride_outer) {
    return (long long)b.outer * stride_outer + (long long)b.inner * stride_inner;
}

// "no offset given" for store_accumulators_plain's optional output offset
constexpr long long kNoBatchOffset = -0x7fffffffffffffffLL - 1;

struct GemmParams {
    const float* A;
    const float* B;
    float* C;           // destination; split-K partial sums go to ws instead
    Epilogue ep;
    float* colsum;      // optional [batch][M]: colsum[m] = sum_k op(A)[m][k] (EXT kernels with transposed A and plain B, no split-K)
    float* ws;          // split-K workspace [batch][splitk][M][N], or nullptr
    int* counters;      // split-K arrival counters [batch][tiles], all zero between launches; nullptr = reduce in a
                        // second kernel
    int M, N, K;
    int lda, ldb, ldc;
    long long strideA, strideB, strideC;     // in elements, between matrices of the inner batch level
    long long strideA2, strideB2, strideC2;  // ... of the outer level (batch z = outer * batch_inner + inner)
    int batch_inner;                         // matrices per outer step (== batch for a plain strided batch)
    int tiles_m, tiles_n;
    int splitk;   // >= 1
    int kchunk;   // K range of one split, multiple of BK
    float alpha, beta;
    int flags;
    int group_m;  // tile rows per swizzle group
    int nz;       // batch * splitk: the grid is one-dimensional, tiles_m * tiles_n * nz workgroups
};

// ---------------------------------------------------------------------------
// Global -> register -> LDS staging of one operand tile of logical shape
// [BK (k)] x [BMN (m or n)].  KCONTIG: global memory is contiguous along k.
// ---------------------------------------------------------------------------
// WAVE_SPLITS_K (k-contiguous operands with BK = 64 or 32): a wavefront covers 16 lines x 16 k (each lane one 16-byte
// vector) instead of 4 lines x 64 k, and the wavefronts of the workgroup split k between them.  With BK = 64 the
// plain assignment would put the four dword stores of a scattered vector on 16 banks (4-way conflicts; 2-way with
// BK = 32); this one reaches 64 distinct banks again.
template <int BMN, int BK, int NT, int PITCH, bool KCONTIG, bool WAVE_SPLITS_K = false>
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
        int vec = tid % VEC_PER_LINE;
        int line = tid / VEC_PER_LINE;
        if constexpr (WAVE_SPLITS_K && KCONTIG) {
            static_assert(!WAVE_SPLITS_K || ((BK == 64 || BK == 32) && NT == 256), "mapping written for 4 wavefronts");
            constexpr int KW = BK / 16;  // wavefronts that split k between them; the others take further lines
            const int wave = tid >> 6, lane = tid & 63;
            vec = 4 * (wave % KW) + (lane >> 4);
            line = (lane & 15) + 16 * (wave / KW);
        }
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
    __device__ __forceinline__ void load_fast_vec(f32x4& r, int v) const {
        const float* p = gptr + (long long)(v * LINE_STEP) * ld;
        __builtin_memcpy(&r, p, 16);
    }

    __device__ __forceinline__ void load_fast(f32x4 (&r)[NV]) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) load_fast_vec(r[v], v);
    }

    // Checked load: elements with m/n >= mn_rem or k >= k_rem read as zero
    // (mn_rem, k_rem are counted from the tile origin) and touch no memory.
    __device__ __forceinline__ void load_safe_vec(f32x4& r, int v, int mn_rem, int k_rem) const {
        const float* p;
        int nval;
        if (KCONTIG) {
            // Rows past the edge re-read the last valid row instead of being zeroed: their
            // products land in rows (columns) of C that are never stored, and the load
            // stays a plain 16-byte vector for every lane of an edge tile.
            const int mn = mn0 + v * LINE_STEP;
            const int mnc = (mn < mn_rem) ? mn : mn_rem - 1;
            p = gptr + (long long)(mnc - mn0) * ld;
            nval = k_rem - k0;
        } else {
            p = gptr + (long long)(v * LINE_STEP) * ld;
            const int k = k0 + v * LINE_STEP;
            nval = (k < k_rem) ? (mn_rem - mn0) : 0;
        }
        f32x4 x;
        if (nval >= 4) {
            // whole vector inside the matrix: the common case even in edge tiles
            __builtin_memcpy(&x, p, 16);
        } else {
            x.x = (nval > 0) ? p[0] : 0.0f;
            x.y = (nval > 1) ? p[1] : 0.0f;
            x.z = (nval > 2) ? p[2] : 0.0f;
            x.w = 0.0f;
        }
        r = x;
    }

    __device__ __forceinline__ void load_safe(f32x4 (&r)[NV], int mn_rem, int k_rem) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) load_safe_vec(r[v], v, mn_rem, k_rem);
    }

    // Per-thread facts about a tile at the ragged edge of m/n, computed once per workgroup: they do not
    // change from k tile to k tile, so full-k tiles of an edge block can be loaded without re-deriving them.
    //
    // Nothing here zero-fills: a row (column) of op(A) (op(B)) past the edge only feeds rows (columns) of C that
    // are never stored, so it may hold any value that can be read without leaving the matrix.  A k-contiguous
    // operand re-reads its last valid row; an m/n-contiguous one reads its vector from a start clamped to
    // `extent - 4` and rotates the elements that are inside the matrix back to their slots.  Both are plain
    // 16-byte loads with no branch.  (Needs an extent of at least 4 along m/n; `usable` says so.)
    struct Edge {
        long long off[KCONTIG ? NV : 1];  // KCONTIG: element offset of vector v from gptr (row clamped);
                                          // otherwise off[0]: element offset of the clamped start from this thread's own
        int shift;                        // !KCONTIG: how far the start was moved back (0..3 matter; more: nothing inside)
        bool usable;
    };
    __device__ __forceinline__ Edge edge_info(int mn_rem, int tile_mn) const {
        Edge e;
        e.shift = 0;
        e.usable = true;
        if (KCONTIG) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int mn = mn0 + v * LINE_STEP;
                e.off[v] = (long long)(((mn < mn_rem) ? mn : mn_rem - 1) - mn0) * ld;
            }
        } else {
            // mn_rem counts from the tile origin; the matrix extent seen from this thread's vector is mn_rem - mn0
            const int last_start = mn_rem - 4;  // latest start (relative to the tile origin) that stays inside
            const int start = (mn0 <= last_start) ? mn0 : last_start;
            e.shift = mn0 - start;
            e.off[0] = (long long)(start - mn0);
            e.usable = (mn_rem >= 4) || (tile_mn > 0);  // the clamped start may reach into the tile before this one
        }
        return e;
    }
    // Load of a full-k tile of an edge block: a plain vector, nothing past the matrix is touched.  For an
    // m/n-contiguous operand the elements arrive `shift` slots late; store_lds_vec_shifted puts them back (doing it
    // here would make the load wait for its own data).
    __device__ __forceinline__ void load_edge_vec(f32x4& r, int v, const Edge& e) const {
        if (KCONTIG)
            __builtin_memcpy(&r, gptr + e.off[v], 16);
        else
            __builtin_memcpy(&r, gptr + (long long)(v * LINE_STEP) * ld + e.off[0], 16);
    }

    // vector v of this thread -> its place in the k-major LDS tile
    __device__ __forceinline__ void store_lds_vec(float* s, const f32x4& r, int v) const {
        if (KCONTIG) {
            float* d = s + k0 * PITCH + (mn0 + v * LINE_STEP);
            d[0 * PITCH] = r.x;
            d[1 * PITCH] = r.y;
            d[2 * PITCH] = r.z;
            d[3 * PITCH] = r.w;
        } else {
            float* d = s + (k0 + v * LINE_STEP) * PITCH + mn0;
            *reinterpret_cast<f32x4*>(d) = r;
        }
    }

    // The same for a vector that was loaded from a start moved back by `sh` elements (load_edge_vec): element j of
    // the wanted vector sits in slot j + sh; slots that would come from beyond slot 3 lie outside the matrix and
    // may hold anything.  sh == 0: as loaded.
    // `any_shift` is uniform over the workgroup (the extent along m/n is not a multiple of 4): without it the
    // vector is stored as loaded and the selects cost nothing.  Returns what was stored.
    __device__ __forceinline__ f32x4 store_lds_vec_shifted(float* s, const f32x4& r, int v, int sh, bool any_shift) const {
        f32x4 y = r;
        if (!KCONTIG && any_shift) {
            y.x = sh == 0 ? r.x : (sh == 1 ? r.y : (sh == 2 ? r.z : r.w));
            y.y = sh == 0 ? r.y : (sh == 1 ? r.z : r.w);
            y.z = sh == 0 ? r.z : r.w;
        }
        store_lds_vec(s, y, v);
        return y;
    }

    __device__ __forceinline__ void store_lds(float* s, const f32x4 (&r)[NV]) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) store_lds_vec(s, r[v], v);
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

// Workgroup barrier that orders LDS traffic only: global loads that are still in
// flight (the register prefetch) must not be waited for here.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Workgroups are handed to the 8 XCDs (each with a private L2) round-robin by linear workgroup id, so the grid is
// one-dimensional and the id is remapped here: every XCD works on one contiguous range of the logical order
// "matrix (batch entry x K split) by matrix, and inside a matrix tile after tile in groups of `group_m` tile
// rows".  Tiles that are resident together then share A row panels and B column panels in their L2, and the tiles
// of one matrix of a strided batch never spread over several XCDs unless a range boundary cuts through it.
struct WorkCoords {
    int zb;              // batch entry * splitk + split
    int tile_m, tile_n;
};
__device__ __forceinline__ WorkCoords work_coords(unsigned lin, int tiles_m, int tiles_n, int nz, int group_m) {
    constexpr unsigned NXCD = 8;
    const unsigned ntiles = (unsigned)(tiles_m * tiles_n);
    const unsigned total = ntiles * (unsigned)nz;  // the host keeps this below 2^31
    const unsigned q = total / NXCD, r = total % NXCD;
    const unsigned xcd = lin % NXCD, local = lin / NXCD;
    const unsigned L = xcd * q + (xcd < r ? xcd : r) + local;
    WorkCoords w;
    unsigned t = L;
    w.zb = 0;
    if (nz > 1) {  // uniform; an unbatched product takes no division
        w.zb = (int)(L / ntiles);
        t = L - (unsigned)w.zb * ntiles;
    }
    // reversed, so the ragged last tile row / column (slower, bounds-checked) is issued first
    const int logical = (int)(ntiles - 1 - t);
    const int per_group = group_m * tiles_n;
    const int g = logical / per_group;
    const int first_m = g * group_m;
    const int gsz = (tiles_m - first_m < group_m) ? (tiles_m - first_m) : group_m;
    const int in_g = logical - g * per_group;
    w.tile_m = first_m + in_g % gsz;
    w.tile_n = in_g / gsz;
    return w;
}

// The order for products whose tiles do unequal work because their k loops start at their first row
// (GEMM_FLAG_K_FROM_M): tile row 0 sums over all of K, the last one over a sliver.  Every XCD owns nz / 8 whole matrices
// (the host checks that the counts divide and that there is one tile column).  Inside an XCD the (tile row, matrix)
// pairs are taken longest first, and the rounds of `cu_per_xcd` workgroups alternate direction, so that the compute
// unit that got the longest item of one round gets the shortest of the next (workgroups of one XCD go to its compute
// units in turn): co-resident workgroups then add up to about the same work everywhere.
__device__ __forceinline__ WorkCoords work_coords_longest_first(unsigned lin, int tiles_m, int nz, int cu_per_xcd) {
    constexpr unsigned NXCD = 8;
    const unsigned xcd = lin % NXCD, local = lin / NXCD;
    const unsigned nm = (unsigned)nz / NXCD;               // matrices per XCD
    const unsigned q = nm * (unsigned)tiles_m;             // items per XCD
    const unsigned round = local / (unsigned)cu_per_xcd, pos = local % (unsigned)cu_per_xcd;
    const unsigned left = q - round * (unsigned)cu_per_xcd;
    const unsigned len = left < (unsigned)cu_per_xcd ? left : (unsigned)cu_per_xcd;
    const unsigned item = round * (unsigned)cu_per_xcd + ((round & 1u) ? len - 1u - pos : pos);
    WorkCoords w;
    w.tile_m = (int)(item / nm);
    w.tile_n = 0;
    w.zb = (int)(xcd * nm + item % nm);
    return w;
}

// TN consecutive floats as one vector access (TN = 1, 2 or 4); the caller has checked alignment.
template <int TN>
__device__ __forceinline__ void load_row_vec(const float* p, float (&v)[TN]) {
    if constexpr (TN == 4) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(p);
        v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
    } else if constexpr (TN == 2) {
        const f32x2 t = *reinterpret_cast<const f32x2*>(p);
        v[0] = t.x, v[1] = t.y;
    } else {
        v[0] = p[0];
    }
}
template <int TN>
__device__ __forceinline__ void store_row_vec(float* p, const float (&v)[TN]) {
    if constexpr (TN == 4) {
        *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
    } else if constexpr (TN == 2) {
        *reinterpret_cast<f32x2*>(p) = f32x2{v[0], v[1]};
    } else {
        p[0] = v[0];
    }
}

// s_waitcnt vmcnt(0) as an instruction the compiler's own wait-count bookkeeping sees (expcnt and lgkmcnt fields at
// their maxima: not waited for).
__device__ __forceinline__ void wait_for_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// One accumulator element, read where it is used.  The operand constraint keeps the element in an accumulation
// register up to this point.  Without it the register allocator, which may hold these values in either half of the
// register file, moves most of a full-size accumulator set (256 values) into ordinary registers right behind the
// k loop and then spills to memory in the write-out.
// Only for the full-size set (PIN): smaller ones live wherever the allocator likes and need no help.
template <bool PIN>
__device__ __forceinline__ float acc_value(float x) {
    if constexpr (PIN) {
        float y;
        asm("v_accvgpr_read_b32 %0, %1" : "=v"(y) : "a"(x));
        return y;
    } else {
        return x;
    }
}

// Write-out of a wavefront whose whole 32*TM x 32*TN patch lies inside the matrix and may be accessed in vectors
// of TN floats:   C = act(alpha * acc + bias + beta * C + gamma * D).
// There are no per-lane tests and no loads under conditions here, so the stores go out back to back.  (In the
// general path every row is its own conditional block, and the compiler's wait-count bookkeeping, which merges the
// paths through those blocks, makes each row wait until the previous row's store has been acknowledged.)
// When old values are needed (beta != 0, or an addend D), rows go in chunks of four and the values of chunk k + 1
// are requested before chunk k is stored, so a load never waits behind the stores issued just before it (the
// compiler may not move loads across stores itself: for all it knows the rows alias).
// c0 / d0 point at the lane's first row (row_base + 4 * TM * lhi) and first column; d0 == nullptr: no addend.
template <int TM, int TN, bool EXT, bool PIN = (TM * TN >= 16)>
__device__ __forceinline__ void store_patch_fast(const f32x16 (&acc)[TM][TN], float* c0, long long ldo, const float* d0,
                                                 long long ldd, float alpha, float beta, float gamma,
                                                 const float (&bv)[TN], int act, float act_param) {
    auto row_off = [&](int k, int e) {  // chunk k = (tile row i, register group g), element e of the group
        const int i = k / 4, r = 4 * (k % 4) + e;
        return (long long)(TM * (8 * (r / 4) + (r % 4)) + i);
    };
    constexpr int CHUNKS = 4 * TM;
    const bool use_c = (beta != 0.0f), use_d = EXT && (d0 != nullptr);
    auto finish = [&](int k, int e, const float (&cv)[TN], const float (&dv)[TN]) {
        const int i = k / 4, r = 4 * (k % 4) + e;
        float v[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            v[j] = alpha * acc_value<PIN>(acc[i][j][r]) + bv[j];
            if (use_c) v[j] += beta * cv[j];
            if constexpr (EXT) {
                if (use_d) v[j] += gamma * dv[j];
                if (act != ACT_NONE) v[j] = leaky_relu(v[j], act_param);
            }
        }
        store_row_vec<TN>(c0 + row_off(k, e) * ldo, v);
    };
    if (!use_c && !use_d) {
        const float zero[TN] = {};
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
#pragma unroll
            for (int e = 0; e < 4; ++e) finish(k, e, zero, zero);
            // keep the arithmetic of one chunk next to its stores: left alone, the scheduler computes all
            // 16 * TM * TN results first, which needs more registers than there are
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }
    float cbuf[2][4][TN] = {}, dbuf[2][4][TN] = {};
    auto request = [&](int k) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (use_c) load_row_vec<TN>(c0 + row_off(k, e) * ldo, cbuf[k & 1][e]);
            if constexpr (EXT) {
                if (use_d) load_row_vec<TN>(d0 + row_off(k, e) * ldd, dbuf[k & 1][e]);
            }
        }
    };
    request(0);
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
        if (k + 1 < CHUNKS) request(k + 1);
#pragma unroll
        for (int e = 0; e < 4; ++e) finish(k, e, cbuf[k & 1][e], dbuf[k & 1][e]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Epilogue shared by the fp32 and bf16-input kernels.  acc[i][j][r] holds
// C[row][col] with  row = row_base + TM*(8*(r/4) + 4*lhi + r%4) + i  and
// col = col0 + j  (row_base = first row of the wavefront, col0 = first of the
// TN consecutive columns this lane owns, lhi = lane / 32).
//
// Without split-K: C = alpha*acc + beta*C + bias (C is read only when beta != 0).
// With split-K the raw partial sums go to workspace slice `zb`.  If arrival
// counters are supplied, the workgroup that arrives last for its tile (per-tile
// atomic counter, release/acquire fences at device scope) adds the splitk
// partial tiles in index order - every partial is re-read from memory, so the
// sum does not depend on which workgroup happens to be last - and writes
// alpha*sum + beta*C + bias.  Otherwise a second kernel does that reduction.
// ---------------------------------------------------------------------------
// Write-out.  Two versions: the plain one (bias, alpha, beta; single-level batch) that every ordinary product
// uses, and the extended one (also gamma * D, (leaky) ReLU, two-level batch) compiled only into the kernels
// instantiated with EXT, so that the extra tests and registers cost the plain product nothing.
// ---------------------------------------------------------------------------
// LEAN: for callers that hold many registers across the call (the streaming kernels keep the next panel in flight):
// the path for patches that stick out of the matrix then takes its compact form.
template <int TM, int TN, bool PIN = (TM * TN >= 16), bool LEAN = false>
__device__ __forceinline__ void store_accumulators_plain(const f32x16 (&acc)[TM][TN], const GemmParams& p, int row_base,
                                                   int col0, int lhi, int zb, int batch, int tile_index,
                                                   long long c_offset = kNoBatchOffset) {
    const bool to_ws = (p.splitk > 1);
    float* out;
    long long ldo;
    float alpha, beta;
    const float* bias;
    bool vec_ok;
    if (to_ws) {
        out = p.ws + (long long)zb * p.M * p.N;
        ldo = p.N;
        alpha = 1.0f;
        beta = 0.0f;
        bias = nullptr;
        vec_ok = (p.flags & GEMM_FLAG_WS_VEC) && (col0 + TN <= p.N);
    } else {
        out = p.C + (c_offset != kNoBatchOffset ? c_offset : (long long)batch * p.strideC);  // c_offset: the caller's own batch walk
        ldo = p.ldc;
        alpha = p.alpha;
        beta = p.beta;
        bias = p.ep.bias;
        vec_ok = (p.flags & GEMM_FLAG_C_VEC) && (col0 + TN <= p.N);
    }

    // a wavefront whose patch lies inside the matrix takes the branch-free write-out
    const int row_w = __builtin_amdgcn_readfirstlane(row_base);
    const int col_w = __builtin_amdgcn_readfirstlane(col0);  // lane 0 owns the wavefront's first column
    const bool ws_or_c_vec = to_ws ? ((p.flags & GEMM_FLAG_WS_VEC) != 0) : ((p.flags & GEMM_FLAG_C_VEC) != 0);
    if (ws_or_c_vec && row_w + 32 * TM <= p.M && col_w + 32 * TN <= p.N) {
        float bv[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = 0.0f;
        if (bias != nullptr) load_row_vec<TN>(bias + col0, bv);
        store_patch_fast<TM, TN, false, PIN>(acc, out + (long long)(row_base + TM * 4 * lhi) * ldo + col0, ldo, nullptr, 0, alpha,
                                        beta, 0.0f, bv, ACT_NONE, 0.0f);
    } else if (!LEAN && ws_or_c_vec && row_w + 32 * TM <= p.M && p.N % TN == 0) {
        // A patch that only sticks out over the right edge of a matrix whose width is a multiple of a lane's TN
        // columns (a lane is then wholly inside or wholly outside): the same write-out with the outside lanes switched
        // off.  A copy of its own: under a lane condition the whole-patch case above measured 3 % slower on products
        // without any edge (2048^3).
        if (col0 + TN <= p.N) {
            float bv[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) bv[j] = 0.0f;
            if (bias != nullptr) load_row_vec<TN>(bias + col0, bv);
            store_patch_fast<TM, TN, false, PIN>(acc, out + (long long)(row_base + TM * 4 * lhi) * ldo + col0, ldo, nullptr, 0,
                                                 alpha, beta, 0.0f, bv, ACT_NONE, 0.0f);
        }
    } else if constexpr (LEAN) {
        // the compact form: old values asked for on the vector path only, element-wise stores with their loads inside
        // the row's condition (a store round trip per row at a ragged right edge, few registers)
        float bv[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = (bias != nullptr && col0 + j < p.N) ? bias[col0 + j] : 0.0f;
        // the bias values are needed (and waited for) here, on every path: otherwise each row's block below
        // would wait for "a load that may still be pending" and with it for the previous row's store
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(bv[j]));

        // Old values (beta != 0) are asked for four rows at a time, from addresses clamped into the matrix and outside
        // the per-row conditions, before any of the four rows is stored: one wait per four rows instead of a
        // load - wait - store round trip per row (the compiler may not move a load across the store of the row
        // before it: for all it knows they alias).
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int rc = 0; rc < 4; ++rc) {
                float cold[4][TN];
                if (vec_ok && beta != 0.0f) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int rq = row_base + TM * (8 * rc + 4 * lhi + q) + i;
                        load_row_vec<TN>(out + (long long)(rq < p.M ? rq : p.M - 1) * ldo + col0, cold[q]);
                    }
                }
#pragma unroll
                for (int r = 4 * rc; r < 4 * rc + 4; ++r) {
                    const int row = row_base + TM * (8 * (r / 4) + 4 * lhi + (r % 4)) + i;
                    if (row >= p.M) continue;
                    float* crow = out + (long long)row * ldo + col0;
                    float v[TN];
#pragma unroll
                    for (int j = 0; j < TN; ++j) v[j] = alpha * acc_value<PIN>(acc[i][j][r]) + bv[j];
                    if (vec_ok) {
                        if (beta != 0.0f) {
#pragma unroll
                            for (int j = 0; j < TN; ++j) v[j] += beta * cold[r % 4][j];
                        }
                        store_row_vec<TN>(crow, v);
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
    } else if (row_w < p.M && col_w < p.N) {  // (a wavefront whose patch lies wholly outside the matrix writes nothing)
        float bv[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = (bias != nullptr && col0 + j < p.N) ? bias[col0 + j] : 0.0f;
        // the bias values are needed (and waited for) here, on every path: otherwise each row's block below
        // would wait for "a load that may still be pending" and with it for the previous row's store
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(bv[j]));

        // Two copies of the loop, chosen by a uniform branch: one for beta == 0 that contains no load at all, one
        // that asks for the old values four rows at a time, from addresses clamped into the matrix and outside the
        // per-row conditions, before any of the four rows is stored.  Stores count like loads in the memory wait
        // counter, so wherever a load's result is awaited the stores issued before it are awaited too: with the load of
        // the old value inside a row's own condition, or merely present under an `if (beta != 0)` that is not
        // taken, a ragged right edge cost a store round trip per row (measured: 1.5 us for the 16 rows of a
        // 64 x 64 tile, against 0.4 us for the branch-free write-out of a whole patch).
        auto rows = [&](auto with_old) {
        constexpr bool OLD = decltype(with_old)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int rc = 0; rc < 4; ++rc) {
                float cold[4][TN];
                if constexpr (OLD) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int rq = row_base + TM * (8 * rc + 4 * lhi + q) + i;
                        const float* src = out + (long long)(rq < p.M ? rq : p.M - 1) * ldo;
                        if (vec_ok) {
                            load_row_vec<TN>(src + col0, cold[q]);
                        } else {
#pragma unroll
                            for (int j = 0; j < TN; ++j) cold[q][j] = src[col0 + j < p.N ? col0 + j : p.N - 1];
                        }
                    }
                }
                // (one address product per block of four rows; the rows of a block lie TM * ldo apart)
                const int row0 = row_base + TM * (8 * rc + 4 * lhi) + i;
                float* const crow0 = out + (long long)row0 * ldo + col0;
#pragma unroll
                for (int r = 4 * rc; r < 4 * rc + 4; ++r) {
                    if (row0 + TM * (r % 4) >= p.M) continue;
                    float* crow = crow0 + (long long)(TM * (r % 4)) * ldo;
                    float v[TN];
#pragma unroll
                    for (int j = 0; j < TN; ++j) v[j] = alpha * acc_value<PIN>(acc[i][j][r]) + bv[j];
                    if constexpr (OLD) {
#pragma unroll
                        for (int j = 0; j < TN; ++j) v[j] += beta * cold[r % 4][j];
                    }
                    if (vec_ok) {
                        store_row_vec<TN>(crow, v);
                    } else {
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            if (col0 + j < p.N) crow[j] = v[j];
                    }
                }
            }
        }
        };  // rows
        if (beta != 0.0f)  // uniform
            rows(std::true_type{});
        else
            rows(std::false_type{});
    }

    if (!to_ws || p.counters == nullptr) return;

    // ---- in-kernel split-K reduction by the last workgroup to arrive ----
    __shared__ int s_is_last;
    __threadfence();  // release: this thread's partial sums are visible device-wide
    __syncthreads();
    if (threadIdx.x == 0) {
        int* cnt = p.counters + (long long)batch * (p.tiles_m * p.tiles_n) + tile_index;
        const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        const int last = (old == p.splitk - 1);
        if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
        s_is_last = last;
    }
    __syncthreads();
    if (!s_is_last) return;
    __threadfence();  // acquire: the other workgroups' partial sums are visible to every thread here

    const long long mn = (long long)p.M * p.N;
    const float* wsb = p.ws + (long long)batch * p.splitk * mn;
    float* Cb = p.C + (long long)batch * p.strideC;
    const bool ws_vec = (p.flags & GEMM_FLAG_WS_VEC) && (col0 + TN <= p.N);
    const bool c_vec = (p.flags & GEMM_FLAG_C_VEC) && (col0 + TN <= p.N);
    float cb[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) cb[j] = (p.ep.bias != nullptr && col0 + j < p.N) ? p.ep.bias[col0 + j] : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = row_base + TM * (8 * (r / 4) + 4 * lhi + (r % 4)) + i;
            if (row >= p.M) continue;
            const float* wrow = wsb + (long long)row * p.N + col0;
            float sum[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) sum[j] = 0.0f;
            for (int sidx = 0; sidx < p.splitk; ++sidx) {
                const float* w = wrow + (long long)sidx * mn;
                if (ws_vec) {
                    float t[TN];
                    load_row_vec<TN>(w, t);
#pragma unroll
                    for (int j = 0; j < TN; ++j) sum[j] += t[j];
                } else {
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        if (col0 + j < p.N) sum[j] += w[j];
                }
            }
            float* crow = Cb + (long long)row * p.ldc + col0;
            if (c_vec) {
                float o[TN];
#pragma unroll
                for (int j = 0; j < TN; ++j) o[j] = p.alpha * sum[j] + cb[j];
                if (p.beta != 0.0f) {
                    float c[TN];
                    load_row_vec<TN>(crow, c);
#pragma unroll
                    for (int j = 0; j < TN; ++j) o[j] += p.beta * c[j];
                }
                store_row_vec<TN>(crow, o);
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if (col0 + j < p.N) {
                        float o = p.alpha * sum[j] + cb[j];
                        if (p.beta != 0.0f) o += p.beta * crow[j];
                        crow[j] = o;
                    }
                }
            }
        }
    }
}

// v[j] = alpha * (A.B)[row][col0 + j] on entry; adds bias, beta * C and gamma * D, applies the activation
// and writes C.  crow / drow point at column col0 of the row; bv holds the bias values of the TN columns.
// v[j] = alpha * (A.B)[row][col0 + j] on entry; adds bias, beta * C and gamma * D, applies the activation
// and writes C.  crow / drow point at column col0 of the row (drow is looked at only if has_d, which like act
// is the same for the whole workgroup, so those tests are scalar branches); bv holds the bias values of the
// TN columns.
template <int TN>
__device__ __forceinline__ void finish_row(float (&v)[TN], float* crow, const float* drow, bool has_d,
                                           const float (&bv)[TN], float beta, float gamma, int act, float act_param,
                                           bool vec_ok, int ncols_left) {
#pragma unroll
    for (int j = 0; j < TN; ++j) v[j] += bv[j];
    if (vec_ok) {
        if (beta != 0.0f) {
            float c[TN];
            load_row_vec<TN>(crow, c);
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] += beta * c[j];
        }
        if (has_d) {
            float d[TN];
            load_row_vec<TN>(drow, d);
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] += gamma * d[j];
        }
        if (act != ACT_NONE) {
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] = leaky_relu(v[j], act_param);
        }
        store_row_vec<TN>(crow, v);
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if (j < ncols_left) {
                float o = v[j];
                if (beta != 0.0f) o += beta * crow[j];
                if (has_d) o += gamma * drow[j];
                if (act != ACT_NONE) o = leaky_relu(o, act_param);
                crow[j] = o;
            }
        }
    }
}

template <int TM, int TN>
__device__ __forceinline__ void store_accumulators_ext(const f32x16 (&acc)[TM][TN], const GemmParams& p, int row_base,
                                                       int col0, int lhi, int zb, int batch, BatchIndex bi,
                                                       int tile_index) {
    const bool to_ws = (p.splitk > 1);
    float* const Cb = p.C + batch_offset(bi, p.strideC, p.strideC2);
    const float* const Db =
        (p.ep.addend != nullptr) ? p.ep.addend + batch_offset(bi, p.ep.strideD, p.ep.strideD2) : nullptr;
    const bool c_vec = (p.flags & GEMM_FLAG_C_VEC) && (col0 + TN <= p.N);
    const bool ws_vec = (p.flags & GEMM_FLAG_WS_VEC) && (col0 + TN <= p.N);

    // One pass over the accumulators serves both destinations (the registers are read in one place only):
    // the final C, or - with split-K - the raw partial sums of workspace slice zb.
    float* out;
    const float* dsrc;
    long long ldo, ldd;
    float alpha, beta, gamma;
    int act;
    bool vec_ok;
    float bv[TN];
    if (to_ws) {
        out = p.ws + (long long)zb * p.M * p.N;
        dsrc = nullptr;
        ldo = p.N, ldd = 0;
        alpha = 1.0f, beta = 0.0f, gamma = 0.0f;
        act = ACT_NONE;
        vec_ok = ws_vec;
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = 0.0f;
    } else {
        out = Cb;
        dsrc = Db;
        ldo = p.ldc, ldd = p.ep.ldd;
        alpha = p.alpha, beta = p.beta, gamma = p.ep.gamma;
        act = p.ep.act;
        vec_ok = c_vec;
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = (p.ep.bias != nullptr && col0 + j < p.N) ? p.ep.bias[col0 + j] : 0.0f;
    }
    // the bias values are needed (and waited for) here, on every path (see store_accumulators_plain)
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(bv[j]));
    const bool has_d = (dsrc != nullptr);
    const int row_w = __builtin_amdgcn_readfirstlane(row_base);
    const int col_w = __builtin_amdgcn_readfirstlane(col0);  // lane 0 owns the wavefront's first column
    const bool ws_or_c_vec = to_ws ? ((p.flags & GEMM_FLAG_WS_VEC) != 0) : ((p.flags & GEMM_FLAG_C_VEC) != 0);
    if (ws_or_c_vec && row_w + 32 * TM <= p.M && col_w + 32 * TN <= p.N) {
        // the wavefront's patch lies inside the matrix: branch-free write-out
        const long long first = (long long)(row_base + TM * 4 * lhi);
        store_patch_fast<TM, TN, true>(acc, out + first * ldo + col0, ldo, has_d ? dsrc + first * ldd + col0 : nullptr, ldd,
                                       alpha, beta, gamma, bv, act, p.ep.act_param);
    } else if (ws_or_c_vec && row_w + 32 * TM <= p.M && p.N % TN == 0) {
        // it sticks out over the right edge only, with every lane wholly inside or wholly outside: the same write-out
        // with the outside lanes switched off (a copy of its own, see store_accumulators_plain)
        if (col0 + TN <= p.N) {
            const long long first = (long long)(row_base + TM * 4 * lhi);
            store_patch_fast<TM, TN, true>(acc, out + first * ldo + col0, ldo, has_d ? dsrc + first * ldd + col0 : nullptr,
                                           ldd, alpha, beta, gamma, bv, act, p.ep.act_param);
        }
    } else if (row_w < p.M && col_w < p.N) {  // (a wavefront whose patch lies wholly outside the matrix writes nothing)
        // as in store_accumulators_plain: a copy of the loop without any load for beta == 0 and no addend, and one that
        // asks for the old values of C and the addend four rows at a time, outside the per-row conditions and from
        // addresses clamped into the matrix, so that no load stands between the stores
        auto rows = [&](auto with_old) {
        constexpr bool OLD = decltype(with_old)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int rc = 0; rc < 4; ++rc) {
                float cold[4][TN], dold[4][TN];
#pragma unroll
                for (int q = 0; q < (OLD ? 4 : 0); ++q) {
                    const int rq = row_base + TM * (8 * rc + 4 * lhi + q) + i;
                    const long long rcl = rq < p.M ? rq : p.M - 1;
                    if (beta != 0.0f) {  // uniform
                        if (vec_ok) {
                            load_row_vec<TN>(out + rcl * ldo + col0, cold[q]);
                        } else {
#pragma unroll
                            for (int j = 0; j < TN; ++j) cold[q][j] = out[rcl * ldo + (col0 + j < p.N ? col0 + j : p.N - 1)];
                        }
                    }
                    if (has_d) {  // uniform
                        if (vec_ok) {
                            load_row_vec<TN>(dsrc + rcl * ldd + col0, dold[q]);
                        } else {
#pragma unroll
                            for (int j = 0; j < TN; ++j) dold[q][j] = dsrc[rcl * ldd + (col0 + j < p.N ? col0 + j : p.N - 1)];
                        }
                    }
                }
                const int row0 = row_base + TM * (8 * rc + 4 * lhi) + i;
                float* const crow0 = out + (long long)row0 * ldo + col0;
#pragma unroll
                for (int r = 4 * rc; r < 4 * rc + 4; ++r) {
                    if (row0 + TM * (r % 4) >= p.M) continue;
                    float* crow = crow0 + (long long)(TM * (r % 4)) * ldo;
                    float v[TN];
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        v[j] = alpha * acc_value<(TM * TN >= 16)>(acc[i][j][r]) + bv[j];
                        if constexpr (OLD) {
                            if (beta != 0.0f) v[j] += beta * cold[r % 4][j];
                            if (has_d) v[j] += gamma * dold[r % 4][j];
                        }
                        if (act != ACT_NONE) v[j] = leaky_relu(v[j], p.ep.act_param);
                    }
                    if (vec_ok) {
                        store_row_vec<TN>(crow, v);
                    } else {
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            if (col0 + j < p.N) crow[j] = v[j];
                    }
                }
            }
        }
        };  // rows
        if (beta != 0.0f || has_d)  // uniform
            rows(std::true_type{});
        else
            rows(std::false_type{});
    }

    if (!to_ws) return;
    if (p.counters == nullptr) return;

    // ---- in-kernel split-K reduction by the last workgroup to arrive ----
    __shared__ int s_is_last;
    __threadfence();  // release: this thread's partial sums are visible device-wide
    __syncthreads();
    if (threadIdx.x == 0) {
        int* cnt = p.counters + (long long)batch * (p.tiles_m * p.tiles_n) + tile_index;
        const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        const int last = (old == p.splitk - 1);
        if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
        s_is_last = last;
    }
    __syncthreads();
    if (!s_is_last) return;
    __threadfence();  // acquire: the other workgroups' partial sums are visible to every thread here

    const long long mn = (long long)p.M * p.N;
    const float* wsb = p.ws + (long long)batch * p.splitk * mn;
    float bias_v[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) bias_v[j] = (p.ep.bias != nullptr && col0 + j < p.N) ? p.ep.bias[col0 + j] : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = row_base + TM * (8 * (r / 4) + 4 * lhi + (r % 4)) + i;
            if (row >= p.M) continue;
            const float* wrow = wsb + (long long)row * p.N + col0;
            float sum[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) sum[j] = 0.0f;
            for (int sidx = 0; sidx < p.splitk; ++sidx) {
                const float* w = wrow + (long long)sidx * mn;
                if (ws_vec) {
                    float t[TN];
                    load_row_vec<TN>(w, t);
#pragma unroll
                    for (int j = 0; j < TN; ++j) sum[j] += t[j];
                } else {
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        if (col0 + j < p.N) sum[j] += w[j];
                }
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) sum[j] *= p.alpha;
            finish_row<TN>(sum, Cb + (long long)row * p.ldc + col0,
                           Db != nullptr ? Db + (long long)row * p.ep.ldd + col0 : nullptr, Db != nullptr, bias_v,
                           p.beta, p.ep.gamma, p.ep.act, p.ep.act_param, c_vec, p.N - col0);
        }
    }
}

template <int TM, int TN, bool EXT>
__device__ __forceinline__ void store_accumulators(const f32x16 (&acc)[TM][TN], const GemmParams& p, int row_base,
                                                   int col0, int lhi, int zb, int batch, BatchIndex bi, int tile_index) {
    if constexpr (EXT)
        store_accumulators_ext<TM, TN>(acc, p, row_base, col0, lhi, zb, batch, bi, tile_index);
    else
        store_accumulators_plain<TM, TN>(acc, p, row_base, col0, lhi, zb, batch, tile_index);
}

template <int TM_, int TN_, int WM_, int WN_, int BK_>
struct TileCfg {
    static constexpr int TM = TM_, TN = TN_, WM = WM_, WN = WN_, BK = BK_;
    static constexpr int BM = TM * WM * 32, BN = TN * WN * 32;
    static constexpr int NT = WM * WN * 64;
    static constexpr int PA = BM + 4, PB = BN + 4;  // LDS row pitch in floats (== 4 mod 16)
    static constexpr int LDS_BYTES = 2 * BK * (PA + PB) * 4;
};

// EXT selects the extended write-out and the two-level batch.  An EXT kernel with transposed A and plain B can
// also produce colsum[m] = sum_k op(A)[m][k] (workgroups of tile column 0, from the A tiles they stage anyway):
// the Linear layer's bias gradient (sum of dy over the batch rows, Prod/CPU/CpuTensor.cs:1736-1740) when the
// product is dW = dy^T . x (Linear.cs:158-164).
template <class CFG, bool TA, bool TB, bool EXT = false>
__global__ void __launch_bounds__(CFG::NT) sgemm_mfma_kernel(const GemmParams p) {
    constexpr bool COLSUM = EXT && TA && !TB;
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

    WorkCoords wc = work_coords(blockIdx.x, p.tiles_m, p.tiles_n, p.nz, p.group_m);
    if constexpr (EXT) {
        if (p.flags & GEMM_FLAG_LONGEST_FIRST) wc = work_coords_longest_first(blockIdx.x, p.tiles_m, p.nz, p.group_m);
    }
    const int tile_m = wc.tile_m, tile_n = wc.tile_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int zb = wc.zb;  // batch * splitk + split
    int batch = zb, split = 0;
    if (p.splitk > 1) {
        batch = zb / p.splitk;
        split = zb - batch * p.splitk;
    }

    int kbeg = split * p.kchunk;
    const int kend = (kbeg + p.kchunk < p.K) ? (kbeg + p.kchunk) : p.K;
    if constexpr (EXT) {
        if (p.flags & GEMM_FLAG_K_FROM_M) {  // uniform
            const int k0 = (m0 / BK) * BK;
            if (k0 > kbeg) kbeg = k0;
        }
    }
    const int klen = kend - kbeg;  // may be <= 0 for a trailing empty split
    const int nk = (klen + BK - 1) / BK;
    const int nk_full = klen > 0 ? klen / BK : 0;

    BatchIndex bi = {0, batch};
    if constexpr (EXT) bi = split_batch(batch, p.batch_inner);
    const float* Ab = p.A + batch_offset(bi, p.strideA, p.strideA2);
    const float* Bb = p.B + batch_offset(bi, p.strideB, p.strideB2);

    const int m_rem = p.M - m0, n_rem = p.N - n0;  // > 0 by construction
    const bool full_mn = (m_rem >= BM) && (n_rem >= BN);

    StageA sa;
    StageB sb;
    sa.init(Ab, p.lda, m0, kbeg, tid);
    sb.init(Bb, p.ldb, n0, kbeg, tid);

    // COLSUM: all of a thread's A vectors cover the same four m (StageA is m-contiguous), one k row each;
    // every staged vector is added here on its way to LDS (tiles past the end of K are zeros).
    f32x4 cs = {0.0f, 0.0f, 0.0f, 0.0f};

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int a_off = wm * (TM * 32) + l32 * TM;
    const int b_off = wn * (TN * 32) + l32 * TN;
    constexpr int KS = BK / 2;                   // MFMA k steps per tile
    constexpr int NP = StageA::NV + StageB::NV;  // LDS store pieces per tile

    // NS register stages per operand (tile t lives in stage t % NS): while tile kt is multiplied out of LDS,
    // tile kt+1 sits in registers and is written to the other LDS buffer in small pieces between MFMAs, and
    // tiles kt+2 .. kt+NS are in flight from global memory.  Each piece's registers are refilled with tile
    // kt+1+NS right after they have been stored, so a global load has NS full tiles of MFMA work to land.
    // Two stages everywhere.  Four were measured for the 64-wide tiles (a tile lasts 512-1024 cycles there, less
    // than a memory latency): 1024 x 1024 x 2048 38.9 -> 37.0 us, but 1024^3 and 1000^3 unchanged or slower (five
    // tiles of prologue loads) and twice the registers (137 against 68: fewer co-resident workgroups).
    //
    // The k loop is one straight-line body of NS tiles with no special cases: tiles at or beyond the end of K are
    // fetched as zeros (no memory access), so a tile count that is not a multiple of two multiplies one tile of zeros.
    constexpr int NS = 2;
    f32x4 ra[NS][StageA::NV], rb[NS][StageB::NV];
    int fetch = 0;  // index of the k tile the stage pointers address; tiles are fetched in order

    // MFMA operand fragments: a ring of NB buffers over k steps, read D = NB-1 steps ahead of their use.
    // With one or two MFMAs per k step a single step (64-128 cycles) does not cover an LDS round trip, so
    // those configurations look three steps ahead.  The ring runs on across k tiles.
    constexpr int MT = TM * TN;           // MFMAs per k step
    constexpr int NB = (MT <= 2) ? 4 : 2;
    constexpr int D = NB - 1;
    static_assert(KS % NB == 0, "the fragment ring must divide the k steps of a tile");
    Frag<TM> fa[NB];
    Frag<TN> fb[NB];
    const float* const a_rd = As + lhi * PA + a_off;
    const float* const b_rd = Bs + lhi * PB + b_off;

    // Edge blocks: per-thread facts for branch-free loads of full-k tiles (see TileStage::Edge).  rot_a / rot_b: how
    // far this thread's vectors of an m/n-contiguous operand arrive shifted; zero when the extent is a multiple of 4
    // (then a vector is either wholly inside or wholly outside, and what lies outside may hold anything).
    // sh_a / sh_b [stage]: the shift of what the register stage currently holds (0: as loaded).
    //
    // Interior blocks and edge blocks run two disjoint copies of everything from here to the end of the k loop
    // (run<true> / run<false>): the edge facts then do not exist on the interior path at all.  With one copy they were
    // live across the interior loop (the edge loops are reachable from it as far as the compiler can tell), and in the
    // configurations that use all 512 registers they were spilled around it, in every block.
    auto run = [&](auto interior_tag) {
    constexpr bool INTERIOR = decltype(interior_tag)::value;
    typename StageA::Edge ea = {};
    typename StageB::Edge eb = {};
    if constexpr (!INTERIOR) {
        ea = sa.edge_info(m_rem, m0);
        eb = sb.edge_info(n_rem, n0);
    }
    const bool edge_ok = !INTERIOR && ea.usable && eb.usable;  // uniform over the workgroup
    // (StageA is k-contiguous when A is not transposed, StageB when B is: their vectors never arrive shifted)
    const bool any_rot_a = !INTERIOR && TA && (p.M % 4 != 0), any_rot_b = !INTERIOR && !TB && (p.N % 4 != 0);
    const int rot_a = any_rot_a ? ea.shift : 0, rot_b = any_rot_b ? eb.shift : 0;
    int sh_a[NS] = {}, sh_b[NS] = {};

    {
        // prologue: tile 0 -> stage 0 -> LDS buffer 0, tiles 1 .. NS-1 -> their stages, tile NS -> stage 0
#pragma unroll
        for (int t = 0; t <= NS; ++t) {
            const int st = t % NS;
            const int k_rem = klen - fetch * BK;
            sh_a[st] = 0;
            sh_b[st] = 0;
            if (INTERIOR && fetch < nk_full) {
                sa.load_fast(ra[st]);
                sb.load_fast(rb[st]);
            } else if (edge_ok && fetch < nk_full) {
#pragma unroll
                for (int v = 0; v < StageA::NV; ++v) sa.load_edge_vec(ra[st][v], v, ea);
#pragma unroll
                for (int v = 0; v < StageB::NV; ++v) sb.load_edge_vec(rb[st][v], v, eb);
                sh_a[st] = rot_a;
                sh_b[st] = rot_b;
            } else {
                sa.load_safe(ra[st], m_rem, k_rem);
                sb.load_safe(rb[st], n_rem, k_rem);
            }
            sa.advance();
            sb.advance();
            ++fetch;
            if (t == 0) {
#pragma unroll
                for (int v = 0; v < StageA::NV; ++v) {
                    if constexpr (INTERIOR) {
                        sa.store_lds_vec(As, ra[0][v], v);
                        if constexpr (COLSUM) cs += ra[0][v];
                    } else {
                        const f32x4 stored = sa.store_lds_vec_shifted(As, ra[0][v], v, sh_a[0], any_rot_a);
                        if constexpr (COLSUM) cs += stored;
                    }
                }
#pragma unroll
                for (int v = 0; v < StageB::NV; ++v) {
                    if constexpr (INTERIOR)
                        sb.store_lds_vec(Bs, rb[0][v], v);
                    else
                        sb.store_lds_vec_shifted(Bs, rb[0][v], v, sh_b[0], any_rot_b);
                }
            }
        }
        lds_barrier();
#pragma unroll
        for (int t = 0; t < D; ++t) {
            fa[t].load(a_rd + (2 * t) * PA);
            fb[t].load(b_rd + (2 * t) * PB);
        }
    }

    // The barrier of a tile sits behind the first MFMA of k step SB = KS - D.  By then this wavefront has
    // issued its last fragment read of the current LDS buffer (for step KS-1, issued at step SB-1) and all its
    // stores of the next tile; once every wavefront is past it, the next tile may be read - the look-ahead
    // reads of steps SB.. go there - and the current buffer may be overwritten by the tile after.
    constexpr int SB = KS - D;
    constexpr int G = SB * MT - (MT >= 2 ? MT / 2 : 1);  // MFMA slots that carry staging work: they end a little
                                                         // before the barrier so its wait finds the stores done
    constexpr int NW = 2 * NP;                           // staging work items per tile: (store, refill) per piece
    static_assert(G >= 1, "no MFMA slot left for staging");

    // One k tile.  P selects the LDS buffer read; the register stage P^1 holds the
    // next tile and is refilled, piece by piece, with tile `fetch`.
    // MODE 0: tile `fetch` is a full tile of an interior block (unchecked loads);
    // MODE 1: a full-k tile of an edge block (branch-free loads through the precomputed edge facts ea / eb);
    // MODE 2: the last tiles of an interior block (each fetch decides between unchecked loads and, at or past the
    //         end of K, checked ones);
    // MODE 3: the last tiles of an edge block (edge loads for full-k tiles, fully checked loads otherwise);
    // MODE 4: MODE 1 for a block none of whose vectors arrives shifted (M and N multiples of 4, or the operand is
    //         k-contiguous): plain LDS stores.  The element selects of the shifted store, executed for nothing, made
    //         the 64-wide-tile kernels VALU-bound in edge blocks (12 instructions per MFMA).
    // MODE 5 / 6: the last tiles of an interior / edge block, when no tile that is still to be multiplied remains to be
    //         fetched: the register stage is stored to LDS and not refilled.  Without any load in it the pair costs what
    //         a pair of the main loop costs (1361 cycles with 64 x 64 tiles); as a pair of MODE 2, whose every slot
    //         chooses between two kinds of load (of tiles beyond the end: zeros), it took 2361.
    // MODE 9: the very last tile of a block with an odd number of tiles: nothing is stored and nothing fetched
    //         (there is no tile after it; the tile of zeros that used to complete the last pair is no longer multiplied).
    // R: the register stage that holds the next tile (it is stored to LDS buffer P ^ 1 and refilled).
    auto k_tile = [&](auto parity, auto stage, auto mode, const typename StageA::Edge& ea,
                      const typename StageB::Edge& eb) {
        constexpr int P = decltype(parity)::value;
        constexpr int Q = P ^ 1;
        constexpr int R = decltype(stage)::value;
        constexpr int MODE = decltype(mode)::value;
        const bool fast = (MODE == 0) || (MODE == 2 && (fetch < nk_full));
        // the tail of an edge block: a full-k tile still takes the branch-free edge loads
        const bool edge_fast = (MODE == 3) && edge_ok && (fetch < nk_full);
        const int k_rem = klen - fetch * BK;
        // The stage stored in this tile holds the tile after this one.  Behind the last tile there is none: the tiles
        // that fetch nothing (MODE 5 / 6) left the stage as it was, and what it holds must not be summed again.
        const bool sum_stored = (MODE != 5 && MODE != 6) || (fetch - NS < nk);
        const float* as = a_rd + P * (BK * PA);
        const float* bs = b_rd + P * (BK * PB);
        float* const as_next = As + Q * (BK * PA);
        float* const bs_next = Bs + Q * (BK * PB);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int m = i * TN + j;      // MFMA slot inside the k step
                    const int gslot = s * MT + m;  // MFMA slot inside the tile
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s % NB].v[i], fb[s % NB].v[j], acc[i][j], 0, 0, 0);
                    // An MFMA occupies its SIMD's matrix pipe for 64 cycles and the wavefront cannot
                    // issue the next one earlier, so whatever is placed between two MFMAs is free
                    // as long as it issues within that shadow.  The non-MFMA work of a tile is
                    // therefore spread thinly over its MFMA slots (the fences pin it there):
                    __builtin_amdgcn_sched_barrier(0);
                    // - behind the first MFMA of a k step: the tile's barrier (step SB only) and the
                    //   LDS reads of the fragments needed D steps later, from this tile or the next;
                    if (m == 0) {
                        if (s == SB) {
                            sa.advance();
                            sb.advance();
                            ++fetch;
                            lds_barrier();
                        }
                        const int t = s + D;
                        if (t < KS) {
                            fa[t % NB].load(as + (2 * t) * PA);
                            fb[t % NB].load(bs + (2 * t) * PB);
                        } else {
                            fa[t % NB].load(a_rd + Q * (BK * PA) + (2 * (t - KS)) * PA);
                            fb[t % NB].load(b_rd + Q * (BK * PB) + (2 * (t - KS)) * PB);
                        }
                    }
                    // - the staging work items (store piece q to LDS, then refill its registers
                    //   from global memory), item w in slot w*G/NW;
                    if (MODE != 9 && gslot < G) {
#pragma unroll
                        for (int w = 0; w < NW; ++w) {
                            if ((w * G) / NW != gslot) continue;
                            const int q = w / 2;
                            const bool is_store = (w % 2 == 0);
                            if (q < StageA::NV) {
                                const int v = q < StageA::NV ? q : 0;
                                if (is_store) {
                                    if constexpr (MODE == 0 || MODE == 2 || MODE == 4 || MODE == 5) {
                                        sa.store_lds_vec(as_next, ra[R][v], v);
                                        if constexpr (COLSUM) {
                                            if (sum_stored) cs += ra[R][v];
                                        }
                                    } else {
                                        const f32x4 stored =
                                            sa.store_lds_vec_shifted(as_next, ra[R][v], v, sh_a[R], any_rot_a);
                                        if constexpr (COLSUM) {
                                            if (sum_stored) cs += stored;
                                        }
                                    }
                                } else if constexpr (MODE == 5 || MODE == 6) {
                                    // nothing left to fetch
                                } else if (MODE == 1 || MODE == 4 || edge_fast)
                                    sa.load_edge_vec(ra[R][v], v, ea);
                                else if (fast)
                                    sa.load_fast_vec(ra[R][v], v);
                                else
                                    sa.load_safe_vec(ra[R][v], v, m_rem, k_rem);
                            } else {
                                const int v = q >= StageA::NV ? q - StageA::NV : 0;
                                if (is_store) {
                                    if constexpr (MODE == 0 || MODE == 2 || MODE == 4 || MODE == 5)
                                        sb.store_lds_vec(bs_next, rb[R][v], v);
                                    else
                                        sb.store_lds_vec_shifted(bs_next, rb[R][v], v, sh_b[R], any_rot_b);
                                } else if constexpr (MODE == 5 || MODE == 6) {
                                    // nothing left to fetch
                                } else if (MODE == 1 || MODE == 4 || edge_fast)
                                    sb.load_edge_vec(rb[R][v], v, eb);
                                else if (fast)
                                    sb.load_fast_vec(rb[R][v], v);
                                else
                                    sb.load_safe_vec(rb[R][v], v, n_rem, k_rem);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        // what stage R holds now was fetched in this tile: remember whether it arrived shifted
        if constexpr (MODE == 1 || MODE == 3) {
            const bool via_edge = (MODE == 1) || edge_fast;
            sh_a[R] = via_edge ? rot_a : 0;
            sh_b[R] = via_edge ? rot_b : 0;
        }
    };

    // NS tiles in a row, starting at a tile index that is a multiple of NS (tile kt reads LDS buffer kt & 1, the
    // next tile sits in stage (kt + 1) % NS).  `limit`: tiles at or past it are skipped, in pairs (NS = 4 only).
    auto tiles = [&](auto mode, int first, int limit, auto mode_of_second) {
        using M = decltype(mode);
        using M2 = decltype(mode_of_second);
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        k_tile(I0{}, std::integral_constant<int, 1 % NS>{}, M{}, ea, eb);
        k_tile(I1{}, std::integral_constant<int, 2 % NS>{}, M2{}, ea, eb);
        if constexpr (NS == 4) {
            if (first + 2 >= limit) return;  // uniform
            k_tile(I0{}, std::integral_constant<int, 3>{}, M{}, ea, eb);
            k_tile(I1{}, std::integral_constant<int, 0>{}, M{}, ea, eb);
        }
    };
    constexpr int kNoLimit = 0x7fffffff;
    // a pair of tiles fetches the tiles NS + 1 and NS + 2 ahead of its first one; once the first of those fetches lies at
    // or beyond nk, nothing needs fetching any more
    static_assert(NS == 2, "the tail loops are written for pairs of tiles");
    // The 256 x 256 tiles, which use every register there is, keep one kind of pair for the whole tail (MODE 2 / 3): with
    // more kinds of pair the compiler spilled 1.2 KB per lane there.  (For the smaller tiles, too, the kinds of pair are
    // kept to a few ifs and loops in a row: chosen in nested branches, one case per shape of the end of K, they doubled
    // the accumulator registers and halved the number of blocks per CU.)
    constexpr bool SPLIT_TAIL = (TM * TN < 16);
    int kt = 0;
    // branch-free groups of NS tiles while all their fetches (tiles kt+NS+1 .. kt+2*NS) are full k tiles,
    // then the last few tiles (K tail included): same body, each fetch chooses checked or unchecked loads
    if constexpr (INTERIOR) {
        // All loads of the prologue are waited for here, once per block.  The compiler derives the wait counts in
        // front of the loop's LDS stores from the loads that may be in flight on any path into the loop; with the
        // prologue's loads among them (issued in an order of its own choosing, some under conditions) it made the
        // first store of every pass wait for ALL loads, including the ones issued a few MFMAs earlier, and the loop
        // ran at one memory latency per pair of tiles (64 x 64 tiles: 885 cycles per tile for 512 cycles of MFMAs).
        // With nothing in flight at the entry the counts are exact (all but the newest NS * NP - 1 loads).
        wait_for_all_loads();
        for (; kt + 2 * NS < nk_full; kt += NS) tiles(std::integral_constant<int, 0>{}, kt, kNoLimit, std::integral_constant<int, 0>{});
        if constexpr (SPLIT_TAIL) {
            // The pairs whose fetches reach the end of K (tiles at or beyond nk are not fetched: an odd number of tiles ends
            // with a tile on its own, below).  An even number of full tiles: the last tile is fetched by the first tile of
            // a pair whose second tile fetches nothing.
            if (kt + NS + 1 < nk_full && kt + 2 * NS >= nk) {
                tiles(std::integral_constant<int, 0>{}, kt, kNoLimit, std::integral_constant<int, 5>{});
                kt += NS;
            }
            // a partial tile at the end of K, fetched by the second tile of a pair (which chooses per fetch) ...
            for (; kt + NS + 2 < nk; kt += NS) tiles(std::integral_constant<int, 2>{}, kt, nk, std::integral_constant<int, 2>{});
            // ... or by the first tile of a pair
            if (kt + NS + 1 < nk) {
                tiles(std::integral_constant<int, 2>{}, kt, nk, std::integral_constant<int, 5>{});
                kt += NS;
            }
            // whole pairs that have nothing to fetch
            for (; kt + 1 < nk; kt += NS) tiles(std::integral_constant<int, 5>{}, kt, nk, std::integral_constant<int, 5>{});
            // an odd number of tiles: the last one by itself (it reads LDS buffer 0: its index is even)
            if (kt < nk)
                k_tile(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, 9>{}, ea, eb);
        } else {
            for (; kt < nk; kt += NS) tiles(std::integral_constant<int, 2>{}, kt, nk, std::integral_constant<int, 2>{});
        }
    } else {
        if (edge_ok && (any_rot_a || any_rot_b)) {  // uniform
            for (; kt + 2 * NS < nk_full; kt += NS) tiles(std::integral_constant<int, 1>{}, kt, kNoLimit, std::integral_constant<int, 1>{});
        } else if (edge_ok) {
            wait_for_all_loads();  // exact wait counts inside the loop, as for interior blocks
            for (; kt + 2 * NS < nk_full; kt += NS) tiles(std::integral_constant<int, 4>{}, kt, kNoLimit, std::integral_constant<int, 4>{});
        }
        if constexpr (SPLIT_TAIL) {
            // pairs whose first tile still has a tile to fetch, whole pairs that fetch nothing, and - an odd number of
            // tiles - the last tile by itself, as in interior blocks
            for (; kt + NS + 1 < nk; kt += NS) tiles(std::integral_constant<int, 3>{}, kt, nk, std::integral_constant<int, 3>{});
            for (; kt + 1 < nk; kt += NS) tiles(std::integral_constant<int, 6>{}, kt, nk, std::integral_constant<int, 6>{});
            if (kt < nk)
                k_tile(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, 9>{}, ea, eb);
        } else {
            for (; kt < nk; kt += NS) tiles(std::integral_constant<int, 3>{}, kt, nk, std::integral_constant<int, 3>{});
        }
    }
    };  // run
    if (full_mn)
        run(std::true_type{});
    else
        run(std::false_type{});

    if constexpr (COLSUM) {
        if (p.colsum != nullptr && tile_n == 0) {  // uniform over the workgroup
            // threads tid, tid + BM/4, ... hold partial sums of the same four m: add them in that order
            constexpr int GROUPS = BM / 4, LINES = NT / GROUPS;
            __syncthreads();  // every wavefront is done reading fragments from LDS
            float* red = smem;  // [LINES][BM]
            *reinterpret_cast<f32x4*>(red + (tid / GROUPS) * BM + (tid % GROUPS) * 4) = cs;
            __syncthreads();
            if (tid < BM && m0 + tid < p.M) {
                float t = 0.0f;
#pragma unroll
                for (int l = 0; l < LINES; ++l) t += red[l * BM + tid];
                p.colsum[(long long)batch * p.M + m0 + tid] = t;
            }
        }
    }

    store_accumulators<TM, TN, EXT>(acc, p, m0 + wm * (TM * 32), n0 + wn * (TN * 32) + TN * l32, lhi, zb, batch, bi,
                                    tile_m * p.tiles_n + tile_n);
}

}  // namespace snhip
