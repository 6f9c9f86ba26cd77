// bf16-input / fp32-accumulate GEMM for gfx950 built on v_mfma_f32_32x32x16_bf16.
//
// Same contract, launch geometry and epilogue as sgemm_mfma.hpp (row-major
// C = alpha*op(A)*op(B) + beta*C + bias over a strided batch; fp32 operands in
// global memory, fp32 C).  The operands are rounded to bf16 (round to nearest
// even, v_cvt_pk_bf16_f32) on their way from registers into LDS, products are
// accumulated in fp32.  The reference has no reduced-precision GEMM; this is
// the variant its benchmark description asks for next to the fp32 path.
//
// LDS layout.  The 32x32x16 MFMA wants 8 consecutive k per lane (lane l supplies
// A[l%32][8*(l/32) .. +7]), so tiles are kept "row-major": As[row][k] in bf16
// with a row pitch of BK+8 elements (an odd number of 16-byte chunks, so the 8
// lanes served per LDS cycle hit different banks).  Logical rows are interleaved
// across the TM (TN) MFMA tiles of a wavefront exactly as in the fp32 kernel
// (row TM*i+t <-> lane i of tile t, which gives each lane TN consecutive columns
// of C), but are stored de-interleaved: physical row = 32*t + i inside the
// wavefront's block of rows.  One ds_read_b128 then yields the 8 k values of one
// MFMA tile row, and both the fragment reads and the staging writes touch
// consecutive physical rows.
//
// Staging.  An operand contiguous along k is loaded as 16-byte vectors along k
// (4 floats -> 4 bf16 -> one ds_write_b64).  An operand contiguous along m/n is
// loaded as 4x4 blocks (4 k rows x 4 consecutive m/n, four 16-byte loads), which
// are transposed in registers for free: each of the 4 rows gets 4 consecutive k
// as one ds_write_b64.
//
// Operands stored as bf16 (TIN = __bf16).  The same kernel reads operands that are already bf16 in memory: a
// 16-byte vector then carries 8 elements, a k-contiguous vector goes to LDS unchanged (one ds_write_b128) and an
// m/n-contiguous operand is handled in units of 4 k rows x 8 columns, transposed in registers into eight
// ds_write_b64.  Half the bytes per element on the way from L2 into LDS is what this variant is for: with fp32
// storage a 256 x 256 tile needs the L2's whole bandwidth to feed the MFMAs at full rate.
#pragma once
#include "sgemm_mfma.hpp"

namespace snhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// logical row (interleaved over T tiles) -> physical LDS row (tile-major)
template <int T>
__device__ __forceinline__ constexpr int phys_row(int logical) {
    const int w = logical / (32 * T), r = logical % (32 * T);
    return w * (32 * T) + 32 * (r % T) + r / T;
}
template <int T>
__device__ __forceinline__ constexpr int logical_row(int phys) {
    const int w = phys / (32 * T), r = phys % (32 * T);
    return w * (32 * T) + T * (r % 32) + r / 32;
}

// Staging of one operand tile of logical shape [BMN rows (m or n)] x [BK (k)].
// T: MFMA tiles per wavefront along this dimension (row interleave factor).
// A "piece" is the unit the pipeline stores to LDS and refills from global
// memory in one go: one vector (KCONTIG) or one 4x4 block (otherwise).
template <int BMN, int BK, int NT, int PITCH, int T, bool KCONTIG, typename TIN = float>
struct BStage {
    static constexpr int EPV = 16 / (int)sizeof(TIN);   // elements per 16-byte vector: 4 (fp32 storage) or 8 (bf16)
    static constexpr int NV = (BK * BMN) / (EPV * NT);  // 16-byte vectors per thread
    static_assert((BK * BMN) % (EPV * NT) == 0, "tile must split evenly over threads");
    // KCONTIG: VPL vectors cover one row; thread = (vec, line); vector v -> physical row line + v*LINE_STEP
    static constexpr int VPL = BK / EPV;
    static constexpr int LINE_STEP = NT / VPL;
    // !KCONTIG: UPL units (4 k rows x EPV columns) cover one block of 4 k rows; thread = (g, kb);
    // unit u -> k block kb + u*KB_STEP
    static constexpr int UPL = BMN / EPV;
    static constexpr int KB_STEP = (NT >= UPL) ? NT / UPL : 1;
    static constexpr int NU = NV / 4;
    static constexpr int NPIECES = KCONTIG ? NV : NU;
    static constexpr int VEC_PER_PIECE = KCONTIG ? 1 : 4;
    // the logical row of vector v must separate into a per-thread part and a per-vector constant (see thread_row)
    static_assert(!KCONTIG || (NT % VPL == 0 && ((LINE_STEP <= 32 && 32 % LINE_STEP == 0) ||
                                                 (LINE_STEP % 32 == 0 && T % (LINE_STEP / 32) == 0))),
                  "unsupported k-contiguous split");
    static_assert(KCONTIG || (NV % 4 == 0 && NT % UPL == 0), "unsupported m/n-contiguous split");

    int line, k0;       // KCONTIG: physical row of vector 0, k offset of this thread's vectors
    int g, kb;          // !KCONTIG: group of EPV logical rows, k block of unit 0
    const TIN* gptr;    // address of vector 0 for the current k tile
    long long ld;

    __device__ __forceinline__ void init(const TIN* base, long long ld_, int tile_mn, int kbeg, int tid) {
        ld = ld_;
        if (KCONTIG) {
            k0 = (tid % VPL) * EPV;
            line = tid / VPL;
            gptr = base + (long long)(tile_mn + thread_row()) * ld + (kbeg + k0);
        } else {
            g = tid % UPL;
            kb = tid / UPL;
            gptr = base + (long long)(kbeg + 4 * kb) * ld + (tile_mn + EPV * g);
        }
    }
    __device__ __forceinline__ void advance() { gptr += KCONTIG ? (long long)BK : (long long)BK * ld; }

    // logical row of vector v (physical row line + v * LINE_STEP) is  row_const(v) + thread_row(): with
    // line = l + 32 * q the thread's part is T * l + q, and q + (tile index of v * LINE_STEP) never carries past T
    __device__ __forceinline__ static constexpr int row_const(int v) { return logical_row<T>(v * LINE_STEP); }
    __device__ __forceinline__ int thread_row() const { return T * (line % 32) + line / 32; }

    __device__ __forceinline__ const TIN* vec_ptr(int v) const {
        if (KCONTIG) return gptr + (long long)row_const(v) * ld;
        return gptr + (long long)(4 * (v / 4) * KB_STEP + (v % 4)) * ld;
    }

    __device__ __forceinline__ void load_fast_vec(f32x4& r, int v) const { __builtin_memcpy(&r, vec_ptr(v), 16); }

    // elements with m/n >= mn_rem or k >= k_rem (counted from the tile origin) read as zero, untouched in memory
    __device__ __forceinline__ void load_safe_vec(f32x4& r, int v, int mn_rem, int k_rem) const {
        const TIN* p = vec_ptr(v);
        int nval;
        if (KCONTIG) {
            // rows past the edge re-read the last valid row (their products are never stored)
            const int mn = row_const(v) + thread_row();
            if (mn >= mn_rem) p = gptr + (long long)(mn_rem - 1 - thread_row()) * ld;
            nval = k_rem - k0;
        } else {
            const int k = 4 * (kb + (v / 4) * KB_STEP) + (v % 4);
            nval = (k < k_rem) ? (mn_rem - EPV * g) : 0;
        }
        f32x4 x;
        if (nval >= EPV) {
            __builtin_memcpy(&x, p, 16);
        } else if constexpr (EPV == 4) {
            x.x = (nval > 0) ? p[0] : 0.0f;
            x.y = (nval > 1) ? p[1] : 0.0f;
            x.z = (nval > 2) ? p[2] : 0.0f;
            x.w = 0.0f;
        } else {
            // bf16 storage: the valid elements one by one as 16-bit words, the rest zero bits (= +0.0)
            const unsigned short* ps = reinterpret_cast<const unsigned short*>(p);
            unsigned int w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const unsigned int lo = (nval > 2 * e) ? ps[2 * e] : 0u;
                const unsigned int hi = (nval > 2 * e + 1) ? ps[2 * e + 1] : 0u;
                w[e] = lo | (hi << 16);
            }
            __builtin_memcpy(&x, w, 16);
        }
        r = x;
    }

    __device__ __forceinline__ void load_piece_fast(f32x4 (&r)[NV], int q) const {
#pragma unroll
        for (int i = 0; i < VEC_PER_PIECE; ++i) load_fast_vec(r[q * VEC_PER_PIECE + i], q * VEC_PER_PIECE + i);
    }
    __device__ __forceinline__ void load_piece_safe(f32x4 (&r)[NV], int q, int mn_rem, int k_rem) const {
#pragma unroll
        for (int i = 0; i < VEC_PER_PIECE; ++i)
            load_safe_vec(r[q * VEC_PER_PIECE + i], q * VEC_PER_PIECE + i, mn_rem, k_rem);
    }

    // round to bf16 and write piece q to the LDS tile s[row][k]
    __device__ __forceinline__ void store_piece(__bf16* s, const f32x4 (&r)[NV], int q) const {
        if constexpr (EPV == 8) {
            if (KCONTIG) {
                *reinterpret_cast<f32x4*>(s + (line + q * LINE_STEP) * PITCH + k0) = r[q];  // 8 k, already bf16
            } else {
                // 4 k rows x 8 columns -> 8 rows of 4 k
                const int kk = 4 * (kb + q * KB_STEP);
                bf16x8 in[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) __builtin_memcpy(&in[i], &r[4 * q + i], 16);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const bf16x4 h = {in[0][e], in[1][e], in[2][e], in[3][e]};
                    *reinterpret_cast<bf16x4*>(s + phys_row<T>(8 * g + e) * PITCH + kk) = h;
                }
            }
        } else if (KCONTIG) {
            const bf16x4 h = __builtin_convertvector(r[q], bf16x4);
            *reinterpret_cast<bf16x4*>(s + (line + q * LINE_STEP) * PITCH + k0) = h;
        } else {
            const int kk = 4 * (kb + q * KB_STEP);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const f32x4 col = {r[4 * q + 0][e], r[4 * q + 1][e], r[4 * q + 2][e], r[4 * q + 3][e]};
                const bf16x4 h = __builtin_convertvector(col, bf16x4);
                *reinterpret_cast<bf16x4*>(s + phys_row<T>(4 * g + e) * PITCH + kk) = h;
            }
        }
    }

    __device__ __forceinline__ void load_fast(f32x4 (&r)[NV]) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) load_fast_vec(r[v], v);
    }
    __device__ __forceinline__ void load_safe(f32x4 (&r)[NV], int mn_rem, int k_rem) const {
#pragma unroll
        for (int v = 0; v < NV; ++v) load_safe_vec(r[v], v, mn_rem, k_rem);
    }
    __device__ __forceinline__ void store_lds(__bf16* s, const f32x4 (&r)[NV]) const {
#pragma unroll
        for (int q = 0; q < NPIECES; ++q) store_piece(s, r, q);
    }
};

template <int TM_, int TN_, int WM_, int WN_, int BK_>
struct BTileCfg {
    static constexpr int TM = TM_, TN = TN_, WM = WM_, WN = WN_, BK = BK_;
    static constexpr int BM = TM * WM * 32, BN = TN * WN * 32;
    static constexpr int NT = WM * WN * 64;
    static constexpr int PITCH = BK + 8;  // bf16 elements; (2*BK+16)/16 is odd for BK a multiple of 16
    static constexpr int LDS_BYTES = 2 * (BM + BN) * PITCH * 2;
    static_assert(BK % 32 == 0, "BK must give an even number of 16-wide k steps");
};

// TIN: how A and B are stored in memory (float, rounded to bf16 on the way into LDS, or __bf16); with __bf16 the
// operand pointers of GemmParams point at bf16 data and leading dimensions / strides count bf16 elements.
template <class CFG, bool TA, bool TB, typename TIN = float>
__global__ void __launch_bounds__(CFG::NT) bgemm_mfma_kernel(const GemmParams p) {
    constexpr int TM = CFG::TM, TN = CFG::TN, WN = CFG::WN, BK = CFG::BK;
    constexpr int BM = CFG::BM, BN = CFG::BN, NT = CFG::NT, PITCH = CFG::PITCH;
    using StageA = BStage<BM, BK, NT, PITCH, TM, !TA, TIN>;
    using StageB = BStage<BN, BK, NT, PITCH, TN, TB, TIN>;

    extern __shared__ __attribute__((aligned(16))) float smem_f[];
    __bf16* const smem = reinterpret_cast<__bf16*>(smem_f);
    __bf16* const As = smem;                    // [2][BM][PITCH]
    __bf16* const Bs = smem + 2 * BM * PITCH;   // [2][BN][PITCH]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, lhi = lane >> 5;

    const WorkCoords wc = work_coords(blockIdx.x, p.tiles_m, p.tiles_n, p.nz, p.group_m);
    const int tile_m = wc.tile_m, tile_n = wc.tile_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int zb = wc.zb;
    int batch = zb, split = 0;
    if (p.splitk > 1) {
        batch = zb / p.splitk;
        split = zb - batch * p.splitk;
    }

    const int kbeg = split * p.kchunk;
    const int kend = (kbeg + p.kchunk < p.K) ? (kbeg + p.kchunk) : p.K;
    const int klen = kend - kbeg;
    const int nk = (klen + BK - 1) / BK;
    const int nk_full = klen / BK;

    const TIN* Ab = reinterpret_cast<const TIN*>(p.A) + (long long)batch * p.strideA;
    const TIN* Bb = reinterpret_cast<const TIN*>(p.B) + (long long)batch * p.strideB;
    const int m_rem = p.M - m0, n_rem = p.N - n0;
    const bool full_mn = (m_rem >= BM) && (n_rem >= BN);

    StageA sa;
    StageB sb;
    sa.init(Ab, p.lda, m0, kbeg, tid);
    sb.init(Bb, p.ldb, n0, kbeg, tid);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    constexpr int KS = BK / 16;                                  // MFMA k steps per tile (even)
    constexpr int MT = TM * TN;                                  // MFMAs per k step
    constexpr int NF = TM + TN;                                  // fragment reads per k step
    constexpr int NP = StageA::NPIECES + StageB::NPIECES;        // staging pieces per tile
    constexpr int MID = MT / 2;                                  // barrier slot in the last k step
    constexpr int G = (KS - 1) * MT + MID;                       // MFMA slots that carry staging pieces

    // Same pipeline as the fp32 kernel: tile kt in LDS buffer kt&1, tile kt+1 in
    // register stage (kt+1)&1, tile kt+2 in flight; pieces of tile kt+1 are written
    // to the other LDS buffer between MFMAs and their registers refilled with tile
    // kt+3.  MFMAs here are 32 cycles long, so the side work is spread over every
    // MFMA slot rather than only behind the first MFMA of a k step.
    f32x4 ra[2][StageA::NV], rb[2][StageB::NV];
    int fetch = 0;
    bf16x8 fa[2][TM], fb[2][TN];
    // physical row of this lane in tile t is  wave block + 32*t + l32
    const __bf16* const a_rd = As + (wm * (TM * 32) + l32) * PITCH + 8 * lhi;
    const __bf16* const b_rd = Bs + (wn * (TN * 32) + l32) * PITCH + 8 * lhi;

    // fragment read f (0..NF-1) of k step s from LDS buffer `buf` into fragment buffer fbuf
    auto read_frag = [&](int f, int s, int buf, int fbuf) {
        if (f < TM)
            fa[fbuf][f < TM ? f : 0] =
                *reinterpret_cast<const bf16x8*>(a_rd + buf * (BM * PITCH) + (32 * f) * PITCH + 16 * s);
        else
            fb[fbuf][f >= TM ? f - TM : 0] =
                *reinterpret_cast<const bf16x8*>(b_rd + buf * (BN * PITCH) + (32 * (f - TM)) * PITCH + 16 * s);
    };

    {
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            const int st = (t == 1) ? 1 : 0;
            const int k_rem = klen - fetch * BK;
            if (full_mn && fetch < nk_full) {
                sa.load_fast(ra[st]);
                sb.load_fast(rb[st]);
            } else {
                sa.load_safe(ra[st], m_rem, k_rem);
                sb.load_safe(rb[st], n_rem, k_rem);
            }
            sa.advance();
            sb.advance();
            ++fetch;
            if (t == 0) {
                sa.store_lds(As, ra[0]);
                sb.store_lds(Bs, rb[0]);
            }
        }
        lds_barrier();
#pragma unroll
        for (int f = 0; f < NF; ++f) read_frag(f, 0, 0, 0);
    }

    auto k_tile = [&](auto parity, auto steady) {
        constexpr int P = decltype(parity)::value;
        constexpr int Q = P ^ 1;
        const bool fast = decltype(steady)::value || (full_mn && (fetch < nk_full));
        const int k_rem = klen - fetch * BK;
        __bf16* const as_next = As + Q * (BM * PITCH);
        __bf16* const bs_next = Bs + Q * (BN * PITCH);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int m = i * TN + j;      // MFMA slot inside the k step
                    const int gslot = s * MT + m;  // MFMA slot inside the tile
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[s & 1][i], fb[s & 1][j], acc[i][j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    // fragments of the next k step, spread over this step's slots
                    if (s + 1 < KS) {
#pragma unroll
                        for (int f = 0; f < NF; ++f)
                            if (f >= (m * NF) / MT && f < ((m + 1) * NF) / MT) read_frag(f, s + 1, P, (s + 1) & 1);
                    }
                    // staging pieces of the next tile, each followed by the refill of its registers
                    if (gslot < G) {
#pragma unroll
                        for (int q = 0; q < NP; ++q) {
                            if (q < (gslot * NP) / G || q >= ((gslot + 1) * NP) / G) continue;
                            if (q < StageA::NPIECES) {
                                const int qa = q < StageA::NPIECES ? q : 0;
                                sa.store_piece(as_next, ra[Q], qa);
                                if (fast)
                                    sa.load_piece_fast(ra[Q], qa);
                                else
                                    sa.load_piece_safe(ra[Q], qa, m_rem, k_rem);
                            } else {
                                const int qb = q >= StageA::NPIECES ? q - StageA::NPIECES : 0;
                                sb.store_piece(bs_next, rb[Q], qb);
                                if (fast)
                                    sb.load_piece_fast(rb[Q], qb);
                                else
                                    sb.load_piece_safe(rb[Q], qb, n_rem, k_rem);
                            }
                        }
                    }
                    if (s + 1 == KS) {
                        if (m == MID) {
                            sa.advance();
                            sb.advance();
                            ++fetch;
                            lds_barrier();
                        }
                        // first fragments of the next tile, spread over the slots behind the barrier
                        if (m >= MID) {
#pragma unroll
                            for (int f = 0; f < NF; ++f)
                                if (f >= ((m - MID) * NF) / (MT - MID) && f < ((m - MID + 1) * NF) / (MT - MID))
                                    read_frag(f, 0, Q, 0);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    int kt = 0;
    if (full_mn) {
        wait_for_all_loads();  // makes the wait counts inside the loop exact (see the fp32 kernel)
        for (; kt + 4 < nk_full; kt += 2) {
            k_tile(P0{}, std::true_type{});
            k_tile(P1{}, std::true_type{});
        }
    }
    for (; kt < nk; kt += 2) {
        k_tile(P0{}, std::false_type{});
        k_tile(P1{}, std::false_type{});
    }

    // Reading the full-size accumulator set through pinned accumulation registers (see acc_value) pays with
    // bf16 storage only: with fp32 storage the k loop needs every ordinary register, and the allocation the
    // pinned write-out leads to puts spill reloads inside that loop (8192^3: 725 against 924 TFLOP/s).
    constexpr bool PIN = (TM * TN >= 16) && (sizeof(TIN) == 2);
    store_accumulators_plain<TM, TN, PIN>(acc, p, m0 + wm * (TM * 32), n0 + wn * (TN * 32) + TN * l32, lhi, zb, batch,
                                          tile_m * p.tiles_n + tile_n);
}

}  // namespace snhip
