// Regularised normal equations (Z^T Z + lambda I) alpha = Z^T y: fp64 Cholesky factorisation
// A = U^T U of the symmetric positive definite matrix, in place in the upper triangle, and the
// two triangular solves.  The reference calls torch.linalg.solve (LU) at this point
// (qml_lightning/models/kernel.py:226-234).
//
// Row-major A with row stride ld, 128-column blocks grouped in panels of 512 rows.  Per block k:
//   1. the block's 128 rows (columns k..F) take the product of the panel's rows above them
//      (fp64 MFMA tile product, depth up to 384);
//   2. one workgroup factors the 128x128 diagonal block in registers and also produces the
//      inverse of the factor (both orientations, kept for the solves);
//   3. U12 = U11^-T A12 as a product with that inverse on the same MFMA tiles.
// After a panel, the trailing matrix takes A22 -= U12^T U12 (512 rows deep) on the tiles on or
// above the diagonal.  The depth of 512 is what makes the trailing update MFMA-bound: at a
// depth of 128 the read-modify-write of the trailing matrix dominates.
// For whole tiles (F a multiple of 128) a panel and the trailing update of the panel before it are ONE
// launch (panel_kernel below); any other F takes a launch per step with the tile kernel of gram.hip.
// Only elements on or above the diagonal are read; below the diagonal only the lower halves of
// the 128x128 diagonal tiles are overwritten.  Flops: F^3/3.
#include <type_traits>
#include <utility>

#include "qmll_common.h"
#include "gram_tiles.h"

// gram.hip: tiles on/above the diagonal of C[n,n] (row stride ldc) += sign * Z^T Z, Z = M rows
// of n columns with row stride ldz
int qmll_internal_syrk_upper(const double* Z, int M, int n, long long ldz, double* C, long long ldc, double sign,
                             hipStream_t stream);
// gram.hip: C[ra,n] = or += sign * Za^T Zb, Za = M x ra (row stride lda), Zb = M x n (row stride ldb)
int qmll_internal_gemm_tn(const double* Za, long long lda, int ra, const double* Zb, long long ldb, int n, int M,
                          double* C, long long ldc, double sign, int overwrite, hipStream_t stream);

namespace {

constexpr int NB = 128;       // block edge
constexpr int OB = 512;       // panel depth of the trailing update
constexpr int PT = 512;           // threads of a factorisation workgroup (and of the tile product's eight wavefronts)
constexpr int SB = 16;            // sub-block edge of the diagonal-block factorisation (one fp64 MFMA tile)
constexpr int NSB = NB / SB;      // sub-blocks per edge
constexpr int NSUB = NSB * (NSB + 1) / 2;     // sub-blocks on or above (or on or below) the diagonal
constexpr int MWAVES = PT / 64 - 1;           // wavefronts that hold sub-blocks; wavefront 0 factors the diagonal ones
constexpr int NSLOT = (2 * NSUB + MWAVES - 1) / MWAVES;
constexpr int SSTRIDE = NB + 16;  // doubles per row of a 16-row strip in LDS (rows 32 banks apart, see gram.hip)
constexpr int DSTRIDE = SB + 1;

typedef double double4_t __attribute__((ext_vector_type(4)));

// LDS of the diagonal-block factorisation, 41 KB
struct PotrfShared {
    double ustrip[SB][SSTRIDE];   // block row K of U
    double wstrip[SB][SSTRIDE];   // block row K of W = L^-1
    double dblk[SB][DSTRIDE];     // the diagonal sub-block about to be factored
    double vblk[SB][DSTRIDE];     // the inverse of its factor
    int failed;
};

__device__ __forceinline__ double value_of_lane(double v, int lane) {
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)b, lane);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(b >> 32), lane);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// Sub-block t of the list the wavefronts 1..7 are dealt their register slots from (wavefront w holds
// t = 7 s + w - 1 in slot s): first the 36 sub-blocks of S on or above the diagonal, row by row, then the
// 36 of W on or below it.  kind 0: S, 1: W.
struct SubId {
    int kind, i, j;
};
constexpr SubId sub_id(int t) {
    SubId b{t >= NSUB ? 1 : 0, 0, 0};
    int u = b.kind ? t - NSUB : t;
    if (!b.kind) {
        while (u >= NSB - b.i) { u -= NSB - b.i; ++b.i; }
        b.j = b.i + u;
    } else {
        while (u >= b.i + 1) { u -= b.i + 1; ++b.i; }
        b.j = u;
    }
    return b;
}

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>); the second form stops at the first false
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}
template <class F, int... Is>
__device__ __forceinline__ bool static_all_impl(F& f, std::integer_sequence<int, Is...>) {
    return (f(std::integral_constant<int, Is>{}) && ...);
}
template <int N, class F>
__device__ __forceinline__ bool static_all(F&& f) {
    return static_all_impl(f, std::make_integer_sequence<int, N>{});
}

// Factor the nb x nb block at (k0,k0) (nb <= 128; the rest is padded with the identity) and invert the factor.
// Blocked right-looking Cholesky on 16 x 16 sub-blocks, S = U^T U, with the same block operations applied to
// the identity: W = L^-1 = U^-T.  The sub-blocks live in registers in the accumulator layout of
// v_mfma_f64_16x16x4_f64 (register r of a lane: row lane/16 + 4r, column lane%16), which is also the layout
// of both operands (row = the summed index), so a sub-block feeds the matrix pipe as it stands.  Wavefronts
// 1..7 hold the 72 sub-blocks, up to eleven each; which ones is fixed at compile time (one instance of the code
// per wavefront), so a finished sub-block's registers are free again and no index is computed at run time.
// Wavefront 0 holds none and does the serial part.  Step K of eight:
//   1. the owner of S(K,K) puts it into LDS; wavefront 0 factors it, a lane per column: sixteen pivots, each
//      a reciprocal square root and the pivot row handed round with v_readlane, no barrier and no LDS inside;
//      the same row operations on the identity give V = U_KK^-1;
//   2. block row K: U(K,J) = V^T S(K,J), W(K,J) = V^T W(K,J), four MFMAs each, to LDS and to memory;
//   3. S(I,J) -= U(K,I)^T U(K,J) and W(I,J) -= U(K,I)^T W(K,J) for the rows I > K.
// 24 barriers instead of the 128 of an elimination pivot by pivot, and the multiply-adds on the matrix pipe.
// Output: upper triangle of the block <- U11; inv[m*128+i] = U11^-1[m,i] = W[i,m]; invT[i*128+m] the same.
// info: 0, or 1 + the index of the first pivot that is not positive (later launches then exit).

// inv[m, 16 K + i] = W[16 K + i, m] for the columns m of block row K, from the strip in LDS: thread = (m, half a
// row of sixteen), 64 contiguous bytes each
__device__ __forceinline__ void store_inverse_columns(int K, double* inv, const PotrfShared& ps) {
    const int m = (int)threadIdx.x >> 1, half = (int)threadIdx.x & 1;
    if (m < (K + 1) * SB) {
#pragma unroll
        for (int q = 0; q < SB / 2; ++q) inv[m * NB + K * SB + half * (SB / 2) + q] = ps.wstrip[half * (SB / 2) + q][m];
    }
}

// wavefront 0: the diagonal sub-blocks, one after the other
__device__ __forceinline__ bool potrf_factor_wave(double* blk, long long ld, int k0, int nb, double* inv, int* info,
                                                  PotrfShared& ps) {
    const int lane = (int)threadIdx.x & 63, l16 = lane & 15;
    for (int K = 0; K < NSB; ++K) {
        __syncthreads();                                               // S(K,K) is in LDS
        // column l16 of the sub-block in d, row l16 of V in w (the four groups of sixteen lanes hold copies)
        double d[SB], w[SB];
#pragma unroll
        for (int i = 0; i < SB; ++i) {
            d[i] = ps.dblk[i][l16];
            w[i] = i == l16 ? 1.0 : 0.0;
        }
        int bad = -1;                                                  // the first pivot that is not positive
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            double piv = value_of_lane(d[j], j);                       // the same value in every lane
            if (!(piv > 0.0)) {
                bad = bad < 0 ? j : bad;
                piv = 1.0;
            }
            // 1/sqrt by the hardware estimate and two Newton steps
            double y = __builtin_amdgcn_rsq(piv);
            const double h = 0.5 * piv;
            y = fma(y, fma(-h * y, y, 0.5), y);
            y = fma(y, fma(-h * y, y, 0.5), y);
            const double u = d[j] * y;                                 // U[j, l16]
            const double wj = w[j] * y;                                // W[j, l16]
            d[j] = u;
            w[j] = wj;
#pragma unroll
            for (int i = j + 1; i < SB; ++i) {
                const double ui = value_of_lane(u, i);                 // U[j, i] = L[i, j]
                d[i] = fma(-ui, u, d[i]);
                w[i] = fma(-ui, wj, w[i]);
                // pins the update to this step (no instruction is emitted): nothing needs w before the end, so
                // left alone the compiler computes all of it there and carries every multiplier of every step
                // in scalar registers it does not have
                asm volatile("" : "+v"(w[i]));
            }
        }
        if (bad >= 0 && lane == 0) {
            *info = k0 + K * SB + bad + 1;
            ps.failed = 1;
        }
        // (every lane stores: the four copies write the same values)
#pragma unroll
        for (int i = 0; i < SB; ++i) {
            ps.vblk[l16][i] = w[i];                                    // V[c, i] = W[i, c]
            const int row = K * SB + i, col = K * SB + l16;
            if (lane < SB && i <= l16 && col < nb) blk[(size_t)row * ld + col] = d[i];
        }
        __syncthreads();                                               // V is in LDS
        if (ps.failed) return false;
        __syncthreads();                                               // block row K is in LDS
        store_inverse_columns(K, inv, ps);
    }
    return true;
}

// wavefront WV = 1..7: its share of the sub-blocks
template <int WV>
__device__ __forceinline__ bool potrf_mfma_wave(double* blk, long long ld, int nb, double* inv, double* invT,
                                                PotrfShared& ps) {
    const int lane = (int)threadIdx.x & 63, l16 = lane & 15, lk = lane >> 4;
    const int ldi = (int)ld;
    // per-lane parts of every address; what is added per sub-block is a constant
    double* const blk_lane = blk + (size_t)lk * ld + l16;
    double* const invT_lane = invT + lk * NB + l16;
    double* const us_lane = &ps.ustrip[lk][l16];
    double* const ws_lane = &ps.wstrip[lk][l16];
    double4_t sub[NSLOT];
    static_for<NSLOT>([&](auto s_) {
        constexpr int s = decltype(s_)::value, t = s * MWAVES + WV - 1;
        if constexpr (t < 2 * NSUB) {
            constexpr SubId b = sub_id(t);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = b.i * SB + lk + 4 * r, col = b.j * SB + l16;
                if constexpr (b.kind == 0) {
                    const int lo = row < col ? row : col, hi = row < col ? col : row;
                    // (32-bit offsets: 128 rows of at most 2^23 doubles)
                    sub[s][r] = hi < nb ? blk[(unsigned)(lo * ldi + hi)] : (row == col ? 1.0 : 0.0);
                } else {
                    sub[s][r] = row == col ? 1.0 : 0.0;
                }
            }
        }
    });
    return static_all<NSB>([&](auto K_) -> bool {
        constexpr int K = decltype(K_)::value;
        static_for<NSLOT>([&](auto s_) {
            constexpr int s = decltype(s_)::value, t = s * MWAVES + WV - 1;
            if constexpr (t < 2 * NSUB) {
                constexpr SubId b = sub_id(t);
                if constexpr (b.kind == 0 && b.i == K && b.j == K) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) ps.dblk[lk + 4 * r][l16] = sub[s][r];
                }
            }
        });
        __syncthreads();                                               // S(K,K) is in LDS
        __syncthreads();                                               // wavefront 0 has factored it: V is in LDS
        if (ps.failed) return false;
        double va[4];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) va[kk] = ps.vblk[4 * kk + lk][l16];
        static_for<NSLOT>([&](auto s_) {
            constexpr int s = decltype(s_)::value, t = s * MWAVES + WV - 1;
            if constexpr (t < 2 * NSUB) {
                constexpr SubId b = sub_id(t);
                if constexpr (b.i == K && (b.kind == 1 || b.j > K)) {
                    double4_t res = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk)
                        res = __builtin_amdgcn_mfma_f64_16x16x4f64(va[kk], sub[s][kk], res, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if constexpr (b.kind == 0) {
                            us_lane[4 * r * SSTRIDE + b.j * SB] = res[r];
                            if (b.j * SB + l16 < nb && K * SB + lk + 4 * r < nb)
                                blk_lane[(size_t)(K * SB + 4 * r) * ld + b.j * SB] = res[r];
                        } else {
                            ws_lane[4 * r * SSTRIDE + b.j * SB] = res[r];
                            invT_lane[(K * SB + 4 * r) * NB + b.j * SB] = res[r];
                        }
                    }
                }
            }
        });
        __syncthreads();                                               // block row K is in LDS
        store_inverse_columns(K, inv, ps);
        static_for<NSLOT>([&](auto s_) {
            constexpr int s = decltype(s_)::value, t = s * MWAVES + WV - 1;
            if constexpr (t < 2 * NSUB) {
                constexpr SubId b = sub_id(t);
                if constexpr (b.i > K && (b.kind == 0 || b.j <= K)) {
                    const double* right = b.kind == 0 ? us_lane : ws_lane;
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) {
                        const double fa = -us_lane[4 * kk * SSTRIDE + b.i * SB];
                        const double fb = right[4 * kk * SSTRIDE + b.j * SB];
                        sub[s] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa, fb, sub[s], 0, 0, 0);
                    }
                }
            }
        });
        return true;
    });
}

// Called by all PT threads of the workgroup.  False when a pivot is not positive (info is then set).
__device__ __forceinline__ bool potrf_block(double* A, long long ld, int k0, int nb, double* inv, double* invT,
                                            int* info, PotrfShared& ps) {
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    double* blk = A + (size_t)k0 * ld + k0;
    // the sub-blocks of inv / invT that stay zero (the others are written when their block row is final)
    for (int e = tid; e < (NSUB - NSB) * SB * SB; e += PT) {
        int b = e / (SB * SB), I = 0;
        const int r = (e / SB) % SB, c = e % SB;
        while (b >= NSB - 1 - I) { b -= NSB - 1 - I; ++I; }
        const int J = I + 1 + b;                                  // I < J
        invT[(I * SB + r) * NB + J * SB + c] = 0.0;
        inv[(J * SB + r) * NB + I * SB + c] = 0.0;
    }
    if (tid == 0) ps.failed = 0;
    bool ok;
    switch (wave) {
        case 0: ok = potrf_factor_wave(blk, ld, k0, nb, inv, info, ps); break;
        case 1: ok = potrf_mfma_wave<1>(blk, ld, nb, inv, invT, ps); break;
        case 2: ok = potrf_mfma_wave<2>(blk, ld, nb, inv, invT, ps); break;
        case 3: ok = potrf_mfma_wave<3>(blk, ld, nb, inv, invT, ps); break;
        case 4: ok = potrf_mfma_wave<4>(blk, ld, nb, inv, invT, ps); break;
        case 5: ok = potrf_mfma_wave<5>(blk, ld, nb, inv, invT, ps); break;
        case 6: ok = potrf_mfma_wave<6>(blk, ld, nb, inv, invT, ps); break;
        default: ok = potrf_mfma_wave<7>(blk, ld, nb, inv, invT, ps); break;
    }
    if (!ok) return false;                                        // every wavefront saw the same flag
    __syncthreads();
    return true;
}

__global__ __launch_bounds__(PT, 4) void potrf_block_kernel(double* A, long long ld, int k0, int nb, double* inv,
                                                         double* invT, int* info) {
    __shared__ PotrfShared ps;
    if (*info != 0) return;
    potrf_block(A, ld, k0, nb, inv, invT, info, ps);
}

// ---- one launch per panel -------------------------------------------------------------------
//
// Steps 1-3 above are eleven dependent launches per panel, each of at most F/128 workgroups and a few
// tens of microseconds, and the trailing update that follows has to wait for them.  For whole 128-column
// tiles a panel is one launch instead, and that launch also carries the trailing update of the panel
// before it.
//
// Column owners.  Workgroup w < (F - P0) / 128 owns the column of tiles w of the panel's rows (columns
// P0 + 128 w ...).  It first gives its tiles the update of the previous panel (rows R0 .. P0 of the
// factor, already final: the part of that panel's trailing update that falls into this panel's rows),
// then walks down its column:
//     wait for "block l factored";  tile(l, w) = U11_l^-T tile(l, w)                      row strip
//     for the block rows b > l of its column: wait for "strip (l, b) done";
//                                              tile(b, w) -= tile(l, b)^T tile(l, w)      update, 128 deep
// and the owner of column l, which reaches its diagonal tile with every update applied, factors it and
// publishes the inverse.  A workgroup only ever waits for owners of columns left of its own, which have
// lower workgroup ids; ids are dispatched in order, so whoever is waited for is running or done,
// whatever the number of workgroups resident at a time.  Every wait is bounded all the same: a wait that
// runs out sets info to -1 and the workgroup leaves.
//
// Head tiles.  Once the trailing matrix is small a launch lasts as long as its slowest owner, and four of an
// owner's fourteen tile products are that first update.  The host then puts workgroups for those tiles in
// front of the owners (one per tile, waiting for nobody); each counts itself into its column's counter
// when done, and an owner starts by waiting for its column's count.
//
// Trailing tiles.  The workgroups after the owners (their count rounded up to a multiple of eight, so
// that the XCD of a tile is what gram_tiles.h deals) take the previous panel's update of the tiles
// on or above the diagonal below this panel, 512 deep, and wait for nobody.  While the panel's chain of
// dependent steps (four factorisations, each waiting for the strip before it) runs on a few CUs, the rest
// of the chip is busy with these.
constexpr int PKB = 16;                 // rows staged per step
constexpr int PSTRIDE = NB + 16;        // doubles per staged row (see gram.hip)
constexpr int P_TPR = PT / PKB;         // threads per staged row
constexpr int P_CPT = NB / P_TPR;       // doubles per thread and row
constexpr int P_UN = P_CPT / 2;         // 16-byte units per thread
constexpr unsigned FLAG_DONE = 1u, FLAG_FAILED = 0x80000000u;   // (a counter never gets near the second)
constexpr int PBLK = OB / NB;                        // blocks per panel
constexpr int FLAGS_PER_PANEL = PBLK + PBLK * PBLK;  // "block l factored": [l]; "strip (l, b) done": [PBLK + l PBLK + b]
constexpr int SPLIT_HEADS_BELOW = 48;       // trailing tiles per edge
constexpr unsigned SPIN_LIMIT = 1u << 21;   // polls of about a microsecond each before a wait gives up

typedef double double2_t __attribute__((ext_vector_type(2)));

struct TileShared {
    double a[2][PKB][PSTRIDE], b[2][PKB][PSTRIDE];
};

// The 128 x 128 tile at C (row stride ldc) = or += sign * Za^T Zb, Za and Zb `depth` rows (a multiple of 16) of 128
// columns; the tile product of gram.hip for whole tiles (same staging, same MFMA order).  C may be Zb
// (depth 128, overwrite): everything is read before anything is written.  Ends with a barrier.
__device__ __forceinline__ void tile_product(const double* Za, long long lda, const double* Zb, long long ldb,
                                             int depth, double* C, long long ldc, double sign, bool overwrite,
                                             TileShared& sm) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave / 4) * 64, wj = (wave % 4) * 32;
    const int l16 = lane & 15, lk = lane >> 4;
    double4_t acc[4][2];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 2; ++q) acc[p][q] = (double4_t){0.0, 0.0, 0.0, 0.0};
    const int lr = tid / P_TPR, lc = (tid % P_TPR) * P_CPT;
    double2_t ra[P_UN], rb[P_UN];
    auto load_panels = [&](int m0) {
        const double2_t* pa = reinterpret_cast<const double2_t*>(Za + (size_t)(m0 + lr) * lda + lc);
        const double2_t* pb = reinterpret_cast<const double2_t*>(Zb + (size_t)(m0 + lr) * ldb + lc);
#pragma unroll
        for (int q = 0; q < P_UN; ++q) ra[q] = pa[q];
#pragma unroll
        for (int q = 0; q < P_UN; ++q) rb[q] = pb[q];
    };
    auto store_panels = [&](int buf) {
        double2_t* da = reinterpret_cast<double2_t*>(&sm.a[buf][lr][lc]);
        double2_t* db = reinterpret_cast<double2_t*>(&sm.b[buf][lr][lc]);
#pragma unroll
        for (int q = 0; q < P_UN; ++q) da[q] = ra[q];
#pragma unroll
        for (int q = 0; q < P_UN; ++q) db[q] = rb[q];
    };
    const int nsteps = depth / PKB;
    load_panels(0);
    store_panels(0);
    __syncthreads();
#pragma unroll 1
    for (int step = 0; step < nsteps; ++step) {
        const int cur = step & 1;
        if (step + 1 < nsteps) load_panels((step + 1) * PKB);   // in flight during the MFMAs
#pragma unroll
        for (int kk = 0; kk < PKB; kk += 4) {
            double fa[4], fb[2];
#pragma unroll
            for (int p = 0; p < 4; ++p) fa[p] = sm.a[cur][kk + lk][wi + p * 16 + l16];
#pragma unroll
            for (int q = 0; q < 2; ++q) fb[q] = sm.b[cur][kk + lk][wj + q * 16 + l16];
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int q = 0; q < 2; ++q)
                    acc[p][q] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[p], fb[q], acc[p][q], 0, 0, 0);
        }
        if (step + 1 < nsteps) store_panels(cur ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                double* c = C + (size_t)(wi + p * 16 + lk + 4 * r) * ldc + wj + q * 16 + l16;
                const double v = sign * acc[p][q][r];
                // (the sum is left to the memory side: no wait for the old value; every element of C takes
                // exactly one addition per launch, so the result does not depend on any order)
                if (overwrite) *c = v;
                else unsafeAtomicAdd(c, v);
            }
    __syncthreads();
}

// every store of the workgroup so far becomes visible to the device, then the flag is set / counted up
__device__ __forceinline__ void publish(unsigned* flag, unsigned value) {
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void publish_one_more(unsigned* counter) {
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// Waits until the word is at least `target` and returns it; a wait that runs out sets info to -1 and
// returns FLAG_FAILED.
__device__ __forceinline__ unsigned await(unsigned* flag, unsigned target, unsigned spin_limit, int* info,
                                          unsigned& seen) {
    if (threadIdx.x == 0) {
        unsigned v = __hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
        for (unsigned n = 0; v < target && n < spin_limit; ++n) {
            __builtin_amdgcn_s_sleep(32);
            v = __hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (v < target) {
            atomicCAS(info, 0, -1);
            v = FLAG_FAILED;
        }
        seen = v;
    }
    __syncthreads();
    const unsigned v = seen;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");    // every wavefront reads what was published
    __syncthreads();                                       // `seen` may be written again
    return v;
}

// Panel rows [P0, P0 + 128 nblk); [R0, P0) are the rows of the panel before it, whose update the trailing
// matrix has not had yet (R0 = P0: nothing outstanding).  Workgroup ids: [0, nhead_pad) the tiles of this
// panel's rows that take that update ("head": column w has min(w, nblk - 1) + 1 of them, columns in order),
// then nown_pad ids for the column owners, then the tiles of the trailing matrix below this panel, nt per edge
// (0: none).  flags: FLAGS_PER_PANEL words, then one counter per column (head tiles done), all zero.
__global__ __launch_bounds__(PT, 4) void panel_kernel(double* A, long long ld, int F, int R0, int P0, int nblk,
                                                      int nhead_pad, int nown, int nown_pad, int nt, TileMap tm,
                                                      double* invs, int* info, unsigned* flags, unsigned spin_limit) {
    // the tile product and the factorisation never run at the same time: one piece of LDS for both, which
    // is what lets two workgroups share a CU (2 x 74 KB)
    __shared__ __attribute__((aligned(16))) union {
        TileShared tile;
        PotrfShared potrf;
    } lds;
    TileShared& sm = lds.tile;
    PotrfShared& ps = lds.potrf;
    __shared__ unsigned seen;
    if (*info != 0) return;
    unsigned* heads_done = flags + FLAGS_PER_PANEL;
    int bid = (int)blockIdx.x;
    if (bid < nhead_pad) {                                   // a head tile: waits for nobody
        int w, b;
        const int tri = nblk * (nblk + 1) / 2;               // the columns of the panel itself form a triangle
        if (bid < tri) {
            w = 0;
            while (bid >= (w + 1) * (w + 2) / 2) ++w;
            b = bid - w * (w + 1) / 2;
        } else {
            w = nblk + (bid - tri) / nblk;
            b = (bid - tri) % nblk;
        }
        const int k0 = P0 + b * NB, j0 = P0 + w * NB;
        if (j0 >= F) return;
        tile_product(A + (size_t)R0 * ld + k0, ld, A + (size_t)R0 * ld + j0, ld, P0 - R0, A + (size_t)k0 * ld + j0, ld,
                     -1.0, false, sm);
        publish_one_more(heads_done + w);
        return;
    }
    bid -= nhead_pad;
    if (bid >= nown_pad) {                                   // a tile of the trailing matrix
        int ti, tj;
        tile_of_block<true>((unsigned)(bid - nown_pad), nt, nt, tm, ti, tj);
        if (ti < 0 || ti > tj) return;
        const int Q = P0 + nblk * NB;
        const int i0 = Q + ti * NB, c0 = Q + tj * NB;
        tile_product(A + (size_t)R0 * ld + i0, ld, A + (size_t)R0 * ld + c0, ld, P0 - R0, A + (size_t)i0 * ld + c0, ld,
                     -1.0, false, sm);
        return;
    }
    // a column owner: owner o < nblk has column o of the panel, the one with its diagonal tile in it; the others
    // have every (nown - nblk)-th column right of the panel
    if (bid >= nown) return;
    const int ncol = (F - P0) / NB;
    const int stride = bid < nblk ? ncol : nown - nblk;
    const int mine = bid < nblk ? bid : nblk - 1;            // last block row with a tile on or above the diagonal
    if (P0 > R0 && nhead_pad > 0) {
        for (int w = bid; w < ncol; w += stride)
            if (await(heads_done + w, (unsigned)(mine + 1), spin_limit, info, seen) == FLAG_FAILED) return;
    } else if (P0 > R0) {                                    // no workgroups for the head tiles: the owner's own work
        for (int w = bid; w < ncol; w += stride)
            for (int b = 0; b <= mine; ++b)
                tile_product(A + (size_t)R0 * ld + P0 + b * NB, ld, A + (size_t)R0 * ld + P0 + w * NB, ld, P0 - R0,
                             A + (size_t)(P0 + b * NB) * ld + P0 + w * NB, ld, -1.0, false, sm);
    }
    unsigned strips_seen = 0u;                               // "strip (l, b) done" flags this workgroup has seen set
    for (int l = 0; l < nblk; ++l) {
        const int k0 = P0 + l * NB;
        double* inv = invs + (size_t)(k0 / NB) * 2 * NB * NB;
        if (l == bid) {                                      // the own diagonal tile: every update is in
            const bool ok = potrf_block(A, ld, k0, NB, inv, inv + NB * NB, info, ps);
            // on failure every workgroup right of this column leaves at this flag, before it could wait for
            // anything that is now never set
            publish(flags + l, ok ? FLAG_DONE : FLAG_FAILED);
            return;
        }
        if (await(flags + l, FLAG_DONE, spin_limit, info, seen) != FLAG_DONE) return;
        for (int w = bid; w < ncol; w += stride) {
            const int j0 = P0 + w * NB;                      // first column of the owned tiles
            double* tile = A + (size_t)k0 * ld + j0;
            tile_product(inv, NB, tile, ld, NB, tile, ld, 1.0, true, sm);
            if (bid < nblk) publish(flags + PBLK + l * PBLK + bid, FLAG_DONE);
            for (int b = l + 1; b <= mine; ++b) {
                const unsigned bit = 1u << (l * PBLK + b);
                if (b != bid && !(strips_seen & bit)) {
                    if (await(flags + PBLK + l * PBLK + b, FLAG_DONE, spin_limit, info, seen) != FLAG_DONE) return;
                    strips_seen |= bit;
                }
                tile_product(A + (size_t)k0 * ld + P0 + b * NB, ld, tile, ld, NB, A + (size_t)(P0 + b * NB) * ld + j0, ld,
                             -1.0, false, sm);
            }
        }
    }
}

__global__ __launch_bounds__(256) void zero_words_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ---- triangular solves with one right-hand side -----------------------------------------
//
// One launch per direction, one workgroup per 128-row block.  Forward, U^T z = b: workgroup k keeps
// acc = b_k - sum_{i<k} U(i,k)^T z_i, taking the tiles U(i,k) in the order of i, then z_k = U11_k^-T acc through
// the stored inverse.  Backward, U x = z: the same from the last block to the first with the tiles U(k,j),
// j > k.  The values handed from workgroup to workgroup are their own flags: z (and the exchange copy of x)
// start out as a NaN with a payload no computation produces, a producer stores its 128 results with
// device-scope atomic stores, and a consumer polls the very values it needs with device-scope atomic loads
// (the tile they multiply is final and already on its way from memory): no fence, no separate flag, one trip
// through memory per step of the chain.  Every workgroup waits only for workgroups with lower ids (the backward
// launch numbers the blocks from the end), so whoever is waited for is running or done; the waits are bounded
// all the same, and one that runs out hands on a NaN, which ends up in the solution instead of a wrong number.
constexpr int ST = 512;            // threads of a solve workgroup
constexpr int SQ = ST / NB;        // row quarters: thread (c = tid % 128, q = tid / 128) has rows 32 q .. 32 q + 31
constexpr int SR = NB / SQ;
constexpr unsigned long long NOT_YET = 0x7FF8C0DEC0DE0001ULL;

__device__ __forceinline__ unsigned long long peek(const double* p) {
    return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void hand_on(double* p, double v) {
    unsigned long long bits = (unsigned long long)__double_as_longlong(v);
    if (bits == NOT_YET) bits ^= 2ULL;                                // (never: keeps a consumer from waiting for ever)
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// out[c] = sum_m M[m,c] vec[m] with the thread's 32 rows of M in registers; the four partial sums through LDS
__device__ __forceinline__ double block_product(const double (&iv)[SR], const double* vec, double (*part)[NB], int c,
                                                int q) {
    double s = 0.0;
#pragma unroll
    for (int m = 0; m < SR; ++m) s = fma(iv[m], vec[SR * q + m], s);
    part[q][c] = s;
    __syncthreads();
    return (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
}

__global__ __launch_bounds__(ST) void fwd_solve_kernel(const double* U, long long ld, int F, const double* invs,
                                                       const double* b, double* z, unsigned spin_limit) {
    __shared__ double part[SQ][NB], vec[NB];
    const int k = (int)blockIdx.x, k0 = k * NB;
    const int tid = threadIdx.x, lane = tid & 63, c = tid & (NB - 1), q = tid / NB;
    const double* inv = invs + (size_t)k * 2 * NB * NB;
    double iv[SR];
#pragma unroll
    for (int m = 0; m < SR; ++m) iv[m] = inv[(SR * q + m) * NB + c];
    const bool colok = k0 + c < F;
    double acc = (q == 0 && colok) ? b[k0 + c] : 0.0;
    for (int i = 0; i < k; ++i) {
        const double* tile = U + (size_t)(i * NB + SR * q) * ld + k0 + c;
        double u[SR];
#pragma unroll
        for (int r = 0; r < SR; ++r) u[r] = colok ? tile[(size_t)r * ld] : 0.0;
        // lane r: row r of this wavefront's quarter of z_i
        const double* mine = z + i * NB + SR * q + (lane & (SR - 1));
        unsigned long long bits = peek(mine);
        for (unsigned n = 0; __builtin_amdgcn_ballot_w64(bits == NOT_YET) != 0ULL && n < spin_limit; ++n) {
            __builtin_amdgcn_s_sleep(4);
            bits = peek(mine);
        }
        const double zr = bits == NOT_YET ? __builtin_nan("") : __longlong_as_double((long long)bits);
#pragma unroll
        for (int r = 0; r < SR; ++r) acc = fma(-u[r], value_of_lane(zr, r), acc);
    }
    part[q][c] = acc;
    __syncthreads();
    if (tid < NB) vec[tid] = (part[0][tid] + part[1][tid]) + (part[2][tid] + part[3][tid]);
    __syncthreads();
    const double zk = block_product(iv, vec, part, c, q);
    if (tid < NB) hand_on(z + k0 + tid, zk);
}

__global__ __launch_bounds__(ST) void bwd_solve_kernel(const double* U, long long ld, int F, int nblk,
                                                       const double* invs, const double* z, double* xs, double* x,
                                                       unsigned spin_limit) {
    __shared__ double part[SQ][NB], vec[NB];
    const int k = nblk - 1 - (int)blockIdx.x, k0 = k * NB;
    const int tid = threadIdx.x, c = tid & (NB - 1), q = tid / NB;
    const int csub = tid & 15, rowgrp = tid >> 4;          // sixteen lanes of eight columns along a row; rows rowgrp + 32 a
    const double* invT = invs + (size_t)k * 2 * NB * NB + NB * NB;
    double iv[SR];
#pragma unroll
    for (int m = 0; m < SR; ++m) iv[m] = invT[(SR * q + m) * NB + c];
    double acc[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) acc[a] = csub == 0 ? z[k0 + rowgrp + 32 * a] : 0.0;
    for (int j = nblk - 1; j > k; --j) {
        const int col0 = j * NB + 8 * csub;
        double u[4][8];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const double* row = U + (size_t)(k0 + rowgrp + 32 * a) * ld + col0;     // k < nblk - 1: a whole block of rows
#pragma unroll
            for (int e = 0; e < 8; ++e) u[a][e] = col0 + e < F ? row[e] : 0.0;
        }
        unsigned long long bits[8];
        bool pending = false;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            bits[e] = peek(xs + col0 + e);
            pending |= bits[e] == NOT_YET;
        }
        for (unsigned n = 0; __builtin_amdgcn_ballot_w64(pending) != 0ULL && n < spin_limit; ++n) {
            __builtin_amdgcn_s_sleep(4);
            pending = false;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                bits[e] = peek(xs + col0 + e);
                pending |= bits[e] == NOT_YET;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const double xv = bits[e] == NOT_YET ? __builtin_nan("") : __longlong_as_double((long long)bits[e]);
#pragma unroll
            for (int a = 0; a < 4; ++a) acc[a] = fma(-u[a][e], xv, acc[a]);
        }
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int m = 8; m >= 1; m >>= 1) acc[a] += __shfl_xor(acc[a], m, 16);
        if (csub == 0) vec[rowgrp + 32 * a] = acc[a];
    }
    __syncthreads();
    const double xk = block_product(iv, vec, part, c, q);
    if (tid < NB) {
        hand_on(xs + k0 + tid, xk);                         // whole blocks: the columns past F are zero
        if (k0 + tid < F) x[k0 + tid] = xk;
    }
}

__global__ __launch_bounds__(256) void fill_words64_kernel(unsigned long long* p, int n, unsigned long long v) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = v;
}

}  // namespace

// device workspace: the inverses of the diagonal blocks (both orientations), z of the forward solve and the
// exchange copy of x of the backward solve (whole blocks each), and the flags of the panel launches (per panel:
// FLAGS_PER_PANEL + one counter per block column)
namespace {
struct Workspace {
    double* invs;
    double* z;
    double* xs;
    unsigned* panel_flags;
    size_t nblk, npanel, bytes;
};
Workspace workspace_layout(void* base, int F) {
    Workspace w;
    w.nblk = ((size_t)F + NB - 1) / NB;
    w.npanel = ((size_t)F + OB - 1) / OB;
    w.invs = reinterpret_cast<double*>(base);
    w.z = w.invs + w.nblk * 2 * NB * NB;
    w.xs = w.z + w.nblk * NB;
    w.panel_flags = reinterpret_cast<unsigned*>(w.xs + w.nblk * NB);
    w.bytes = (w.nblk * 2 * NB * NB + 2 * w.nblk * NB) * sizeof(double) +
              w.npanel * (FLAGS_PER_PANEL + w.nblk) * sizeof(unsigned) + 256;
    return w;
}
}  // namespace

extern "C" size_t qmll_cholesky_workspace_bytes(int F) {
    if (F <= 0) return 0;
    return workspace_layout(nullptr, F).bytes;
}

namespace {

// rows [k0, k0+nb) of the panel that starts at P0: update from the panel's rows above, factor the
// diagonal block, solve the row strip to its right
int factor_block(double* A, int F, long long ld, int P0, int k0, double* invs, int* info, hipStream_t stream) {
    const int nb = F - k0 < NB ? F - k0 : NB;
    double* inv = invs + (size_t)(k0 / NB) * 2 * NB * NB;
    if (k0 > P0) {
        const double* above = A + (size_t)P0 * ld + k0;
        const int rc = qmll_internal_gemm_tn(above, ld, nb, above, ld, F - k0, k0 - P0, A + (size_t)k0 * ld + k0, ld,
                                             -1.0, 0, stream);
        if (rc != QMLL_OK) return rc;
    }
    hipLaunchKernelGGL(potrf_block_kernel, dim3(1), dim3(PT), 0, stream, A, ld, k0, nb, inv, inv + NB * NB, info);
    QMLL_CHECK_LAUNCH("qmll_cholesky_f64");
    const int n = F - k0 - nb;
    if (n > 0) {
        double* A12 = A + (size_t)k0 * ld + k0 + NB;
        return qmll_internal_gemm_tn(inv, NB, NB, A12, ld, n, NB, A12, ld, 1.0, 1, stream);
    }
    return QMLL_OK;
}

}  // namespace

extern "C" int qmll_cholesky_f64(double* A, int F, long long ld, void* workspace, int* info, qmll_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    QMLL_REQUIRE(F > 0 && ld >= F, QMLL_ERR_INVALID, "qmll_cholesky_f64: bad size F=%d ld=%lld", F, ld);
    QMLL_REQUIRE(ld < (1LL << 23), QMLL_ERR_INVALID, "qmll_cholesky_f64: row stride %lld too large", ld);
    QMLL_REQUIRE(A && workspace && info, QMLL_ERR_INVALID, "qmll_cholesky_f64: null pointer");
    QMLL_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, QMLL_ERR_INVALID,
                 "qmll_cholesky_f64: the workspace must be 16-byte aligned");
    const Workspace ws = workspace_layout(workspace, F);
    double* invs = ws.invs;
    // whole tiles and 16-byte loads: one launch per panel, which also carries the trailing update of the panel
    // before it; otherwise a launch per step
    const bool whole_tiles = F % NB == 0 && ld % 2 == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0;
    if (whole_tiles) {
        unsigned* flags = ws.panel_flags;
        const int per_panel = FLAGS_PER_PANEL + (int)ws.nblk;
        const int nflags = (F + OB - 1) / OB * per_panel;
        hipLaunchKernelGGL(zero_words_kernel, dim3((nflags + 255) / 256), dim3(256), 0, stream, flags, nflags);
        QMLL_CHECK_LAUNCH("qmll_cholesky_f64");
        for (int P0 = 0; P0 < F; P0 += OB) {
            const int pend = P0 + OB < F ? P0 + OB : F;       // this panel: rows [P0, pend)
            const int R0 = P0 >= OB ? P0 - OB : 0;            // the panel before it
            const int nblk = (pend - P0) / NB;
            const int ncol = (F - P0) / NB;                   // columns of tiles from the panel's first to the last
            const int nt = P0 > R0 ? (F - pend) / NB : 0;
            const int nown = ncol;
            // The head tiles (this panel's rows of the update of the panel before) go to workgroups of their own
            // once the trailing matrix is small, where a launch lasts as long as its slowest owner: four head tiles
            // and ten strip / update products in a row, 540 us, against a chain of four factorisations of 390.
            // While the trailing tiles keep the chip busy for longer than that, the owners take their head tiles
            // themselves and no slot waits for another.
            const bool split_heads = P0 > R0 && nt <= SPLIT_HEADS_BELOW;
            const int nown_pad = (nown + NXCD - 1) / NXCD * NXCD;
            const int nhead = split_heads ? nblk * (nblk + 1) / 2 + (ncol - nblk) * nblk : 0;
            const int nhead_pad = (nhead + NXCD - 1) / NXCD * NXCD;
            long long per_xcd = 0;
            TileMap tm = gram_tile_map(nt > 0 ? nt : 1, nt > 0 ? nt : 1, true, per_xcd);
            const long long grid = (long long)nhead_pad + nown_pad + (nt > 0 ? per_xcd * NXCD : 0);
            QMLL_REQUIRE(grid < 2147483647LL, QMLL_ERR_INVALID, "qmll_cholesky_f64: too many tiles");
            hipLaunchKernelGGL(panel_kernel, dim3((unsigned)grid), dim3(PT), 0, stream, A, ld, F, R0, P0, nblk, nhead_pad,
                               nown, nown_pad, nt, tm, invs, info, flags + (size_t)(P0 / OB) * per_panel, SPIN_LIMIT);
            QMLL_CHECK_LAUNCH("qmll_cholesky_f64");
        }
        return QMLL_OK;
    }
    for (int P0 = 0; P0 < F; P0 += OB) {
        const int pend = P0 + OB < F ? P0 + OB : F;           // this panel: rows [P0, pend)
        for (int k0 = P0; k0 < pend; k0 += NB) {
            const int rc = factor_block(A, F, ld, P0, k0, invs, info, stream);
            if (rc != QMLL_OK) return rc;
        }
        if (pend >= F) break;
        const int rc = qmll_internal_syrk_upper(A + (size_t)P0 * ld + pend, pend - P0, F - pend, ld,
                                                A + (size_t)pend * ld + pend, ld, -1.0, stream);
        if (rc != QMLL_OK) return rc;
    }
    return QMLL_OK;
}

extern "C" int qmll_cholesky_solve_f64(const double* U, int F, long long ld, void* workspace, double* b,
                                       qmll_stream_t stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    QMLL_REQUIRE(F > 0 && ld >= F, QMLL_ERR_INVALID, "qmll_cholesky_solve_f64: bad size F=%d ld=%lld", F, ld);
    QMLL_REQUIRE(U && workspace && b, QMLL_ERR_INVALID, "qmll_cholesky_solve_f64: null pointer");
    const Workspace ws = workspace_layout(workspace, F);
    const int nblk = (int)ws.nblk;
    // z and the exchange copy of x are contiguous: "not yet" everywhere
    hipLaunchKernelGGL(fill_words64_kernel, dim3((2 * nblk * NB + 255) / 256), dim3(256), 0, stream,
                       reinterpret_cast<unsigned long long*>(ws.z), 2 * nblk * NB, NOT_YET);
    QMLL_CHECK_LAUNCH("qmll_cholesky_solve_f64");
    // U^T z = b, then U x = z with x into b
    hipLaunchKernelGGL(fwd_solve_kernel, dim3(nblk), dim3(ST), 0, stream, U, ld, F, ws.invs, b, ws.z, SPIN_LIMIT);
    QMLL_CHECK_LAUNCH("qmll_cholesky_solve_f64");
    hipLaunchKernelGGL(bwd_solve_kernel, dim3(nblk), dim3(ST), 0, stream, U, ld, F, nblk, ws.invs, ws.z, ws.xs, b,
                       SPIN_LIMIT);
    QMLL_CHECK_LAUNCH("qmll_cholesky_solve_f64");
    return QMLL_OK;
}
