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
constexpr int GR = 32, GC = 16;   // potrf thread grid: thread (ti,tj) owns rows ti + 32 a, columns tj + 16 b
constexpr int PT = GR * GC;       // threads of a factorisation workgroup (and of the tile product's eight wavefronts)

// Factor the nb x nb block at (k0,k0) (nb <= 128; the rest is padded with the identity).
// Elimination without square roots on a symmetric copy held in registers, A = L D L^T: in step j
// row r > j takes S[r,:] -= (S[j,r]/S[j,j]) S[j,:]; the same row operations applied to the
// identity give T = L^-1.  At the end U[j,c] = S[j,c]/sqrt(D_j) and U^-1[m,i] = T[i,m]/sqrt(D_i).
// Rows are dealt cyclically (32 x 16 threads, 4 x 8 elements each), so the shrinking active window
// stays balanced; the pivot row travels through LDS, one barrier per step.  Only the 32 x 16-element
// groups that hold live data are kept: for row group a the column groups b >= 2a of S and b <= 2a + 1 of T,
// forty values per thread, which with a step's temporaries stays inside the 128 registers of a kernel that
// runs two workgroups of 512 per CU.
// The kernel is bound by its chain of 128 dependent steps (barrier, pivot row through LDS, reciprocal), not
// by arithmetic: without the elimination's multiply-adds it still takes three quarters of its time.
// Output: upper triangle of the block <- U11; inv[m*128+i] = U11^-1[m,i]; invT[i*128+m] the same.
// info: 0, or 1 + the index of the first pivot that is not positive (later launches then exit).
struct PotrfShared {
    double rowS[2][NB], rowT[2][NB], dsq[NB];
};

// Called by all PT threads of the workgroup.  False when a pivot is not positive (info is then set).
__device__ __forceinline__ bool potrf_block(double* A, long long ld, int k0, int nb, double* inv, double* invT,
                                            int* info, PotrfShared& ps) {
    auto& rowS = ps.rowS;
    auto& rowT = ps.rowT;
    auto& dsq = ps.dsq;
    const int tid = threadIdx.x;
    const int ti = tid / GC, tj = tid % GC;
    double* blk = A + (size_t)k0 * ld + k0;
    double st[4][10];
#define S_(a, b) st[a][(b) + 2]
#define T_(a, b) st[a][b]
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int r = a * GR + ti;
#pragma unroll
        for (int b = 2 * a; b < 8; ++b) {
            const int c = b * GC + tj;
            const int lo = r < c ? r : c, hi = r < c ? c : r;
            S_(a, b) = hi < nb ? blk[(size_t)lo * ld + hi] : (r == c ? 1.0 : 0.0);
        }
#pragma unroll
        for (int b = 0; b <= 2 * a + 1; ++b) T_(a, b) = (r == b * GC + tj) ? 1.0 : 0.0;
    }
    // reciprocal by the hardware estimate and two Newton steps (full fp64 accuracy up to a couple of
    // ulps) instead of the much longer IEEE division sequence: it sits on the serial path of every step
    auto reciprocal = [](double v) {
        double ip = __builtin_amdgcn_rcp(v);
        ip = fma(fma(-v, ip, 1.0), ip, ip);
        return fma(fma(-v, ip, 1.0), ip, ip);
    };
    // (the row group of the pivot is a template constant, not a loop variable the unroller may or may not
    // fix: with it dynamic the register array goes to scratch memory)
    auto eliminate = [&](auto ja_) -> bool {
        constexpr int ja = decltype(ja_)::value;
        for (int jj = 0; jj < GR; ++jj) {
            const int j = ja * GR + jj, buf = jj & 1;
            if (ti == jj) {
#pragma unroll
                for (int b = 2 * ja; b < 8; ++b) rowS[buf][b * GC + tj] = S_(ja, b);
#pragma unroll
                for (int b = 0; b <= 2 * ja + 1; ++b) rowT[buf][b * GC + tj] = T_(ja, b);
            }
            __syncthreads();   // the other copy was last read in the step before, which ended at this barrier
            const double piv = rowS[buf][j];
            if (!(piv > 0.0)) {                       // the same value in every thread: uniform exit
                if (tid == 0) *info = k0 + j + 1;
                return false;
            }
            const double ip = reciprocal(piv);
            double rv[8], tv[8], f[4];
#pragma unroll
            for (int b = 2 * ja; b < 8; ++b) rv[b] = rowS[buf][b * GC + tj];
#pragma unroll
            for (int b = 0; b <= 2 * ja + 1; ++b) tv[b] = rowT[buf][b * GC + tj];
#pragma unroll
            for (int a = ja; a < 4; ++a) {
                const int r = a * GR + ti;
                f[a] = r > j ? rowS[buf][r] * ip : 0.0;
            }
#pragma unroll
            for (int a = ja; a < 4; ++a) {
#pragma unroll
                for (int b = 2 * a; b < 8; ++b) S_(a, b) = fma(-f[a], rv[b], S_(a, b));
#pragma unroll
                for (int b = 0; b <= 2 * ja + 1; ++b) T_(a, b) = fma(-f[a], tv[b], T_(a, b));
            }
        }
        return true;
    };
    if (!eliminate(std::integral_constant<int, 0>{}) || !eliminate(std::integral_constant<int, 1>{}) ||
        !eliminate(std::integral_constant<int, 2>{}) || !eliminate(std::integral_constant<int, 3>{}))
        return false;
    // 1/sqrt(D_r) of every row, from the threads that hold the diagonal
    if (tj == ti % GC) {
#pragma unroll
        for (int a = 0; a < 4; ++a) dsq[a * GR + ti] = 1.0 / sqrt(ti < GC ? S_(a, 2 * a) : S_(a, 2 * a + 1));
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int r = a * GR + ti;
        const double dr = dsq[r];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const int c = b * GC + tj;
            if (b >= 2 * a && c >= r && c < nb) blk[(size_t)r * ld + c] = S_(a, b) * dr;
            const double v = b <= 2 * a + 1 ? T_(a, b) * dr : 0.0;     // U^-1[c,r]
            invT[r * NB + c] = v;
            inv[c * NB + r] = v;
        }
    }
    return true;
}
#undef S_
#undef T_

__global__ __launch_bounds__(PT) void potrf_block_kernel(double* A, long long ld, int k0, int nb, double* inv,
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
constexpr unsigned FLAG_DONE = 1u, FLAG_FAILED = 2u;
constexpr int PBLK = OB / NB;                        // blocks per panel
constexpr int FLAGS_PER_PANEL = PBLK + PBLK * PBLK;  // "block l factored": [l]; "strip (l, b) done": [PBLK + l PBLK + b]
constexpr unsigned SPIN_LIMIT = 1u << 21;   // polls of about a microsecond each before a wait gives up

typedef double double2_t __attribute__((ext_vector_type(2)));
typedef double double4_t __attribute__((ext_vector_type(4)));

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
                *c = overwrite ? v : *c + v;
            }
    __syncthreads();
}

// every store of the workgroup so far becomes visible to the device, then the flag is set
__device__ __forceinline__ void publish(unsigned* flag, unsigned value) {
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// true once the flag says done; false when its owner failed or the wait ran out (info <- -1)
__device__ __forceinline__ bool await(unsigned* flag, unsigned spin_limit, int* info, unsigned& seen) {
    if (threadIdx.x == 0) {
        unsigned v = __hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
        for (unsigned n = 0; v == 0u && n < spin_limit; ++n) {
            __builtin_amdgcn_s_sleep(32);
            v = __hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (v == 0u) {
            atomicCAS(info, 0, -1);
            v = FLAG_FAILED;
        }
        seen = v;
    }
    __syncthreads();
    const unsigned v = seen;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");    // every wavefront reads what the owner published
    __syncthreads();                                       // `seen` may be written again
    return v == FLAG_DONE;
}

// Panel rows [P0, P0 + 128 nblk); [R0, P0) are the rows of the panel before it, whose update the trailing
// matrix has not had yet (R0 = P0: nothing outstanding).  nown_pad: ids reserved for the column owners;
// nt: tiles per edge of the trailing matrix below this panel (0: none).  flags: FLAGS_PER_PANEL words, zero.
__global__ __launch_bounds__(PT, 4) void panel_kernel(double* A, long long ld, int F, int R0, int P0, int nblk,
                                                      int nown_pad, int nt, TileMap tm, double* invs, int* info,
                                                      unsigned* flags, unsigned spin_limit) {
    __shared__ __attribute__((aligned(16))) TileShared sm;
    __shared__ PotrfShared ps;
    __shared__ unsigned seen;
    if (*info != 0) return;
    const int bid = (int)blockIdx.x;
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
    const int j0 = P0 + bid * NB;                            // first column of the owned tiles
    if (j0 >= F) return;
    const int mine = bid < nblk ? bid : nblk - 1;            // last block row with a tile on or above the diagonal
    if (P0 > R0) {
        for (int b = 0; b <= mine; ++b) {
            const int k0 = P0 + b * NB;
            tile_product(A + (size_t)R0 * ld + k0, ld, A + (size_t)R0 * ld + j0, ld, P0 - R0, A + (size_t)k0 * ld + j0, ld,
                         -1.0, false, sm);
        }
    }
    for (int l = 0; l < nblk; ++l) {
        const int k0 = P0 + l * NB;
        double* tile = A + (size_t)k0 * ld + j0;
        double* inv = invs + (size_t)(k0 / NB) * 2 * NB * NB;
        if (k0 == j0) {                                      // the own diagonal tile: every update is in
            const bool ok = potrf_block(A, ld, k0, NB, inv, inv + NB * NB, info, ps);
            // on failure every workgroup right of this column leaves at this flag, before it could wait for
            // anything that is now never set
            publish(flags + l, ok ? FLAG_DONE : FLAG_FAILED);
            return;
        }
        if (!await(flags + l, spin_limit, info, seen)) return;
        tile_product(inv, NB, tile, ld, NB, tile, ld, 1.0, true, sm);
        if (bid < nblk) publish(flags + PBLK + l * PBLK + bid, FLAG_DONE);
        for (int b = l + 1; b <= mine; ++b) {
            if (b != bid && !await(flags + PBLK + l * PBLK + b, spin_limit, info, seen)) return;
            tile_product(A + (size_t)k0 * ld + P0 + b * NB, ld, tile, ld, NB, A + (size_t)(P0 + b * NB) * ld + j0, ld, -1.0,
                         false, sm);
        }
    }
}

__global__ __launch_bounds__(256) void zero_words_kernel(unsigned* p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ---- triangular solves with one right-hand side -----------------------------------------

// Block k of U^T z = b: z_k = U11^-T b_k (product with the stored inverse, recomputed by every
// workgroup), then b[j] -= sum_r U[k0+r, j] z_k[r] for the columns j right of the block
// (thread = column).  Workgroup 0 stores z_k into z.
__global__ __launch_bounds__(256) void fwd_step_kernel(const double* __restrict__ U, long long ld, int k0, int nb,
                                                       int F, const double* __restrict__ inv, double* __restrict__ b,
                                                       double* __restrict__ z) {
    __shared__ double rs[NB], xs[NB];
    const int tid = threadIdx.x;
    if (tid < NB) rs[tid] = tid < nb ? b[k0 + tid] : 0.0;
    __syncthreads();
    if (tid < NB) {
        double s0 = 0.0, s1 = 0.0;
        for (int m = 0; m < NB; m += 2) {
            s0 = fma(inv[m * NB + tid], rs[m], s0);
            s1 = fma(inv[(m + 1) * NB + tid], rs[m + 1], s1);
        }
        xs[tid] = s0 + s1;
        if (blockIdx.x == 0 && tid < nb) z[k0 + tid] = s0 + s1;
    }
    __syncthreads();
    const int j = k0 + NB + blockIdx.x * 256 + tid;
    if (j >= F) return;
    const double* col = U + (size_t)k0 * ld + j;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
#pragma unroll 8
    for (int r = 0; r < NB; r += 4) {
        s0 = fma(col[(size_t)r * ld], xs[r], s0);
        s1 = fma(col[(size_t)(r + 1) * ld], xs[r + 1], s1);
        s2 = fma(col[(size_t)(r + 2) * ld], xs[r + 2], s2);
        s3 = fma(col[(size_t)(r + 3) * ld], xs[r + 3], s3);
    }
    b[j] -= (s0 + s1) + (s2 + s3);
}

// Block k of U x = z: x_k = U11^-1 z_k (z_k already holds every later block's contribution), then
// z[i] -= sum_c U[i, k0+c] x_k[c] for the rows i above the block: 16 lanes per row, 8 columns per
// lane, 64 rows per workgroup.  Workgroup 0 stores x_k into x.
constexpr int BWD_ROWS = 64;
__global__ __launch_bounds__(256) void bwd_step_kernel(const double* __restrict__ U, long long ld, int k0, int nb,
                                                       const double* __restrict__ invT, double* __restrict__ z,
                                                       double* __restrict__ x) {
    __shared__ double zs[NB], xs[NB];
    const int tid = threadIdx.x;
    if (tid < NB) zs[tid] = tid < nb ? z[k0 + tid] : 0.0;
    __syncthreads();
    if (tid < NB) {
        double s0 = 0.0, s1 = 0.0;
        for (int i = 0; i < NB; i += 2) {
            s0 = fma(invT[i * NB + tid], zs[i], s0);
            s1 = fma(invT[(i + 1) * NB + tid], zs[i + 1], s1);
        }
        xs[tid] = tid < nb ? s0 + s1 : 0.0;
        if (blockIdx.x == 0 && tid < nb) x[k0 + tid] = s0 + s1;
    }
    __syncthreads();
    const int sub = tid & 15;
    double xv[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) xv[q] = xs[sub * 8 + q];
    for (int rr = tid >> 4; rr < BWD_ROWS; rr += 16) {
        const int i = blockIdx.x * BWD_ROWS + rr;     // uniform over the 16 lanes of a row
        double sacc = 0.0;
        if (i < k0) {
            const double* row = U + (size_t)i * ld + k0 + sub * 8;
#pragma unroll
            for (int q = 0; q < 8; ++q)
                if (sub * 8 + q < nb) sacc = fma(row[q], xv[q], sacc);
        }
#pragma unroll
        for (int m = 8; m >= 1; m >>= 1) sacc += __shfl_xor(sacc, m, 16);
        if (i < k0 && sub == 0) z[i] -= sacc;
    }
}

}  // namespace

extern "C" size_t qmll_cholesky_workspace_bytes(int F) {
    if (F <= 0) return 0;
    const size_t nblk = ((size_t)F + NB - 1) / NB;
    const size_t npanel = ((size_t)F + OB - 1) / OB;
    return (nblk * 2 * NB * NB + (size_t)F) * sizeof(double) + npanel * FLAGS_PER_PANEL * sizeof(unsigned) + 256;
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
    QMLL_REQUIRE(A && workspace && info, QMLL_ERR_INVALID, "qmll_cholesky_f64: null pointer");
    QMLL_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0, QMLL_ERR_INVALID,
                 "qmll_cholesky_f64: the workspace must be 16-byte aligned");
    double* invs = reinterpret_cast<double*>(workspace);
    // whole tiles and 16-byte loads: one launch per panel, which also carries the trailing update of the panel
    // before it; otherwise a launch per step
    const bool whole_tiles = F % NB == 0 && ld % 2 == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0;
    if (whole_tiles) {
        const size_t nblk_all = (size_t)F / NB;
        unsigned* flags = reinterpret_cast<unsigned*>(invs + nblk_all * 2 * NB * NB + (size_t)F);
        const int nflags = (F + OB - 1) / OB * FLAGS_PER_PANEL;
        hipLaunchKernelGGL(zero_words_kernel, dim3((nflags + 255) / 256), dim3(256), 0, stream, flags, nflags);
        QMLL_CHECK_LAUNCH("qmll_cholesky_f64");
        for (int P0 = 0; P0 < F; P0 += OB) {
            const int pend = P0 + OB < F ? P0 + OB : F;       // this panel: rows [P0, pend)
            const int R0 = P0 >= OB ? P0 - OB : 0;            // the panel before it
            const int nown = (F - P0) / NB;
            const int nown_pad = (nown + NXCD - 1) / NXCD * NXCD;
            const int nt = P0 > R0 ? (F - pend) / NB : 0;
            long long per_xcd = 0;
            TileMap tm = gram_tile_map(nt > 0 ? nt : 1, nt > 0 ? nt : 1, true, per_xcd);
            const long long grid = nown_pad + (nt > 0 ? per_xcd * NXCD : 0);
            QMLL_REQUIRE(grid < 2147483647LL, QMLL_ERR_INVALID, "qmll_cholesky_f64: too many tiles");
            hipLaunchKernelGGL(panel_kernel, dim3((unsigned)grid), dim3(PT), 0, stream, A, ld, F, R0, P0, (pend - P0) / NB,
                               nown_pad, nt, tm, invs, info, flags + (size_t)(P0 / OB) * FLAGS_PER_PANEL, SPIN_LIMIT);
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
    double* invs = reinterpret_cast<double*>(workspace);
    const size_t nblk = ((size_t)F + NB - 1) / NB;
    double* z = invs + nblk * 2 * NB * NB;
    // U^T z = b, blocks in ascending order (b is used up)
    for (int k0 = 0; k0 < F; k0 += NB) {
        const int nb = F - k0 < NB ? F - k0 : NB;
        const int n = F - k0 - nb;
        const double* inv = invs + (size_t)(k0 / NB) * 2 * NB * NB;
        const int grid = n > 0 ? (n + 255) / 256 : 1;
        hipLaunchKernelGGL(fwd_step_kernel, dim3(grid), dim3(256), 0, stream, U, ld, k0, nb, F, inv, b, z);
        QMLL_CHECK_LAUNCH("qmll_cholesky_solve_f64");
    }
    // U x = z, blocks in descending order, x into b
    const int last = (F - 1) / NB * NB;
    for (int k0 = last; k0 >= 0; k0 -= NB) {
        const int nb = F - k0 < NB ? F - k0 : NB;
        const double* invT = invs + (size_t)(k0 / NB) * 2 * NB * NB + NB * NB;
        const int grid = k0 > 0 ? (k0 + BWD_ROWS - 1) / BWD_ROWS : 1;
        hipLaunchKernelGGL(bwd_step_kernel, dim3(grid), dim3(256), 0, stream, U, ld, k0, nb, invT, z, b);
        QMLL_CHECK_LAUNCH("qmll_cholesky_solve_f64");
    }
    return QMLL_OK;
}
