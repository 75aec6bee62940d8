// Regularised normal equations (Z^T Z + lambda I) alpha = Z^T y: fp64 Cholesky factorisation
// A = U^T U of the symmetric positive definite matrix, in place in the upper triangle, and the
// two triangular solves.  The reference calls torch.linalg.solve (LU) at this point
// (qml_lightning/models/kernel.py:226-234).
//
// Row-major A with row stride ld, 128-column blocks grouped in panels of 512 rows.  Per block k:
//   1. the block's 128 rows (columns k..F) take the product of the panel's rows above them
//      (fp64 MFMA tile kernel of gram.hip, depth up to 384);
//   2. potrf_block_kernel: one workgroup factors the 128x128 diagonal block in registers and
//      also produces the inverse of the factor (both orientations, kept for the solves);
//   3. U12 = U11^-T A12 as a product with that inverse on the same MFMA kernel.
// After a panel, the trailing matrix takes A22 -= U12^T U12 (512 rows deep) on the tiles on or
// above the diagonal.  The depth of 512 is what makes the trailing update MFMA-bound: at a
// depth of 128 the read-modify-write of the trailing matrix dominates.
// Only elements on or above the diagonal are read; below the diagonal only the lower halves of
// the 128x128 diagonal tiles are overwritten.  Flops: F^3/3.
#include <type_traits>

#include "qmll_common.h"

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
constexpr int G = 16;         // potrf thread grid edge: thread (ti,tj) owns rows ti+16a, columns tj+16b

// Factor the nb x nb block at (k0,k0) (nb <= 128; the rest is padded with the identity).
// Elimination without square roots on a symmetric copy held in registers, A = L D L^T: in step j
// row r > j takes S[r,:] -= (S[j,r]/S[j,j]) S[j,:]; the same row operations applied to the
// identity give T = L^-1.  At the end U[j,c] = S[j,c]/sqrt(D_j) and U^-1[m,i] = T[i,m]/sqrt(D_i).
// Rows are dealt cyclically (16 x 16 threads, 8 x 8 elements each), so the shrinking active window
// stays balanced; the pivot row travels through LDS, one barrier per step.  Only the 16x16-element
// groups that hold live data are touched: the upper ones of S, the lower ones of T.
// Output: upper triangle of the block <- U11; inv[m*128+i] = U11^-1[m,i]; invT[i*128+m] the same.
// info: 0, or 1 + the index of the first pivot that is not positive (later launches then exit).
__global__ __launch_bounds__(256) void potrf_block_kernel(double* __restrict__ A, long long ld, int k0, int nb,
                                                          double* __restrict__ inv, double* __restrict__ invT,
                                                          int* __restrict__ info) {
    __shared__ double rowS[2][2][NB], rowT[2][2][NB], dsq[NB];
    if (*info != 0) return;
    const int tid = threadIdx.x;
    const int ti = tid / G, tj = tid % G;
    double* blk = A + (size_t)k0 * ld + k0;
    // one array for both: S(a,b), b >= a, the upper 16 x 16-element groups of the symmetric copy; T(a,b), b <= a,
    // the lower groups of L^-1 (two [8][8] arrays, half empty, end up in scratch memory beside the step's temporaries)
    double st[8][9];
#define S_(a, b) st[a][(b) + 1]
#define T_(a, b) st[a][b]
#pragma unroll
    for (int a = 0; a < 8; ++a) {
#pragma unroll
        for (int b = a; b < 8; ++b) {
            const int r = a * G + ti, c = b * G + tj;
            const int lo = r < c ? r : c, hi = r < c ? c : r;
            S_(a, b) = hi < nb ? blk[(size_t)lo * ld + hi] : (r == c ? 1.0 : 0.0);
        }
#pragma unroll
        for (int b = 0; b <= a; ++b) T_(a, b) = (a == b && ti == tj) ? 1.0 : 0.0;
    }
    // reciprocal by the hardware estimate and two Newton steps (full fp64 accuracy up to a couple of
    // ulps) instead of the much longer IEEE division sequence: it sits on the serial path of every step
    auto reciprocal = [](double v) {
        double ip = __builtin_amdgcn_rcp(v);
        ip = fma(fma(-v, ip, 1.0), ip, ip);
        return fma(fma(-v, ip, 1.0), ip, ip);
    };
    // Two pivots per barrier.  The kernel is bound by its chain of dependent steps (barrier, pivot row
    // through LDS, reciprocal: 44 of 59 us remain when the elimination's multiply-adds are taken out), not by
    // arithmetic.  Rows j and j+1 are published as they stand before step j; every thread forms what step j
    // would have made of row j+1 (row1 - l row0, l = S[j,j+1] / S[j,j]) and applies both eliminations: the
    // same operations in the same order as one pivot at a time, hence the same bits.  Halving the barriers
    // buys less than their share (59 -> 53 us per block, 45.0 -> 44.2 ms per factorisation at 16 384): the LDS
    // reads and the two reciprocals, the second of which waits for the first, are what a step is made of.
    // (the register block index is a template constant, not a loop variable the unroller may or may not fix:
    // with it dynamic the register arrays go to scratch memory)
    auto eliminate = [&](auto ja_) -> bool {
        constexpr int ja = decltype(ja_)::value;
        for (int jj = 0; jj < G; jj += 2) {
            const int j = ja * G + jj, buf = (jj >> 1) & 1;
            if (ti == jj || ti == jj + 1) {
                const int which = ti - jj;
#pragma unroll
                for (int b = ja; b < 8; ++b) rowS[buf][which][b * G + tj] = S_(ja, b);
#pragma unroll
                for (int b = 0; b <= ja; ++b) rowT[buf][which][b * G + tj] = T_(ja, b);
            }
            __syncthreads();   // the other copy was last read in the step before, which ended at this barrier
            const double piv0 = rowS[buf][0][j];
            if (!(piv0 > 0.0)) {                      // the same value in every thread: uniform exit
                if (tid == 0) *info = k0 + j + 1;
                return false;
            }
            const double ip0 = reciprocal(piv0);
            const double a01 = rowS[buf][0][j + 1];
            const double l = a01 * ip0;
            const double piv1 = fma(-l, a01, rowS[buf][1][j + 1]);
            if (!(piv1 > 0.0)) {
                if (tid == 0) *info = k0 + j + 2;
                return false;
            }
            const double ip1 = reciprocal(piv1);
            double rv0[8], rv1[8], tv0[8], tv1[8], f0[8], f1[8];
#pragma unroll
            for (int b = ja; b < 8; ++b) {
                rv0[b] = rowS[buf][0][b * G + tj];
                rv1[b] = fma(-l, rv0[b], rowS[buf][1][b * G + tj]);
            }
#pragma unroll
            for (int b = 0; b <= ja; ++b) {
                tv0[b] = rowT[buf][0][b * G + tj];
                tv1[b] = fma(-l, tv0[b], rowT[buf][1][b * G + tj]);
            }
#pragma unroll
            for (int a = ja; a < 8; ++a) {
                const int r = a * G + ti;
                const double c0 = rowS[buf][0][r];
                f0[a] = r > j ? c0 * ip0 : 0.0;
                f1[a] = r > j + 1 ? fma(-l, c0, rowS[buf][1][r]) * ip1 : 0.0;
            }
#pragma unroll
            for (int a = ja; a < 8; ++a) {
#pragma unroll
                for (int b = a; b < 8; ++b) S_(a, b) = fma(-f1[a], rv1[b], fma(-f0[a], rv0[b], S_(a, b)));
#pragma unroll
                for (int b = 0; b <= ja; ++b) T_(a, b) = fma(-f1[a], tv1[b], fma(-f0[a], tv0[b], T_(a, b)));
            }
        }
        return true;
    };
    if (!eliminate(std::integral_constant<int, 0>{}) || !eliminate(std::integral_constant<int, 1>{}) ||
        !eliminate(std::integral_constant<int, 2>{}) || !eliminate(std::integral_constant<int, 3>{}) ||
        !eliminate(std::integral_constant<int, 4>{}) || !eliminate(std::integral_constant<int, 5>{}) ||
        !eliminate(std::integral_constant<int, 6>{}) || !eliminate(std::integral_constant<int, 7>{}))
        return;
    // 1/sqrt(D_r) of every row, from the threads on the diagonal
    if (ti == tj) {
#pragma unroll
        for (int a = 0; a < 8; ++a) dsq[a * G + ti] = 1.0 / sqrt(S_(a, a));
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < 8; ++a) {
        const int r = a * G + ti;
        const double dr = dsq[r];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const int c = b * G + tj;
            if (b >= a && c >= r && c < nb) blk[(size_t)r * ld + c] = S_(a, b) * dr;
            const double v = b <= a ? T_(a, b) * dr : 0.0;     // U^-1[c,r]
            invT[r * NB + c] = v;
            inv[c * NB + r] = v;
        }
    }
}
#undef S_
#undef T_

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
    return (nblk * 2 * NB * NB + (size_t)F) * sizeof(double) + 256;
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
    hipLaunchKernelGGL(potrf_block_kernel, dim3(1), dim3(256), 0, stream, A, ld, k0, nb, inv, inv + NB * NB, info);
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
