// Normal-equation accumulation Z^T Z / Z^T y on the fp64 matrix cores of gfx950.
// Replaces the torch.matmul calls of qml_lightning/models/kernel.py:172-192 and
// qml_lightning/cuda/utils_kernel.cu:70-129 (matmul_and_reduce) of the reference.
//
// C[i,j] += sum_m Z[m,i] Z[m,j].  Z is row-major [M,F], so for a fixed m both operand
// fragments are contiguous in memory: the A fragment of v_mfma_f64_16x16x4_f64 (16 rows i
// x 4 steps k) is Z[m0+k, i0+i] and the B fragment is Z[m0+k, j0+j]; no transpose is
// ever materialised.  A workgroup (512 threads, 8 wavefronts) owns a 128x128 tile of C;
// each wavefront keeps a 64x32 sub-tile (4x2 MFMA tiles, 64 accumulator registers; four wavefronts
// per SIMD hold the matrix pipe busier than two with 64x64 sub-tiles did) and
// the two 128-wide column panels of Z are staged through LDS KB rows at a time with the
// next panel's global loads in flight during the MFMAs.  In the symmetric mode only tiles
// on or above the diagonal are computed; the mirror image is copied by a separate pass
// (gram_mirror_kernel), once per call or once after the caller's last batch.  Algorithmic work: M*F*(F+1) flops, 8*M*F bytes read once (re-reads of a
// panel by the tiles of one row/column are served from L2: consecutive workgroup ids walk
// along a tile row).
#include "qmll_common.h"
#include "gram_tiles.h"

namespace {

typedef double double4_t __attribute__((ext_vector_type(4)));
typedef double double2_t __attribute__((ext_vector_type(2)));

constexpr int KB = 16;        // rows of Z staged per step
constexpr int NWAVE = 8;      // wavefronts per workgroup: 2 along i x NWAVE/2 along j
constexpr int GT = 64 * NWAVE;
constexpr int WJ = NWAVE / 2;            // wavefronts along j
constexpr int NQ = TILE / WJ / 16;       // 16-column MFMA tiles per wavefront along j (4 along i)
constexpr int TPR = GT / KB;             // threads per staged row
constexpr int CPT = TILE / TPR;          // doubles per thread and row
constexpr int UN = CPT / 2;              // 16-byte units per thread
// doubles per staged row: 128 + 16, i.e. consecutive rows start 32 banks apart, so the two
// k-rows a half-wavefront reads in one ds_read_b64 never share a bank
constexpr int LDS_STRIDE = TILE + 16;
// GUARD: some panel sticks out of the matrix (F or the row block not a multiple of 128, or
// odd F): every element load is bounds-checked.  !GUARD: whole panels, 16-byte vector loads.
// GEN: general operands for the Cholesky updates (separate A operand Za, row strides, sign,
// overwrite).  !GEN is the Gram product proper: both operands are Z, every stride is F, C += Z^T Z;
// the strides and the second pointer are then compile-time aliases, which keeps its address
// arithmetic and register use as they were tuned.
template <bool SYM, bool GUARD, bool GEN>
__global__ __launch_bounds__(GT, 2) void gram_kernel(const double* __restrict__ Z, int M, int F, int f0, int f1,
                                                      int nti, int ntj, TileMap tm, double* __restrict__ C,
                                                      long long ldz_, long long ldc_, double sign_,
                                                      const double* __restrict__ Za_, long long lda_, int overwrite_) {
    unsigned bid = blockIdx.x;
    const bool split = GEN && tm.pieces > 1;          // one of several row ranges of a tile, to the workspace
    if (split) {
        const unsigned piece = bid % (unsigned)tm.pieces;
        bid = tm.tail_first + bid / (unsigned)tm.pieces;
        const long long m0 = (long long)piece * tm.piece_rows;
        const long long left = (long long)M - m0;
        M = left < 0 ? 0 : (int)(left < tm.piece_rows ? left : tm.piece_rows);
        if (M > 0) {
            Z += (size_t)m0 * ldz_;
            Za_ += (size_t)m0 * lda_;
        }
    }
    const long long ldz = GEN ? ldz_ : (long long)F, ldc = GEN ? ldc_ : (long long)F, lda = GEN ? lda_ : (long long)F;
    const double sign = GEN ? sign_ : 1.0;
    const double* __restrict__ Za = GEN ? Za_ : Z;
    const int overwrite = GEN ? overwrite_ : 0;
    // two copies of each staged panel: the next one is written while the current one is read,
    // one barrier per step (2 x 2 x 18 KB per workgroup, two workgroups of eight wavefronts per CU)
    __shared__ __attribute__((aligned(16))) double sA[2][KB][LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) double sB[2][KB][LDS_STRIDE];

    int ti, tj;
    tile_of_block<SYM>(bid, nti, ntj, tm, ti, tj);
    if (ti < 0 || (SYM && ti > tj)) return;
    if (split && M <= 0) {           // a row range past the end: its partial tile is zero
        for (int e = threadIdx.x; e < TILE * TILE; e += GT) C[(size_t)blockIdx.x * (TILE * TILE) + e] = 0.0;
        return;
    }
    const int i0 = f0 + ti * TILE;   // first feature of the A panel (rows of C)
    const int j0 = tj * TILE;        // first feature of the B panel (columns of C)
    const int ilim = SYM ? F : f1;
    const bool same = SYM && ti == tj;
    constexpr bool interior = !GUARD;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wi = (wave / WJ) * 64, wj = (wave % WJ) * (16 * NQ);   // wavefront's 64 x 16 NQ sub-tile
    const int l16 = lane & 15, lk = lane >> 4;

    double4_t acc[4][NQ];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < NQ; ++q) acc[p][q] = (double4_t){0.0, 0.0, 0.0, 0.0};

    // global -> register staging: KB x 128 doubles per panel = 2048 = 512 threads x 4:
    // thread t loads row t/32, columns (t%32)*4 .. +4
    const int lr = tid / TPR;
    const int lc = (tid % TPR) * CPT;
    double2_t ra[UN], rb[UN];
    bool loaded_rowok = true;

    auto load_panels = [&](int m0) {
        const int m = m0 + lr;
        const bool rowok = m < M;
        if constexpr (interior) {
            // rows past the end are read from the last row (always valid memory) and zeroed
            const size_t mr = (size_t)(rowok ? m : M - 1);
            const double2_t* pa = reinterpret_cast<const double2_t*>(Za + mr * lda + i0 + lc);
            const double2_t* pb = reinterpret_cast<const double2_t*>(Z + mr * ldz + j0 + lc);
            // nothing may consume the loaded values before the MFMAs of the current panel
            // have been issued, so the zeroing of tail rows happens at the LDS store
            loaded_rowok = rowok;
#pragma unroll
            for (int q = 0; q < UN; ++q) ra[q] = pa[q];
            if (!same) {
#pragma unroll
                for (int q = 0; q < UN; ++q) rb[q] = pb[q];
            }
        } else {
            const double* zr = Z + (size_t)m * ldz;
            const double* zar = Za + (size_t)m * lda;
#pragma unroll
            for (int q = 0; q < UN; ++q) {
                const int ca = i0 + lc + 2 * q;
                ra[q].x = (rowok && ca < ilim) ? zar[ca] : 0.0;
                ra[q].y = (rowok && ca + 1 < ilim) ? zar[ca + 1] : 0.0;
                const int cb = j0 + lc + 2 * q;
                rb[q].x = (rowok && cb < F) ? zr[cb] : 0.0;
                rb[q].y = (rowok && cb + 1 < F) ? zr[cb + 1] : 0.0;
            }
        }
    };
    auto store_panels = [&](int buf) {
        double2_t* da = reinterpret_cast<double2_t*>(&sA[buf][lr][lc]);
        double2_t* db = reinterpret_cast<double2_t*>(&sB[buf][lr][lc]);
        if (__builtin_expect(loaded_rowok, 1)) {
#pragma unroll
            for (int q = 0; q < UN; ++q) da[q] = ra[q];
            if (!same) {
#pragma unroll
                for (int q = 0; q < UN; ++q) db[q] = rb[q];
            }
        } else {   // a row past the end of Z (last step only) contributes zeros
            const double2_t zero = {0.0, 0.0};
#pragma unroll
            for (int q = 0; q < UN; ++q) da[q] = zero;
            if (!same) {
#pragma unroll
                for (int q = 0; q < UN; ++q) db[q] = zero;
            }
        }
    };

    const int nsteps = (M + KB - 1) / KB;
    load_panels(0);
    store_panels(0);
    __syncthreads();
    for (int step = 0; step < nsteps; ++step) {
        const int cur = step & 1;
        const double(*pa)[LDS_STRIDE] = sA[cur];
        const double(*pb)[LDS_STRIDE] = same ? sA[cur] : sB[cur];
        if (step + 1 < nsteps) load_panels((step + 1) * KB);   // in flight during the MFMAs
#pragma unroll
        for (int kk = 0; kk < KB; kk += 4) {
            double fa[4], fb[NQ];
#pragma unroll
            for (int p = 0; p < 4; ++p) fa[p] = pa[kk + lk][wi + p * 16 + l16];
#pragma unroll
            for (int q = 0; q < NQ; ++q) fb[q] = pb[kk + lk][wj + q * 16 + l16];
#pragma unroll
            for (int p = 0; p < 4; ++p)
#pragma unroll
                for (int q = 0; q < NQ; ++q)
                    acc[p][q] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[p], fb[q], acc[p][q], 0, 0, 0);
        }
        // the other copy was last read in the previous step, which every wavefront left
        // through the barrier below
        if (step + 1 < nsteps) store_panels(cur ^ 1);
        __syncthreads();
    }

    // accumulator layout of v_mfma_f64_16x16x4_f64 (measured on gfx950): register r of a
    // lane holds row lane/16 + 4r of column lane%16
#pragma unroll
    for (int p = 0; p < 4; ++p) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int gi = i0 + wi + p * 16 + lk + 4 * r;
                const int gj = j0 + wj + q * 16 + l16;
                if (gi < ilim && gj < F) {
                    const double v = sign * acc[p][q][r];
                    if (split) {
                        C[(size_t)blockIdx.x * (TILE * TILE) + (size_t)(gi - i0) * TILE + (gj - j0)] = v;
                    } else if (SYM) {
                        C[(size_t)gi * ldc + gj] += v;             // the mirror image is a separate pass
                    } else if (overwrite) {
                        C[(size_t)(gi - f0) * ldc + gj] = v;
                    } else {
                        C[(size_t)(gi - f0) * ldc + gj] += v;
                    }
                }
            }
        }
    }
}

// C[j,i] = C[i,j] for every element of the tiles strictly above the diagonal (32x32 blocks
// transposed through LDS, both sides coalesced).  The symmetric kernel accumulates only tiles
// on or above the diagonal; copying instead of adding twice keeps the two triangles
// bit-identical and replaces 128-byte-strided read-modify-writes in the kernel's epilogue.
constexpr int MT = 32;
__global__ __launch_bounds__(256) void gram_mirror_kernel(double* __restrict__ C, int F) {
    __shared__ double t[MT][MT + 1];
    const int bi = blockIdx.y, bj = blockIdx.x;            // block row / column, 32 x 32 each
    if (bi / (TILE / MT) >= bj / (TILE / MT)) return;      // only tiles strictly above the diagonal
    const int tx = threadIdx.x % MT, ty = threadIdx.x / MT;
    for (int r = ty; r < MT; r += 256 / MT) {
        const int gi = bi * MT + r, gj = bj * MT + tx;
        t[r][tx] = (gi < F && gj < F) ? C[(size_t)gi * F + gj] : 0.0;
    }
    __syncthreads();
    for (int r = ty; r < MT; r += 256 / MT) {
        const int gj = bj * MT + r, gi = bi * MT + tx;
        if (gi < F && gj < F) C[(size_t)gj * F + gi] = t[tx][r];
    }
}

// C tile += the partial tiles of its row ranges, added in the order of the ranges (split launch of the
// last tiles of the symmetric mode); one workgroup per tile id from tail_first on
__global__ __launch_bounds__(256) void gram_tail_reduce_kernel(const double* __restrict__ ws, int nt, TileMap tm, int F,
                                                                double* __restrict__ C, long long ldc) {
    int ti, tj;
    tile_of_block<true>(tm.tail_first + blockIdx.x, nt, nt, tm, ti, tj);
    if (ti < 0 || ti > tj) return;
    const double* w = ws + (size_t)blockIdx.x * tm.pieces * (TILE * TILE);
    for (int e = threadIdx.x; e < TILE * TILE; e += 256) {
        const int gi = ti * TILE + e / TILE, gj = tj * TILE + e % TILE;
        if (gi < F && gj < F) {
            double sum = 0.0;
            for (int p = 0; p < tm.pieces; ++p) sum += w[(size_t)p * (TILE * TILE) + e];
            C[(size_t)gi * ldc + gj] += sum;
        }
    }
}

// ZTy[f] += sum_m Z[m,f] y[m] for f in [f0,f1): thread = feature, rows split over grid.y
constexpr int GV_ROWS = 512;
__global__ __launch_bounds__(256) void gemv_t_kernel(const double* __restrict__ Z, const double* __restrict__ y, int M,
                                                      int F, int f0, int f1, double* __restrict__ out) {
    const int f = f0 + blockIdx.x * 256 + threadIdx.x;
    if (f >= f1) return;
    const int m0 = blockIdx.y * GV_ROWS;
    const int m1 = min(M, m0 + GV_ROWS);
    double s = 0.0;
    for (int m = m0; m < m1; ++m) s = fma(Z[(size_t)m * F + f], y[m], s);
    unsafeAtomicAdd(&out[f], s);
}

// C += double(A.B) with the fp32 Kahan inner sum of the reference (utils_kernel.cu:104-117)
constexpr int MR = 16;
__global__ __launch_bounds__(MR* MR) void matmul_and_reduce_kernel(const float* __restrict__ A,
                                                                   const float* __restrict__ B, int Ar, int K, int Bc,
                                                                   double* __restrict__ C) {
    __shared__ float As[MR][MR + 1];
    __shared__ float Bs[MR][MR + 1];
    const int tx = threadIdx.x % MR, ty = threadIdx.x / MR;
    const int row = blockIdx.y * MR + ty, col = blockIdx.x * MR + tx;
    float sum = 0.0f, c = 0.0f;
    for (int k0 = 0; k0 < K; k0 += MR) {
        As[ty][tx] = (row < Ar && k0 + tx < K) ? A[(size_t)row * K + k0 + tx] : 0.0f;
        Bs[ty][tx] = (k0 + ty < K && col < Bc) ? B[(size_t)(k0 + ty) * Bc + col] : 0.0f;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < MR; ++k) {
            const float yv = __builtin_fmaf(As[ty][k], Bs[k][tx], -c);
            const float t = sum + yv;
            c = (t - sum) - yv;
            sum = t;
        }
        __syncthreads();
    }
    if (row < Ar && col < Bc) C[(size_t)row * Bc + col] += (double)sum;
}

}  // namespace

// Z: M rows of F used columns, row stride ldz; C: row stride ldc; C += sign * Z^T Z
// bytes of workspace that let the symmetric launch split its last tiles (see below): at most one
// workgroup slot's worth of partial tiles, ids without a tile included
constexpr size_t GRAM_WS_TILES = 1024;
constexpr size_t GRAM_WS_BYTES = GRAM_WS_TILES * TILE * TILE * sizeof(double);

static int gram_launch(const double* Z, const double* y, int M, int F, int f0, int f1, bool sym, bool mirror, double* C,
                       double* ZTy, hipStream_t stream, const char* who, long long ldz = 0, long long ldc = 0,
                       double sign = 1.0, const double* Za = nullptr, long long lda = 0, int overwrite = 0,
                       double* ws = nullptr, size_t ws_bytes = 0) {
    if (ldz == 0) ldz = F;
    if (ldc == 0) ldc = F;
    if (!Za) {   // the Gram product: both operands are Z
        Za = Z;
        lda = ldz;
    }
    QMLL_REQUIRE(M >= 0 && F > 0, QMLL_ERR_INVALID, "%s: bad size M=%d F=%d", who, M, F);
    QMLL_REQUIRE(0 <= f0 && f0 < f1 && (f1 <= F || (Za && Za != Z)), QMLL_ERR_INVALID,
                 "%s: bad feature range [%d,%d) of %d", who, f0, f1, F);
    if (M == 0) return QMLL_OK;
    QMLL_REQUIRE(Z && C, QMLL_ERR_INVALID, "%s: null pointer", who);
    QMLL_REQUIRE((y == nullptr) == (ZTy == nullptr), QMLL_ERR_INVALID, "%s: y and ZTy must both be given or both be NULL",
                 who);
    const int ntj = (F + TILE - 1) / TILE;
    const int nti = sym ? ntj : (f1 - f0 + TILE - 1) / TILE;
    // super-tiles are dealt round-robin to the XCDs; ids of tiles outside the matrix exit at once
    long long per_xcd;
    TileMap tm = gram_tile_map(nti, ntj, sym, per_xcd);
    long long nblocks = per_xcd * NXCD;
    QMLL_REQUIRE(nblocks < 2147483647LL, QMLL_ERR_INVALID, "%s: too many tiles", who);
    // The tiles run in rounds of one per workgroup slot (two per CU); when the last round is less
    // than half full its tiles are cut into row ranges that fill the slots, each range writing a
    // partial tile to the workspace, and a small kernel adds the partial tiles in the order of the
    // ranges: the sums stay deterministic.  At F = 16 384 that is 64 of 8256 tiles in 8 ranges each,
    // 16.1 rounds instead of 17.
    TileMap tail = tm;
    long long ntail_ids = 0;
    if (sym && ws && M >= 2048) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) {
            const long long slots = 2LL * cus;
            const long long ntiles = (long long)ntj * (ntj + 1) / 2;
            const long long left = ntiles % slots;
            if (ntiles > slots && left > 0 && 2 * left <= slots) {
                // the ids of the last `left` tiles (ids past the last tile or without one are skipped over)
                long long b = nblocks, found = 0;
                while (b > 0 && found < left) {
                    int ti, tj;
                    tile_of_block<true>((unsigned)(b - 1), nti, ntj, tm, ti, tj);
                    if (ti >= 0 && ti <= tj) ++found;
                    --b;
                }
                const long long ids = nblocks - b;
                long long pieces = slots / left;
                if (pieces > 8) pieces = 8;
                if (found == left && pieces > 1 && (size_t)(ids * pieces) * TILE * TILE * sizeof(double) <= ws_bytes) {
                    tail.pieces = (int)pieces;
                    tail.piece_rows = (int)((((long long)M + pieces - 1) / pieces + KB - 1) / KB * KB);
                    tail.tail_first = (unsigned)b;
                    ntail_ids = ids;
                    nblocks = b;      // the ordinary launch stops before the tail
                }
            }
        }
    }
    const bool guard = (F % TILE) != 0 || ((f1 - f0) % TILE) != 0 || (f0 % 2) != 0 || (ldz % 2) != 0 ||
                       (lda % 2) != 0 || (reinterpret_cast<uintptr_t>(Z) % 16) != 0 ||
                       (reinterpret_cast<uintptr_t>(Za) % 16) != 0;
    const dim3 grid((unsigned)nblocks), block(GT);
    const bool gen = Za != Z || ldz != F || ldc != F || lda != F || sign != 1.0 || overwrite != 0;
#define QMLL_GRAM_LAUNCH(S, G, E)                                                                              \
    hipLaunchKernelGGL((gram_kernel<S, G, E>), grid, block, 0, stream, Z, M, F, sym ? 0 : f0, sym ? F : f1, nti, \
                       ntj, tm, C, ldz, ldc, sign, Za, lda, overwrite)
    if (gen) {
        if (sym && !guard) QMLL_GRAM_LAUNCH(true, false, true);
        else if (sym) QMLL_GRAM_LAUNCH(true, true, true);
        else if (!guard) QMLL_GRAM_LAUNCH(false, false, true);
        else QMLL_GRAM_LAUNCH(false, true, true);
    } else {
        if (sym && !guard) QMLL_GRAM_LAUNCH(true, false, false);
        else if (sym) QMLL_GRAM_LAUNCH(true, true, false);
        else if (!guard) QMLL_GRAM_LAUNCH(false, false, false);
        else QMLL_GRAM_LAUNCH(false, true, false);
    }
#undef QMLL_GRAM_LAUNCH
    QMLL_CHECK_LAUNCH(who);
    if (ntail_ids > 0) {
        const dim3 tgrid((unsigned)(ntail_ids * tail.pieces));
        if (guard)
            hipLaunchKernelGGL((gram_kernel<true, true, true>), tgrid, block, 0, stream, Z, M, F, 0, F, nti, ntj, tail, ws,
                               ldz, ldc, sign, Za, lda, overwrite);
        else
            hipLaunchKernelGGL((gram_kernel<true, false, true>), tgrid, block, 0, stream, Z, M, F, 0, F, nti, ntj, tail, ws,
                               ldz, ldc, sign, Za, lda, overwrite);
        QMLL_CHECK_LAUNCH(who);
        hipLaunchKernelGGL(gram_tail_reduce_kernel, dim3((unsigned)ntail_ids), dim3(256), 0, stream, ws, ntj, tail, F, C, ldc);
        QMLL_CHECK_LAUNCH(who);
    }
    if (sym && mirror && ldc == F) {
        const unsigned nb = (unsigned)((F + MT - 1) / MT);
        hipLaunchKernelGGL(gram_mirror_kernel, dim3(nb, nb), dim3(256), 0, stream, C, F);
        QMLL_CHECK_LAUNCH(who);
    }
    if (y) {
        dim3 grid((f1 - f0 + 255) / 256, (M + GV_ROWS - 1) / GV_ROWS);
        hipLaunchKernelGGL(gemv_t_kernel, grid, dim3(256), 0, stream, Z, y, M, F, f0, f1, ZTy);
        QMLL_CHECK_LAUNCH(who);
    }
    return QMLL_OK;
}

extern "C" int qmll_gram_f64(const double* Z, const double* y, int M, int F, double* ZTZ, double* ZTy,
                             qmll_stream_t stream) {
    return gram_launch(Z, y, M, F, 0, F > 0 ? F : 1, true, true, ZTZ, ZTy, (hipStream_t)stream, "qmll_gram_f64");
}

extern "C" int qmll_gram_upper_f64(const double* Z, const double* y, int M, int F, double* ZTZ, double* ZTy,
                                   qmll_stream_t stream) {
    return gram_launch(Z, y, M, F, 0, F > 0 ? F : 1, true, false, ZTZ, ZTy, (hipStream_t)stream, "qmll_gram_upper_f64");
}

extern "C" size_t qmll_gram_workspace_bytes(void) { return GRAM_WS_BYTES; }

extern "C" int qmll_gram_upper_ws_f64(const double* Z, const double* y, int M, int F, double* ZTZ, double* ZTy,
                                      double* workspace, size_t workspace_bytes, qmll_stream_t stream) {
    return gram_launch(Z, y, M, F, 0, F > 0 ? F : 1, true, false, ZTZ, ZTy, (hipStream_t)stream, "qmll_gram_upper_ws_f64", 0, 0,
                       1.0, nullptr, 0, 0, workspace, workspace_bytes);
}

extern "C" int qmll_gram_mirror_f64(double* ZTZ, int F, qmll_stream_t stream) {
    QMLL_REQUIRE(F > 0, QMLL_ERR_INVALID, "qmll_gram_mirror_f64: bad size F=%d", F);
    QMLL_REQUIRE(ZTZ, QMLL_ERR_INVALID, "qmll_gram_mirror_f64: null pointer");
    const unsigned nb = (unsigned)((F + MT - 1) / MT);
    QMLL_REQUIRE(nb <= 65535, QMLL_ERR_INVALID, "qmll_gram_mirror_f64: F=%d too large", F);
    hipLaunchKernelGGL(gram_mirror_kernel, dim3(nb, nb), dim3(256), 0, (hipStream_t)stream, ZTZ, F);
    QMLL_CHECK_LAUNCH("qmll_gram_mirror_f64");
    return QMLL_OK;
}

extern "C" int qmll_gram_tile_f64(const double* Z, const double* y, int M, int F, int f0, int f1, double* ZTZ_tile,
                                  double* ZTy, qmll_stream_t stream) {
    return gram_launch(Z, y, M, F, f0, f1, false, false, ZTZ_tile, ZTy, (hipStream_t)stream, "qmll_gram_tile_f64");
}

extern "C" int qmll_matmul_and_reduce(const float* A, const float* B, int Ar, int K, int Bc, double* C,
                                      qmll_stream_t stream) {
    QMLL_REQUIRE(Ar >= 0 && K >= 0 && Bc >= 0, QMLL_ERR_INVALID, "qmll_matmul_and_reduce: bad size %d %d %d", Ar, K, Bc);
    if (Ar == 0 || Bc == 0) return QMLL_OK;
    QMLL_REQUIRE(A && B && C, QMLL_ERR_INVALID, "qmll_matmul_and_reduce: null pointer");
    dim3 grid((Bc + MR - 1) / MR, (Ar + MR - 1) / MR);
    QMLL_REQUIRE(grid.y <= 65535, QMLL_ERR_INVALID, "qmll_matmul_and_reduce: too many rows (%d)", Ar);
    hipLaunchKernelGGL(matmul_and_reduce_kernel, grid, dim3(MR * MR), 0, (hipStream_t)stream, A, B, Ar, K, Bc, C);
    QMLL_CHECK_LAUNCH("qmll_matmul_and_reduce");
    return QMLL_OK;
}

// used by solve.hip: tiles on or above the diagonal of C[n,n] += sign * Z^T Z with strided operands
int qmll_internal_syrk_upper(const double* Z, int M, int n, long long ldz, double* C, long long ldc, double sign,
                             hipStream_t stream) {
    return gram_launch(Z, nullptr, M, n, 0, n, true, false, C, nullptr, stream, "qmll_cholesky_f64", ldz, ldc, sign);
}

// used by solve.hip: C[ra, n] (row stride ldc) = or += sign * Za^T Zb, Za = M rows of ra columns
// (row stride lda), Zb = M rows of n columns (row stride ldb).  With overwrite set and
// ra <= 128, C may be Zb itself: one workgroup owns each 128-column strip and reads all of it
// before it writes.
int qmll_internal_gemm_tn(const double* Za, long long lda, int ra, const double* Zb, long long ldb, int n, int M,
                          double* C, long long ldc, double sign, int overwrite, hipStream_t stream) {
    return gram_launch(Zb, nullptr, M, n, 0, ra, false, false, C, nullptr, stream, "qmll_cholesky_f64", ldb, ldc, sign,
                       Za, lda, overwrite);
}
