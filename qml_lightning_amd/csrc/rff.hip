// Random Fourier features and their derivative rows (fp64, as the reference's training
// route computes them).  Replaces qml_lightning/cuda/random_features_kernel.cu:5-94.
//
// Two kinds of kernels:
//  * thread = feature column f; a workgroup owns 256 consecutive features and a chunk of
//    rows (atoms, or the 3 x TJ derivative rows of one atom), whose fp32 inputs sit in LDS
//    and are read by broadcast, so each W[k,f] load (coalesced over the workgroup) is reused
//    for every row of the chunk.  Any atom order; molecule sums through fp64 atomics.
//  * rff_derivative_mfma_kernel, for molecule-major atoms: a workgroup owns (molecule, 64
//    feature columns, up to 63 derivative rows).  Each wavefront keeps its 16 columns of W as
//    MFMA B fragments in registers for the whole molecule; per atom the 63 derivative rows
//    plus the atom's own x row (whose product is the sine argument) form one 64 x d A tile
//    in LDS, multiplied with v_mfma_f64_16x16x4_f64; the per-atom product is scaled by the
//    sine column factor and summed over the molecule's atoms in registers, so G is
//    read-modify-written once per element and no atomics are needed.
#include "qmll_common.h"

namespace {

constexpr int RT = 256;     // threads = features per workgroup
constexpr int RA = 8;       // atoms per workgroup (features kernel)
constexpr int TJ = 8;       // target atoms per workgroup (derivative kernel)

__global__ __launch_bounds__(RT) void rff_features_kernel(const float* __restrict__ x, const double* __restrict__ W,
                                                           const double* __restrict__ b,
                                                           const int* __restrict__ mol_index, int A, int d, int F,
                                                           int nmol, double* __restrict__ Zf) {
    extern __shared__ float sx[];   // [RA][d]
    const int a0 = blockIdx.x * RA;
    const int na = min(RA, A - a0);
    for (int t = threadIdx.x; t < na * d; t += RT) sx[t] = x[(size_t)a0 * d + t];
    __syncthreads();
    const int f = blockIdx.y * RT + threadIdx.x;
    if (f >= F) return;
    double acc[RA];
#pragma unroll
    for (int r = 0; r < RA; ++r) acc[r] = 0.0;
    for (int k = 0; k < d; ++k) {
        const double w = W[(size_t)k * F + f];
#pragma unroll
        for (int r = 0; r < RA; ++r)
            if (r < na) acc[r] = fma((double)sx[r * d + k], w, acc[r]);
    }
    const double norm = sqrt(2.0 / (double)F);
    const double bf = b[f];
    int cur = -1;
    double run = 0.0;
#pragma unroll
    for (int r = 0; r < RA; ++r) {
        if (r < na) {
            const int mol = mol_index[a0 + r];
            if (mol != cur) {
                if (cur >= 0 && cur < nmol) unsafeAtomicAdd(&Zf[(size_t)cur * F + f], run);
                cur = mol;
                run = 0.0;
            }
            run += norm * cos(acc[r] + bf);
        }
    }
    if (cur >= 0 && cur < nmol) unsafeAtomicAdd(&Zf[(size_t)cur * F + f], run);
}

__global__ __launch_bounds__(RT) void rff_derivative_kernel(const float* __restrict__ x, const float* __restrict__ grad,
                                                             const double* __restrict__ W, const double* __restrict__ b,
                                                             const int* __restrict__ mol_index, int n, int d, int F,
                                                             int nmol, int njc, double* __restrict__ G) {
    extern __shared__ float sm[];   // [d] x row, then [TJ*3][d] derivative rows
    float* sx = sm;
    float* sg = sm + d;
    const size_t a = blockIdx.x / njc;
    const int j0 = (blockIdx.x % njc) * TJ;
    const int nj = min(TJ, n - j0);
    for (int t = threadIdx.x; t < d; t += RT) sx[t] = x[a * d + t];
    for (int t = threadIdx.x; t < nj * 3 * d; t += RT) sg[t] = grad[((a * n + j0) * 3) * d + t];
    __syncthreads();
    const int mol = mol_index[a];
    const int f = blockIdx.y * RT + threadIdx.x;
    if (f >= F || mol < 0 || mol >= nmol) return;
    double s0 = 0.0;
    double acc[TJ * 3];
#pragma unroll
    for (int r = 0; r < TJ * 3; ++r) acc[r] = 0.0;
    for (int k = 0; k < d; ++k) {
        const double w = W[(size_t)k * F + f];
        s0 = fma((double)sx[k], w, s0);
#pragma unroll
        for (int r = 0; r < TJ * 3; ++r)
            if (r < nj * 3) acc[r] = fma((double)sg[r * d + k], w, acc[r]);
    }
    const double fd = sqrt(2.0 / (double)F) * sin(s0 + b[f]);
#pragma unroll
    for (int r = 0; r < TJ * 3; ++r) {
        if (r < nj * 3 && acc[r] != 0.0) {
            const int j = j0 + r / 3, c = r % 3;
            unsafeAtomicAdd(&G[(((size_t)mol * n + j) * 3 + c) * F + f], fd * acc[r]);
        }
    }
}

typedef double double4_t __attribute__((ext_vector_type(4)));

constexpr int MROWS = 64;   // A-tile rows: 63 derivative rows + the atom's x row
constexpr int MPAD = 4;     // floats of padding per LDS row: 16 rows x 4 k land in 64 distinct banks

// grid (ceil(F/64), nmol, ceil(3n/63)), 256 threads.
template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D <= 128 ? 2 : 1))) void rff_derivative_mfma_kernel(const float* __restrict__ x,
                                                                  const float* __restrict__ grad,
                                                                  const double* __restrict__ W,
                                                                  const double* __restrict__ b,
                                                                  const int* __restrict__ seg, int n, int F,
                                                                  double* __restrict__ G) {
    constexpr int LD = D + MPAD;
    constexpr int KS = D / 4;                 // MFMA k-steps
    constexpr int V4 = MROWS * D / 4 / 256;   // float4 loads per thread per tile
    __shared__ __attribute__((aligned(16))) float tile[MROWS * LD];

    const int mol = blockIdx.y;
    const int a_begin = seg[mol], a_end = seg[mol + 1];
    if (a_begin >= a_end) return;
    const int rows3n = 3 * n;
    const int row0 = blockIdx.z * (MROWS - 1);
    const int nrows = min(MROWS - 1, rows3n - row0);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int l16 = lane & 15, lk = lane >> 4;
    const int f = blockIdx.x * 64 + wave * 16 + l16;
    const bool fok = f < F;

    // B fragments of this wavefront's 16 columns, all of K, resident for the whole molecule
    double wreg[KS];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) wreg[kk] = fok ? W[(size_t)(kk * 4 + lk) * F + f] : 0.0;
    const double bf = fok ? b[f] : 0.0;
    const double norm = sqrt(2.0 / (double)F);

    double4_t gacc[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) gacc[p] = (double4_t){0.0, 0.0, 0.0, 0.0};

    // tile element owned by this thread in load slot v: float4 number v*256 + tid
    float4 stage[V4];
    auto fetch = [&](int a) {
#pragma unroll
        for (int v = 0; v < V4; ++v) {
            const int idx = v * 256 + threadIdx.x;
            const int row = idx / (D / 4), c4 = idx % (D / 4);
            float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row < nrows)
                val = *reinterpret_cast<const float4*>(grad + ((size_t)a * rows3n + row0 + row) * D + c4 * 4);
            else if (row == MROWS - 1)
                val = *reinterpret_cast<const float4*>(x + (size_t)a * D + c4 * 4);
            stage[v] = val;
        }
    };
    fetch(a_begin);
    for (int a = a_begin; a < a_end; ++a) {
        __syncthreads();   // the previous atom's fragments have been read
#pragma unroll
        for (int v = 0; v < V4; ++v) {
            const int idx = v * 256 + threadIdx.x;
            const int row = idx / (D / 4), c4 = idx % (D / 4);
            *reinterpret_cast<float4*>(&tile[row * LD + c4 * 4]) = stage[v];
        }
        __syncthreads();
        if (a + 1 < a_end) fetch(a + 1);   // in flight during the MFMAs

        double4_t pacc[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) pacc[p] = (double4_t){0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const double av = (double)tile[(p * 16 + l16) * LD + kk * 4 + lk];
                pacc[p] = __builtin_amdgcn_mfma_f64_16x16x4f64(av, wreg[kk], pacc[p], 0, 0, 0);
            }
        }
        // accumulator register r of a 16x16 block holds row lane/16 + 4r, column lane%16:
        // the x row (tile row 63) is register 3 of block 3 in lanes 48..63
        const double s0 = __shfl(pacc[3][3], 48 + l16, 64);
        const double fd = norm * sin(s0 + bf);
#pragma unroll
        for (int p = 0; p < 4; ++p) gacc[p] += fd * pacc[p];
    }
    if (!fok) return;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = p * 16 + lk + 4 * r;
            if (row < nrows) {
                double* dst = G + ((size_t)mol * rows3n + row0 + row) * F + f;
                *dst += gacc[p][r];
            }
        }
    }
}

}  // namespace

extern "C" int qmll_rff_features(const float* x, const double* W, const double* b, const int* mol_index, int A, int d,
                                 int F, int nmol, double* Zf, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && d > 0 && F > 0 && nmol >= 0, QMLL_ERR_INVALID, "qmll_rff_features: bad size A=%d d=%d F=%d", A,
                 d, F);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(x && W && b && mol_index && Zf, QMLL_ERR_INVALID, "qmll_rff_features: null pointer");
    QMLL_REQUIRE((size_t)RA * d * sizeof(float) <= 64 * 1024, QMLL_ERR_INVALID, "qmll_rff_features: d=%d too large", d);
    QMLL_REQUIRE((F + RT - 1) / RT <= 65535, QMLL_ERR_INVALID, "qmll_rff_features: F=%d too large", F);
    dim3 grid((A + RA - 1) / RA, (F + RT - 1) / RT);
    hipLaunchKernelGGL(rff_features_kernel, grid, dim3(RT), (size_t)RA * d * sizeof(float), (hipStream_t)stream, x, W, b,
                       mol_index, A, d, F, nmol, Zf);
    QMLL_CHECK_LAUNCH("qmll_rff_features");
    return QMLL_OK;
}

extern "C" int qmll_rff_derivative_features(const float* x, const float* grad, const double* W, const double* b,
                                            const int* mol_index, const int* seg_offsets, int A, int n, int d, int F,
                                            int nmol, double* G, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && n >= 0 && d > 0 && F > 0 && nmol >= 0, QMLL_ERR_INVALID,
                 "qmll_rff_derivative_features: bad size A=%d n=%d d=%d F=%d", A, n, d, F);
    if (A == 0 || n == 0 || nmol == 0) return QMLL_OK;
    QMLL_REQUIRE(x && grad && W && b && (mol_index || seg_offsets) && G, QMLL_ERR_INVALID,
                 "qmll_rff_derivative_features: null pointer");
    if (seg_offsets && (d == 64 || d == 128 || d == 256)) {
        const int rg = (3 * n + MROWS - 2) / (MROWS - 1);
        QMLL_REQUIRE(nmol <= 65535 && rg <= 65535, QMLL_ERR_INVALID,
                     "qmll_rff_derivative_features: grid too large (nmol=%d n=%d)", nmol, n);
        dim3 grid((F + 63) / 64, nmol, rg);
        if (d == 64)
            hipLaunchKernelGGL(rff_derivative_mfma_kernel<64>, grid, dim3(256), 0, (hipStream_t)stream, x, grad, W, b,
                               seg_offsets, n, F, G);
        else if (d == 128)
            hipLaunchKernelGGL(rff_derivative_mfma_kernel<128>, grid, dim3(256), 0, (hipStream_t)stream, x, grad, W, b,
                               seg_offsets, n, F, G);
        else
            hipLaunchKernelGGL(rff_derivative_mfma_kernel<256>, grid, dim3(256), 0, (hipStream_t)stream, x, grad, W, b,
                               seg_offsets, n, F, G);
        QMLL_CHECK_LAUNCH("qmll_rff_derivative_features");
        return QMLL_OK;
    }
    QMLL_REQUIRE(mol_index, QMLL_ERR_INVALID,
                 "qmll_rff_derivative_features: mol_index is needed when d=%d is not 64, 128 or 256", d);
    const size_t lds = (size_t)(1 + TJ * 3) * d * sizeof(float);
    QMLL_REQUIRE(lds <= 64 * 1024, QMLL_ERR_INVALID, "qmll_rff_derivative_features: d=%d too large", d);
    const int njc = (n + TJ - 1) / TJ;
    QMLL_REQUIRE((long long)A * njc < 2147483647LL && (F + RT - 1) / RT <= 65535, QMLL_ERR_INVALID,
                 "qmll_rff_derivative_features: grid too large");
    dim3 grid((unsigned)(A * njc), (F + RT - 1) / RT);
    hipLaunchKernelGGL(rff_derivative_kernel, grid, dim3(RT), lds, (hipStream_t)stream, x, grad, W, b, mol_index, n, d, F,
                       nmol, njc, G);
    QMLL_CHECK_LAUNCH("qmll_rff_derivative_features");
    return QMLL_OK;
}
