// Random Fourier features and their derivative rows (fp64, as the reference's training
// route computes them).  Replaces qml_lightning/cuda/random_features_kernel.cu:5-94.
//
// Thread = feature column f; a workgroup owns 256 consecutive features and a chunk of
// rows (atoms, or the 3 x TJ derivative rows of one atom), whose fp32 inputs sit in LDS
// and are read by broadcast, so each W[k,f] load (coalesced over the workgroup) is reused
// for every row of the chunk.
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
                                            const int* mol_index, int A, int n, int d, int F, int nmol, double* G,
                                            qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && n >= 0 && d > 0 && F > 0 && nmol >= 0, QMLL_ERR_INVALID,
                 "qmll_rff_derivative_features: bad size A=%d n=%d d=%d F=%d", A, n, d, F);
    if (A == 0 || n == 0) return QMLL_OK;
    QMLL_REQUIRE(x && grad && W && b && mol_index && G, QMLL_ERR_INVALID, "qmll_rff_derivative_features: null pointer");
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
