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


// ---- fused predict path ------------------------------------------------------------------
// e[a] = sqrt(2/F) sum_f alpha_f cos(x_a . W_t[:,f] + b_t[f]),  gx[a,:] = d e[a] / d x_a, for
// element-sorted rows x [A,d] (tiles of 128 atoms share the element t, so one W).  Replaces
// the per-element matmul + cos + index_add + matmul(alpha) of the reference's TorchScript
// forward (qml_lightning/models/random_features.py:88-100) and its autograd transpose
// without ever writing the [atoms, F] feature matrix.
//
// Two chained matrix-core products per 32-feature chunk of W (staged in LDS):
// S^T[f,a] = W^T x^T  ->  P[f,a] = -norm alpha_f sin(S + b_f)  ->  GX^T[k,a] += W P.
// Everything is kept transposed so that the accumulator registers of the first product (row
// = feature, column = atom) are exactly the B operand the second one needs (contraction
// index = feature): P never leaves the registers.  x^T (B operand of the first product)
// stays in registers for the whole kernel, GX^T in accumulators.
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int RE_T = 256;        // threads: 4 wavefronts x 32 atoms
constexpr int RE_M = 128;        // atoms per workgroup
constexpr int RE_FC = 32;        // features per staged chunk (one block of 32 rows)

// The products run on the half-precision matrix cores.  v_mfma_f32_32x32x16_f16 runs 13 times as fast per
// flop as v_mfma_f32_32x32x2_f32 (40 against 64 clocks for eight times the flops), so each fp32 operand is split into two fp16 parts (hi = the value
// rounded to fp16, lo = the rounded rest: 22 bits together) and a product becomes three matrix
// instructions, hi.hi + hi.lo + lo.hi, accumulated in fp32; lo.lo is below the rounding of the sum.
// fp16 has five exponent bits, so every operand is scaled by a power of two first (exact): x by the
// wavefront's 2^kx (largest |x| of its 32 atoms to [2^13, 2^14)), alpha by the workgroup's 2^kp (largest
// |alpha| norm of its feature range), every chunk of W by its own 2^kw (largest |W| of the chunk); the
// sine argument, the chunk's contribution to the gradient and the outputs take the inverse factors.
// fp16 subnormals are kept by the matrix cores, so small entries beside large ones lose only bits
// below 2^-38 of the largest.
//
// W is a constant of the model, so it is split ONCE (rff_presplit_kernel) into the very bytes the
// predict kernel wants in LDS: per element and 32-feature chunk an image holding the chunk twice,
// feature-major with k contiguous (A operand of the first product, rows = features) and k-major with
// the chunk's 32 features contiguous (A operand of the second, rows = k), the features in the order in
// which the first product's accumulator registers hold them (register r of half h: feature
// 8(r/4) + 4h + r%4), so the split P goes straight from registers into the B operand; hi and lo parts
// each, row padding included.  The predict kernel then moves an image into LDS with direct
// global-to-LDS loads (no registers, no vector instructions), the next chunk's while this one is
// multiplied.
template <int D>
struct RffImage {
    static constexpr int LD1 = D + 8;                // halves per row of the feature-major copy
    static constexpr int LD2 = RE_FC + 8;            // halves per row of the k-major copy
    static constexpr int W1H = 0, W1L = RE_FC * LD1, W2H = 2 * RE_FC * LD1, W2L = W2H + D * LD2;
    static constexpr int HALVES = W2L + D * LD2;
    static constexpr int BYTES = HALVES * 2;         // 37888 (D = 128), 19456 (D = 64): whole KiB
    static constexpr int BLOCKS = BYTES / 1024;      // 1 KiB = one wavefront's 64 x 16-byte load
    static_assert(BYTES % 1024 == 0, "an image is moved in 1 KiB blocks");
};

// One workgroup per (chunk, element): the chunk's power of two, then the image through LDS.
template <int D>
__global__ __launch_bounds__(RE_T) void rff_presplit_kernel(const float* __restrict__ W, int F, _Float16* __restrict__ images,
                                                            int* __restrict__ exponents) {
    using Img = RffImage<D>;
    constexpr int NP = D / 64;                // pairs of adjacent k rows staged per thread
    __shared__ __attribute__((aligned(16))) _Float16 img[Img::HALVES];
    __shared__ float swmax[RE_T / 64];
    const int chunk = blockIdx.x, type = blockIdx.y, nchunks = gridDim.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* Wt = W + (size_t)type * D * F;
    const int f0 = chunk * RE_FC;
    // thread -> features sf .. sf+3 of the rows k0 = 2 (tid / 8) + 64 p and k0 + 1
    const int sf = (tid & 7) * 4, skp = 2 * (tid >> 3);
    // place of features sf .. sf+3 in a row of the k-major copy: f = 16 t + 8 c + 4 h' + e -> 16 t + 8 h' + 4 c + e
    const int pos2 = (sf & 16) | ((sf & 4) << 1) | ((sf & 8) >> 1);
    float4 stage[NP][2];
    float m = 0.0f;
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            stage[p][r] = *reinterpret_cast<const float4*>(Wt + (size_t)(skp + 64 * p + r) * F + f0 + sf);
            m = fmaxf(fmaxf(fmaxf(m, fabsf(stage[p][r].x)), fmaxf(fabsf(stage[p][r].y), fabsf(stage[p][r].z))),
                      fabsf(stage[p][r].w));
        }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if (lane == 0) swmax[wave] = m;
    for (int t = tid; t < Img::HALVES / 2; t += RE_T) reinterpret_cast<unsigned*>(img)[t] = 0u;    // row padding
    __syncthreads();
    const int kw = scale_exponent(fmaxf(fmaxf(swmax[0], swmax[1]), fmaxf(swmax[2], swmax[3])));
    const float sw = pow2i(kw);
    if (tid == 0) exponents[type * nchunks + chunk] = kw;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int k0 = skp + 64 * p;
        const float w0[4] = {stage[p][0].x * sw, stage[p][0].y * sw, stage[p][0].z * sw, stage[p][0].w * sw};
        const float w1[4] = {stage[p][1].x * sw, stage[p][1].y * sw, stage[p][1].z * sw, stage[p][1].w * sw};
        half4_t r0h, r0l, r1h, r1l;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            _Float16 a, c;
            split_f16(w0[e], a, c);
            r0h[e] = a; r0l[e] = c;
            split_f16(w1[e], a, c);
            r1h[e] = a; r1l[e] = c;
            *reinterpret_cast<half2_t*>(&img[Img::W1H + (sf + e) * Img::LD1 + k0]) = (half2_t){r0h[e], r1h[e]};
            *reinterpret_cast<half2_t*>(&img[Img::W1L + (sf + e) * Img::LD1 + k0]) = (half2_t){r0l[e], r1l[e]};
        }
        *reinterpret_cast<half4_t*>(&img[Img::W2H + k0 * Img::LD2 + pos2]) = r0h;
        *reinterpret_cast<half4_t*>(&img[Img::W2L + k0 * Img::LD2 + pos2]) = r0l;
        *reinterpret_cast<half4_t*>(&img[Img::W2H + (k0 + 1) * Img::LD2 + pos2]) = r1h;
        *reinterpret_cast<half4_t*>(&img[Img::W2L + (k0 + 1) * Img::LD2 + pos2]) = r1l;
    }
    __syncthreads();
    float4* dst = reinterpret_cast<float4*>(images + (size_t)(type * nchunks + chunk) * Img::HALVES);
    for (int t = tid; t < Img::BYTES / 16; t += RE_T) dst[t] = reinterpret_cast<const float4*>(img)[t];
}

template <int D, bool WITH_GRAD>
__global__ __launch_bounds__(RE_T) __attribute__((amdgpu_waves_per_eu(2))) void rff_energy_sorted_f16_kernel(
    const float* __restrict__ x, const int* __restrict__ type_offsets, const int* __restrict__ sorted_slots,
    const _Float16* __restrict__ images, const int* __restrict__ exponents, const float* __restrict__ b,
    const float* __restrict__ alpha, int ne, int F, float norm, float* __restrict__ e_slots, float* __restrict__ gx) {
    using Img = RffImage<D>;
    constexpr int LD1 = Img::LD1, LD2 = Img::LD2;
    constexpr int KS = D / 16;                // matrix instructions along k per product term
    // two images, this chunk's and the next one's, as two arrays of their own: the compiler then knows
    // that the loads into one do not touch what is read from the other and does not wait for them
    __shared__ __attribute__((aligned(16))) _Float16 simg0[Img::HALVES], simg1[Img::HALVES];
    __shared__ __attribute__((aligned(16))) float sba[2 * 2 * RE_FC];     // [2][2][RE_FC]: b / 2 pi, alpha norm 2^kp of the two chunks

    int type = -1, row0 = 0, rows = 0;
    {
        int bidx = blockIdx.x;
        for (int t = 0; t < ne; ++t) {
            const int o0 = type_offsets[t], o1 = type_offsets[t + 1];
            const int nt = (o1 - o0 + RE_M - 1) / RE_M;
            if (bidx < nt) {
                type = t;
                row0 = o0 + bidx * RE_M;
                rows = min(RE_M, o1 - row0);
                break;
            }
            bidx -= nt;
        }
    }
    if (type < 0) return;
    const float* bt = b + (size_t)type * F;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 31, h = lane >> 5;
    const int arow = 32 * wave + i;
    const bool aok = arow < rows;
    const int fsplit = F / (int)gridDim.y;
    const int fbeg = (int)blockIdx.y * fsplit, fend = fbeg + fsplit;
    const int nchunks = F / RE_FC;
    // a scalar base and one per-lane offset: the loads then need no per-lane 64-bit addresses
    const unsigned char* img0 = reinterpret_cast<const unsigned char*>(images) + (size_t)type * nchunks * Img::BYTES;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const unsigned lane16 = (unsigned)lane * 16u;
    const int* kws = exponents + type * nchunks;
    // chunk `c` of this element into LDS copy `par`: every wavefront moves the 1 KiB blocks wave, wave + 4, ...
    // (64 lanes x 16 bytes per instruction, written to LDS at block start + 16 lane)
    auto dma = [&](int c, _Float16* to) {
        const unsigned char* src = img0 + (size_t)c * Img::BYTES;
        unsigned char* dst = reinterpret_cast<unsigned char*>(to);
#pragma unroll
        for (int u0 = 0; u0 < Img::BLOCKS; u0 += RE_T / 64) {
            const int u = u0 + wave_s;
            if (u < Img::BLOCKS)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + u * 1024 + lane16),
                                                 (__attribute__((address_space(3))) void*)(dst + u * 1024), 16, 0, 0);
        }
    };
    dma(fbeg / RE_FC, simg0);

    // x^T as the B operand of the first product: instruction j contracts k = 16 j + 8 h + (0..7)
    half8_t xh[KS], xl[KS];
    float inv_sx;
    {
        float xv[KS][8];
        const float* xr = x + (size_t)(row0 + (aok ? arow : 0)) * D + 8 * h;
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            const float4 v0 = aok ? *reinterpret_cast<const float4*>(xr + 16 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 v1 = aok ? *reinterpret_cast<const float4*>(xr + 16 * j + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
            xv[j][0] = v0.x; xv[j][1] = v0.y; xv[j][2] = v0.z; xv[j][3] = v0.w;
            xv[j][4] = v1.x; xv[j][5] = v1.y; xv[j][6] = v1.z; xv[j][7] = v1.w;
#pragma unroll
            for (int q = 0; q < 8; ++q) m = fmaxf(m, fabsf(xv[j][q]));
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
        if (__builtin_expect(not_finite(m), 0)) {        // an infinity among the rows: the largest finite entry
            m = 0.0f;
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int q = 0; q < 8; ++q) m = fmaxf(m, finite_abs(xv[j][q]));
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
        }
        const int kx = scale_exponent(m);
        const float sx = pow2i(kx);
        inv_sx = pow2i(-kx);
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                _Float16 a, c;
                split_f16(xv[j][q] * sx, a, c);
                xh[j][q] = a;
                xl[j][q] = c;
            }
    }
    // the workgroup's alpha scale (every wavefront finds the same value)
    float sp, inv_sp;
    {
        float m = 0.0f;
        for (int f = fbeg + lane; f < fend; f += 64) m = fmaxf(m, fabsf(alpha[f]));
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
        const int kp = scale_exponent(m * norm);
        sp = pow2i(kp);
        inv_sp = pow2i(-kp);
    }
    if (tid < RE_FC) {
        sba[tid] = bt[fbeg + tid] * 0.15915494309189535f;
        sba[RE_FC + tid] = alpha[fbeg + tid] * norm * sp;
    }

    float16_t gacc[D / 32];
    if constexpr (WITH_GRAD) {
#pragma unroll
        for (int blk = 0; blk < D / 32; ++blk)
#pragma unroll
            for (int r = 0; r < 16; ++r) gacc[blk][r] = 0.0f;
    }
    float energy = 0.0f;

    // one chunk: `img` holds it, the next one is loaded into `other`
    auto round = [&](int f0, int par, const _Float16* img, _Float16* other) {
        const bool more = f0 + RE_FC < fend;
        // this chunk's image has landed (every wavefront waits for its own loads, then for the others),
        // and the other copy, read in the round before, is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // b and alpha of the next chunk are requested before its image so that waiting for them does
        // not wait for the image; they go to LDS at the end of the round
        float bnext = 0.0f, anext = 0.0f;
        if (more && tid < RE_FC) {
            bnext = bt[f0 + RE_FC + tid];
            anext = alpha[f0 + RE_FC + tid];
        }
        if (more) dma(f0 / RE_FC + 1, other);
        const _Float16 *sW1h = img + Img::W1H, *sW1l = img + Img::W1L, *sW2h = img + Img::W2H, *sW2l = img + Img::W2L;
        const float* sb = sba + par * 2 * RE_FC;
        const float* sa = sb + RE_FC;
        const int kw = kws[f0 / RE_FC];
        const float inv_sw = pow2i(-kw);

        // first product: 2^(kx + kw) S^T (32 features x 32 atoms)
        const float inv_sxw = inv_sx * inv_sw;
        float16_t sacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[r] = 0.0f;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            const half8_t ah = *reinterpret_cast<const half8_t*>(&sW1h[i * LD1 + 16 * j + 8 * h]);
            const half8_t al = *reinterpret_cast<const half8_t*>(&sW1l[i * LD1 + 16 * j + 8 * h]);
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, xh[j], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, xl[j], sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, xh[j], sacc, 0, 0, 0);
        }
        // accumulator register r: feature 8(r/4) + 4h + r%4 of the chunk, atom = lane%32.  The sine
        // argument is formed in REVOLUTIONS (b arrives divided by 2 pi, the product takes 1 / 2 pi with its
        // inverse scales): v_sin_f32 / v_cos_f32 reduce the range themselves up to 256 revolutions; the
        // rounding of the argument, |arg| 6e-8 radians, is that of an fp32 argument in radians.  Beyond
        // 1500 radians whole revolutions are taken off first (u - rint(u) is exact in fp32).
        constexpr float UMAX = 1500.0f * 0.15915494309189535f;
        const float crev = inv_sxw * 0.15915494309189535f;
        float umax = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 bv = *reinterpret_cast<const float4*>(&sb[8 * q + 4 * h]);
            const float bq[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                sacc[4 * q + e] = fmaf(sacc[4 * q + e], crev, bq[e]);
                umax = fmaxf(umax, fabsf(sacc[4 * q + e]));
            }
        }
        if (__builtin_expect(__any(umax > UMAX), 0)) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (fabsf(sacc[r]) > UMAX) sacc[r] -= rintf(sacc[r]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 av = *reinterpret_cast<const float4*>(&sa[8 * q + 4 * h]);
            const float aq[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float u = sacc[4 * q + e];
                const float sn = __builtin_amdgcn_sinf(u), cs = __builtin_amdgcn_cosf(u);
                energy = fmaf(aq[e], cs, energy);
                sacc[4 * q + e] = -aq[e] * sn;           // 2^kp P
            }
        }
        if constexpr (WITH_GRAD) {
            // second product: 2^kp GX^T[k, a] += 2^-kw sum_f 2^kw W[k, f] 2^kp P[f, a]; instruction t contracts the
            // features of registers 8 t .. 8 t + 7.  The chunk's contribution is summed from zero and
            // added to the running sums by the vector unit: the matrix instruction aligns its products
            // to the accumulator it is given, and against a sum over a thousand chunks their low bits
            // would be cut off
            half8_t ph[2], pl[2];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    _Float16 a, c;
                    split_f16(sacc[8 * t + q], a, c);
                    ph[t][q] = a;
                    pl[t][q] = c;
                }
#pragma unroll
            for (int blk = 0; blk < D / 32; ++blk) {
                float16_t part;
#pragma unroll
                for (int r = 0; r < 16; ++r) part[r] = 0.0f;
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const half8_t ah = *reinterpret_cast<const half8_t*>(&sW2h[(32 * blk + i) * LD2 + 16 * t + 8 * h]);
                    const half8_t al = *reinterpret_cast<const half8_t*>(&sW2l[(32 * blk + i) * LD2 + 16 * t + 8 * h]);
                    part = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, ph[t], part, 0, 0, 0);
                    part = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, pl[t], part, 0, 0, 0);
                    part = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, ph[t], part, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) gacc[blk][r] = fmaf(part[r], inv_sw, gacc[blk][r]);
            }
        }
        if (more && tid < RE_FC) {
            float* nb = sba + (par ^ 1) * 2 * RE_FC;
            nb[tid] = bnext * 0.15915494309189535f;
            nb[RE_FC + tid] = anext * norm * sp;
        }
    };
    for (int f0 = fbeg; f0 < fend; f0 += 2 * RE_FC) {
        round(f0, 0, simg0, simg1);
        if (f0 + RE_FC < fend) round(f0 + RE_FC, 1, simg1, simg0);
    }

    energy = (energy + __shfl_xor(energy, 32, 64)) * inv_sp;
    if (gridDim.y == 1) {
        if (h == 0 && aok) e_slots[sorted_slots[row0 + arow]] = energy;
        if constexpr (WITH_GRAD) {
            if (aok) {
                float* gr = gx + (size_t)(row0 + arow) * D;
#pragma unroll
                for (int blk = 0; blk < D / 32; ++blk)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        *reinterpret_cast<float4*>(gr + 32 * blk + 8 * q + 4 * h) =
                            make_float4(gacc[blk][4 * q] * inv_sp, gacc[blk][4 * q + 1] * inv_sp,
                                        gacc[blk][4 * q + 2] * inv_sp, gacc[blk][4 * q + 3] * inv_sp);
            }
        }
    } else {
        // the feature parts add into zero-filled outputs
        if (h == 0 && aok) atomicAdd(&e_slots[sorted_slots[row0 + arow]], energy);
        if constexpr (WITH_GRAD) {
            if (aok) {
                float* gr = gx + (size_t)(row0 + arow) * D;
#pragma unroll
                for (int blk = 0; blk < D / 32; ++blk)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        atomicAdd(gr + 32 * blk + 8 * (r / 4) + 4 * h + (r % 4), gacc[blk][r] * inv_sp);
            }
        }
    }
}

__global__ void zero_fill_kernel(float* __restrict__ p, size_t n) {
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (size_t)gridDim.x * blockDim.x) p[t] = 0.0f;
}

// rows past the last atom of a known element carry a zero gradient
__global__ void zero_tail_rows_kernel(const int* __restrict__ type_offsets, int ne, int A, int d, float* __restrict__ gx) {
    const int total = type_offsets[ne];
    const size_t n = (size_t)(A - total) * d;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (size_t)gridDim.x * blockDim.x)
        gx[(size_t)total * d + t] = 0.0f;
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

// bytes of the pre-split form of W [ne, d, F]: the images, then one exponent per image
static size_t rff_image_bytes(int d) { return d == 64 ? (size_t)RffImage<64>::BYTES : (size_t)RffImage<128>::BYTES; }

extern "C" size_t qmll_rff_presplit_bytes(int ne, int d, int F) {
    if (ne <= 0 || F <= 0 || F % RE_FC != 0 || (d != 64 && d != 128)) return 0;
    const size_t n = (size_t)ne * (F / RE_FC);
    return n * rff_image_bytes(d) + n * sizeof(int);
}

extern "C" int qmll_rff_presplit(const float* W, int ne, int d, int F, void* out, size_t out_bytes, qmll_stream_t stream) {
    QMLL_REQUIRE(ne > 0 && F > 0, QMLL_ERR_INVALID, "qmll_rff_presplit: bad size ne=%d F=%d", ne, F);
    QMLL_REQUIRE(d == 64 || d == 128, QMLL_ERR_INVALID, "qmll_rff_presplit: d=%d is not 64 or 128", d);
    QMLL_REQUIRE(F % RE_FC == 0, QMLL_ERR_INVALID, "qmll_rff_presplit: F=%d is not a multiple of %d", F, RE_FC);
    QMLL_REQUIRE(W && out, QMLL_ERR_INVALID, "qmll_rff_presplit: null pointer");
    QMLL_REQUIRE(out_bytes >= qmll_rff_presplit_bytes(ne, d, F), QMLL_ERR_INVALID,
                 "qmll_rff_presplit: output of %zu bytes, %zu are needed", out_bytes, qmll_rff_presplit_bytes(ne, d, F));
    QMLL_REQUIRE((((uintptr_t)W | (uintptr_t)out) & 15) == 0, QMLL_ERR_INVALID,
                 "qmll_rff_presplit: W and the output must be 16-byte aligned");
    const int nchunks = F / RE_FC;
    QMLL_REQUIRE(ne <= 65535, QMLL_ERR_INVALID, "qmll_rff_presplit: ne=%d too large", ne);
    _Float16* images = (_Float16*)out;
    int* exponents = (int*)((char*)out + (size_t)ne * nchunks * rff_image_bytes(d));
    const dim3 grid(nchunks, ne);
    if (d == 64)
        hipLaunchKernelGGL(rff_presplit_kernel<64>, grid, dim3(RE_T), 0, (hipStream_t)stream, W, F, images, exponents);
    else
        hipLaunchKernelGGL(rff_presplit_kernel<128>, grid, dim3(RE_T), 0, (hipStream_t)stream, W, F, images, exponents);
    QMLL_CHECK_LAUNCH("qmll_rff_presplit");
    return QMLL_OK;
}

extern "C" int qmll_rff_energy_sorted(const float* x, const int* type_offsets, const int* sorted_slots, const void* W_split,
                                      const float* b, const float* alpha, int A, int ne, int d, int F, float* e_slots,
                                      float* gx, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && ne > 0 && d > 0 && F > 0, QMLL_ERR_INVALID, "qmll_rff_energy_sorted: bad size A=%d ne=%d d=%d F=%d",
                 A, ne, d, F);
    QMLL_REQUIRE(d == 64 || d == 128, QMLL_ERR_INVALID, "qmll_rff_energy_sorted: d=%d is not 64 or 128", d);
    QMLL_REQUIRE(F % RE_FC == 0, QMLL_ERR_INVALID, "qmll_rff_energy_sorted: F=%d is not a multiple of %d", F, RE_FC);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(x && type_offsets && sorted_slots && W_split && b && alpha && e_slots, QMLL_ERR_INVALID,
                 "qmll_rff_energy_sorted: null pointer");
    QMLL_REQUIRE((((uintptr_t)x | (uintptr_t)W_split | (uintptr_t)gx) & 15) == 0, QMLL_ERR_INVALID,
                 "qmll_rff_energy_sorted: x, W_split and gx must be 16-byte aligned");
    const _Float16* images = (const _Float16*)W_split;
    const int* exponents = (const int*)((const char*)W_split + (size_t)ne * (F / RE_FC) * rff_image_bytes(d));
    const float norm = sqrtf(2.0f / (float)F);
    hipStream_t st = (hipStream_t)stream;
    // Two workgroups fit a CU (two wavefronts per SIMD) and all run the same chunk loop, so the launch takes ceil(workgroups / 512) rounds of 1/fs of a tile's work
    // when the features are split over fs workgroups per tile.  fs is the power of two up to
    // 64 with the shortest estimate (a larger one has to win by 5 %): 672 tiles take 2 rounds
    // with fs = 1 and 21/16 with fs = 16; one molecule takes 1/64 instead of 1.  For fs > 1
    // the parts add their energies and gradients into zero-filled outputs with fp32 atomics
    // (from fs = 4 on the order of the terms, hence the last bit, varies from run to run).
    const int tiles = (A + RE_M - 1) / RE_M, slots = 2 * 256;
    auto rounds = [&](int k) { return (double)(((long long)(tiles + ne) * k + slots - 1) / slots) / k; };
    int fs = 1;
    for (int k = 2; k <= 64 && F % (k * RE_FC) == 0; k *= 2)
        if (rounds(k) < 0.95 * rounds(fs)) fs = k;
    const dim3 grid(tiles + ne, fs);
    if (fs > 1 && gx) {
        hipLaunchKernelGGL(zero_fill_kernel, dim3(1024), dim3(256), 0, st, gx, (size_t)A * d);
        QMLL_CHECK_LAUNCH("qmll_rff_energy_sorted");
    }
#define CALL(DD)                                                                                                     \
    if (gx)                                                                                                          \
        hipLaunchKernelGGL((rff_energy_sorted_f16_kernel<DD, true>), grid, dim3(RE_T), 0, st, x, type_offsets,         \
                           sorted_slots, images, exponents, b, alpha, ne, F, norm, e_slots, gx);                      \
    else                                                                                                             \
        hipLaunchKernelGGL((rff_energy_sorted_f16_kernel<DD, false>), grid, dim3(RE_T), 0, st, x, type_offsets,        \
                           sorted_slots, images, exponents, b, alpha, ne, F, norm, e_slots, gx);
    if (d == 64) {
        CALL(64)
    } else {
        CALL(128)
    }
#undef CALL
    QMLL_CHECK_LAUNCH("qmll_rff_energy_sorted");
    if (gx) {
        hipLaunchKernelGGL(zero_tail_rows_kernel, dim3(64), dim3(256), 0, st, type_offsets, ne, A, d, gx);
        QMLL_CHECK_LAUNCH("qmll_rff_energy_sorted");
    }
    return QMLL_OK;
}
