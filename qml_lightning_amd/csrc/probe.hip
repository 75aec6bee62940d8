// Measured ceilings of the device the library runs on: plain fill and copy kernels (HBM), a loop
// of independent matrix-core instructions in fp64, fp32 and fp16, and a loop of independent
// transcendental instructions.  The benchmark divides each kernel's rate by these next to the
// nominal peaks; the copy kernel is also the known-size reference for scaling the FETCH_SIZE /
// WRITE_SIZE counters of a profiler run.  No counterpart in the reference.
#include "qmll_common.h"

namespace {

typedef double double4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

constexpr int PT = 256;

typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int UNR = 4;   // 16-byte accesses in flight per thread: a workgroup moves 16 KB

// streaming kernels: every thread issues UNR independent 16-byte accesses (consecutive threads
// touch consecutive 16 bytes), with the nontemporal hint the library's own streaming kernels use
__global__ __launch_bounds__(PT) void probe_fill_kernel(floatx4* __restrict__ dst, size_t n4, float v) {
    const floatx4 val = {v, v, v, v};
    const size_t base = (size_t)blockIdx.x * (PT * UNR) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const size_t i = base + (size_t)u * PT;
        if (i < n4) __builtin_nontemporal_store(val, dst + i);
    }
}

__global__ __launch_bounds__(PT) void probe_copy_kernel(const floatx4* __restrict__ src, floatx4* __restrict__ dst,
                                                         size_t n4) {
    const size_t base = (size_t)blockIdx.x * (PT * UNR) + threadIdx.x;
    floatx4 v[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const size_t i = base + (size_t)u * PT;
        if (i < n4) v[u] = __builtin_nontemporal_load(src + i);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const size_t i = base + (size_t)u * PT;
        if (i < n4) __builtin_nontemporal_store(v[u], dst + i);
    }
}

// sixteen independent accumulator tiles per wavefront fed from four A and four B fragments, the
// shape of a 64 x 64 sub-tile of a matrix product: the matrix pipe never waits for a result
__global__ __launch_bounds__(PT, 2) void probe_mfma_f64_kernel(int iters, double* __restrict__ out) {
    double fa[4], fb[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        fa[p] = 1e-3 * (double)((threadIdx.x & 7) + p + 1);
        fb[p] = 1e-3 * (double)((threadIdx.x & 3) + 2 * p + 1);
    }
    double4_t acc[4][4];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[p][q] = (double4_t){0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[p][q] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[p], fb[q], acc[p][q], 0, 0, 0);
    }
    double s = 0.0;
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q) s += acc[p][q][0] + acc[p][q][1] + acc[p][q][2] + acc[p][q][3];
    out[(size_t)blockIdx.x * PT + threadIdx.x] = s;
}

__global__ __launch_bounds__(PT) void probe_mfma_f32_kernel(int iters, float* __restrict__ out) {
    const float a = 1e-3f * (float)(threadIdx.x & 7), b = 1e-3f * (float)(threadIdx.x & 3);
    float16_t c0, c1;
#pragma unroll
    for (int r = 0; r < 16; ++r) c0[r] = c1[r] = 0.0f;
    for (int it = 0; it < iters; ++it) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c1, 0, 0, 0);
        c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, c1, 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += c0[r] + c1[r];
    out[(size_t)blockIdx.x * PT + threadIdx.x] = s;
}

// the instruction of the split-operand products (projection, random Fourier features): two
// independent 32 x 32 accumulator tiles per wavefront, fp16 operands, fp32 accumulation
__global__ __launch_bounds__(PT) void probe_mfma_f16_kernel(int iters, float* __restrict__ out) {
    half8_t a, b;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        a[k] = (_Float16)(1e-3f * (float)((threadIdx.x + k) & 7));
        b[k] = (_Float16)(1e-3f * (float)((threadIdx.x + 2 * k) & 3));
    }
    float16_t c0, c1;
#pragma unroll
    for (int r = 0; r < 16; ++r) c0[r] = c1[r] = 0.0f;
    for (int it = 0; it < iters; ++it) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c1, 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += c0[r] + c1[r];
    out[(size_t)blockIdx.x * PT + threadIdx.x] = s;
}

// eight independent chains of v_exp_f32 per lane (arguments stay in [-1, 0])
__global__ __launch_bounds__(PT) void probe_exp_kernel(int iters, float* __restrict__ out) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = -0.01f * (float)(threadIdx.x % 61 + k);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = -__builtin_amdgcn_exp2f(v[k]);
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) s += v[k];
    out[(size_t)blockIdx.x * PT + threadIdx.x] = s;
}

// ---- instruction mixes -------------------------------------------------------------------
// Straight-line loops of the instruction classes the fused SORF kernel issues, alone and mixed,
// on independent registers: what a wavefront instruction of each class costs a SIMD.  One
// iteration of MIX_FUSED stands for one stack of one wavefront of that kernel at 128 components
// (8 registers per lane, four atoms per wavefront): 82 plain fp32 + 64 DPP fmac + 16
// transcendental instructions, counted in its ISA.
enum { MIX_PLAIN = 0, MIX_DPP = 1, MIX_TRANS = 2, MIX_FUSED = 3, MIX_COUNT = 4 };

template <int N>
__device__ __forceinline__ void plain_ops(float (&v)[8], float c) {
#pragma unroll
    for (int k = 0; k < N; ++k) v[k & 7] = fmaf(v[k & 7], c, 0.25f);
}
template <int N>
__device__ __forceinline__ void dpp_ops(float (&v)[8], float c) {
#pragma unroll
    for (int k = 0; k < N; ++k)
        asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(v[k & 7]) : "v"(c));
}
template <int N>
__device__ __forceinline__ void trans_ops(float (&v)[8]) {
#pragma unroll
    for (int k = 0; k < N; ++k) v[k & 7] = __builtin_amdgcn_sinf(v[k & 7]);
}

template <int MIX>
__global__ __launch_bounds__(PT) void probe_mix_kernel(int iters, float* __restrict__ out) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = 0.001f * (float)((threadIdx.x & 31) + k);
    const float c = (threadIdx.x & 1) ? -0.5f : 0.5f;
    for (int it = 0; it < iters; ++it) {
        if constexpr (MIX == MIX_PLAIN) plain_ops<128>(v, c);
        if constexpr (MIX == MIX_DPP) dpp_ops<128>(v, c);
        if constexpr (MIX == MIX_TRANS) trans_ops<128>(v);
        if constexpr (MIX == MIX_FUSED) {
            // forward: sign multiply + register stages, in-row stages, argument, sincos, products;
            // adjoint: register stages, in-row stages, accumulate
            plain_ops<28>(v, c);
            dpp_ops<32>(v, c);
            plain_ops<8>(v, c);
            trans_ops<16>(v);
            plain_ops<18>(v, c);
            dpp_ops<32>(v, c);
            plain_ops<28>(v, c);
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) s += v[k];
    out[(size_t)blockIdx.x * PT + threadIdx.x] = s;
}

constexpr int PROBE_CUS = 256;
constexpr int PROBE_MAX_BLOCKS_PER_CU = 16;

}  // namespace

extern "C" int qmll_probe_fill(float* dst, size_t nfloats, float value, qmll_stream_t stream) {
    QMLL_REQUIRE(dst && nfloats % 4 == 0 && ((uintptr_t)dst & 15) == 0, QMLL_ERR_INVALID,
                 "qmll_probe_fill: needs a 16-byte aligned buffer of a multiple of 4 floats");
    if (nfloats == 0) return QMLL_OK;
    const size_t n4 = nfloats / 4;
    hipLaunchKernelGGL(probe_fill_kernel, dim3((unsigned)((n4 + PT * UNR - 1) / (PT * UNR))), dim3(PT), 0, (hipStream_t)stream,
                       reinterpret_cast<floatx4*>(dst), n4, value);
    QMLL_CHECK_LAUNCH("qmll_probe_fill");
    return QMLL_OK;
}

extern "C" int qmll_probe_copy(const float* src, float* dst, size_t nfloats, qmll_stream_t stream) {
    QMLL_REQUIRE(src && dst && nfloats % 4 == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0, QMLL_ERR_INVALID,
                 "qmll_probe_copy: needs 16-byte aligned buffers of a multiple of 4 floats");
    if (nfloats == 0) return QMLL_OK;
    const size_t n4 = nfloats / 4;
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)((n4 + PT * UNR - 1) / (PT * UNR))), dim3(PT), 0, (hipStream_t)stream,
                       reinterpret_cast<const floatx4*>(src), reinterpret_cast<floatx4*>(dst), n4);
    QMLL_CHECK_LAUNCH("qmll_probe_copy");
    return QMLL_OK;
}

extern "C" size_t qmll_probe_out_bytes(void) {
    return (size_t)PROBE_CUS * PROBE_MAX_BLOCKS_PER_CU * PT * sizeof(double);
}

extern "C" double qmll_probe_rate(int which, int iters, int blocks_per_cu, void* out, qmll_stream_t stream) {
    // returns the number of operations the launch performs (flop for the matrix loops,
    // exponentials for which = 2); negative on error
    if (!out || iters <= 0 || blocks_per_cu < 1 || blocks_per_cu > PROBE_MAX_BLOCKS_PER_CU) {
        qmll_set_error("qmll_probe_rate: null output, no iterations, or blocks_per_cu outside 1..%d", PROBE_MAX_BLOCKS_PER_CU);
        return -1.0;
    }
    const int PROBE_BLOCKS = PROBE_CUS * blocks_per_cu;
    const double waves = (double)PROBE_BLOCKS * (PT / 64);
    double ops;
    if (which == 0) {
        hipLaunchKernelGGL(probe_mfma_f64_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (double*)out);
        ops = waves * iters * 16.0 * (2.0 * 16 * 16 * 4);
    } else if (which == 1) {
        hipLaunchKernelGGL(probe_mfma_f32_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (float*)out);
        ops = waves * iters * 4.0 * (2.0 * 32 * 32 * 2);
    } else if (which == 2) {
        hipLaunchKernelGGL(probe_exp_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (float*)out);
        ops = waves * 64.0 * iters * 8.0;
    } else if (which == 3) {
        hipLaunchKernelGGL(probe_mfma_f16_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (float*)out);
        ops = waves * iters * 4.0 * (2.0 * 32 * 32 * 16);
    } else {
        qmll_set_error("qmll_probe_rate: which = %d (0: fp64 matrix loop, 1: fp32 matrix loop, 2: exp loop, 3: fp16 matrix loop)", which);
        return -1.0;
    }
    if (hipGetLastError() != hipSuccess) {
        qmll_set_error("qmll_probe_rate: launch failed");
        return -1.0;
    }
    return ops;
}

extern "C" double qmll_probe_mix(int mix, int iters, int blocks_per_cu, void* out, qmll_stream_t stream) {
    // returns the number of wavefront-iterations per SIMD the launch performs (wavefronts per SIMD
    // x iters): duration x clock / that = SIMD clocks per iteration of the mix; negative on error
    if (!out || iters <= 0 || blocks_per_cu < 1 || blocks_per_cu > PROBE_MAX_BLOCKS_PER_CU || mix < 0 || mix >= MIX_COUNT) {
        qmll_set_error("qmll_probe_mix: mix outside 0..%d, null output, no iterations, or blocks_per_cu outside 1..%d",
                       MIX_COUNT - 1, PROBE_MAX_BLOCKS_PER_CU);
        return -1.0;
    }
    const dim3 grid(PROBE_CUS * blocks_per_cu), block(PT);
    float* o = (float*)out;
    hipStream_t st = (hipStream_t)stream;
    switch (mix) {
        case MIX_PLAIN: hipLaunchKernelGGL(probe_mix_kernel<MIX_PLAIN>, grid, block, 0, st, iters, o); break;
        case MIX_DPP: hipLaunchKernelGGL(probe_mix_kernel<MIX_DPP>, grid, block, 0, st, iters, o); break;
        case MIX_TRANS: hipLaunchKernelGGL(probe_mix_kernel<MIX_TRANS>, grid, block, 0, st, iters, o); break;
        default: hipLaunchKernelGGL(probe_mix_kernel<MIX_FUSED>, grid, block, 0, st, iters, o); break;
    }
    if (hipGetLastError() != hipSuccess) {
        qmll_set_error("qmll_probe_mix: launch failed");
        return -1.0;
    }
    return (double)blocks_per_cu * iters;
}
