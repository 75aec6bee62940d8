// Measured ceilings of the device the library runs on: plain fill and copy kernels (HBM), a loop
// of independent matrix-core instructions in fp64 and fp32, and a loop of independent
// transcendental instructions.  The benchmark divides each kernel's rate by these next to the
// nominal peaks; the copy kernel is also the known-size reference for scaling the FETCH_SIZE /
// WRITE_SIZE counters of a profiler run.  No counterpart in the reference.
#include "qmll_common.h"

namespace {

typedef double double4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int PT = 256;

__global__ __launch_bounds__(PT) void probe_fill_kernel(float4* __restrict__ dst, size_t n4, float v) {
    const float4 val = make_float4(v, v, v, v);
    for (size_t i = (size_t)blockIdx.x * PT + threadIdx.x; i < n4; i += (size_t)gridDim.x * PT) dst[i] = val;
}

__global__ __launch_bounds__(PT) void probe_copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst,
                                                         size_t n4) {
    for (size_t i = (size_t)blockIdx.x * PT + threadIdx.x; i < n4; i += (size_t)gridDim.x * PT) dst[i] = src[i];
}

// four independent accumulator tiles per wavefront, so the matrix pipe never waits for a result
__global__ __launch_bounds__(PT) void probe_mfma_f64_kernel(int iters, double* __restrict__ out) {
    const double a = 1e-3 * (double)(threadIdx.x & 7), b = 1e-3 * (double)(threadIdx.x & 3);
    double4_t c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
    for (int it = 0; it < iters; ++it) {
        c0 = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c3, 0, 0, 0);
    }
    const double4_t s = c0 + c1 + c2 + c3;
    out[(size_t)blockIdx.x * PT + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
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

constexpr int PROBE_BLOCKS = 256 * 16;   // 16 workgroups of 4 wavefronts per CU: 16 wavefronts per SIMD queued, 8 resident

}  // namespace

extern "C" int qmll_probe_fill(float* dst, size_t nfloats, float value, qmll_stream_t stream) {
    QMLL_REQUIRE(dst && nfloats % 4 == 0 && ((uintptr_t)dst & 15) == 0, QMLL_ERR_INVALID,
                 "qmll_probe_fill: needs a 16-byte aligned buffer of a multiple of 4 floats");
    if (nfloats == 0) return QMLL_OK;
    hipLaunchKernelGGL(probe_fill_kernel, dim3(256 * 32), dim3(PT), 0, (hipStream_t)stream, reinterpret_cast<float4*>(dst),
                       nfloats / 4, value);
    QMLL_CHECK_LAUNCH("qmll_probe_fill");
    return QMLL_OK;
}

extern "C" int qmll_probe_copy(const float* src, float* dst, size_t nfloats, qmll_stream_t stream) {
    QMLL_REQUIRE(src && dst && nfloats % 4 == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0, QMLL_ERR_INVALID,
                 "qmll_probe_copy: needs 16-byte aligned buffers of a multiple of 4 floats");
    if (nfloats == 0) return QMLL_OK;
    hipLaunchKernelGGL(probe_copy_kernel, dim3(256 * 32), dim3(PT), 0, (hipStream_t)stream,
                       reinterpret_cast<const float4*>(src), reinterpret_cast<float4*>(dst), nfloats / 4);
    QMLL_CHECK_LAUNCH("qmll_probe_copy");
    return QMLL_OK;
}

extern "C" size_t qmll_probe_out_bytes(void) { return (size_t)PROBE_BLOCKS * PT * sizeof(double); }

extern "C" double qmll_probe_rate(int which, int iters, void* out, qmll_stream_t stream) {
    // returns the number of operations the launch performs (flop for the matrix loops,
    // exponentials for which = 2); negative on error
    if (!out || iters <= 0) {
        qmll_set_error("qmll_probe_rate: null output or no iterations");
        return -1.0;
    }
    const double waves = (double)PROBE_BLOCKS * (PT / 64);
    double ops;
    if (which == 0) {
        hipLaunchKernelGGL(probe_mfma_f64_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (double*)out);
        ops = waves * iters * 4.0 * (2.0 * 16 * 16 * 4);
    } else if (which == 1) {
        hipLaunchKernelGGL(probe_mfma_f32_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (float*)out);
        ops = waves * iters * 4.0 * (2.0 * 32 * 32 * 2);
    } else if (which == 2) {
        hipLaunchKernelGGL(probe_exp_kernel, dim3(PROBE_BLOCKS), dim3(PT), 0, (hipStream_t)stream, iters, (float*)out);
        ops = waves * 64.0 * iters * 8.0;
    } else {
        qmll_set_error("qmll_probe_rate: which = %d (0: fp64 matrix loop, 1: fp32 matrix loop, 2: exp loop)", which);
        return -1.0;
    }
    if (hipGetLastError() != hipSuccess) {
        qmll_set_error("qmll_probe_rate: launch failed");
        return -1.0;
    }
    return ops;
}
