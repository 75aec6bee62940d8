// SORF (sign diagonal . fast Walsh-Hadamard stacks), cos features and their derivatives
// for gfx950.  Replaces qml_lightning/cuda/hadamard_kernel.cu of the reference
// (kernels :5-102, :204-312, :424-539, :541-585, :587-717, :778-839).
//
// A length-d transform lives in the registers of one wavefront: lane L holds the EPL =
// d/64 consecutive elements L*EPL .. L*EPL+EPL-1 (d < 64: 64/d transforms share a
// wavefront, one element per lane).  Butterflies over the low log2(EPL) index bits are
// register-to-register; the six lane-index bits go through DPP (xor 1, 2, 8), ds_swizzle
// (xor 4, 16) and a cross-half exchange (xor 32).  The stages of a Walsh-Hadamard
// transform commute, so this order gives the reference's natural-order result.  The
// H/sqrt(d) scalings of the T chained transforms and the coefficient normalisation are
// folded into one multiply.  No LDS is used for the transform itself.
//
// Two-op contract (coefficients materialised, [A,S,d] fp32): both ops are HBM bound,
// 4d + 4Sd bytes per atom forward.  The fused kernel keeps coefficients in registers and is
// VALU bound (one sincos per feature).
#include <type_traits>

#include "qmll_common.h"

namespace {

template <int EPL>
__device__ __forceinline__ void load_vec(float (&v)[EPL], const float* __restrict__ p) {
    if constexpr (EPL == 1) {
        v[0] = p[0];
    } else if constexpr (EPL == 2) {
        const float2 t = *reinterpret_cast<const float2*>(p);
        v[0] = t.x;
        v[1] = t.y;
    } else {
#pragma unroll
        for (int q = 0; q < EPL / 4; ++q) {
            const float4 t = reinterpret_cast<const float4*>(p)[q];
            v[4 * q + 0] = t.x;
            v[4 * q + 1] = t.y;
            v[4 * q + 2] = t.z;
            v[4 * q + 3] = t.w;
        }
    }
}

template <int EPL>
__device__ __forceinline__ void store_vec(const float (&v)[EPL], float* __restrict__ p) {
    if constexpr (EPL == 1) {
        p[0] = v[0];
    } else if constexpr (EPL == 2) {
        *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
    } else {
#pragma unroll
        for (int q = 0; q < EPL / 4; ++q)
            reinterpret_cast<float4*>(p)[q] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
    }
}

// Streaming accesses for data that is read or written once (coefficient and gradient
// arrays of gigabytes): the nontemporal hint keeps them from displacing the reusable
// operands in the caches; measured +10 % on the read+write feature kernels.
template <int V>
__device__ __forceinline__ void load_stream(float (&v)[V], const float* p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    if constexpr (V == 1) {
        v[0] = __builtin_nontemporal_load(p);
    } else if constexpr (V == 2) {
        const f2 t = __builtin_nontemporal_load(reinterpret_cast<const f2*>(p));
        v[0] = t[0];
        v[1] = t[1];
    } else {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
            const f4 t = __builtin_nontemporal_load(reinterpret_cast<const f4*>(p) + q);
            v[4 * q + 0] = t[0];
            v[4 * q + 1] = t[1];
            v[4 * q + 2] = t[2];
            v[4 * q + 3] = t[3];
        }
    }
}

template <int V>
__device__ __forceinline__ void store_stream(const float (&v)[V], float* p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    if constexpr (V == 1) {
        __builtin_nontemporal_store(v[0], p);
    } else if constexpr (V == 2) {
        f2 t = {v[0], v[1]};
        __builtin_nontemporal_store(t, reinterpret_cast<f2*>(p));
    } else {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
            f4 t = {v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
            __builtin_nontemporal_store(t, reinterpret_cast<f4*>(p) + q);
        }
    }
}

// One radix-2 stage across lanes: lanes with bit MASK clear get v + partner, the others
// partner - v.  The own value's sign is flipped with a per-lane mask (one xor), so the
// add can take the partner straight from the DPP / swizzle network.
template <int MASK>
__device__ __forceinline__ float butterfly(float v, int lane) {
    const float p = lane_xor<MASK>(v);
    const int sm = (lane & MASK) ? (int)0x80000000 : 0;
    return p + __int_as_float(__float_as_int(v) ^ sm);
}

// Radix-2 stage across lanes 16 or 32 apart for TWO registers at once, on the gfx950 lane
// swap instructions: v_permlane16_swap exchanges the odd 16-lane rows of `a` with the even
// rows of `b` (v_permlane32_swap: the upper half of `a` with the lower half of `b`), after
// which partner values sit in the same lane of a and b; one add, one subtract, and the
// same swap again puts sums and differences back in place.  No LDS crossbar round trip.
template <int MASK>
__device__ __forceinline__ void butterfly_pair(float& a, float& b) {
    typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
    uint2_t r;
    if constexpr (MASK == 16)
        r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    else
        r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    const float x = __uint_as_float(r[0]), y = __uint_as_float(r[1]);
    const float sum = x + y, dif = x - y;
    if constexpr (MASK == 16)
        r = __builtin_amdgcn_permlane16_swap(__float_as_uint(sum), __float_as_uint(dif), false, false);
    else
        r = __builtin_amdgcn_permlane32_swap(__float_as_uint(sum), __float_as_uint(dif), false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
}

// unnormalised Walsh-Hadamard transform of the d = EPL*LANES values held by LANES lanes
template <int EPL, int LANES>
__device__ __forceinline__ void fwht_wave(float (&v)[EPL], int lane) {
#pragma unroll
    for (int h = 1; h < EPL; h <<= 1) {
#pragma unroll
        for (int q = 0; q < EPL; ++q) {
            if ((q & h) == 0) {
                const float a = v[q], b = v[q + h];
                v[q] = a + b;
                v[q + h] = a - b;
            }
        }
    }
#pragma unroll
    for (int q = 0; q < EPL; ++q) {
        float t = v[q];
        if constexpr (LANES > 1) t = butterfly<1>(t, lane);
        if constexpr (LANES > 2) t = butterfly<2>(t, lane);
        if constexpr (LANES > 4) t = butterfly<4>(t, lane);
        if constexpr (LANES > 8) t = butterfly<8>(t, lane);
        if constexpr (EPL == 1) {
            if constexpr (LANES > 16) t = butterfly<16>(t, lane);
            if constexpr (LANES > 32) t = butterfly<32>(t, lane);
        }
        v[q] = t;
    }
    if constexpr (EPL >= 2) {
#pragma unroll
        for (int q = 0; q < EPL; q += 2) {
            if constexpr (LANES > 16) butterfly_pair<16>(v[q], v[q + 1]);
            if constexpr (LANES > 32) butterfly_pair<32>(v[q], v[q + 1]);
        }
    }
}

// Two ways to lay a length-d transform over a wavefront.
//  Wide: all 64 lanes share one transform (d >= 64), d/64 elements per lane: consecutive
//        lanes touch consecutive memory, best for the kernels that stream coefficients.
//  Deep: 32 elements per lane, d/32 lanes per transform, 64/(d/32) transforms side by side:
//        five of the log2(d) stages are register-to-register and only log2(d/32) go across
//        lanes, best for the fused kernel, which is bound by instruction issue.
template <int D_, int EPL_>
struct ShapeT {
    static constexpr int d = D_;
    static constexpr int EPL = EPL_;
    static constexpr int LANES = D_ / EPL_;
    static constexpr int G = 64 / LANES;   // transforms per wavefront
};
template <int LOG2D>
using Shape = ShapeT<(1 << LOG2D), ((1 << LOG2D) >= 64 ? (1 << LOG2D) / 64 : 1)>;
template <int LOG2D>
using DeepShape = ShapeT<(1 << LOG2D), ((1 << LOG2D) >= 32 ? 32 : (1 << LOG2D))>;

// forward chain for stack s: v <- prod_m H diag(D[m,s]) v   (unnormalised)
template <typename Sh>
__device__ __forceinline__ void chain_forward(float (&v)[Sh::EPL], const float* __restrict__ D, int S, int T,
                                              int s, int e0, int lane) {
    for (int m = 0; m < T; ++m) {
        float dv[Sh::EPL];
        load_vec<Sh::EPL>(dv, D + ((size_t)m * S + s) * Sh::d + e0);
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) v[q] *= dv[q];
        fwht_wave<Sh::EPL, Sh::LANES>(v, lane);
    }
}

// adjoint chain: v <- prod_{m=T-1..0} diag(D[m,s]) H v   (unnormalised)
template <typename Sh>
__device__ __forceinline__ void chain_adjoint(float (&v)[Sh::EPL], const float* __restrict__ D, int S, int T,
                                              int s, int e0, int lane) {
    for (int m = T - 1; m >= 0; --m) {
        fwht_wave<Sh::EPL, Sh::LANES>(v, lane);
        float dv[Sh::EPL];
        load_vec<Sh::EPL>(dv, D + ((size_t)m * S + s) * Sh::d + e0);
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) v[q] *= dv[q];
    }
}

constexpr int SORF_THREADS = 256;
constexpr int SORF_WAVES = SORF_THREADS / 64;

// ---- two-op contract: coefficients ------------------------------------------------
template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void sorf_forward_kernel(const float* __restrict__ x,
                                                                     const float* __restrict__ D, int S, int T,
                                                                     float scale, float* __restrict__ out) {
    using Sh = Shape<LOG2D>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / Sh::LANES, l = lane % Sh::LANES;
    const int e0 = l * Sh::EPL;
    const size_t a = blockIdx.x;
    float xv[Sh::EPL];
    load_vec<Sh::EPL>(xv, x + a * Sh::d + e0);
    const int step = SORF_WAVES * gridDim.y * Sh::G;
    for (int s = (blockIdx.y * SORF_WAVES + wave) * Sh::G + sub; s < S; s += step) {
        float v[Sh::EPL];
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) v[q] = xv[q];
        chain_forward<Sh>(v, D, S, T, s, e0, lane);
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) v[q] *= scale;
        store_vec<Sh::EPL>(v, out + (a * S + s) * Sh::d + e0);
    }
}

// ---- two-op contract: adjoint summed over stacks ----------------------------------
template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void sorf_adjoint_kernel(const float* __restrict__ g,
                                                                     const float* __restrict__ D, int S, int T,
                                                                     float scale, float* __restrict__ gx) {
    using Sh = Shape<LOG2D>;
    __shared__ float red[SORF_WAVES][Sh::d];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / Sh::LANES, l = lane % Sh::LANES;
    const int e0 = l * Sh::EPL;
    const size_t a = blockIdx.x;
    float acc[Sh::EPL];
#pragma unroll
    for (int q = 0; q < Sh::EPL; ++q) acc[q] = 0.0f;
    for (int s = wave * Sh::G + sub; s < S; s += SORF_WAVES * Sh::G) {
        float v[Sh::EPL];
        load_vec<Sh::EPL>(v, g + (a * S + s) * Sh::d + e0);
        chain_adjoint<Sh>(v, D, S, T, s, e0, lane);
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) acc[q] += v[q];
    }
    // fold the 64/d transforms that share a wavefront (d < 64)
    if constexpr (Sh::G > 1) {
#pragma unroll
        for (int mask = Sh::LANES; mask < 64; mask <<= 1) acc[0] += __shfl_xor(acc[0], mask, 64);
    }
    if (sub == 0) {
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) red[wave][e0 + q] = acc[q];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < Sh::d; e += SORF_THREADS) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < SORF_WAVES; ++w) t += red[w][e];
        gx[a * Sh::d + e] = scale * t;
    }
}

// ---- fused predict path ------------------------------------------------------------
// Wide layout (coalesced loads of D, bias and alpha).  Per stack: sign diagonal, transform,
// one sincos per feature, energy and d(energy)/d(coefficient), adjoint transform,
// accumulate; the four wavefronts of a workgroup split the stacks and meet in LDS.  (The
// deep layout has fewer cross-lane stages but its 128-byte-strided per-lane loads of the
// three per-feature arrays cost more than the butterflies save: measured 1.7x slower.)
//
// Two addressing modes.  Per element (types == NULL): x is [A,d], the weights belong to
// one element, atom a writes e_atom[out_index ? out_index[a] : a] and gx[a,:].  Typed
// (types != NULL): x is [N, ne*d] with one d-wide block per element type, out_index[a] is
// the slot (row) of atom a, types[slot] picks the block and the element's D / bias, and
// the gradient goes to the same block of gx [N, ne*d]; all elements run in one launch.
template <int LOG2D, bool WITH_GRAD>
__global__ __launch_bounds__(SORF_THREADS) void sorf_energy_fused_kernel(
    const float* __restrict__ x, const float* __restrict__ D, const float* __restrict__ bias,
    const float* __restrict__ alpha, const int* __restrict__ out_index, const int* __restrict__ types,
    const int* __restrict__ type_offsets, int ne, int S, int T, float scale, float normf, float* __restrict__ e_atom,
    float* __restrict__ gx) {
    using Sh = Shape<LOG2D>;
    __shared__ float red[SORF_WAVES][Sh::d];
    __shared__ float ered[SORF_WAVES];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / Sh::LANES, l = lane % Sh::LANES;
    const int e0 = l * Sh::EPL;
    const size_t a = blockIdx.x;
    const size_t slot = out_index ? (size_t)out_index[a] : a;
    size_t xoff = a * Sh::d;          // row of x / gx that belongs to this atom
    if (type_offsets != nullptr) {
        // atoms sorted by element: x and gx are compact [A,d] in that order, atom a belongs to
        // the type whose range [type_offsets[t], type_offsets[t+1]) holds it
        if ((int)a >= type_offsets[ne]) {     // past the last atom of a known element
            if constexpr (WITH_GRAD)
                for (int e = threadIdx.x; e < Sh::d; e += SORF_THREADS) gx[xoff + e] = 0.0f;
            return;
        }
        int t = 0;
        while (t + 1 < ne && (int)a >= type_offsets[t + 1]) ++t;
        D += (size_t)t * T * S * Sh::d;
        bias += (size_t)t * S * Sh::d;
    } else if (types != nullptr) {
        const int t = types[slot];
        if (t < 0 || t >= ne) {        // element not in the model: contributes nothing
            if (threadIdx.x == 0) e_atom[slot] = 0.0f;
            return;
        }
        xoff = (slot * ne + t) * Sh::d;
        D += (size_t)t * T * S * Sh::d;
        bias += (size_t)t * S * Sh::d;
    }
    float xv[Sh::EPL], acc[Sh::EPL];
    load_vec<Sh::EPL>(xv, x + xoff + e0);
#pragma unroll
    for (int q = 0; q < Sh::EPL; ++q) acc[q] = 0.0f;
    float energy = 0.0f;
    constexpr int STEP = SORF_WAVES * Sh::G;
    if (T == 1) {
        // one transform per stack (the usual case): the sign diagonal serves the forward and
        // the adjoint pass, and the three per-feature vectors of the NEXT stack are fetched
        // while this stack is being computed
        int s = wave * Sh::G + sub;
        float dv[Sh::EPL], bv[Sh::EPL], av[Sh::EPL];
        if (s < S) {
            load_vec<Sh::EPL>(dv, D + (size_t)s * Sh::d + e0);
            load_vec<Sh::EPL>(bv, bias + (size_t)s * Sh::d + e0);
            load_vec<Sh::EPL>(av, alpha + (size_t)s * Sh::d + e0);
        }
        for (; s < S; s += STEP) {
            float dn[Sh::EPL], bn[Sh::EPL], an[Sh::EPL];
            const int sn = s + STEP < S ? s + STEP : s;      // last round re-reads its own row
            load_vec<Sh::EPL>(dn, D + (size_t)sn * Sh::d + e0);
            load_vec<Sh::EPL>(bn, bias + (size_t)sn * Sh::d + e0);
            load_vec<Sh::EPL>(an, alpha + (size_t)sn * Sh::d + e0);
            float v[Sh::EPL];
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) v[q] = xv[q] * dv[q];
            fwht_wave<Sh::EPL, Sh::LANES>(v, lane);
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) {
                float sn_, cs;
                sincos_f32(fmaf(v[q], scale, bv[q]), &sn_, &cs);
                const float w = av[q] * normf;
                energy = fmaf(w, cs, energy);
                v[q] = -w * sn_;                          // d E / d coefficient
            }
            if constexpr (WITH_GRAD) {
                fwht_wave<Sh::EPL, Sh::LANES>(v, lane);
#pragma unroll
                for (int q = 0; q < Sh::EPL; ++q) acc[q] = fmaf(v[q], dv[q], acc[q]);
            }
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) {
                dv[q] = dn[q];
                bv[q] = bn[q];
                av[q] = an[q];
            }
        }
    } else {
        for (int s = wave * Sh::G + sub; s < S; s += STEP) {
            float v[Sh::EPL];
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) v[q] = xv[q];
            chain_forward<Sh>(v, D, S, T, s, e0, lane);
            float bv[Sh::EPL], av[Sh::EPL];
            load_vec<Sh::EPL>(bv, bias + (size_t)s * Sh::d + e0);
            load_vec<Sh::EPL>(av, alpha + (size_t)s * Sh::d + e0);
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) {
                float sn_, cs;
                sincos_f32(fmaf(v[q], scale, bv[q]), &sn_, &cs);
                const float w = av[q] * normf;
                energy = fmaf(w, cs, energy);
                v[q] = -w * sn_;
            }
            if constexpr (WITH_GRAD) {
                chain_adjoint<Sh>(v, D, S, T, s, e0, lane);
#pragma unroll
                for (int q = 0; q < Sh::EPL; ++q) acc[q] += v[q];
            }
        }
    }
    energy = wave_sum(energy);
    if (lane == 0) ered[wave] = energy;
    if constexpr (WITH_GRAD) {
        // fold the G transforms that ran side by side in this wavefront
#pragma unroll
        for (int mask = Sh::LANES; mask < 64; mask <<= 1) {
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) acc[q] += __shfl_xor(acc[q], mask, 64);
        }
        if (sub == 0) {
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) red[wave][e0 + q] = acc[q];
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < SORF_WAVES; ++w) t += ered[w];
        e_atom[slot] = t;
    }
    if constexpr (WITH_GRAD) {
        for (int e = threadIdx.x; e < Sh::d; e += SORF_THREADS) {
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < SORF_WAVES; ++w) t += red[w][e];
            gx[xoff + e] = scale * t;
        }
    }
}

// ---- fused kernel, instruction-lean variant (one transform per stack, 64 <= d <= 256) ----
// The generic kernel above spends ~75 vector instructions per coefficient; this one ~22 plus two
// transcendental issues:
//  * a transform lives in ONE ROW of 16 lanes, d/16 registers per lane, so the four rows of a
//    wavefront hold four atoms and only four butterfly stages cross lanes (none crosses rows);
//    the other log2(d/16) stages are register-to-register.
//  * each cross-lane stage is ONE v_fmac_f32_dpp, w += c * w[partner], c = +-1 per lane.
//    Lanes that should hold (partner - own) hold its negative instead; the pending sign of a
//    lane is the same after every full transform (parity of its four stage bits), so it is
//    folded into per-lane constants.  The third stage pairs lane i with i^7 (row_half_mirror,
//    a single DPP control; i^4 is none), which is the standard transform if logical index
//    bits (c0,c1,c2,c3) sit at lane (c0^c2) + 2(c1^c2) + 4 c2 + 8 c3: a fixed permutation of
//    where each lane loads from.
//  * sin and cos come from the transcendental unit, fed with arg / 2 pi (revolutions).
//  * the four atoms of a workgroup share each stack's sign diagonal, bias and alpha (one
//    load serves all rows), which divides the L2 traffic for those vectors -- the limit of a
//    one-atom-per-workgroup mapping -- by four.
#define QMLL_DPP_STAGE4(CTRL, w0, w1, w2, w3, c)                                                 \
    asm("s_nop 1\n\t"                                                                            \
        "v_fmac_f32_dpp %0, %0, %4 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %1, %1, %4 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %2, %2, %4 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %3, %3, %4 " CTRL " row_mask:0xf bank_mask:0xf"                          \
        : "+v"(w0), "+v"(w1), "+v"(w2), "+v"(w3)                                                 \
        : "v"(c))

// eight registers behind one pair of wait states (the hazard is between the instruction that
// wrote a register and the first DPP read of it; inside the block every read is at least
// eight instructions behind its write in the block before)
#define QMLL_DPP_STAGE8(CTRL, w, g, c)                                                           \
    asm("s_nop 1\n\t"                                                                            \
        "v_fmac_f32_dpp %0, %0, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %1, %1, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %2, %2, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %3, %3, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %4, %4, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %5, %5, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %6, %6, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                      \
        "v_fmac_f32_dpp %7, %7, %8 " CTRL " row_mask:0xf bank_mask:0xf"                          \
        : "+v"(w[g]), "+v"(w[g + 1]), "+v"(w[g + 2]), "+v"(w[g + 3]), "+v"(w[g + 4]), "+v"(w[g + 5]),     \
          "+v"(w[g + 6]), "+v"(w[g + 7])                                                         \
        : "v"(c))

// the four in-row stages for NV registers (NV a multiple of 4); cs[k] = -1 in lanes whose
// stage bit k is set, +1 elsewhere
template <int NV>
__device__ __forceinline__ void row_stages(float (&w)[NV], const float (&cs)[4]) {
    if constexpr (NV % 8 == 0) {
#pragma unroll
        for (int g = 0; g < NV; g += 8) QMLL_DPP_STAGE8("quad_perm:[1,0,3,2]", w, g, cs[0]);
#pragma unroll
        for (int g = 0; g < NV; g += 8) QMLL_DPP_STAGE8("quad_perm:[2,3,0,1]", w, g, cs[1]);
#pragma unroll
        for (int g = 0; g < NV; g += 8) QMLL_DPP_STAGE8("row_half_mirror", w, g, cs[2]);
#pragma unroll
        for (int g = 0; g < NV; g += 8) QMLL_DPP_STAGE8("row_ror:8", w, g, cs[3]);
    } else {
#pragma unroll
        for (int g = 0; g < NV; g += 4) QMLL_DPP_STAGE4("quad_perm:[1,0,3,2]", w[g], w[g + 1], w[g + 2], w[g + 3], cs[0]);
#pragma unroll
        for (int g = 0; g < NV; g += 4) QMLL_DPP_STAGE4("quad_perm:[2,3,0,1]", w[g], w[g + 1], w[g + 2], w[g + 3], cs[1]);
#pragma unroll
        for (int g = 0; g < NV; g += 4) QMLL_DPP_STAGE4("row_half_mirror", w[g], w[g + 1], w[g + 2], w[g + 3], cs[2]);
#pragma unroll
        for (int g = 0; g < NV; g += 4) QMLL_DPP_STAGE4("row_ror:8", w[g], w[g + 1], w[g + 2], w[g + 3], cs[3]);
    }
}

template <int EPL>
__device__ __forceinline__ void register_stages(float* v) {
#pragma unroll
    for (int h = 1; h < EPL; h <<= 1) {
#pragma unroll
        for (int q = 0; q < EPL; ++q) {
            if ((q & h) == 0) {
                const float a = v[q], b = v[q + h];
                v[q] = a + b;
                v[q + h] = a - b;
            }
        }
    }
}

// sum over the 16 lanes of a row, result in every lane of the row
__device__ __forceinline__ float row_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false));   // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));   // row_ror:8
    return v;
}

// Per-lane constants of the 16-lanes-per-transform layout: which row (transform) of the
// wavefront the lane belongs to, where its elements sit in the vector, the +-1 factors of
// the four in-row stages and the sign left pending after a full transform.  A lane holds
// EPL/4 groups of four consecutive elements, group q at q*64 + 4*pos (pos = the lane's
// permuted place in the row, which makes row_half_mirror a radix-2 stage): a 16-byte
// access per lane then covers 256 contiguous bytes per row.  Index bits 0-1 and the bits
// from 6 up are the register stages, bits 2-5 the in-row stages; the stages of a
// Walsh-Hadamard transform commute, so the natural-order result is unchanged.
template <int EPL>
struct RowLanes {
    int row, i16, e0;
    float cs[4];
    float sigma;
    __device__ __forceinline__ explicit RowLanes(int lane) {
        row = lane >> 4;
        i16 = lane & 15;
        const int c2 = (i16 >> 2) & 1, c0 = (i16 & 1) ^ c2, c1 = ((i16 >> 1) & 1) ^ c2, c3 = i16 >> 3;
        e0 = (c0 | (c1 << 1) | (c2 << 2) | (c3 << 3)) * 4;
        cs[0] = c0 ? -1.0f : 1.0f;
        cs[1] = c1 ? -1.0f : 1.0f;
        cs[2] = c2 ? -1.0f : 1.0f;
        cs[3] = c3 ? -1.0f : 1.0f;
        sigma = ((c0 + c1 + c2 + c3) & 1) ? -1.0f : 1.0f;
    }
};

// streaming forms of the two helpers below
template <int EPL>
__device__ __forceinline__ void load_row_stream(float (&v)[EPL], const float* __restrict__ p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int q = 0; q < EPL / 4; ++q) {
        const f4 t = __builtin_nontemporal_load(reinterpret_cast<const f4*>(p + q * 64));
        v[4 * q + 0] = t[0];
        v[4 * q + 1] = t[1];
        v[4 * q + 2] = t[2];
        v[4 * q + 3] = t[3];
    }
}

template <int EPL>
__device__ __forceinline__ void store_row_stream(const float (&v)[EPL], float* __restrict__ p) {
    typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int q = 0; q < EPL / 4; ++q) {
        f4 t = {v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
        __builtin_nontemporal_store(t, reinterpret_cast<f4*>(p + q * 64));
    }
}

// the lane's EPL elements of the vector at p (p already includes the lane's e0)
template <int EPL>
__device__ __forceinline__ void load_row(float (&v)[EPL], const float* __restrict__ p) {
#pragma unroll
    for (int q = 0; q < EPL / 4; ++q) {
        const float4 t = *reinterpret_cast<const float4*>(p + q * 64);
        v[4 * q + 0] = t.x;
        v[4 * q + 1] = t.y;
        v[4 * q + 2] = t.z;
        v[4 * q + 3] = t.w;
    }
}

template <int EPL>
__device__ __forceinline__ void store_row(const float (&v)[EPL], float* __restrict__ p) {
#pragma unroll
    for (int q = 0; q < EPL / 4; ++q)
        *reinterpret_cast<float4*>(p + q * 64) = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
}

constexpr int ROWS_NA = 4;   // atoms per workgroup = rows of 16 lanes per wavefront

// MULTI: more than one transform per stack (T > 1); the first sign diagonal stays in registers
// as for T = 1, the later ones are fetched where they are used (forward and again in the adjoint).
// NW: wavefronts per workgroup, which share out the stacks (16 for a few atoms: a molecule then takes
// a quarter of the time, its stacks being the only parallelism there is).
template <int LOG2D, bool WITH_GRAD, bool MULTI, int NW = SORF_WAVES>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(LOG2D >= 8 ? 4 : 1, 8))) void sorf_energy_rows_kernel(
    const float* __restrict__ x, const float* __restrict__ D, const float* __restrict__ bias,
    const float* __restrict__ alpha, const float* __restrict__ bias_absmax, const int* __restrict__ out_index,
    const int* __restrict__ type_offsets, int ne, int A, int S, int T_, float scale, float normf,
    float* __restrict__ e_atom, float* __restrict__ gx) {
    const int T = MULTI ? T_ : 1;
    constexpr int d = 1 << LOG2D;
    constexpr int EPL = d / 16;                 // registers per lane
    constexpr int NA = ROWS_NA;
    static_assert(EPL >= 4 && EPL % 4 == 0, "groups of four butterfly chains per lane");
    __shared__ float red[NW][NA][d];
    __shared__ float ered[NW][NA];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // the NA consecutive atoms of this workgroup; with type_offsets they never straddle two types
    int row0, rows;
    if (type_offsets != nullptr) {
        int b = blockIdx.x, t = 0;
        rows = 0;
        for (; t < ne; ++t) {
            const int o0 = type_offsets[t], o1 = type_offsets[t + 1];
            const int nt = (o1 - o0 + NA - 1) / NA;
            if (b < nt) {
                row0 = o0 + b * NA;
                rows = min(NA, o1 - row0);
                break;
            }
            b -= nt;
        }
        if (rows == 0) {
            // a workgroup past the last tile (the launch adds at least one): its share of the gradient
            // rows past the last atom of a known element, which are zero
            if constexpr (WITH_GRAD) {
                const int spare = b, nspare = (int)gridDim.x - ((int)blockIdx.x - b);
                for (int r = type_offsets[ne] + spare; r < A; r += nspare)
                    for (int c = threadIdx.x; c < d; c += 64 * NW) gx[(size_t)r * d + c] = 0.0f;
            }
            return;
        }
        D += (size_t)t * T * S * d;
        bias += (size_t)t * S * d;
    } else {
        row0 = blockIdx.x * NA;
        rows = min(NA, A - row0);
        if (rows <= 0) return;
    }

    // this lane's row (atom) and the vector elements it holds
    const RowLanes<EPL> L(lane);
    const int row = L.row, i16 = L.i16, e0 = L.e0;
    const float (&cs)[4] = L.cs;
    const float sigma = L.sigma;                                     // pending sign after a transform
    const float scale_l = scale * sigma;
    const bool valid = row < rows;

    float xv[EPL], acc[EPL];
    load_row<EPL>(xv, x + (size_t)(row0 + (valid ? row : 0)) * d + e0);
#pragma unroll
    for (int p = 0; p < EPL; ++p) {
        if (!valid) xv[p] = 0.0f;
        acc[p] = 0.0f;
    }
    float energy = 0.0f;

    if constexpr (!MULTI) {
        // One transform per stack.  The coefficients are carried in REVOLUTIONS: x is scaled by
        // scale / 2 pi once per atom, so the argument of v_sin_f32 / v_cos_f32 is a single fma per
        // coefficient.  The network leaves sigma * (H v) in a lane (sigma = the lane's pending
        // sign); instead of multiplying it out, the lane works with u' = sigma * u:
        //     u' = (H v)_computed + (sigma / 2 pi) * bias,   cos(u') = cos(u),  sin(u') = sigma sin(u).
        // The gradient entering the adjoint transform is then sigma * g.  The transposed network
        // (the same stages with the stage constants negated: (I + diag(c) P)^T = I - diag(c) P,
        // because the partner lane has the opposite stage bit) computes H (sigma * in), i.e. H g
        // itself, with no sign left pending.
        constexpr float INV2PI = 0.15915494309189535f;
        const float xs = scale * INV2PI;
        const float csig = sigma * INV2PI;
        float ncs[4] = {-cs[0], -cs[1], -cs[2], -cs[3]};
#pragma unroll
        for (int q = 0; q < 4; ++q) asm("" : "+v"(ncs[q]));   // kept in registers, not negated again in every stack
#pragma unroll
        for (int p = 0; p < EPL; ++p) xv[p] *= xs;
        // v_sin_f32 / v_cos_f32 reduce the range themselves up to 256 revolutions.  The rounding of
        // the argument, |arg| * 6e-8 radians, is the size of the rounding of an fp32 argument in
        // radians; measured against fp64 the energies and gradients are as close as with an exact
        // Cody-Waite reduction in front (5e-7 at |arg| ~ 16, 2e-6 at ~100).  Beyond 1500 radians the
        // whole revolutions are taken off first: u - rint(u) is exact in fp32.
        constexpr float UMAX = 1500.0f * INV2PI;
        // Every coefficient of an atom is bounded by sum_q |x_q| (the butterflies only add and subtract)
        // plus the largest |bias| (a constant of the model, handed in when the caller knows it): where
        // that bound stays below UMAX for the four atoms of the wavefront, which is the rule, no stack
        // needs to look at its arguments.  Without the bias bound every stack checks them.
        bool track = true;
        if (bias_absmax != nullptr) {
            float bound = 0.0f;
#pragma unroll
            for (int p = 0; p < EPL; ++p) bound += fabsf(xv[p]);
            bound = fmaf(*bias_absmax, INV2PI, row_sum(bound));
            track = __any(!(bound <= UMAX));       // a NaN bound keeps the checks
        }
        // dnext / next: the sign diagonal of the stack after this one and where it sits.  It is fetched one
        // stack ahead (it is the first thing a stack needs): at the start of this stack, or, with sixteen
        // registers per lane (d = 256), in its middle, when bias and alpha are done with and their registers
        // free (a fourth wavefront per SIMD instead of three)
        constexpr bool LATE_DIAGONAL = EPL >= 16;
        auto stack = [&](auto tracked, const float (&dcur)[EPL], float (&dnext)[EPL], const float* next, size_t off) {
            constexpr bool TRACK = decltype(tracked)::value;
            float bv[EPL], av[EPL];
            load_row<EPL>(bv, bias + off);                   // the same for the four rows
            load_row<EPL>(av, alpha + off);
            if constexpr (!LATE_DIAGONAL) load_row<EPL>(dnext, next);
            float v[EPL];
#pragma unroll
            for (int p = 0; p < EPL; ++p) v[p] = xv[p] * dcur[p];
            register_stages<EPL>(v);
            row_stages<EPL>(v, cs);
            float u[EPL], umax = 0.0f;
#pragma unroll
            for (int p = 0; p < EPL; ++p) {
                u[p] = fmaf(bv[p], csig, v[p]);
                if constexpr (TRACK) umax = fmaxf(umax, fabsf(u[p]));
            }
#pragma unroll
            for (int p = 0; p < EPL; ++p) {
                const float sn = __builtin_amdgcn_sinf(u[p]), cs_ = __builtin_amdgcn_cosf(u[p]);
                energy = fmaf(av[p], cs_, energy);
                v[p] = av[p] * sn;                           // sigma * (-(d E / d coefficient) / normf)
            }
            if constexpr (TRACK) {
                if (__builtin_expect(__any(umax > UMAX), 0)) {
#pragma unroll
                    for (int p = 0; p < EPL; ++p) {
                        if (fabsf(u[p]) > UMAX) {
                            const float c0_ = __builtin_amdgcn_cosf(u[p]);
                            const float ur = u[p] - rintf(u[p]);
                            const float sn = __builtin_amdgcn_sinf(ur), cs_ = __builtin_amdgcn_cosf(ur);
                            energy += av[p] * (cs_ - c0_);
                            v[p] = av[p] * sn;
                        }
                    }
                }
            }
            if constexpr (LATE_DIAGONAL) load_row<EPL>(dnext, next);
            if constexpr (WITH_GRAD) {
                register_stages<EPL>(v);
                row_stages<EPL>(v, ncs);
#pragma unroll
                for (int p = 0; p < EPL; ++p) acc[p] = fmaf(v[p], dcur[p], acc[p]);
            }
        };
        // two stacks per round with the sign diagonals in two register sets that swap roles: the
        // diagonal of a stack is fetched one stack ahead (it is the first thing a stack needs),
        // bias and alpha at the start of their own stack (needed after the transform)
        auto stacks = [&](auto tracked) {
            float d0[EPL], d1[EPL];
            int s = wave;
            if (s < S) load_row<EPL>(d0, D + (size_t)s * d + e0);
            while (s < S) {
                stack(tracked, d0, d1, D + (size_t)(s + NW < S ? s + NW : s) * d + e0, (size_t)s * d + e0);
                s += NW;
                if (s >= S) break;
                stack(tracked, d1, d0, D + (size_t)(s + NW < S ? s + NW : s) * d + e0, (size_t)s * d + e0);
                s += NW;
            }
        };
        if (track)
            stacks(std::true_type{});
        else
            stacks(std::false_type{});
        energy = row_sum(energy);
        if (i16 == 0) ered[wave][row] = energy;
        if constexpr (WITH_GRAD) {
            // no sign is pending, and the scaling of x does not enter d E / d coefficient
#pragma unroll
            for (int p = 0; p < EPL; ++p) red[wave][row][(p >> 2) * 64 + e0 + (p & 3)] = acc[p];
        }
    } else {
    // per stack: the sign diagonal is fetched one stack ahead (it is the first thing a stack
    // needs), bias and alpha at the start of their own stack (needed after the transform)
    float dv[EPL], bv[EPL], av[EPL];
    int s = wave;
    if (s < S) load_row<EPL>(dv, D + (size_t)s * d + e0);
    for (; s < S; s += NW) {
        const size_t off = (size_t)s * d + e0;               // the same for the four rows
        load_row<EPL>(bv, bias + off);
        load_row<EPL>(av, alpha + off);
        float dn[EPL];
        load_row<EPL>(dn, D + (size_t)(s + NW < S ? s + NW : s) * d + e0);

        float v[EPL];
#pragma unroll
        for (int p = 0; p < EPL; ++p) v[p] = xv[p] * dv[p];
        register_stages<EPL>(v);
        row_stages<EPL>(v, cs);
        for (int m = 1; m < T; ++m) {
            float dm[EPL];
            load_row<EPL>(dm, D + ((size_t)m * S + s) * d + e0);
#pragma unroll
            for (int p = 0; p < EPL; ++p) v[p] *= dm[p] * sigma;
            register_stages<EPL>(v);
            row_stages<EPL>(v, cs);
        }

        float arg[EPL], amax = 0.0f;
#pragma unroll
        for (int p = 0; p < EPL; ++p) {
            arg[p] = fmaf(v[p], scale_l, bv[p]);
            amax = fmaxf(amax, fabsf(arg[p]));
        }
        // arg / 2 pi goes to the transcendental unit directly (see the one-transform branch)
#pragma unroll
        for (int p = 0; p < EPL; ++p) {
            const float u = arg[p] * 0.15915494309189535f;
            const float sn = __builtin_amdgcn_sinf(u), cs_ = __builtin_amdgcn_cosf(u);
            energy = fmaf(av[p], cs_, energy);
            v[p] = av[p] * sn;                               // -(d E / d coefficient) / normf
        }
        if (__builtin_expect(__any(amax > 1500.0f), 0)) {
            // beyond the unit's own range: exact reduction first, the library routine past 3.2e4
#pragma unroll
            for (int p = 0; p < EPL; ++p) {
                if (fabsf(arg[p]) > 1500.0f) {
                    const float c0_ = __builtin_amdgcn_cosf(arg[p] * 0.15915494309189535f);
                    float sn, cs_;
                    sincos_hw(arg[p], &sn, &cs_);
                    if (fabsf(arg[p]) > 32000.0f) sincos_large(arg[p], &sn, &cs_);
                    energy += av[p] * (cs_ - c0_);
                    v[p] = av[p] * sn;
                }
            }
        }
        if constexpr (WITH_GRAD) {
            register_stages<EPL>(v);
            row_stages<EPL>(v, cs);
            for (int m = T - 1; m >= 1; --m) {
                float dm[EPL];
                load_row<EPL>(dm, D + ((size_t)m * S + s) * d + e0);
#pragma unroll
                for (int p = 0; p < EPL; ++p) v[p] *= dm[p] * sigma;
                register_stages<EPL>(v);
                row_stages<EPL>(v, cs);
            }
#pragma unroll
            for (int p = 0; p < EPL; ++p) acc[p] = fmaf(v[p], dv[p], acc[p]);
        }
#pragma unroll
        for (int p = 0; p < EPL; ++p) dv[p] = dn[p];
    }
    energy = row_sum(energy);
    if (i16 == 0) ered[wave][row] = energy;
    if constexpr (WITH_GRAD) {
#pragma unroll
        for (int p = 0; p < EPL; ++p) red[wave][row][(p >> 2) * 64 + e0 + (p & 3)] = acc[p] * sigma;
    }
    }
    __syncthreads();
    if (threadIdx.x < rows) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) t += ered[w][threadIdx.x];
        const int a = row0 + threadIdx.x;
        e_atom[out_index ? out_index[a] : a] = normf * t;
    }
    if constexpr (WITH_GRAD) {
        const float gscale = -scale * normf;
        for (int e = threadIdx.x; e < rows * d; e += 64 * NW) {
            const int j = e / d, c = e % d;
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) t += red[w][j][c];
            gx[(size_t)(row0 + j) * d + c] = gscale * t;
        }
    }
}


// ---- two-op contract in the 16-lane-row layout (64 <= d <= 256) ---------------------------
// The four rows of a wavefront carry four consecutive stacks of ONE atom, so a workgroup has
// 16 stacks in flight and every lane moves d/16 consecutive floats (16-byte accesses, a row
// covers one contiguous d-float vector).  Eight or more independent butterfly chains per
// lane and the next stack's operands in flight hide the memory latency that bounds a
// one-transform-per-wavefront mapping.
constexpr int ROWS_STACKS = SORF_WAVES * 4;   // stacks in flight per workgroup

constexpr int FWD_NA = 8;   // atoms per workgroup of the forward kernel: each diagonal row read serves eight outputs

template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void sorf_forward_rows_kernel(const float* __restrict__ x,
                                                                          const float* __restrict__ D, int A, int S,
                                                                          int T, float scale, float* __restrict__ out) {
    constexpr int d = 1 << LOG2D;
    constexpr int EPL = d / 16;
    __shared__ __attribute__((aligned(16))) float xs[FWD_NA][d];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const RowLanes<EPL> L(lane);
    const int a0 = blockIdx.x * FWD_NA;
    const int na = min(FWD_NA, A - a0);
    for (int e = threadIdx.x; e < na * (d / 4); e += SORF_THREADS)
        reinterpret_cast<float4*>(&xs[0][0])[e] = reinterpret_cast<const float4*>(x + (size_t)a0 * d)[e];
    __syncthreads();
    const int step = ROWS_STACKS * gridDim.y;
    const float fin = scale * L.sigma;
    int sb = blockIdx.y * ROWS_STACKS + wave * 4;          // first stack of this wavefront's four
    if (sb >= S) return;
    int s = min(sb + L.row, S - 1);
    float dv[EPL];
    load_row<EPL>(dv, D + (size_t)s * d + L.e0);
    for (; sb < S; sb += step) {
        const bool live = sb + L.row < S;
        const int sn = min(sb + step + L.row, S - 1);
        float dn[EPL];
        load_row<EPL>(dn, D + (size_t)sn * d + L.e0);       // first diagonal of the next round
        for (int j = 0; j < na; ++j) {
            float v[EPL];
            load_row<EPL>(v, &xs[j][L.e0]);
#pragma unroll
            for (int p = 0; p < EPL; ++p) v[p] *= dv[p];
            register_stages<EPL>(v);
            row_stages<EPL>(v, L.cs);
            for (int m = 1; m < T; ++m) {
                float dm[EPL];
                load_row<EPL>(dm, D + ((size_t)m * S + s) * d + L.e0);
#pragma unroll
                for (int p = 0; p < EPL; ++p) v[p] *= dm[p] * L.sigma;
                register_stages<EPL>(v);
                row_stages<EPL>(v, L.cs);
            }
#pragma unroll
            for (int p = 0; p < EPL; ++p) v[p] *= fin;
            if (live) store_row_stream<EPL>(v, out + ((size_t)(a0 + j) * S + s) * d + L.e0);
        }
        s = sn;
#pragma unroll
        for (int p = 0; p < EPL; ++p) dv[p] = dn[p];
    }
}

template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void sorf_adjoint_rows_kernel(const float* __restrict__ g,
                                                                          const float* __restrict__ D, int S, int T,
                                                                          float scale, float* __restrict__ gx) {
    constexpr int d = 1 << LOG2D;
    constexpr int EPL = d / 16;
    __shared__ float red[ROWS_STACKS][d];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const RowLanes<EPL> L(lane);
    const size_t a = blockIdx.x;
    float acc[EPL];
#pragma unroll
    for (int p = 0; p < EPL; ++p) acc[p] = 0.0f;
    int sb = wave * 4;
    if (sb < S) {
        int s = min(sb + L.row, S - 1);
        float v[EPL], dv[EPL];
        load_row_stream<EPL>(v, g + (a * S + s) * d + L.e0);
        load_row<EPL>(dv, D + ((size_t)(T - 1) * S + s) * d + L.e0);
        for (; sb < S; sb += ROWS_STACKS) {
            const bool live = sb + L.row < S;
            const int sn = min(sb + ROWS_STACKS + L.row, S - 1);
            float vn[EPL], dn[EPL];
            load_row_stream<EPL>(vn, g + (a * S + sn) * d + L.e0);
            load_row<EPL>(dn, D + ((size_t)(T - 1) * S + sn) * d + L.e0);
            register_stages<EPL>(v);
            row_stages<EPL>(v, L.cs);
            for (int m = T - 1; m > 0; --m) {
                // v <- true value of diag(D[m]) H v, then the next transform
#pragma unroll
                for (int p = 0; p < EPL; ++p) v[p] *= dv[p] * L.sigma;
                load_row<EPL>(dv, D + ((size_t)(m - 1) * S + s) * d + L.e0);
                register_stages<EPL>(v);
                row_stages<EPL>(v, L.cs);
            }
            if (live) {
#pragma unroll
                for (int p = 0; p < EPL; ++p) acc[p] = fmaf(v[p], dv[p], acc[p]);
            }
            s = sn;
#pragma unroll
            for (int p = 0; p < EPL; ++p) {
                v[p] = vn[p];
                dv[p] = dn[p];
            }
        }
    }
#pragma unroll
    for (int p = 0; p < EPL; ++p) red[wave * 4 + L.row][(p >> 2) * 64 + L.e0 + (p & 3)] = acc[p] * L.sigma;
    __syncthreads();
    for (int e = threadIdx.x; e < d; e += SORF_THREADS) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < ROWS_STACKS; ++w) t += red[w][e];
        gx[a * d + e] = scale * t;
    }
}

// ---- derivative (force) features ----------------------------------------------------
// One workgroup per (atom a, target atom j): for x in 0..2 and every stack, the chain of
// u = input_derivative[a,j,x,:] times cos_derivs[a,:] is added into G[mol(a),j,x,:].
// Several atoms of one molecule add into the same row, hence the fp64 atomics (the
// reference does the same, hadamard_kernel.cu:712).  All-zero u rows (targets that are
// not neighbours of a) are skipped.
template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void derivative_features_kernel(
    const double* __restrict__ cos_derivs, double normalisation, const int* __restrict__ mol_index,
    const float* __restrict__ input_derivative, const float* __restrict__ D, int n, int S, int T, float hscale,
    double* __restrict__ G) {
    using Sh = Shape<LOG2D>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / Sh::LANES, l = lane % Sh::LANES;
    const int e0 = l * Sh::EPL;
    const size_t a = blockIdx.x / n;
    const int j = blockIdx.x % n;
    const int mol = mol_index[a];
    const size_t F = (size_t)S * Sh::d;
    for (int xc = 0; xc < 3; ++xc) {
        float uv[Sh::EPL];
        load_vec<Sh::EPL>(uv, input_derivative + ((a * n + j) * 3 + xc) * Sh::d + e0);
        float nz = 0.0f;
#pragma unroll
        for (int q = 0; q < Sh::EPL; ++q) nz += fabsf(uv[q]);
        if (__ballot(nz != 0.0f) == 0ull) continue;    // wave-uniform: nothing to add
        double* Grow = G + (((size_t)mol * n + j) * 3 + xc) * F;
        for (int s = wave * Sh::G + sub; s < S; s += SORF_WAVES * Sh::G) {
            float v[Sh::EPL];
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) v[q] = uv[q];
            chain_forward<Sh>(v, D, S, T, s, e0, lane);
#pragma unroll
            for (int q = 0; q < Sh::EPL; ++q) {
                const size_t f = (size_t)s * Sh::d + e0 + q;
                const double val = normalisation * cos_derivs[a * F + f] * (double)(v[q] * hscale);
                unsafeAtomicAdd(&Grow[f], val);
            }
        }
    }
}

// Segmented, atomic-free variant for molecule-major atoms: seg[mol]..seg[mol+1] are the
// atoms of molecule `mol`.  A wavefront owns (molecule, stack): it keeps the sin
// coefficients of a chunk of the molecule's atoms for that stack in registers, walks the
// 3n target rows, sums the chained transforms of the chunk's atoms in registers and adds
// the row slice into G once (each G element has exactly one owner, so a plain
// read-modify-write is enough and the sum order is fixed).
template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void derivative_features_seg_kernel(
    const double* __restrict__ cos_derivs, double normalisation, const int* __restrict__ seg,
    const float* __restrict__ input_derivative, const float* __restrict__ D, int n, int S, int T, float hscale,
    double* __restrict__ G) {
    using Sh = Shape<LOG2D>;
    constexpr int AC = Sh::EPL >= 16 ? 1 : (Sh::EPL >= 4 ? 4 : 8);   // atoms per register chunk
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / Sh::LANES, l = lane % Sh::LANES;
    const int e0 = l * Sh::EPL;
    const int mol = blockIdx.x;
    const int a0 = seg[mol], a1 = seg[mol + 1];
    if (a1 <= a0) return;
    const size_t F = (size_t)S * Sh::d;
    const int step = SORF_WAVES * gridDim.y * Sh::G;
    const double scale = normalisation * (double)hscale;
    for (int s = (blockIdx.y * SORF_WAVES + wave) * Sh::G + sub; s < S; s += step) {
        for (int ac = a0; ac < a1; ac += AC) {
            const int na = min(AC, a1 - ac);
            float cdv[AC][Sh::EPL];
#pragma unroll
            for (int i = 0; i < AC; ++i)
#pragma unroll
                for (int q = 0; q < Sh::EPL; ++q)
                    cdv[i][q] = i < na ? (float)cos_derivs[(size_t)(ac + i) * F + (size_t)s * Sh::d + e0 + q] : 0.0f;
            for (int jx = 0; jx < 3 * n; ++jx) {
                float acc[Sh::EPL];
#pragma unroll
                for (int q = 0; q < Sh::EPL; ++q) acc[q] = 0.0f;
                bool any = false;
#pragma unroll
                for (int i = 0; i < AC; ++i) {
                    if (i < na) {
                        float v[Sh::EPL];
                        load_vec<Sh::EPL>(v, input_derivative + (((size_t)(ac + i) * n) * 3 + jx) * Sh::d + e0);
                        float nz = 0.0f;
#pragma unroll
                        for (int q = 0; q < Sh::EPL; ++q) nz += fabsf(v[q]);
                        if (__ballot(nz != 0.0f) != 0ull) {
                            any = true;
                            chain_forward<Sh>(v, D, S, T, s, e0, lane);
#pragma unroll
                            for (int q = 0; q < Sh::EPL; ++q) acc[q] = fmaf(cdv[i][q], v[q], acc[q]);
                        }
                    }
                }
                if (any) {
                    double* g = G + (((size_t)mol * n) * 3 + jx) * F + (size_t)s * Sh::d + e0;
#pragma unroll
                    for (int q = 0; q < Sh::EPL; ++q) g[q] += scale * (double)acc[q];
                }
            }
        }
    }
}

// The same in the 16-lane-row layout (64 <= d <= 256): the four rows of a wavefront are four
// consecutive stacks, whose sign diagonals stay in registers for the whole molecule; every
// lane runs d/16 independent butterfly chains with single-instruction DPP stages (28 issue
// clocks per element instead of 60 for the one-transform-per-wavefront form), the projected
// derivative row of an atom is loaded once for the four stacks, and the sine coefficients of
// up to DF_AC atoms sit in registers while the 3n target rows are walked.
template <int LOG2D>
__global__ __launch_bounds__(SORF_THREADS) void derivative_features_rows_kernel(
    const double* __restrict__ cos_derivs, double normalisation, const int* __restrict__ seg,
    const float* __restrict__ input_derivative, const float* __restrict__ D, int n, int S, int T, float hscale,
    double* __restrict__ G) {
    constexpr int d = 1 << LOG2D;
    constexpr int EPL = d / 16;
    constexpr int AC = EPL >= 16 ? 4 : 8;       // atoms whose sine coefficients are held in registers
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const RowLanes<EPL> L(lane);
    const int mol = blockIdx.x;
    const int a0 = seg[mol], a1 = seg[mol + 1];
    if (a1 <= a0) return;
    const size_t F = (size_t)S * d;
    const double scale = normalisation * (double)hscale;
    const int step = ROWS_STACKS * gridDim.y;
    for (int sb = blockIdx.y * ROWS_STACKS + wave * 4; sb < S; sb += step) {
        const bool live = sb + L.row < S;
        const int s = min(sb + L.row, S - 1);
        float dv[EPL];
        load_row<EPL>(dv, D + (size_t)s * d + L.e0);                 // first diagonal of the chain
        for (int ac = a0; ac < a1; ac += AC) {
            const int na = min(AC, a1 - ac);
            float cdv[AC][EPL];
#pragma unroll
            for (int i = 0; i < AC; ++i) {
                const double* src = cos_derivs + (size_t)(ac + min(i, na - 1)) * F + (size_t)s * d + L.e0;
#pragma unroll
                for (int p = 0; p < EPL; ++p)
                    cdv[i][p] = i < na ? (float)src[(p >> 2) * 64 + (p & 3)] * L.sigma : 0.0f;   // pending sign folded in
            }
            for (int jx = 0; jx < 3 * n; ++jx) {
                float acc[EPL];
#pragma unroll
                for (int p = 0; p < EPL; ++p) acc[p] = 0.0f;
                bool any = false;
#pragma unroll
                for (int i = 0; i < AC; ++i) {
                    if (i < na) {
                        float v[EPL];
                        load_row<EPL>(v, input_derivative + (((size_t)(ac + i) * n) * 3 + jx) * d + L.e0);
                        float nz = 0.0f;
#pragma unroll
                        for (int p = 0; p < EPL; ++p) nz += fabsf(v[p]);
                        if (__ballot(nz != 0.0f) != 0ull) {              // an all-zero row adds nothing
                            any = true;
#pragma unroll
                            for (int p = 0; p < EPL; ++p) v[p] *= dv[p];
                            register_stages<EPL>(v);
                            row_stages<EPL>(v, L.cs);
                            for (int m = 1; m < T; ++m) {
                                float dm[EPL];
                                load_row<EPL>(dm, D + ((size_t)m * S + s) * d + L.e0);
#pragma unroll
                                for (int p = 0; p < EPL; ++p) v[p] *= dm[p] * L.sigma;
                                register_stages<EPL>(v);
                                row_stages<EPL>(v, L.cs);
                            }
#pragma unroll
                            for (int p = 0; p < EPL; ++p) acc[p] = fmaf(cdv[i][p], v[p], acc[p]);
                        }
                    }
                }
                if (any && live) {
                    double* g = G + (((size_t)mol * n) * 3 + jx) * F + (size_t)s * d + L.e0;
#pragma unroll
                    for (int q = 0; q < EPL / 4; ++q) {
                        double2* gq = reinterpret_cast<double2*>(g + q * 64);
                        double2 lo = gq[0], hi = gq[1];
                        lo.x += scale * (double)acc[4 * q];
                        lo.y += scale * (double)acc[4 * q + 1];
                        hi.x += scale * (double)acc[4 * q + 2];
                        hi.y += scale * (double)acc[4 * q + 3];
                        gq[0] = lo;
                        gq[1] = hi;
                    }
                }
            }
        }
    }
}

// All elements of a batch in one launch.  The per-element form above walks G once per element
// and per chunk of DF_AC atoms (read + write of the molecule's 3n x F block each time: four
// passes for C9H8O4), which is what bounds it.  Here a workgroup owns (molecule, four stacks):
// the sine coefficients of ALL the molecule's atoms for those stacks sit in LDS (read from
// memory once), its wavefronts share out the 3n target rows, each row's sum over the atoms
// stays in registers, and every G element is written once (overwrite) or read and written once.
// Workgroup ids are dealt round-robin over the 8 XCDs, so the id keeps a molecule's stack
// groups on one XCD: the molecule's projected Jacobian rows (read by every stack group) then
// come out of that XCD's L2.
constexpr int DF_MAXE = 8;
constexpr int DFT_THREADS = 512;
constexpr int DFT_WAVES = DFT_THREADS / 64;
constexpr int DFT_LDS_BYTES = 64 * 1024;      // most that one workgroup takes; a molecule with more atoms takes several passes
struct DfElements {
    const double* cd[DF_MAXE];   // sine coefficients [A_e, F]
    const float* id[DF_MAXE];    // projected Jacobian rows [A_e, n, 3, d]
    const float* D[DF_MAXE];     // sign diagonals [T, S, d]
    const int* seg[DF_MAXE];     // first atom of each molecule in the element's list [nmol + 1]
    int ne;
};

template <int LOG2D>
__global__ __launch_bounds__(DFT_THREADS) void derivative_features_typed_rows_kernel(
    DfElements E, double normalisation, int n, int S, int T, float hscale, int nmol, int ngroups, int cap,
    int overwrite, double* __restrict__ G) {
    constexpr int d = 1 << LOG2D;
    constexpr int EPL = d / 16;
    constexpr int Q = EPL / 4;
    typedef float f4 __attribute__((ext_vector_type(4)));
    extern __shared__ f4 dft_cdv[];              // [cap][Q][64 lanes]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const RowLanes<EPL> L(lane);
    const int b = blockIdx.x;
    const int mol = (b / (8 * ngroups)) * 8 + (b & 7);
    if (mol >= nmol) return;
    const int sb = ((b >> 3) % ngroups) * 4;
    const bool live = sb + L.row < S;
    const int s = min(sb + L.row, S - 1);
    const size_t F = (size_t)S * d;
    const double scale = normalisation * (double)hscale;
    const int nrows = 3 * n;
    const size_t rstride = (size_t)n * 3 * d;    // between the Jacobian rows of consecutive atoms
    int ntot = 0;
    for (int e = 0; e < E.ne; ++e) ntot += E.seg[e][mol + 1] - E.seg[e][mol];
    int c0 = 0;
    do {
        const int c1 = min(c0 + cap, ntot);
        if (c0 > 0) __syncthreads();
        // sine coefficients of atoms c0..c1 (counted element by element) -> LDS, sign folded in
        int base = 0;
        for (int e = 0; e < E.ne; ++e) {
            const int a0 = E.seg[e][mol], cnt = E.seg[e][mol + 1] - a0;
            const int lo = max(c0, base), hi = min(c1, base + cnt);
            for (int t = lo + ((wave - (lo - c0)) & (DFT_WAVES - 1)); t < hi; t += DFT_WAVES) {
                const double* src = E.cd[e] + (size_t)(a0 + t - base) * F + (size_t)s * d + L.e0;
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    const double2 x = *reinterpret_cast<const double2*>(src + q * 64);
                    const double2 y = *reinterpret_cast<const double2*>(src + q * 64 + 2);
                    f4 c = {(float)x.x * L.sigma, (float)x.y * L.sigma, (float)y.x * L.sigma, (float)y.y * L.sigma};
                    dft_cdv[((t - c0) * Q + q) * 64 + lane] = c;
                }
            }
            base += cnt;
        }
        __syncthreads();
        for (int jx = wave; jx < nrows; jx += DFT_WAVES) {
            float acc[EPL];
#pragma unroll
            for (int p = 0; p < EPL; ++p) acc[p] = 0.0f;
            bool any = false;
            base = 0;
            for (int e = 0; e < E.ne; ++e) {
                const int a0 = E.seg[e][mol], cnt = E.seg[e][mol + 1] - a0;
                const int lo = max(c0, base), hi = min(c1, base + cnt);
                if (lo < hi) {
                    const float* De = E.D[e];
                    float dv[EPL];
                    load_row<EPL>(dv, De + (size_t)s * d + L.e0);         // first diagonal of the chain
                    const float* row = E.id[e] + ((size_t)(a0 + lo - base) * n * 3 + jx) * d + L.e0;
                    float v[EPL];
                    load_row<EPL>(v, row);
                    for (int t = lo; t < hi; ++t) {
                        float vn[EPL];                                     // next atom's row, in flight
                        row += rstride;
                        if (t + 1 < hi) {
                            load_row<EPL>(vn, row);
                        } else {
#pragma unroll
                            for (int p = 0; p < EPL; ++p) vn[p] = 0.0f;
                        }
                        float nz = 0.0f;
#pragma unroll
                        for (int p = 0; p < EPL; ++p) nz += fabsf(v[p]);
                        if (__ballot(nz != 0.0f) != 0ull) {                // an all-zero row adds nothing
                            any = true;
#pragma unroll
                            for (int p = 0; p < EPL; ++p) v[p] *= dv[p];
                            register_stages<EPL>(v);
                            row_stages<EPL>(v, L.cs);
                            for (int m = 1; m < T; ++m) {
                                float dm[EPL];
                                load_row<EPL>(dm, De + ((size_t)m * S + s) * d + L.e0);
#pragma unroll
                                for (int p = 0; p < EPL; ++p) v[p] *= dm[p] * L.sigma;
                                register_stages<EPL>(v);
                                row_stages<EPL>(v, L.cs);
                            }
#pragma unroll
                            for (int q = 0; q < Q; ++q) {
                                const f4 c = dft_cdv[((t - c0) * Q + q) * 64 + lane];
                                acc[4 * q] = fmaf(c[0], v[4 * q], acc[4 * q]);
                                acc[4 * q + 1] = fmaf(c[1], v[4 * q + 1], acc[4 * q + 1]);
                                acc[4 * q + 2] = fmaf(c[2], v[4 * q + 2], acc[4 * q + 2]);
                                acc[4 * q + 3] = fmaf(c[3], v[4 * q + 3], acc[4 * q + 3]);
                            }
                        }
#pragma unroll
                        for (int p = 0; p < EPL; ++p) v[p] = vn[p];
                    }
                }
                base += cnt;
            }
            const bool fresh = overwrite && c0 == 0;                       // G holds nothing yet
            if (live && (any || fresh)) {
                double* g = G + (((size_t)mol * n) * 3 + jx) * F + (size_t)s * d + L.e0;
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    double2* gq = reinterpret_cast<double2*>(g + q * 64);
                    double2 lo2 = {0.0, 0.0}, hi2 = {0.0, 0.0};
                    if (!fresh) {
                        lo2 = gq[0];
                        hi2 = gq[1];
                    }
                    lo2.x += scale * (double)acc[4 * q];
                    lo2.y += scale * (double)acc[4 * q + 1];
                    hi2.x += scale * (double)acc[4 * q + 2];
                    hi2.y += scale * (double)acc[4 * q + 3];
                    gq[0] = lo2;
                    gq[1] = hi2;
                }
            }
        }
        c0 += cap;
    } while (c0 < ntot);
}

// ---- elementwise feature kernels ----------------------------------------------------
// Thread = V consecutive feature columns (V = 4: 16-byte loads/stores; V = 1 when F is not
// a multiple of 4), workgroup = (atom chunk, feature tile).  The forward kernel keeps a
// running sum while consecutive atoms belong to the same molecule and flushes it with one
// atomic when the molecule changes: atoms arrive molecule-major, so this is about one
// atomic per (molecule, feature) instead of one per (atom, feature).
constexpr int CF_THREADS = 256;
constexpr int CF_ATOMS = 16;

template <int V>
__device__ __forceinline__ void load_f(float (&v)[V], const float* p) {
    load_vec<V>(v, p);
}

template <typename OutT, int V>
__global__ __launch_bounds__(CF_THREADS) void cos_features_kernel(const float* __restrict__ coeffs,
                                                                   const float* __restrict__ bias,
                                                                   const int* __restrict__ mol_index,
                                                                   const int* __restrict__ seg, int A, int F,
                                                                   int nmol, float normf, OutT* __restrict__ Zf) {
    // with a segment table this kernel only runs when the table is flagged invalid
    if (seg != nullptr && seg[nmol + 1] == 0) return;
    const int f = (blockIdx.y * CF_THREADS + threadIdx.x) * V;
    if (f >= F) return;
    const int a0 = blockIdx.x * CF_ATOMS;
    const int a1 = min(A, a0 + CF_ATOMS);
    float b[V];
    load_f<V>(b, bias + f);
    int cur = -1;
    OutT run[V];
#pragma unroll
    for (int q = 0; q < V; ++q) run[q] = 0;
    // coefficients of the next two atoms are in flight while the current one is evaluated
    float c0[V], c1[V];
    load_f<V>(c0, coeffs + (size_t)a0 * F + f);
    load_f<V>(c1, coeffs + (size_t)min(a0 + 1, a1 - 1) * F + f);
    for (int a = a0; a < a1; ++a) {
        float c[V], c2[V];
        load_f<V>(c2, coeffs + (size_t)min(a + 2, a1 - 1) * F + f);
#pragma unroll
        for (int q = 0; q < V; ++q) {
            c[q] = c0[q];
            c0[q] = c1[q];
            c1[q] = c2[q];
        }
        const int mol = mol_index[a];
        if (mol != cur) {
            if (cur >= 0 && cur < nmol) {
#pragma unroll
                for (int q = 0; q < V; ++q) unsafeAtomicAdd(&Zf[(size_t)cur * F + f + q], run[q]);
            }
            cur = mol;
#pragma unroll
            for (int q = 0; q < V; ++q) run[q] = 0;
        }
#pragma unroll
        for (int q = 0; q < V; ++q) {
            run[q] += (OutT)(cos_hw(c[q] + b[q]) * normf);
        }
    }
    if (cur >= 0 && cur < nmol) {
#pragma unroll
        for (int q = 0; q < V; ++q) unsafeAtomicAdd(&Zf[(size_t)cur * F + f + q], run[q]);
    }
}

// Offsets of the molecule segments of a molecule-major atom list: seg[m] = first atom whose
// molecule index is >= m (seg[nmol] = A).  seg[nmol+1] is raised when the list is not
// ascending or holds an index outside [0,nmol): the segments are then meaningless.  The
// caller zero-fills seg; one thread per boundary (A+1 of them) writes the entries it owns.
__global__ void segment_offsets_kernel(const int* __restrict__ mol_index, int A, int nmol, int* __restrict__ seg) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t > A) return;
    const int prev = t == 0 ? -1 : mol_index[t - 1];
    const int cur = t == A ? nmol : mol_index[t];
    if (prev > cur || cur < 0 || cur > nmol || (t < A && cur == nmol)) {
        seg[nmol + 1] = 1;
        return;
    }
    for (int m = prev + 1; m <= cur; ++m) seg[m] = t;
}

// Segmented, atomic-free cos features for molecule-major atoms: workgroup = (molecule,
// feature tile); the molecule's atoms are streamed with four rows in flight, summed in
// registers in atom order and added into Zf once (each Zf element has one owner).  Does
// nothing when the segment table is flagged invalid; the atomic kernel then does the work.
template <typename OutT, int V>
__global__ __launch_bounds__(CF_THREADS) void cos_features_seg_kernel(const float* __restrict__ coeffs,
                                                                       const float* __restrict__ bias,
                                                                       const int* __restrict__ seg, int F, int nmol,
                                                                       float normf, OutT* __restrict__ Zf) {
    if (seg[nmol + 1] != 0) return;
    const int mol = blockIdx.x;
    const int f = (blockIdx.y * CF_THREADS + threadIdx.x) * V;
    const int a0 = seg[mol], a1 = seg[mol + 1];
    if (f >= F || a1 <= a0) return;
    float b[V];
    load_f<V>(b, bias + f);
    OutT run[V];
#pragma unroll
    for (int q = 0; q < V; ++q) run[q] = 0;
    constexpr int U = 4;
    for (int a = a0; a < a1; a += U) {
        float c[U][V];
#pragma unroll
        for (int u = 0; u < U; ++u) load_stream<V>(c[u], coeffs + (size_t)min(a + u, a1 - 1) * F + f);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (a + u < a1) {
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    run[q] += (OutT)(cos_hw(c[u][q] + b[q]) * normf);
                }
            }
        }
    }
    OutT* z = Zf + (size_t)mol * F + f;
#pragma unroll
    for (int q = 0; q < V; ++q) z[q] += run[q];
}

template <int V>
__global__ __launch_bounds__(CF_THREADS) void cos_features_backward_kernel(const float* __restrict__ gZ,
                                                                            const float* __restrict__ coeffs,
                                                                            const float* __restrict__ bias,
                                                                            const int* __restrict__ mol_index, int A,
                                                                            int F, int nmol, float normf,
                                                                            float* __restrict__ gc) {
    const int f = (blockIdx.y * CF_THREADS + threadIdx.x) * V;
    if (f >= F) return;
    const int a0 = blockIdx.x * CF_ATOMS;
    const int a1 = min(A, a0 + CF_ATOMS);
    float b[V];
    load_f<V>(b, bias + f);
    constexpr int U = 4;   // atoms in flight per thread
    int cur = -1;          // molecule whose gradient row is in gl
    float gl[V];
#pragma unroll
    for (int q = 0; q < V; ++q) gl[q] = 0.0f;
    for (int a = a0; a < a1; a += U) {
        float c[U][V], g[U][V];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int aa = min(a + u, a1 - 1);
            const int mol = mol_index[aa];
            load_stream<V>(c[u], coeffs + (size_t)aa * F + f);
            if (mol != cur) {          // workgroup-uniform: atoms arrive molecule-major
                cur = mol;
                if (mol >= 0 && mol < nmol) {
                    load_f<V>(gl, gZ + (size_t)mol * F + f);
                } else {
#pragma unroll
                    for (int q = 0; q < V; ++q) gl[q] = 0.0f;
                }
            }
#pragma unroll
            for (int q = 0; q < V; ++q) g[u][q] = gl[q];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (a + u < a1) {
                float o[V];
#pragma unroll
                for (int q = 0; q < V; ++q) {
                    o[q] = g[u][q] * -sin_hw(c[u][q] + b[q]) * normf;
                }
                store_stream<V>(o, gc + (size_t)(a + u) * F + f);
            }
        }
    }
}

template <int V>
__global__ __launch_bounds__(CF_THREADS) void sin_coeffs_kernel(const float* __restrict__ coeffs,
                                                                 const float* __restrict__ bias, int A, int F,
                                                                 float normf, double* __restrict__ out) {
    const int f = (blockIdx.y * CF_THREADS + threadIdx.x) * V;
    if (f >= F) return;
    const int a0 = blockIdx.x * CF_ATOMS;
    const int a1 = min(A, a0 + CF_ATOMS);
    float b[V];
    load_f<V>(b, bias + f);
    for (int a = a0; a < a1; ++a) {
        float c[V];
        load_stream<V>(c, coeffs + (size_t)a * F + f);
        double* o = out + (size_t)a * F + f;
#pragma unroll
        for (int q = 0; q < V; ++q) o[q] = (double)(sin_hw(c[q] + b[q]) * normf);
    }
}

int check_sorf(const char* who, int A, int d, int S, int T) {
    QMLL_REQUIRE(A >= 0 && S > 0 && T > 0, QMLL_ERR_INVALID, "%s: bad size A=%d S=%d T=%d", who, A, S, T);
    QMLL_REQUIRE(qmll_is_pow2(d), QMLL_ERR_NOT_POW2, "%s: input size must be power of 2. (got %d)", who, d);
    QMLL_REQUIRE(d >= 2 && d <= 2048, QMLL_ERR_INVALID, "%s: transform length %d outside [2, 2048]", who, d);
    return QMLL_OK;
}

// total scale of T chained H/sqrt(d) transforms
float hnorm(int d, int T) { return powf(2.0f, -0.5f * (float)qmll_log2(d) * (float)T); }

#define DISPATCH_LOG2D(log2d, CALL)   \
    switch (log2d) {                  \
        case 1: { CALL(1); } break;   \
        case 2: { CALL(2); } break;   \
        case 3: { CALL(3); } break;   \
        case 4: { CALL(4); } break;   \
        case 5: { CALL(5); } break;   \
        case 6: { CALL(6); } break;   \
        case 7: { CALL(7); } break;   \
        case 8: { CALL(8); } break;   \
        case 9: { CALL(9); } break;   \
        case 10: { CALL(10); } break; \
        case 11: { CALL(11); } break; \
        default: break;               \
    }

}  // namespace

extern "C" int qmll_sorf_forward(const float* x, const float* D, int A, int d, int S, int T, float normalisation,
                                 float* out, qmll_stream_t stream) {
    int rc = check_sorf("qmll_sorf_forward", A, d, S, T);
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(x && D && out, QMLL_ERR_INVALID, "qmll_sorf_forward: null pointer");
    const float scale = normalisation * hnorm(d, T);
    if (d >= 64 && d <= 256) {
        // stacks are split over enough workgroups to keep ~16k of them in the launch
        const int nb = (A + FWD_NA - 1) / FWD_NA;
        int ny = (16384 + nb - 1) / nb;
        if (ny > (S + ROWS_STACKS - 1) / ROWS_STACKS) ny = (S + ROWS_STACKS - 1) / ROWS_STACKS;
        const dim3 grid(nb, ny);
        switch (qmll_log2(d)) {
            case 6: hipLaunchKernelGGL(sorf_forward_rows_kernel<6>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, x, D, A, S, T, scale, out); break;
            case 7: hipLaunchKernelGGL(sorf_forward_rows_kernel<7>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, x, D, A, S, T, scale, out); break;
            default: hipLaunchKernelGGL(sorf_forward_rows_kernel<8>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, x, D, A, S, T, scale, out); break;
        }
        QMLL_CHECK_LAUNCH("qmll_sorf_forward");
        return QMLL_OK;
    }
    const int G = d >= 64 ? 1 : 64 / d;
    int ny = (S + SORF_WAVES * G - 1) / (SORF_WAVES * G);
    if (ny > 8) ny = 8;   // each wavefront streams >= S/32 stacks: keeps the x row and D hot
    dim3 grid(A, ny);
#define CALL(L) \
    hipLaunchKernelGGL(sorf_forward_kernel<L>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, x, D, S, T, scale, out)
    DISPATCH_LOG2D(qmll_log2(d), CALL)
#undef CALL
    QMLL_CHECK_LAUNCH("qmll_sorf_forward");
    return QMLL_OK;
}

extern "C" int qmll_sorf_adjoint(const float* g, const float* D, int A, int d, int S, int T, float normalisation,
                                 float* gx, qmll_stream_t stream) {
    int rc = check_sorf("qmll_sorf_adjoint", A, d, S, T);
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(g && D && gx, QMLL_ERR_INVALID, "qmll_sorf_adjoint: null pointer");
    const float scale = normalisation * hnorm(d, T);
    if (d >= 64 && d <= 256) {
        switch (qmll_log2(d)) {
            case 6: hipLaunchKernelGGL(sorf_adjoint_rows_kernel<6>, dim3(A), dim3(SORF_THREADS), 0, (hipStream_t)stream, g, D, S, T, scale, gx); break;
            case 7: hipLaunchKernelGGL(sorf_adjoint_rows_kernel<7>, dim3(A), dim3(SORF_THREADS), 0, (hipStream_t)stream, g, D, S, T, scale, gx); break;
            default: hipLaunchKernelGGL(sorf_adjoint_rows_kernel<8>, dim3(A), dim3(SORF_THREADS), 0, (hipStream_t)stream, g, D, S, T, scale, gx); break;
        }
        QMLL_CHECK_LAUNCH("qmll_sorf_adjoint");
        return QMLL_OK;
    }
#define CALL(L) \
    hipLaunchKernelGGL(sorf_adjoint_kernel<L>, dim3(A), dim3(SORF_THREADS), 0, (hipStream_t)stream, g, D, S, T, scale, gx)
    DISPATCH_LOG2D(qmll_log2(d), CALL)
#undef CALL
    QMLL_CHECK_LAUNCH("qmll_sorf_adjoint");
    return QMLL_OK;
}

static int launch_fused(const char* who, const float* x, const float* D, const float* bias, const float* alpha,
                        const float* bias_absmax, const int* out_index, const int* types, const int* type_offsets, int ne, int A, int d, int S,
                        int T, float normalisation, float* e_atom, float* gx, hipStream_t stream) {
    const float scale = normalisation * hnorm(d, T);
    const float normf = sqrtf(2.0f / ((float)S * (float)d));
    if (d >= 64 && d <= 256 && types == nullptr) {
        // 4 to 16 registers per lane, atoms groupable by element: the instruction-lean kernel
        // (four atoms per workgroup)
        // with type offsets: up to ne tiles more than A / 4 (every type rounds up), and 1 to 64 workgroups
        // that zero the gradient rows past the last atom of a known element
        const int zero_groups = A >= 65536 ? 64 : (A >> 10) + 1;
        const dim3 grid((A + ROWS_NA - 1) / ROWS_NA + (type_offsets ? ne + zero_groups : 0));
        // up to some 1500 atoms the chip has idle SIMDs: sixteen wavefronts per workgroup share out the stacks
        // (measured at d = 128, 128 stacks: 17.4 -> 13.8 us at 1008 atoms, equal at 2016, slower from 2688 on)
        const bool few = A <= 1536 && S >= 64 && d <= 128 && T == 1;
#define LAUNCH_ROWS(L, G, M)                                                                                       \
    if (few && !(M))                                                                                               \
        hipLaunchKernelGGL((sorf_energy_rows_kernel<L, G, false, ((L) <= 7 ? 16 : SORF_WAVES)>), grid, dim3(1024), \
                           0, stream, x, D, bias,                                                                  \
                           alpha, bias_absmax, out_index, type_offsets, ne, A, S, T, scale, normf, e_atom, gx);    \
    else                                                                                                           \
        hipLaunchKernelGGL((sorf_energy_rows_kernel<L, G, M>), grid, dim3(SORF_THREADS), 0, stream, x, D, bias,    \
                           alpha, bias_absmax, out_index, type_offsets, ne, A, S, T, scale, normf, e_atom, gx)
#define CALL_ROWS(L)                                    \
    if (gx && T == 1) { LAUNCH_ROWS(L, true, false); }  \
    else if (gx) { LAUNCH_ROWS(L, true, true); }        \
    else if (T == 1) { LAUNCH_ROWS(L, false, false); }  \
    else { LAUNCH_ROWS(L, false, true); }
        switch (qmll_log2(d)) {
            case 6: { CALL_ROWS(6); } break;
            case 7: { CALL_ROWS(7); } break;
            case 8: { CALL_ROWS(8); } break;
            default: break;
        }
#undef LAUNCH_ROWS
#undef CALL_ROWS
        QMLL_CHECK_LAUNCH(who);
        return QMLL_OK;
    }
#define CALL(L)                                                                                                  \
    if (gx)                                                                                                      \
        hipLaunchKernelGGL((sorf_energy_fused_kernel<L, true>), dim3(A), dim3(SORF_THREADS), 0, stream, x, D,    \
                           bias, alpha, out_index, types, type_offsets, ne, S, T, scale, normf, e_atom, gx);     \
    else                                                                                                         \
        hipLaunchKernelGGL((sorf_energy_fused_kernel<L, false>), dim3(A), dim3(SORF_THREADS), 0, stream, x, D,   \
                           bias, alpha, out_index, types, type_offsets, ne, S, T, scale, normf, e_atom, gx)
    DISPATCH_LOG2D(qmll_log2(d), CALL)
#undef CALL
    QMLL_CHECK_LAUNCH(who);
    return QMLL_OK;
}

extern "C" int qmll_sorf_energy_fused(const float* x, const float* D, const float* bias, const float* alpha,
                                      const int* out_index, int A, int d, int S, int T, float normalisation,
                                      float* e_atom, float* gx, qmll_stream_t stream) {
    int rc = check_sorf("qmll_sorf_energy_fused", A, d, S, T);
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(x && D && bias && alpha && e_atom, QMLL_ERR_INVALID, "qmll_sorf_energy_fused: null pointer");
    return launch_fused("qmll_sorf_energy_fused", x, D, bias, alpha, nullptr, out_index, nullptr, nullptr, 1, A, d, S, T, normalisation,
                        e_atom, gx, (hipStream_t)stream);
}

extern "C" int qmll_sorf_energy_typed(const float* x_all, const int* types, const int* atom_slots, const float* D,
                                      const float* bias, const float* alpha, int A, int N, int ne, int d, int S, int T,
                                      float normalisation, float* e_slots, float* gx_all, qmll_stream_t stream) {
    int rc = check_sorf("qmll_sorf_energy_typed", A, d, S, T);
    if (rc) return rc;
    QMLL_REQUIRE(N >= 0 && ne > 0, QMLL_ERR_INVALID, "qmll_sorf_energy_typed: bad size N=%d ne=%d", N, ne);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(x_all && types && atom_slots && D && bias && alpha && e_slots, QMLL_ERR_INVALID,
                 "qmll_sorf_energy_typed: null pointer");
    return launch_fused("qmll_sorf_energy_typed", x_all, D, bias, alpha, nullptr, atom_slots, types, nullptr, ne, A, d, S, T,
                        normalisation, e_slots, gx_all, (hipStream_t)stream);
}

extern "C" int qmll_sorf_energy_sorted(const float* x, const int* type_offsets, const int* sorted_slots, const float* D,
                                       const float* bias, const float* alpha, const float* bias_absmax, int A, int ne, int d,
                                       int S, int T, float normalisation, float* e_slots, float* gx, qmll_stream_t stream) {
    int rc = check_sorf("qmll_sorf_energy_sorted", A, d, S, T);
    if (rc) return rc;
    QMLL_REQUIRE(ne > 0, QMLL_ERR_INVALID, "qmll_sorf_energy_sorted: bad size ne=%d", ne);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(x && type_offsets && sorted_slots && D && bias && alpha && e_slots, QMLL_ERR_INVALID,
                 "qmll_sorf_energy_sorted: null pointer");
    return launch_fused("qmll_sorf_energy_sorted", x, D, bias, alpha, bias_absmax, sorted_slots, nullptr, type_offsets, ne, A, d, S, T,
                        normalisation, e_slots, gx, (hipStream_t)stream);
}

extern "C" int qmll_derivative_features(const double* cos_derivs, double normalisation, const int* mol_index,
                                        const int* seg_offsets, const float* input_derivative, const float* D, int A,
                                        int n, int d, int S, int T, int nmol, double* G, qmll_stream_t stream) {
    int rc = check_sorf("qmll_derivative_features", A, d, S, T);
    if (rc) return rc;
    QMLL_REQUIRE(n >= 0 && nmol >= 0, QMLL_ERR_INVALID, "qmll_derivative_features: bad size n=%d nmol=%d", n, nmol);
    if (A == 0 || n == 0 || nmol == 0) return QMLL_OK;
    QMLL_REQUIRE(cos_derivs && input_derivative && D && G, QMLL_ERR_INVALID, "qmll_derivative_features: null pointer");
    QMLL_REQUIRE(mol_index || seg_offsets, QMLL_ERR_INVALID,
                 "qmll_derivative_features: need mol_index or seg_offsets");
    const float hscale = hnorm(d, T);
    if (seg_offsets && d >= 64 && d <= 256) {
        // 16 stacks in flight per workgroup; the stacks are split over enough workgroups to
        // keep a few thousand of them in the launch
        int ny = (4096 + nmol - 1) / nmol;
        if (ny > (S + ROWS_STACKS - 1) / ROWS_STACKS) ny = (S + ROWS_STACKS - 1) / ROWS_STACKS;
        const dim3 grid(nmol, ny);
        switch (qmll_log2(d)) {
            case 6: hipLaunchKernelGGL(derivative_features_rows_kernel<6>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, cos_derivs, normalisation, seg_offsets, input_derivative, D, n, S, T, hscale, G); break;
            case 7: hipLaunchKernelGGL(derivative_features_rows_kernel<7>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, cos_derivs, normalisation, seg_offsets, input_derivative, D, n, S, T, hscale, G); break;
            default: hipLaunchKernelGGL(derivative_features_rows_kernel<8>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream, cos_derivs, normalisation, seg_offsets, input_derivative, D, n, S, T, hscale, G); break;
        }
    } else if (seg_offsets) {
        const int G_ = d >= 64 ? 1 : 64 / d;
        int ny = (S + SORF_WAVES * G_ - 1) / (SORF_WAVES * G_);
        if (ny > 65535) ny = 65535;
        dim3 grid(nmol, ny);
#define CALL(L)                                                                                                     \
    hipLaunchKernelGGL(derivative_features_seg_kernel<L>, grid, dim3(SORF_THREADS), 0, (hipStream_t)stream,         \
                       cos_derivs, normalisation, seg_offsets, input_derivative, D, n, S, T, hscale, G)
        DISPATCH_LOG2D(qmll_log2(d), CALL)
#undef CALL
    } else {
        QMLL_REQUIRE((long long)A * n < 2147483647LL, QMLL_ERR_INVALID, "qmll_derivative_features: A*n too large");
#define CALL(L)                                                                                                   \
    hipLaunchKernelGGL(derivative_features_kernel<L>, dim3((unsigned)(A * n)), dim3(SORF_THREADS), 0,             \
                       (hipStream_t)stream, cos_derivs, normalisation, mol_index, input_derivative, D, n, S, T, \
                       hscale, G)
        DISPATCH_LOG2D(qmll_log2(d), CALL)
#undef CALL
    }
    QMLL_CHECK_LAUNCH("qmll_derivative_features");
    return QMLL_OK;
}

extern "C" int qmll_derivative_features_typed(const qmll_df_element* elements, int ne, double normalisation, int n,
                                              int d, int S, int T, int nmol, int overwrite, double* G,
                                              qmll_stream_t stream) {
    int rc = check_sorf("qmll_derivative_features_typed", 0, d, S, T);
    if (rc) return rc;
    QMLL_REQUIRE(n >= 0 && nmol >= 0 && ne >= 0, QMLL_ERR_INVALID,
                 "qmll_derivative_features_typed: bad size n=%d nmol=%d ne=%d", n, nmol, ne);
    QMLL_REQUIRE(ne <= DF_MAXE, QMLL_ERR_INVALID, "qmll_derivative_features_typed: at most %d elements per call (got %d)",
                 DF_MAXE, ne);
    QMLL_REQUIRE(d >= 64 && d <= 256, QMLL_ERR_INVALID,
                 "qmll_derivative_features_typed: projected dimension %d outside [64, 256]", d);
    if (n == 0 || nmol == 0) return QMLL_OK;
    if (ne == 0 && !overwrite) return QMLL_OK;       // with overwrite, no element still means G = 0
    QMLL_REQUIRE(G && (elements || ne == 0), QMLL_ERR_INVALID, "qmll_derivative_features_typed: null pointer");
    DfElements E;
    E.ne = ne;
    for (int e = 0; e < ne; ++e) {
        QMLL_REQUIRE(elements[e].cos_derivs && elements[e].input_derivative && elements[e].D && elements[e].seg_offsets,
                     QMLL_ERR_INVALID, "qmll_derivative_features_typed: null pointer in element %d", e);
        E.cd[e] = elements[e].cos_derivs;
        E.id[e] = elements[e].input_derivative;
        E.D[e] = elements[e].D;
        E.seg[e] = elements[e].seg_offsets;
    }
    for (int e = ne; e < DF_MAXE; ++e) {
        E.cd[e] = nullptr;
        E.id[e] = nullptr;
        E.D[e] = nullptr;
        E.seg[e] = nullptr;
    }
    const float hscale = hnorm(d, T);
    const int ngroups = (S + 3) / 4;
    const int per_atom = 4 * d * (int)sizeof(float);             // LDS bytes of one atom's four stacks
    int cap = DFT_LDS_BYTES / per_atom;               // atoms per pass over the target rows
    if (cap > n) cap = n;
    const long long nblocks = (long long)((nmol + 7) / 8) * 8 * ngroups;
    QMLL_REQUIRE(nblocks <= 0x7fffffffLL, QMLL_ERR_INVALID,
                 "qmll_derivative_features_typed: %d molecules x %d stacks exceed the grid", nmol, S);
    const dim3 grid((unsigned)nblocks);
    const size_t lds = (size_t)cap * per_atom;
#define CALL(L)                                                                                                    \
    hipLaunchKernelGGL(derivative_features_typed_rows_kernel<L>, grid, dim3(DFT_THREADS), lds, (hipStream_t)stream, \
                       E, normalisation, n, S, T, hscale, nmol, ngroups, cap, overwrite, G)
    switch (qmll_log2(d)) {
        case 6: CALL(6); break;
        case 7: CALL(7); break;
        default: CALL(8); break;
    }
#undef CALL
    QMLL_CHECK_LAUNCH("qmll_derivative_features_typed");
    return QMLL_OK;
}

static int check_feat(const char* who, int A, int F, int nmol) {
    QMLL_REQUIRE(A >= 0 && F > 0 && nmol >= 0, QMLL_ERR_INVALID, "%s: bad size A=%d F=%d nmol=%d", who, A, F, nmol);
    QMLL_REQUIRE(F <= 65535 * CF_THREADS, QMLL_ERR_INVALID, "%s: too many features (%d)", who, F);
    return QMLL_OK;
}

// grid for the elementwise kernels: x = atom chunks, y = feature tiles of 256*V columns
static dim3 feat_grid(int A, int F, int V) {
    return dim3((A + CF_ATOMS - 1) / CF_ATOMS, (F + CF_THREADS * V - 1) / (CF_THREADS * V));
}

// launches of the forward feature kernels: segmented when a segment table is given (with
// the atomic kernel behind it for a table flagged invalid), atomic otherwise
template <typename OutT>
static int launch_cos_features(const char* who, const float* coeffs, const float* bias, const int* mol_index,
                               const int* seg, int A, int F, int nmol, OutT* Zf, hipStream_t stream) {
    int rc = check_feat(who, A, F, nmol);
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(coeffs && bias && mol_index && Zf, QMLL_ERR_INVALID, "%s: null pointer", who);
    const float normf = sqrtf(2.0f / (float)F);
    if (seg != nullptr && nmol > 0) {
        // small batches take one column per thread so that the grid still fills the device
        const bool wide = F % 4 == 0 && (long long)nmol * ((F + CF_THREADS * 4 - 1) / (CF_THREADS * 4)) >= 2048;
        if (wide)
            hipLaunchKernelGGL((cos_features_seg_kernel<OutT, 4>), dim3(nmol, (F + CF_THREADS * 4 - 1) / (CF_THREADS * 4)),
                               dim3(CF_THREADS), 0, stream, coeffs, bias, seg, F, nmol, normf, Zf);
        else
            hipLaunchKernelGGL((cos_features_seg_kernel<OutT, 1>), dim3(nmol, (F + CF_THREADS - 1) / CF_THREADS),
                               dim3(CF_THREADS), 0, stream, coeffs, bias, seg, F, nmol, normf, Zf);
        QMLL_CHECK_LAUNCH(who);
    }
    if (F % 4 == 0)
        hipLaunchKernelGGL((cos_features_kernel<OutT, 4>), feat_grid(A, F, 4), dim3(CF_THREADS), 0, stream, coeffs,
                           bias, mol_index, seg, A, F, nmol, normf, Zf);
    else
        hipLaunchKernelGGL((cos_features_kernel<OutT, 1>), feat_grid(A, F, 1), dim3(CF_THREADS), 0, stream, coeffs,
                           bias, mol_index, seg, A, F, nmol, normf, Zf);
    QMLL_CHECK_LAUNCH(who);
    return QMLL_OK;
}

extern "C" int qmll_segment_offsets(const int* mol_index, int A, int nmol, int* seg, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && nmol >= 0, QMLL_ERR_INVALID, "qmll_segment_offsets: bad size A=%d nmol=%d", A, nmol);
    QMLL_REQUIRE(seg && (mol_index || A == 0), QMLL_ERR_INVALID, "qmll_segment_offsets: null pointer");
    hipLaunchKernelGGL(segment_offsets_kernel, dim3(A / 256 + 1), dim3(256), 0, (hipStream_t)stream, mol_index, A, nmol,
                       seg);
    QMLL_CHECK_LAUNCH("qmll_segment_offsets");
    return QMLL_OK;
}

extern "C" int qmll_cos_features_f32(const float* coeffs, const float* bias, const int* mol_index, const int* seg,
                                     int A, int F, int nmol, float* Zf, qmll_stream_t stream) {
    return launch_cos_features<float>("qmll_cos_features_f32", coeffs, bias, mol_index, seg, A, F, nmol, Zf,
                                      (hipStream_t)stream);
}

extern "C" int qmll_cos_features_f64(const float* coeffs, const float* bias, const int* mol_index, const int* seg,
                                     int A, int F, int nmol, double* Zf, qmll_stream_t stream) {
    return launch_cos_features<double>("qmll_cos_features_f64", coeffs, bias, mol_index, seg, A, F, nmol, Zf,
                                       (hipStream_t)stream);
}

extern "C" int qmll_cos_features_backward(const float* gZ, const float* coeffs, const float* bias,
                                          const int* mol_index, int A, int F, int nmol, float* gc,
                                          qmll_stream_t stream) {
    int rc = check_feat("qmll_cos_features_backward", A, F, nmol);
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(gZ && coeffs && bias && mol_index && gc, QMLL_ERR_INVALID, "qmll_cos_features_backward: null pointer");
    const float normf = sqrtf(2.0f / (float)F);
    if (F % 4 == 0)
        hipLaunchKernelGGL(cos_features_backward_kernel<4>, feat_grid(A, F, 4), dim3(CF_THREADS), 0,
                           (hipStream_t)stream, gZ, coeffs, bias, mol_index, A, F, nmol, normf, gc);
    else
        hipLaunchKernelGGL(cos_features_backward_kernel<1>, feat_grid(A, F, 1), dim3(CF_THREADS), 0,
                           (hipStream_t)stream, gZ, coeffs, bias, mol_index, A, F, nmol, normf, gc);
    QMLL_CHECK_LAUNCH("qmll_cos_features_backward");
    return QMLL_OK;
}

extern "C" int qmll_sin_coeffs_f64(const float* coeffs, const float* bias, int A, int F, double* out,
                                   qmll_stream_t stream) {
    int rc = check_feat("qmll_sin_coeffs_f64", A, F, 0);
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(coeffs && bias && out, QMLL_ERR_INVALID, "qmll_sin_coeffs_f64: null pointer");
    const float normf = sqrtf(2.0f / (float)F);
    if (F % 4 == 0)
        hipLaunchKernelGGL(sin_coeffs_kernel<4>, feat_grid(A, F, 4), dim3(CF_THREADS), 0, (hipStream_t)stream, coeffs,
                           bias, A, F, normf, out);
    else
        hipLaunchKernelGGL(sin_coeffs_kernel<1>, feat_grid(A, F, 1), dim3(CF_THREADS), 0, (hipStream_t)stream, coeffs,
                           bias, A, F, normf, out);
    QMLL_CHECK_LAUNCH("qmll_sin_coeffs_f64");
    return QMLL_OK;
}
