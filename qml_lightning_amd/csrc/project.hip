// Per-element projection of the representation on the fp32 matrix cores of gfx950, and
// the element sort that feeds it.  Replaces, for the whole batch at once, the per-element
// boolean-mask gather + torch.matmul(rep, reductor) of
// qml_lightning/representations/dimensionality_reduction.py:47-72 as it is called from
// qml_lightning/models/hadamard_features.py:99-108 (and its autograd transpose).
//
// Atoms are first ordered by element type (stable counting sort, two small kernels), so a
// tile of 128 consecutive atoms shares one reductor.  typed_gemm_kernel then computes
//     C[row, :] = A[row, :] . B_type      (B row-major [K,N])            forward,  or
//     C[row, :] = A[row, :] . B_type^T    (B row-major [N,K])            backward
// with v_mfma_f32_32x32x2f32; rows of A can be gathered and rows of C scattered through the
// sorted slot list, so neither the gathered representation nor a zero-padded
// [slots, elements*d] intermediate is ever materialised.  Only real atoms of known
// elements are touched: no work is spent on padding or on the other elements' reductors.
#include <mutex>

#include "qmll_common.h"

namespace {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int MAXNE = 32;     // element types the sort supports
constexpr int ST = 256;       // threads = atoms per workgroup of the sort

// ---- sort by element type ---------------------------------------------------------------
// counts[b*ne + e] = atoms of type e among atoms b*256 .. b*256+255
__global__ __launch_bounds__(ST) void type_count_kernel(const int* __restrict__ types, const int* __restrict__ slots,
                                                         int A, int ne, int* __restrict__ counts) {
    __shared__ int wcnt[ST / 64][MAXNE];
    const int a = blockIdx.x * ST + threadIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = a < A ? types[slots[a]] : -1;
    for (int e = 0; e < ne; ++e) {
        const unsigned long long m = __ballot(t == e);
        if (lane == 0) wcnt[wave][e] = __popcll(m);
    }
    __syncthreads();
    if (threadIdx.x < ne) {
        int s = 0;
#pragma unroll
        for (int w = 0; w < ST / 64; ++w) s += wcnt[w][threadIdx.x];
        counts[blockIdx.x * ne + threadIdx.x] = s;
    }
}

// sorted[pos] = slot of the atom, pos = start of its type + atoms of that type before it
// (in workgroups before this one, in wavefronts before this one, in lanes before this one)
__global__ __launch_bounds__(ST) void type_place_kernel(const int* __restrict__ types, const int* __restrict__ slots,
                                                         int A, int ne, const int* __restrict__ counts, int nb,
                                                         int* __restrict__ sorted, int* __restrict__ offsets) {
    __shared__ int before[MAXNE], total[MAXNE], start[MAXNE + 1];
    __shared__ int wcnt[ST / 64][MAXNE];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.x;
    if (threadIdx.x < MAXNE) before[threadIdx.x] = total[threadIdx.x] = 0;
    __syncthreads();
    for (int e = 0; e < ne; ++e) {
        int sb = 0, sa = 0;
        for (int q = threadIdx.x; q < nb; q += ST) {
            const int c = counts[q * ne + e];
            sa += c;
            if (q < b) sb += c;
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            sb += __shfl_xor(sb, m, 64);
            sa += __shfl_xor(sa, m, 64);
        }
        if (lane == 0) {
            atomicAdd(&before[e], sb);
            atomicAdd(&total[e], sa);
        }
    }
    const int a = b * ST + threadIdx.x;
    const int slot = a < A ? slots[a] : 0;
    const int t = a < A ? types[slot] : -1;
    int rank = 0;
    for (int e = 0; e < ne; ++e) {
        const unsigned long long m = __ballot(t == e);
        if (lane == 0) wcnt[wave][e] = __popcll(m);
        if (t == e) rank = __popcll(m & ((1ull << lane) - 1ull));
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int s = 0;
        for (int e = 0; e < ne; ++e) {
            start[e] = s;
            s += total[e];
        }
        start[ne] = s;
    }
    __syncthreads();
    if (b == 0 && threadIdx.x <= ne) offsets[threadIdx.x] = start[threadIdx.x];
    if (t >= 0 && t < ne) {
        int pos = start[t] + before[t] + rank;
        for (int w = 0; w < wave; ++w) pos += wcnt[w][t];
        sorted[pos] = slot;
    }
    // entries past the last typed atom name a valid slot, so gathers through them stay in bounds
    for (int i = start[ne] + a; i < A; i += nb * ST) sorted[i] = 0;
}

// slot of listed atom a in the padded [B, n] layout
__global__ __launch_bounds__(256) void atom_slots_kernel(const int* __restrict__ atomIDs, const int* __restrict__ molIDs,
                                                         int n, int A, int* __restrict__ slots) {
    const int a = blockIdx.x * 256 + threadIdx.x;
    if (a < A) slots[a] = molIDs[a] * n + atomIDs[a];
}

// The whole sort in one workgroup for up to 1024 listed atoms (a molecule, a few dozen molecules):
// slot = molIDs * n + atomIDs, count, prefix and placement without a second launch or a workspace.
constexpr int SORT_SMALL = 1024;
__global__ __launch_bounds__(SORT_SMALL) void type_sort_small_kernel(const int* __restrict__ types,
                                                                     const int* __restrict__ atomIDs,
                                                                     const int* __restrict__ molIDs, int n, int A, int ne,
                                                                     int* __restrict__ sorted, int* __restrict__ offsets) {
    __shared__ int wcnt[SORT_SMALL / 64][MAXNE];   // atoms of type e in wavefront w, then: of earlier wavefronts
    __shared__ int total[MAXNE], start[MAXNE + 1];
    const int a = threadIdx.x, lane = a & 63, wave = a >> 6;
    const int slot = a < A ? molIDs[a] * n + atomIDs[a] : 0;
    const int t = a < A ? types[slot] : -1;
    int rank = 0;
    for (int e = 0; e < ne; ++e) {
        const unsigned long long m = __ballot(t == e);
        if (lane == 0) wcnt[wave][e] = __popcll(m);
        if (t == e) rank = __popcll(m & ((1ull << lane) - 1ull));
    }
    __syncthreads();
    if (a < ne) {          // thread e: exclusive prefix of its type over the wavefronts
        int s = 0;
        for (int w = 0; w < SORT_SMALL / 64; ++w) {
            const int c = wcnt[w][a];
            wcnt[w][a] = s;
            s += c;
        }
        total[a] = s;
    }
    __syncthreads();
    if (a == 0) {
        int s = 0;
        for (int e = 0; e < ne; ++e) {
            start[e] = s;
            s += total[e];
        }
        start[ne] = s;
    }
    __syncthreads();
    if (a <= ne) offsets[a] = start[a];
    if (t >= 0 && t < ne) sorted[start[t] + wcnt[wave][t] + rank] = slot;
    // entries past the last typed atom name a valid slot, so gathers through them stay in bounds
    for (int i = start[ne] + a; i < A; i += SORT_SMALL) sorted[i] = 0;
}

// index of charge z in a species list, -1 when it is not there (the rule of element_types_kernel)
__device__ __forceinline__ int species_index(float z, const float* __restrict__ species, int ns) {
    const int q = (int)z;
    int t = -1;
    for (int j = 0; j < ns; ++j)
        if (q == (int)species[j]) t = j;
    return t;
}

// Everything a small padded batch needs before its first compute kernel, in ONE workgroup: the element
// index of every slot by the representation's species list (and, when the model keeps its own list, by
// that one too), the listed atoms sorted by the index the model goes by (stable, as
// type_sort_small_kernel; up to PREP_CHUNKS rounds of 1024 atoms), and a float range set to zero.
// Padded slots (beyond natoms of their molecule) get index 0.
constexpr int PREP_CHUNKS = 4;
__global__ __launch_bounds__(SORT_SMALL) void prepare_small_kernel(
    const float* __restrict__ Z, const int* __restrict__ natoms, const float* __restrict__ species, int ns,
    const float* __restrict__ model_species, int ne, const int* __restrict__ atomIDs, const int* __restrict__ molIDs, int B,
    int n, int A, int* __restrict__ types, int* __restrict__ sort_types, int* __restrict__ sorted, int* __restrict__ offsets,
    float* __restrict__ zero, int zero_count) {
    __shared__ int wcnt[PREP_CHUNKS][SORT_SMALL / 64][MAXNE];   // atoms of type e in (chunk, wavefront), then: before it
    __shared__ int total[MAXNE], start[MAXNE + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunks = (A + SORT_SMALL - 1) / SORT_SMALL;
    for (int idx = tid; idx < B * n; idx += SORT_SMALL) {
        const int m = idx / n;
        const bool real = idx - m * n < natoms[m];
        types[idx] = real ? species_index(Z[idx], species, ns) : 0;
        if (model_species) sort_types[idx] = real ? species_index(Z[idx], model_species, ne) : 0;
    }
    for (int i = tid; i < zero_count; i += SORT_SMALL) zero[i] = 0.0f;
    int slot[PREP_CHUNKS], t[PREP_CHUNKS], rank[PREP_CHUNKS];
#pragma unroll
    for (int k = 0; k < PREP_CHUNKS; ++k) {
        slot[k] = 0;
        t[k] = -1;
        rank[k] = 0;
        if (k < chunks) {
            const int a = k * SORT_SMALL + tid;
            if (a < A) {
                const int m = molIDs[a], i = atomIDs[a];
                slot[k] = m * n + i;
                t[k] = i < natoms[m] ? (model_species ? species_index(Z[slot[k]], model_species, ne)
                                                      : species_index(Z[slot[k]], species, ns))
                                     : 0;
            }
            for (int e = 0; e < ne; ++e) {
                const unsigned long long mk = __ballot(t[k] == e);
                if (lane == 0) wcnt[k][wave][e] = __popcll(mk);
                if (t[k] == e) rank[k] = __popcll(mk & ((1ull << lane) - 1ull));
            }
        }
    }
    __syncthreads();
    if (tid < ne) {          // thread e: exclusive prefix of its type over the chunks and wavefronts
        int sum = 0;
        for (int k = 0; k < chunks; ++k)
            for (int w = 0; w < SORT_SMALL / 64; ++w) {
                const int c = wcnt[k][w][tid];
                wcnt[k][w][tid] = sum;
                sum += c;
            }
        total[tid] = sum;
    }
    __syncthreads();
    if (tid == 0) {
        int sum = 0;
        for (int e = 0; e < ne; ++e) {
            start[e] = sum;
            sum += total[e];
        }
        start[ne] = sum;
    }
    __syncthreads();
    if (tid <= ne) offsets[tid] = start[tid];
#pragma unroll
    for (int k = 0; k < PREP_CHUNKS; ++k)
        if (k < chunks && t[k] >= 0 && t[k] < ne) sorted[start[t[k]] + wcnt[k][wave][t[k]] + rank[k]] = slot[k];
    // entries past the last typed atom name a valid slot, so gathers through them stay in bounds
    for (int i = start[ne] + tid; i < A; i += SORT_SMALL) sorted[i] = 0;
}

// The same bookkeeping for a large batch, short of the sort itself: element indices of every slot, the
// slot of every listed atom, the zero fill; one grid-stride launch instead of three or four
__global__ __launch_bounds__(256) void prepare_large_kernel(const float* __restrict__ Z, const int* __restrict__ natoms,
                                                            const float* __restrict__ species, int ns,
                                                            const float* __restrict__ model_species, int ne,
                                                            const int* __restrict__ atomIDs, const int* __restrict__ molIDs,
                                                            size_t nslots, int n, int A, int* __restrict__ types,
                                                            int* __restrict__ sort_types, int* __restrict__ slots,
                                                            float* __restrict__ zero, size_t zero_count) {
    const size_t first = (size_t)blockIdx.x * 256 + threadIdx.x, step = (size_t)gridDim.x * 256;
    for (size_t idx = first; idx < nslots; idx += step) {
        const size_t m = idx / n;
        const bool real = (int)(idx - m * n) < natoms[m];
        types[idx] = real ? species_index(Z[idx], species, ns) : 0;
        if (model_species) sort_types[idx] = real ? species_index(Z[idx], model_species, ne) : 0;
    }
    if (slots)
        for (size_t a = first; a < (size_t)A; a += step) slots[a] = molIDs[a] * n + atomIDs[a];
    for (size_t i = first; i < zero_count; i += step) zero[i] = 0.0f;
}

__global__ __launch_bounds__(256) void zero_floats_kernel(float* __restrict__ p, size_t count) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (size_t)gridDim.x * 256) p[i] = 0.0f;
}


// ---- typed GEMM -------------------------------------------------------------------------
constexpr int PT = 256;            // threads (4 wavefronts, each 32 rows x 64 columns)
constexpr int PM = 128;            // rows per workgroup
constexpr int PN = 64;             // columns per workgroup (PNT = 128 where the caller picks the wide tile)
constexpr int PK = 32;             // contraction chunk staged in LDS
constexpr int PKS = PK + 4;        // LDS row stride of k-contiguous tiles: 16-byte reads of 16
                                   // consecutive rows fall into 16 distinct groups of 4 banks

// which sorted rows a workgroup owns: tiles never straddle two types.  group: rows per sorted
// entry (1 for one row per atom; the offsets count entries)
__device__ __forceinline__ bool tile_of_block(const int* __restrict__ offsets, int ne, int b, int& type, int& row0,
                                              int& rows, int group = 1) {
    for (int t = 0; t < ne; ++t) {
        const int o0 = offsets[t] * group, o1 = offsets[t + 1] * group;
        const int nt = (o1 - o0 + PM - 1) / PM;
        if (b < nt) {
            type = t;
            row0 = o0 + b * PM;
            rows = min(PM, o1 - row0);
            return true;
        }
        b -= nt;
    }
    return false;
}

// BT = false: B_type is [K,N] row-major (ldb = row length); BT = true: B_type is [N,K].
// VEC: all leading dimensions, K and N are multiples of 4 and the bases are 16-byte aligned.
// PNT: columns per workgroup, 64 or 128.  The wide tile reads the A rows once instead of twice
// and halves the number of workgroups, each twice as long.
template <bool BT, bool VEC, int PNT>
// the forward kernel gains 15 % from a fifth wavefront per SIMD (at most 96 registers); the
// transpose does not fit more than four, the wide tile three
__global__ __launch_bounds__(PT) __attribute__((amdgpu_waves_per_eu(PNT > 64 ? 3 : (BT ? 4 : 5)))) void typed_gemm_kernel(const float* __restrict__ A, int lda,
                                                         const int* __restrict__ a_rows, const float* __restrict__ Bm,
                                                         size_t b_type_stride, int ldb, float* __restrict__ C, int ldc,
                                                         const int* __restrict__ c_rows,
                                                         const int* __restrict__ offsets, int ne, int K, int N,
                                                         int group = 1) {
    // group > 1: every sorted entry stands for `group` consecutive rows, entry e of the list being rows
    // a_rows[e] * group ... of A and rows e * group ... of C (the 3n derivative rows of an atom)
    __shared__ __attribute__((aligned(16))) float sA[PM * PKS];
    constexpr int NJ = PNT / 32;       // 32-column MFMA blocks per wavefront
    __shared__ __attribute__((aligned(16))) float sB[BT ? PNT * PKS : PK * PNT];   // BT: [PNT][PKS]; else [PK][PNT], rotated rows
    int type, row0, rows;
    if (!tile_of_block(offsets, ne, blockIdx.x, type, row0, rows, group)) return;
    const int col0 = blockIdx.y * PNT;
    const float* Bt = Bm + (size_t)type * b_type_stride;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 31, h = lane >> 5;

    // staging: A tile 128 rows x 32 k = 1024 float4, thread -> rows tid/8 + 32v, k4 = tid%8
    const int ar = tid >> 3, ak = (tid & 7) * 4;
    const float* arow[4];
    bool arow_ok[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int r = ar + 32 * v;
        arow_ok[v] = r < rows;
        size_t src = 0;
        if (arow_ok[v]) {
            if (group > 1) {
                const int e = (row0 + r) / group;
                src = (size_t)a_rows[e] * group + (size_t)(row0 + r - e * group);
            } else {
                src = (size_t)(a_rows ? a_rows[row0 + r] : row0 + r);
            }
        }
        arow[v] = A + src * lda;
    }
    // B tile: !BT 32 k x PNT n = 8 PNT float4 -> k = tid/(PNT/4) + (1024/PNT) v, n4 = tid%(PNT/4)
    //          BT PNT n x 32 k = 8 PNT float4 -> n = tid/8 + 32v,  k4 = tid%8
    constexpr int NQ = PNT / 4;        // float4 per B row (!BT)
    constexpr int KV = PT / NQ;        // B rows staged per pass (!BT): 16 or 8
    const int bk = BT ? (tid & 7) * 4 : (tid / NQ);
    const int bn = BT ? (tid >> 3) : (tid % NQ) * 4;

    float4 ra[4], rb[NJ];
    auto load4 = [&](const float* p, int first, int limit) -> float4 {
        // elements first..first+3 of a row, zero beyond `limit`
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (VEC) {
            if (first < limit) v = *reinterpret_cast<const float4*>(p + first);
        } else {
            if (first < limit) v.x = p[first];
            if (first + 1 < limit) v.y = p[first + 1];
            if (first + 2 < limit) v.z = p[first + 2];
            if (first + 3 < limit) v.w = p[first + 3];
        }
        return v;
    };
    auto fetch = [&](int k0) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
            ra[v] = arow_ok[v] ? load4(arow[v], k0 + ak, K) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int v = 0; v < NJ; ++v) {
            if (BT) {
                const int n = col0 + bn + 32 * v;
                rb[v] = n < N ? load4(Bt + (size_t)n * ldb, k0 + bk, K) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                const int k = k0 + bk + KV * v;
                rb[v] = k < K ? load4(Bt + (size_t)k * ldb, col0 + bn, N) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int v = 0; v < 4; ++v) *reinterpret_cast<float4*>(&sA[(ar + 32 * v) * PKS + ak]) = ra[v];
#pragma unroll
        for (int v = 0; v < NJ; ++v) {
            if (BT) {
                *reinterpret_cast<float4*>(&sB[(bn + 32 * v) * PKS + bk]) = rb[v];
            } else {
                // rows 16..31 are rotated by 32 columns: the two wavefront halves, which read
                // rows k and k+16 in one instruction, then use disjoint banks
                const int k = bk + KV * v;
                *reinterpret_cast<float4*>(&sB[k * PNT + ((bn + (k >= 16 ? 32 : 0)) & (PNT - 1))]) = rb[v];
            }
        }
    };

    float16_t acc[NJ];
#pragma unroll
    for (int jt = 0; jt < NJ; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[jt][r] = 0.0f;

    const int nchunks = (K + PK - 1) / PK;
    fetch(0);
    for (int c = 0; c < nchunks; ++c) {
        __syncthreads();
        stash();
        __syncthreads();
        if (c + 1 < nchunks) fetch((c + 1) * PK);
        // MFMA step s contracts k = s (lanes 0-31) and k = 16 + s (lanes 32-63) of the chunk;
        // the order of the contraction index is free, and this one lets a lane read its 16
        // A values (and, transposed, B values) as four 16-byte LDS loads
        // four k-steps at a time: 4 A values and 2 x 4 B values live, not the whole chunk
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 va = *reinterpret_cast<const float4*>(&sA[(32 * wave + i) * PKS + 16 * h + 4 * q]);
            const float af[4] = {va.x, va.y, va.z, va.w};
            float bf[NJ][4];
#pragma unroll
            for (int jt = 0; jt < NJ; ++jt) {
                if (BT) {
                    const float4 v = *reinterpret_cast<const float4*>(&sB[(i + 32 * jt) * PKS + 16 * h + 4 * q]);
                    bf[jt][0] = v.x; bf[jt][1] = v.y; bf[jt][2] = v.z; bf[jt][3] = v.w;
                } else {
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        bf[jt][s] = sB[(4 * q + s + 16 * h) * PNT + ((i + 32 * jt + 32 * h) & (PNT - 1))];
                }
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
                for (int jt = 0; jt < NJ; ++jt)
                    acc[jt] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s], bf[jt][s], acc[jt], 0, 0, 0);
            }
        }
    }

    // accumulator register r of v_mfma_f32_32x32x2f32 holds row 8(r/4) + 4(lane/32) + r%4,
    // column lane%32 (probed on gfx950)
#pragma unroll
    for (int jt = 0; jt < NJ; ++jt) {
        const int col = col0 + 32 * jt + i;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 32 * wave + 8 * (r / 4) + 4 * h + (r % 4);
            if (row < rows && col < N) {
                const int dst = c_rows ? c_rows[row0 + row] : row0 + row;
                C[(size_t)dst * ldc + col] = acc[jt][r];
            }
        }
    }
}

// ---- projections on the half-precision matrix cores -------------------------------------------
// v_mfma_f32_32x32x16_f16 does eight times the flops of the fp32 instruction in 40 clocks against 64,
// so both operands are taken as two fp16 parts (hi = the value rounded to fp16, lo = the rounded
// rest: 22 bits together) behind exact power-of-two scales, and a product term is three matrix
// instructions, hi.hi + hi.lo + lo.hi, accumulated in fp32.
//
// The reductors are constants of the model: they are split ONCE (reductor_presplit_*_kernel) into the
// very bytes the two kernels keep in LDS, "images" that the kernels move with direct global-to-LDS
// loads (no registers, no vector instructions), the next one while the current one is multiplied:
//   forward  image (element, 32-k chunk c, 128-column block): columns x k, k contiguous, hi then lo
//            parts, the chunk behind one power of two (its exponent in a table beside the images);
//   backward image (element, block of 32 rows of U = 32 columns of the product): rows x k, hi then lo,
//            every row behind its own power of two, the 32 inverse factors at the image's end.
// The rows that change from call to call (representation rows forward, gradient rows backward) are
// read from HBM straight into the register layout of the matrix instruction's A operand (lane (i, h)
// holds row i, eight consecutive k), scaled by the power of two of the wavefront's 32 rows and split in
// registers: they never pass through LDS, and no barrier waits on them.
constexpr int FWD_LDH = PK + 8;                       // halves per column of a forward image
constexpr int FWD_IMG_HALVES = 2 * 128 * FWD_LDH;     // hi and lo
constexpr int FWD_IMG_BYTES = FWD_IMG_HALVES * 2;     // 20480
static_assert(FWD_IMG_BYTES % 1024 == 0, "an image is moved in 1 KiB blocks");
template <int K>
struct BwdImage {
    static constexpr int LDB = K + 8;                 // halves per row
    static constexpr int HALVES = 2 * 32 * LDB;       // hi and lo
    static constexpr int SINV = HALVES * 2;           // byte offset of the 32 inverse factors
    static constexpr int BYTES = (SINV + 32 * 4 + 1023) / 1024 * 1024;    // 18432 (K = 128), 10240 (K = 64)
};

// one wavefront's share of a 1 KiB-blocked image: blocks wave, wave + 4, ... (64 lanes x 16 bytes each)
template <int BYTES>
__device__ __forceinline__ void image_to_lds(const unsigned char* __restrict__ src, void* dst, int wave_s, unsigned lane16) {
#pragma unroll
    for (int u0 = 0; u0 < BYTES / 1024; u0 += PT / 64) {
        const int u = u0 + wave_s;
        if (u < BYTES / 1024)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + u * 1024 + lane16),
                                             (__attribute__((address_space(3))) void*)((unsigned char*)dst + u * 1024), 16, 0,
                                             0);
    }
}

// forward images: workgroup = (chunk, column block, element)
__global__ __launch_bounds__(PT) void reductor_presplit_fwd_kernel(const float* __restrict__ U, int R, int d, int ncb,
                                                                    _Float16* __restrict__ images, int* __restrict__ exponents) {
    __shared__ __attribute__((aligned(16))) _Float16 img[FWD_IMG_HALVES];
    __shared__ float smax[PT / 64];
    const int c = blockIdx.x / ncb, cb = blockIdx.x % ncb, type = blockIdx.y, nchunks = gridDim.x / ncb;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* Ut = U + (size_t)type * R * d;
    // thread -> columns (tid/8)*4 .. +3, rows k = 2 (tid%8) + 16 u and the next one
    const int bn = (tid >> 3) * 4, bkp = 2 * (tid & 7);
    float4 rb[2][2];
    float m = 0.0f;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int k = c * PK + bkp + 16 * u + e;
            rb[u][e] = k < R ? *reinterpret_cast<const float4*>(Ut + (size_t)k * d + cb * 128 + bn) : make_float4(0.f, 0.f, 0.f, 0.f);
            m = fmaxf(fmaxf(fmaxf(m, fabsf(rb[u][e].x)), fmaxf(fabsf(rb[u][e].y), fabsf(rb[u][e].z))), fabsf(rb[u][e].w));
        }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if (lane == 0) smax[wave] = m;
    for (int t = tid; t < FWD_IMG_HALVES / 2; t += PT) reinterpret_cast<unsigned*>(img)[t] = 0u;     // column padding
    __syncthreads();
    const int kb = scale_exponent(fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3])));
    const float sb = pow2i(kb);
    const int index = (type * nchunks + c) * ncb + cb;
    if (tid == 0) exponents[index] = kb;
    const float bv[2][2][4] = {{{rb[0][0].x, rb[0][0].y, rb[0][0].z, rb[0][0].w}, {rb[0][1].x, rb[0][1].y, rb[0][1].z, rb[0][1].w}},
                               {{rb[1][0].x, rb[1][0].y, rb[1][0].z, rb[1][0].w}, {rb[1][1].x, rb[1][1].y, rb[1][1].z, rb[1][1].w}}};
#pragma unroll
    for (int cc = 0; cc < 4; ++cc)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            _Float16 h0, l0, h1, l1;
            split_f16(bv[u][0][cc] * sb, h0, l0);
            split_f16(bv[u][1][cc] * sb, h1, l1);
            *reinterpret_cast<half2_t*>(&img[(bn + cc) * FWD_LDH + bkp + 16 * u]) = (half2_t){h0, h1};
            *reinterpret_cast<half2_t*>(&img[128 * FWD_LDH + (bn + cc) * FWD_LDH + bkp + 16 * u]) = (half2_t){l0, l1};
        }
    __syncthreads();
    float4* dst = reinterpret_cast<float4*>(images + (size_t)index * FWD_IMG_HALVES);
    for (int t = tid; t < FWD_IMG_BYTES / 16; t += PT) dst[t] = reinterpret_cast<const float4*>(img)[t];
}

// backward images: workgroup = (block of 32 rows of U, element)
template <int K>
__global__ __launch_bounds__(PT) void reductor_presplit_bwd_kernel(const float* __restrict__ U, int R,
                                                                    unsigned char* __restrict__ images) {
    using Img = BwdImage<K>;
    constexpr int NV = K / 32;
    __shared__ __attribute__((aligned(16))) unsigned char img[Img::BYTES];
    const int b = blockIdx.x, type = blockIdx.y, nblk = gridDim.x;
    const int tid = threadIdx.x;
    const float* Ut = U + (size_t)type * R * K;
    _Float16* ih = reinterpret_cast<_Float16*>(img);
    _Float16* il = ih + 32 * Img::LDB;
    float* sinv = reinterpret_cast<float*>(img + Img::SINV);
    for (int t = tid; t < Img::BYTES / 4; t += PT) reinterpret_cast<unsigned*>(img)[t] = 0u;
    __syncthreads();
    // thread -> row tid/8 of the block, floats (tid%8)*4 + 32 v
    const int bn = tid >> 3, bk = (tid & 7) * 4;
    const int n = 32 * b + bn;
    float4 rb[NV];
    float m = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        rb[v] = n < R ? *reinterpret_cast<const float4*>(Ut + (size_t)n * K + bk + 32 * v) : make_float4(0.f, 0.f, 0.f, 0.f);
        m = fmaxf(fmaxf(fmaxf(m, fabsf(rb[v].x)), fmaxf(fabsf(rb[v].y), fabsf(rb[v].z))), fabsf(rb[v].w));
    }
    m = fmaxf(m, lane_xor<1>(m));            // the eight lanes of a row are neighbours
    m = fmaxf(m, lane_xor<2>(m));
    m = fmaxf(m, lane_xor<4>(m));
    const int kb = scale_exponent(m);
    const float sb = pow2i(kb);
    if ((tid & 7) == 0) sinv[bn] = pow2i(-kb);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const float w[4] = {rb[v].x * sb, rb[v].y * sb, rb[v].z * sb, rb[v].w * sb};
        half4_t wh, wl;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            _Float16 a, c;
            split_f16(w[e], a, c);
            wh[e] = a;
            wl[e] = c;
        }
        *reinterpret_cast<half4_t*>(&ih[bn * Img::LDB + bk + 32 * v]) = wh;
        *reinterpret_cast<half4_t*>(&il[bn * Img::LDB + bk + 32 * v]) = wl;
    }
    __syncthreads();
    float4* dst = reinterpret_cast<float4*>(images + (size_t)(type * nblk + b) * Img::BYTES);
    for (int t = tid; t < Img::BYTES / 16; t += PT) dst[t] = reinterpret_cast<const float4*>(img)[t];
}

// 2^-(ka + kb) applied to a chunk's product as it is added to the running sums: one factor when it is
// a float, two multiplies at the ends of the exponent range (operands near the largest or smallest floats)
__device__ __forceinline__ void add_scaled(float16_t& acc, const float16_t& part, int ka, int kb) {
    const int ks = ka + kb;
    if (ks >= -126 && ks <= 126) {
        const float inv = pow2i(-ks);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = fmaf(part[r], inv, acc[r]);
    } else {
        const float ia = pow2i(-ka), ib = pow2i(-kb);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = fmaf(part[r] * ia, ib, acc[r]);
    }
}

// Forward product x = rep . U_type, 128 x 128 tiles (A [rows, K] gathered through a_rows; K a multiple
// of 4, N a multiple of 128, 16-byte aligned bases).  Per chunk of 32 k: the wavefront's 32 rows take
// the power of two of their largest entry and are split in registers, the chunk of U arrives as its
// image; a chunk's product is summed from zero and added to the running sums by the vector unit with
// the inverse factor (which also keeps the low bits of a small chunk beside a large sum).
__global__ __launch_bounds__(PT) __attribute__((amdgpu_waves_per_eu(3))) void typed_gemm_f16_kernel(
    const float* __restrict__ A, int lda, const int* __restrict__ a_rows, const _Float16* __restrict__ images,
    const int* __restrict__ exponents, float* __restrict__ C, int ldc, const int* __restrict__ offsets, int ne, int K, int N,
    int group) {
    // the two images as arrays of their own: the compiler then knows that the loads into one do not
    // touch what is read from the other
    __shared__ __attribute__((aligned(16))) _Float16 sB0[FWD_IMG_HALVES], sB1[FWD_IMG_HALVES];
    int type, row0, rows;
    if (!tile_of_block(offsets, ne, blockIdx.x, type, row0, rows, group)) return;
    const int col0 = blockIdx.y * 128, ncb = gridDim.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 31, h = lane >> 5;
    const int nchunks = (K + PK - 1) / PK;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const unsigned lane16 = (unsigned)lane * 16u;
    const unsigned char* img0 = reinterpret_cast<const unsigned char*>(images) +
                                ((size_t)type * nchunks * ncb + blockIdx.y) * FWD_IMG_BYTES;
    const int* exps = exponents + (size_t)type * nchunks * ncb + blockIdx.y;
    image_to_lds<FWD_IMG_BYTES>(img0, sB0, wave_s, lane16);

    // this lane's row of A: row 32 wave + i, of each chunk the k = 16 s + 8 h + (0..7), s = 0, 1
    const int r = 32 * wave + i;
    const bool rok = r < rows;
    size_t src = 0;
    if (rok) {
        if (group > 1) {
            const int e = (row0 + r) / group;
            src = (size_t)a_rows[e] * group + (size_t)(row0 + r - e * group);
        } else {
            src = (size_t)(a_rows ? a_rows[row0 + r] : row0 + r);
        }
    }
    const float* arow = A + src * lda + 8 * h;
    float4 ra[2][2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int k = k0 + 16 * s2 + 8 * h + 4 * e;
                ra[s2][e] = (rok && k < K) ? *reinterpret_cast<const float4*>(arow + k0 + 16 * s2 + 4 * e) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
    };
    auto max4 = [](float m, float4 v) { return fmaxf(fmaxf(fmaxf(m, fabsf(v.x)), fmaxf(fabsf(v.y), fabsf(v.z))), fabsf(v.w)); };

    float16_t acc[4];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[jt][q] = 0.0f;

    fetch(0);
    // one chunk: its image is in `cur`, the next one is loaded into `other`
    auto round = [&](int c, const _Float16* cur, _Float16* other) {
        // the rows of this chunk: the wavefront's power of two, two fp16 parts each
        float ma = max4(max4(max4(max4(0.0f, ra[0][0]), ra[0][1]), ra[1][0]), ra[1][1]);
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) ma = fmaxf(ma, __shfl_xor(ma, o, 64));
        if (__builtin_expect(not_finite(ma), 0)) {       // an infinity among the rows: the largest finite entry
            ma = 0.0f;
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                for (int e = 0; e < 2; ++e)
                    ma = fmaxf(fmaxf(fmaxf(ma, finite_abs(ra[s2][e].x)), fmaxf(finite_abs(ra[s2][e].y), finite_abs(ra[s2][e].z))),
                               finite_abs(ra[s2][e].w));
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) ma = fmaxf(ma, __shfl_xor(ma, o, 64));
        }
        const int ka = scale_exponent(ma);
        const float sa = pow2i(ka);
        half8_t ahv[2], alv[2];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const float w[8] = {ra[s2][0].x * sa, ra[s2][0].y * sa, ra[s2][0].z * sa, ra[s2][0].w * sa,
                                ra[s2][1].x * sa, ra[s2][1].y * sa, ra[s2][1].z * sa, ra[s2][1].w * sa};
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                _Float16 a_, c_;
                split_f16(w[q], a_, c_);
                ahv[s2][q] = a_;
                alv[s2][q] = c_;
            }
        }
        // this chunk's image has landed (every wavefront waits for its own loads, then for the others),
        // and the other copy, read in the round before, is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (c + 1 < nchunks) {
            image_to_lds<FWD_IMG_BYTES>(img0 + (size_t)(c + 1) * ncb * FWD_IMG_BYTES, other, wave_s, lane16);
            fetch((c + 1) * PK);
        }
        const int kb = exps[(size_t)c * ncb];
        const _Float16* sBh = cur;
        const _Float16* sBl = cur + 128 * FWD_LDH;
#pragma unroll
        for (int j0 = 0; j0 < 4; j0 += 2) {
            float16_t part[2];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int q = 0; q < 16; ++q) part[jj][q] = 0.0f;
#pragma unroll
            for (int s2 = 0; s2 < PK / 16; ++s2) {
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const half8_t bhv = *reinterpret_cast<const half8_t*>(&sBh[(32 * (j0 + jj) + i) * FWD_LDH + 16 * s2 + 8 * h]);
                    const half8_t blv = *reinterpret_cast<const half8_t*>(&sBl[(32 * (j0 + jj) + i) * FWD_LDH + 16 * s2 + 8 * h]);
                    part[jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(alv[s2], bhv, part[jj], 0, 0, 0);
                    part[jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahv[s2], blv, part[jj], 0, 0, 0);
                    part[jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahv[s2], bhv, part[jj], 0, 0, 0);
                }
            }
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) add_scaled(acc[j0 + jj], part[jj], ka, kb);
        }
    };
    for (int c = 0; c < nchunks; c += 2) {
        round(c, sB0, sB1);
        if (c + 1 < nchunks) round(c + 1, sB1, sB0);
    }

#pragma unroll
    for (int jt = 0; jt < 4; ++jt) {
        const int col = col0 + 32 * jt + i;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int row = 32 * wave + 8 * (q / 4) + 4 * h + (q % 4);
            if (row < rows && col < N) C[(size_t)(row0 + row) * ldc + col] = acc[jt][q];
        }
    }
}

// Transpose product for a short contraction (K = projected dimension 64 or 128):
//     C[c_rows[row], :] = A[row, :] . U_type^T,   A [rows, K] (the gradient rows), U_type [N, K] row-major.
// A wavefront keeps its 32 rows of A in registers for the whole kernel (two fp16 parts behind the
// wavefront's power of two), so every row of A is read exactly once; the workgroup walks the N columns
// in blocks of 32, each block's image arriving in LDS while the previous block is multiplied, and every
// 32 x 32 block of C leaves straight from the accumulators through the two inverse factors.
template <int K>
__global__ __launch_bounds__(PT) void typed_gemm_bt_rows_f16_kernel(const float* __restrict__ A,
                                                                     const unsigned char* __restrict__ images,
                                                                     float* __restrict__ C, int ldc,
                                                                     const int* __restrict__ c_rows,
                                                                     const int* __restrict__ offsets, int ne, int N) {
    using Img = BwdImage<K>;
    constexpr int KS = K / 16;         // matrix instructions along k per product term
    constexpr int LDB = Img::LDB;
    __shared__ __attribute__((aligned(16))) unsigned char sI0[Img::BYTES], sI1[Img::BYTES];
    int type, row0, rows;
    if (!tile_of_block(offsets, ne, blockIdx.x, type, row0, rows)) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 31, h = lane >> 5;
    const int nblk = (N + 31) / 32;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const unsigned lane16 = (unsigned)lane * 16u;
    const unsigned char* img0 = images + (size_t)type * nblk * Img::BYTES;
    image_to_lds<Img::BYTES>(img0, sI0, wave_s, lane16);

    const int r = 32 * wave + i;
    const bool rok = r < rows;
    // instruction j contracts k = 16 j + 8 h + (0..7)
    half8_t ah[KS], al[KS];
    float inv_sa;
    {
        float av[KS][8];
        const float* ap = A + (size_t)(row0 + (rok ? r : 0)) * K + 8 * h;
        float m = 0.0f;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            const float4 v0 = rok ? *reinterpret_cast<const float4*>(ap + 16 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 v1 = rok ? *reinterpret_cast<const float4*>(ap + 16 * j + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
            av[j][0] = v0.x; av[j][1] = v0.y; av[j][2] = v0.z; av[j][3] = v0.w;
            av[j][4] = v1.x; av[j][5] = v1.y; av[j][6] = v1.z; av[j][7] = v1.w;
#pragma unroll
            for (int q = 0; q < 8; ++q) m = fmaxf(m, fabsf(av[j][q]));
        }
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
        if (__builtin_expect(not_finite(m), 0)) {        // an infinity among the rows: the largest finite entry
            m = 0.0f;
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int q = 0; q < 8; ++q) m = fmaxf(m, finite_abs(av[j][q]));
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
        }
        const int ka = scale_exponent(m);
        const float sa = pow2i(ka);
        inv_sa = pow2i(-ka);
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                _Float16 a, c;
                split_f16(av[j][q] * sa, a, c);
                ah[j][q] = a;
                al[j][q] = c;
            }
    }
    int dst[16];                        // destination rows of the 16 accumulator registers
#pragma unroll
    for (int q = 0; q < 16; ++q) {
        const int row = 32 * wave + 8 * (q / 4) + 4 * h + (q % 4);
        dst[q] = row < rows ? (c_rows ? c_rows[row0 + row] : row0 + row) : -1;
    }
    // one block of 32 columns: its image is in `cur`, the next one is loaded into `other`
    auto round = [&](int b, const unsigned char* cur, unsigned char* other) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (b + 1 < nblk) image_to_lds<Img::BYTES>(img0 + (size_t)(b + 1) * Img::BYTES, other, wave_s, lane16);
        float16_t acc;
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[q] = 0.0f;
        const _Float16* bph = reinterpret_cast<const _Float16*>(cur) + i * LDB + 8 * h;
        const _Float16* bpl = bph + 32 * LDB;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            const half8_t bh = *reinterpret_cast<const half8_t*>(bph + 16 * j);
            const half8_t bl = *reinterpret_cast<const half8_t*>(bpl + 16 * j);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[j], bh, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[j], bl, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[j], bh, acc, 0, 0, 0);
        }
        const float sinv = reinterpret_cast<const float*>(cur + Img::SINV)[i];
        const int col = 32 * b + i;
        if (col < N) {
            // the two inverse factors one after the other: their product need not be a float
#pragma unroll
            for (int q = 0; q < 16; ++q)
                if (dst[q] >= 0) C[(size_t)dst[q] * ldc + col] = acc[q] * inv_sa * sinv;
        }
    };
    for (int b = 0; b < nblk; b += 2) {
        round(b, sI0, sI1);
        if (b + 1 < nblk) round(b + 1, sI1, sI0);
    }
}

// sums[m] = sum_i values[m*n + i]: thread = row (the per-molecule energy of a padded batch)
__device__ __forceinline__ void row_sums(const float* __restrict__ values, int B, int n, float* __restrict__ sums, int chunk) {
    const int m = chunk * 256 + threadIdx.x;
    if (m >= B) return;
    float acc = 0.0f;
    for (int i = 0; i < n; ++i) acc += values[(size_t)m * n + i];
    sums[m] = acc;
}
// rows of real atoms whose element the model does not know get a zero gradient
// (lane = slot; the rare untyped slots of a wavefront are then zeroed row by row by all lanes)
__device__ __forceinline__ void zero_untyped_rows(const int* __restrict__ types, int N, int ne, int R,
                                                  float* __restrict__ out, int chunk) {
    const int slot = chunk * 256 + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int t = slot < N ? types[slot] : 0;
    unsigned long long todo = __ballot(slot < N && (t < 0 || t >= ne));
    while (todo) {
        const int l = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const size_t row = (size_t)(slot - lane + l) * R;
        for (int c = lane; c < R; c += 64) out[row + c] = 0.0f;
    }
}

__global__ __launch_bounds__(256) void zero_untyped_rows_kernel(const int* __restrict__ types, int N, int ne, int R,
                                                                float* __restrict__ out, int zero_groups,
                                                                const float* __restrict__ e_slots, int B, int n,
                                                                float* __restrict__ energies) {
    if ((int)blockIdx.x < zero_groups)
        zero_untyped_rows(types, N, ne, R, out, blockIdx.x);
    else                                               // workgroups past the slots: the per-molecule energy sums
        row_sums(e_slots, B, n, energies, (int)blockIdx.x - zero_groups);
}

// Small batches (a molecule to a few thousand atoms): the tiled kernels above run a few workgroups
// through ten dependent load-and-multiply steps, 17-26 us for 21 atoms and 20 / 14-18 us (forward /
// transposed) up to 8000.  Here a workgroup takes one to eight atoms of one element and spreads the
// contraction over its threads, so all loads of an atom are in flight at once and a reductor read serves
// the workgroup's atoms.  Beyond these limits the reductor re-reads from L2 (R d floats per workgroup)
// outweigh the latency: measured at R d = 40 000, forward 9 against 20 us at 2000 atoms, 12 against 20 at
// 4000, 15 against 21 at 5400 (eight atoms per workgroup; four were not tried there), 25 against 21 at
// 8000; transposed 12 against 14 at 2000, 16 against 18 at 4000, 20 against 18 at 5400
constexpr int SMALL_ATOMS = 4096;
constexpr size_t SMALL_READS = 192u << 20;   // floats of reductor per atom times atoms
__host__ inline bool small_batch(int A, int R, int d) { return A <= SMALL_ATOMS && (size_t)A * R * d <= SMALL_READS; }
constexpr int SMALL_KS = 8;        // slices of the contraction in project_small_kernel

__device__ __forceinline__ int type_of_position(const int* __restrict__ type_offsets, int ne, int p) {
    int e = 0;
    while (e + 1 < ne && p >= type_offsets[e + 1]) ++e;
    return e;
}

// NA consecutive sorted atoms of one element for workgroup b (tiles never straddle two elements)
template <int NA>
__device__ __forceinline__ bool small_tile(const int* __restrict__ type_offsets, int ne, int b, int& e, int& row0, int& rows) {
    for (int t = 0; t < ne; ++t) {
        const int o0 = type_offsets[t], o1 = type_offsets[t + 1];
        const int nt = (o1 - o0 + NA - 1) / NA;
        if (b < nt) {
            e = t;
            row0 = o0 + b * NA;
            rows = min(NA, o1 - row0);
            return true;
        }
        b -= nt;
    }
    return false;                                      // a tile beyond the sorted list
}

// x[p, :] = rep[slot(p), :] . U_e: thread = (contraction slice, four columns), slices folded through LDS;
// a workgroup takes NA atoms of one element, so a reductor read serves them all
template <int NA>
__global__ __launch_bounds__(256) void project_small_kernel(const float* __restrict__ rep,
                                                            const int* __restrict__ sorted_slots,
                                                            const int* __restrict__ type_offsets,
                                                            const float* __restrict__ reductors, int ne, int R, int d,
                                                            float* __restrict__ x) {
    extern __shared__ float sm[];
    const int R4 = (R + 3) & ~3;
    float* srow = sm;                                  // [NA][R4]
    float* spart = sm + NA * R4;                       // [SMALL_KS][NA][d]
    const int tid = threadIdx.x;
    int e, row0, rows;
    if (!small_tile<NA>(type_offsets, ne, blockIdx.x, e, row0, rows)) return;
    for (int a = 0; a < NA; ++a) {
        const float* row = rep + (size_t)sorted_slots[row0 + (a < rows ? a : 0)] * R;
        for (int k = tid; k < R; k += 256) srow[a * R4 + k] = a < rows ? row[k] : 0.0f;
    }
    __syncthreads();
    const float* U = reductors + (size_t)e * R * d;
    const int ks = tid >> 5, l32 = tid & 31;
    for (int c4 = l32; c4 < d / 4; c4 += 32) {
        float4 acc[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) acc[a] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
        for (int k = ks; k < R; k += SMALL_KS) {
            const float4 u = *reinterpret_cast<const float4*>(U + (size_t)k * d + 4 * c4);
#pragma unroll
            for (int a = 0; a < NA; ++a) {
                const float r = srow[a * R4 + k];
                acc[a].x = fmaf(r, u.x, acc[a].x);
                acc[a].y = fmaf(r, u.y, acc[a].y);
                acc[a].z = fmaf(r, u.z, acc[a].z);
                acc[a].w = fmaf(r, u.w, acc[a].w);
            }
        }
#pragma unroll
        for (int a = 0; a < NA; ++a) *reinterpret_cast<float4*>(spart + ((size_t)ks * NA + a) * d + 4 * c4) = acc[a];
    }
    __syncthreads();
    for (int i = tid; i < rows * d; i += 256) {
        const int a = i / d, c = i - a * d;
        float sum = 0.0f;
#pragma unroll
        for (int q = 0; q < SMALL_KS; ++q) sum += spart[((size_t)q * NA + a) * d + c];
        x[(size_t)(row0 + a) * d + c] = sum;
    }
}

// g_rep[slot(p), :] = gx[p, :] . U_e^T: thread = output entry r, its reductor row is contiguous.  A
// workgroup takes NA consecutive sorted atoms of one element (tiles never straddle two elements), so a
// reductor row read serves NA atoms: with one atom per workgroup 1008 atoms read 160 MB of reductors from
// L2 (20 us), with eight 20 MB.  Workgroups past the tiles zero the rows of slots whose type is outside
// [0, ne), 256 slots each, and after those, when asked, sum the per-slot energies of 256 molecules each.
template <int NA>
__global__ __launch_bounds__(256) void project_bt_small_kernel(const float* __restrict__ gx,
                                                               const int* __restrict__ sorted_slots,
                                                               const int* __restrict__ type_offsets,
                                                               const float* __restrict__ reductors, int ne, int R, int d,
                                                               float* __restrict__ g_rep, int tiles,
                                                               const int* __restrict__ types, int N, int zero_groups,
                                                               const float* __restrict__ e_slots, int B, int n,
                                                               float* __restrict__ energies) {
    extern __shared__ float sm[];                      // [NA][d]
    if ((int)blockIdx.x >= tiles + zero_groups) {      // spare workgroups: the per-molecule energy sums
        row_sums(e_slots, B, n, energies, (int)blockIdx.x - tiles - zero_groups);
        return;
    }
    if ((int)blockIdx.x >= tiles) {
        zero_untyped_rows(types, N, ne, R, g_rep, (int)blockIdx.x - tiles);
        return;
    }
    const int tid = threadIdx.x;
    int e, row0, rows;
    if (!small_tile<NA>(type_offsets, ne, blockIdx.x, e, row0, rows)) return;
    for (int i = tid; i < NA * d; i += 256) sm[i] = i < rows * d ? gx[(size_t)row0 * d + i] : 0.0f;
    __syncthreads();
    const float* U = reductors + (size_t)e * R * d;
    const float4* g4 = reinterpret_cast<const float4*>(sm);
    const int d4 = d / 4;
    for (int r = tid; r < R; r += 256) {
        const float4* u4 = reinterpret_cast<const float4*>(U + (size_t)r * d);
        float a0[NA], a1[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) a0[a] = a1[a] = 0.0f;
#pragma unroll 4
        for (int c4 = 0; c4 < d4; ++c4) {
            const float4 u = u4[c4];
#pragma unroll
            for (int a = 0; a < NA; ++a) {
                const float4 g = g4[a * d4 + c4];
                a0[a] = fmaf(u.x, g.x, fmaf(u.y, g.y, a0[a]));
                a1[a] = fmaf(u.z, g.z, fmaf(u.w, g.w, a1[a]));
            }
        }
#pragma unroll
        for (int a = 0; a < NA; ++a)
            if (a < rows) g_rep[(size_t)sorted_slots[row0 + a] * R + r] = a0[a] + a1[a];
    }
}

__global__ void zero_ints_kernel(int* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

extern "C" size_t qmll_sort_by_type_workspace(int A, int ne) {
    if (A <= 0 || ne <= 0) return 0;
    return (size_t)((A + ST - 1) / ST) * (size_t)ne * sizeof(int);
}

extern "C" int qmll_sort_by_type(const int* types, const int* slots, int A, int ne, void* workspace,
                                 size_t workspace_bytes, int* sorted_slots, int* type_offsets, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && ne > 0 && ne <= MAXNE, QMLL_ERR_INVALID, "qmll_sort_by_type: bad size A=%d ne=%d (at most %d types)",
                 A, ne, MAXNE);
    QMLL_REQUIRE(type_offsets, QMLL_ERR_INVALID, "qmll_sort_by_type: null pointer");
    if (A == 0) {
        hipLaunchKernelGGL(zero_ints_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, type_offsets, ne + 1);
        QMLL_CHECK_LAUNCH("qmll_sort_by_type");
        return QMLL_OK;
    }
    QMLL_REQUIRE(types && slots && sorted_slots && workspace, QMLL_ERR_INVALID, "qmll_sort_by_type: null pointer");
    QMLL_REQUIRE(workspace_bytes >= qmll_sort_by_type_workspace(A, ne), QMLL_ERR_INVALID,
                 "qmll_sort_by_type: workspace of %zu bytes, %zu needed", workspace_bytes,
                 qmll_sort_by_type_workspace(A, ne));
    const int nb = (A + ST - 1) / ST;
    int* counts = static_cast<int*>(workspace);
    hipLaunchKernelGGL(type_count_kernel, dim3(nb), dim3(ST), 0, (hipStream_t)stream, types, slots, A, ne, counts);
    QMLL_CHECK_LAUNCH("qmll_sort_by_type");
    hipLaunchKernelGGL(type_place_kernel, dim3(nb), dim3(ST), 0, (hipStream_t)stream, types, slots, A, ne, counts, nb,
                       sorted_slots, type_offsets);
    QMLL_CHECK_LAUNCH("qmll_sort_by_type");
    return QMLL_OK;
}

extern "C" size_t qmll_sort_atoms_workspace(int A, int ne) {
    if (A <= SORT_SMALL) return 0;
    return qmll_sort_by_type_workspace(A, ne) + sizeof(int) * (size_t)(A > 0 ? A : 0);
}

extern "C" int qmll_sort_atoms_by_type(const int* types, const int* atomIDs, const int* molIDs, int n, int A, int ne,
                                       void* workspace, size_t workspace_bytes, int* sorted_slots, int* type_offsets,
                                       qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && n > 0 && ne > 0 && ne <= MAXNE, QMLL_ERR_INVALID,
                 "qmll_sort_atoms_by_type: bad size A=%d n=%d ne=%d (at most %d types)", A, n, ne, MAXNE);
    QMLL_REQUIRE(type_offsets, QMLL_ERR_INVALID, "qmll_sort_atoms_by_type: null pointer");
    if (A == 0) {
        hipLaunchKernelGGL(zero_ints_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, type_offsets, ne + 1);
        QMLL_CHECK_LAUNCH("qmll_sort_atoms_by_type");
        return QMLL_OK;
    }
    QMLL_REQUIRE(types && atomIDs && molIDs && sorted_slots, QMLL_ERR_INVALID, "qmll_sort_atoms_by_type: null pointer");
    if (A <= SORT_SMALL) {
        hipLaunchKernelGGL(type_sort_small_kernel, dim3(1), dim3(SORT_SMALL), 0, (hipStream_t)stream, types, atomIDs,
                           molIDs, n, A, ne, sorted_slots, type_offsets);
        QMLL_CHECK_LAUNCH("qmll_sort_atoms_by_type");
        return QMLL_OK;
    }
    const size_t need = qmll_sort_atoms_workspace(A, ne);
    QMLL_REQUIRE(workspace && workspace_bytes >= need, QMLL_ERR_INVALID,
                 "qmll_sort_atoms_by_type: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    // the slots go behind the counts of the general sort
    const size_t counts_bytes = qmll_sort_by_type_workspace(A, ne);
    int* slots = reinterpret_cast<int*>(static_cast<char*>(workspace) + counts_bytes);
    hipLaunchKernelGGL(atom_slots_kernel, dim3((A + 255) / 256), dim3(256), 0, (hipStream_t)stream, atomIDs, molIDs, n, A,
                       slots);
    QMLL_CHECK_LAUNCH("qmll_sort_atoms_by_type");
    return qmll_sort_by_type(types, slots, A, ne, workspace, counts_bytes, sorted_slots, type_offsets, stream);
}

extern "C" int qmll_prepare_batch(const float* Z, const int* natoms, const float* species, int nspecies,
                                  const float* model_species, int ne, const int* atomIDs, const int* molIDs, int B, int n,
                                  int A, void* workspace, size_t workspace_bytes, int* types, int* sort_types,
                                  int* sorted_slots, int* type_offsets, float* zero, size_t zero_count, qmll_stream_t stream) {
    QMLL_REQUIRE(B >= 0 && n >= 0 && A >= 0 && nspecies > 0 && ne > 0 && ne <= MAXNE, QMLL_ERR_INVALID,
                 "qmll_prepare_batch: bad size B=%d n=%d A=%d nspecies=%d ne=%d (at most %d types)", B, n, A, nspecies, ne,
                 MAXNE);
    QMLL_REQUIRE(model_species || ne == nspecies, QMLL_ERR_INVALID,
                 "qmll_prepare_batch: %d model elements for %d species and no model species given", ne, nspecies);
    QMLL_REQUIRE(type_offsets && species && (zero || zero_count == 0), QMLL_ERR_INVALID, "qmll_prepare_batch: null pointer");
    QMLL_REQUIRE(!model_species || sort_types || (size_t)B * n == 0, QMLL_ERR_INVALID,
                 "qmll_prepare_batch: model species without a sort_types output");
    const size_t slots = (size_t)B * n;
    if (A > 0 && A <= PREP_CHUNKS * SORT_SMALL && slots > 0 && slots <= 65536 && zero_count <= 262144) {
        QMLL_REQUIRE(Z && natoms && atomIDs && molIDs && types && sorted_slots, QMLL_ERR_INVALID,
                     "qmll_prepare_batch: null pointer");
        hipLaunchKernelGGL(prepare_small_kernel, dim3(1), dim3(SORT_SMALL), 0, (hipStream_t)stream, Z, natoms, species, nspecies,
                           model_species, ne, atomIDs, molIDs, B, n, A, types, sort_types, sorted_slots, type_offsets, zero,
                           (int)zero_count);
        QMLL_CHECK_LAUNCH("qmll_prepare_batch");
        return QMLL_OK;
    }
    if (A == 0 || slots == 0) {               // nothing listed: clear what was asked and write the offsets
        int rc = qmll_element_types(Z, natoms, species, B, n, nspecies, types, stream);
        if (rc != QMLL_OK) return rc;
        if (model_species) {
            rc = qmll_element_types(Z, natoms, model_species, B, n, ne, sort_types, stream);
            if (rc != QMLL_OK) return rc;
        }
        if (zero_count > 0) {
            const size_t groups = (zero_count + 255) / 256;
            hipLaunchKernelGGL(zero_floats_kernel, dim3((unsigned)(groups < 4096 ? groups : 4096)), dim3(256), 0,
                               (hipStream_t)stream, zero, zero_count);
            QMLL_CHECK_LAUNCH("qmll_prepare_batch");
        }
        return qmll_sort_atoms_by_type(model_species ? sort_types : types, atomIDs, molIDs, n > 0 ? n : 1, 0, ne, workspace,
                                       workspace_bytes, sorted_slots, type_offsets, stream);
    }
    QMLL_REQUIRE(Z && natoms && atomIDs && molIDs && types && sorted_slots, QMLL_ERR_INVALID,
                 "qmll_prepare_batch: null pointer");
    // few listed atoms in a batch with many slots (heavy padding): the one-workgroup sort needs no workspace and
    // builds the slots itself; else they go behind the counts of the general sort, as in qmll_sort_atoms_by_type
    const bool one_workgroup_sort = A <= SORT_SMALL;
    const size_t need = qmll_sort_atoms_workspace(A, ne);
    QMLL_REQUIRE(one_workgroup_sort || (workspace && workspace_bytes >= need), QMLL_ERR_INVALID,
                 "qmll_prepare_batch: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    const size_t counts_bytes = qmll_sort_by_type_workspace(A, ne);
    int* atom_slots = one_workgroup_sort ? nullptr : reinterpret_cast<int*>(static_cast<char*>(workspace) + counts_bytes);
    size_t work = slots > zero_count ? slots : zero_count;
    if ((size_t)A > work) work = (size_t)A;
    const size_t groups = (work + 255) / 256;
    hipLaunchKernelGGL(prepare_large_kernel, dim3((unsigned)(groups < 8192 ? groups : 8192)), dim3(256), 0, (hipStream_t)stream,
                       Z, natoms, species, nspecies, model_species, ne, atomIDs, molIDs, slots, n, A, types, sort_types,
                       atom_slots, zero, zero_count);
    QMLL_CHECK_LAUNCH("qmll_prepare_batch");
    if (one_workgroup_sort)
        return qmll_sort_atoms_by_type(model_species ? sort_types : types, atomIDs, molIDs, n, A, ne, nullptr, 0, sorted_slots,
                                       type_offsets, stream);
    return qmll_sort_by_type(model_species ? sort_types : types, atom_slots, A, ne, workspace, counts_bytes, sorted_slots,
                             type_offsets, stream);
}

// ---- the same sort for callers that cannot allocate -------------------------------------
// The per-workgroup counts live in a file-scope device array instead of a caller workspace.
// Every GPU the library runs on holds its own copy at its own address until the process
// ends; the address is looked up once per device and only that pointer is ever handed to a
// kernel (the array's name in host code is a host-side stand-in, not a device address).
constexpr int SCRATCH_INTS = QMLL_SORT_NOALLOC_MAX_COUNTS;
constexpr int MAX_DEVICES = 64;
static __device__ __align__(256) int scratch[SCRATCH_INTS];

namespace {
std::mutex scratch_mutex;
int* scratch_ptr[MAX_DEVICES] = {};

// device address of `scratch` on the current device (nullptr + error text on failure)
int* scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        qmll_set_error("qmll_sort_by_type_noalloc: no usable current device (%d)", dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            qmll_set_error("qmll_sort_by_type_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return nullptr;
        }
        scratch_ptr[dev] = static_cast<int*>(p);
    }
    return scratch_ptr[dev];
}
}  // namespace

extern "C" int qmll_sort_by_type_noalloc(const int* types, const int* slots, int A, int ne, int* sorted_slots,
                                         int* type_offsets, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && ne > 0 && ne <= MAXNE, QMLL_ERR_INVALID,
                 "qmll_sort_by_type_noalloc: bad size A=%d ne=%d (at most %d types)", A, ne, MAXNE);
    const long long need = (long long)((A + ST - 1) / ST) * ne;
    QMLL_REQUIRE(need <= (long long)SCRATCH_INTS, QMLL_ERR_INVALID,
                 "qmll_sort_by_type_noalloc: A=%d atoms of ne=%d types need %lld counters, the built-in scratch holds %d "
                 "(ceil(A/%d)*ne must not exceed it); use qmll_sort_by_type with a workspace",
                 A, ne, need, SCRATCH_INTS, ST);
    int* counts = scratch_of_current_device();
    if (!counts) return QMLL_ERR_LAUNCH;
    // every counter the placement kernel reads is written by the counting kernel of the same
    // call, so nothing of the previous call's contents needs clearing
    return qmll_sort_by_type(types, slots, A, ne, counts, (size_t)SCRATCH_INTS * sizeof(int), sorted_slots, type_offsets,
                             stream);
}

// layout of the prepared reductors: forward images, backward images, forward exponents
struct SplitLayout {
    size_t fwd_bytes, bwd_bytes, exp_bytes;
    int nchunks, ncb, nblk;
    size_t bwd_image;
    size_t total() const { return fwd_bytes + bwd_bytes + exp_bytes; }
};
static SplitLayout split_layout(int ne, int R, int d) {
    SplitLayout L{};
    if (ne <= 0 || R <= 0 || d <= 0 || R % 4 != 0) return L;
    L.nchunks = (R + PK - 1) / PK;
    L.nblk = (R + 31) / 32;
    if (d % 128 == 0) {
        L.ncb = d / 128;
        L.fwd_bytes = (size_t)ne * L.nchunks * L.ncb * FWD_IMG_BYTES;
        L.exp_bytes = ((size_t)ne * L.nchunks * L.ncb * sizeof(int) + 15) / 16 * 16;
    }
    if (d == 64 || d == 128) {
        L.bwd_image = d == 64 ? (size_t)BwdImage<64>::BYTES : (size_t)BwdImage<128>::BYTES;
        L.bwd_bytes = (size_t)ne * L.nblk * L.bwd_image;
    }
    return L;
}

extern "C" size_t qmll_reductor_presplit_bytes(int ne, int R, int d) { return split_layout(ne, R, d).total(); }

extern "C" int qmll_reductor_presplit(const float* reductors, int ne, int R, int d, void* out, size_t out_bytes,
                                      qmll_stream_t stream) {
    QMLL_REQUIRE(ne > 0 && R > 0 && d > 0 && ne <= 65535, QMLL_ERR_INVALID, "qmll_reductor_presplit: bad size ne=%d R=%d d=%d", ne, R, d);
    const SplitLayout L = split_layout(ne, R, d);
    QMLL_REQUIRE(L.total() > 0, QMLL_ERR_INVALID,
                 "qmll_reductor_presplit: no kernel takes prepared reductors of R=%d (a multiple of 4) x d=%d (64 or a multiple of 128)", R, d);
    QMLL_REQUIRE(reductors && out && aligned16(reductors) && aligned16(out), QMLL_ERR_INVALID,
                 "qmll_reductor_presplit: null or unaligned pointer");
    QMLL_REQUIRE(out_bytes >= L.total(), QMLL_ERR_INVALID, "qmll_reductor_presplit: output of %zu bytes, %zu are needed",
                 out_bytes, L.total());
    unsigned char* base = (unsigned char*)out;
    if (L.fwd_bytes) {
        hipLaunchKernelGGL(reductor_presplit_fwd_kernel, dim3(L.nchunks * L.ncb, ne), dim3(PT), 0, (hipStream_t)stream,
                           reductors, R, d, L.ncb, (_Float16*)base, (int*)(base + L.fwd_bytes + L.bwd_bytes));
        QMLL_CHECK_LAUNCH("qmll_reductor_presplit");
    }
    if (L.bwd_bytes) {
        if (d == 64)
            hipLaunchKernelGGL(reductor_presplit_bwd_kernel<64>, dim3(L.nblk, ne), dim3(PT), 0, (hipStream_t)stream, reductors,
                               R, base + L.fwd_bytes);
        else
            hipLaunchKernelGGL(reductor_presplit_bwd_kernel<128>, dim3(L.nblk, ne), dim3(PT), 0, (hipStream_t)stream, reductors,
                               R, base + L.fwd_bytes);
        QMLL_CHECK_LAUNCH("qmll_reductor_presplit");
    }
    return QMLL_OK;
}

extern "C" int qmll_project_typed(const float* rep, const int* sorted_slots, const int* type_offsets,
                                  const float* reductors, const void* reductors_split, int A, int ne, int R, int d, float* x,
                                  qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && ne > 0 && R > 0 && d > 0, QMLL_ERR_INVALID, "qmll_project_typed: bad size A=%d ne=%d R=%d d=%d", A,
                 ne, R, d);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(rep && sorted_slots && type_offsets && reductors && x, QMLL_ERR_INVALID,
                 "qmll_project_typed: null pointer");
    const bool vec = R % 4 == 0 && d % 4 == 0 && aligned16(rep) && aligned16(reductors);
    if (vec && small_batch(A, R, d)) {
        // several atoms of one element per workgroup from some hundreds of atoms on, while their rows and partial
        // sums fit in LDS
        const size_t per_atom = sizeof(float) * (((size_t)R + 3) / 4 * 4 + (size_t)SMALL_KS * d);
        // (measured at 312 x 128: one atom 8.4 us at 1008 atoms and 12.8 at 2016, two 8.1 / 8.7, four 10.2 / 10.7 and
        // 11.8 at 4032, where two take 13.8; eight are never the fastest: the loads here are coalesced, the
        // multiplications of a workgroup are what grows)
        int na = A <= 768 ? 1 : (A <= 2304 ? 2 : 4);
        while (na > 1 && na * per_atom > 64 * 1024) na >>= 1;
        if (per_atom <= 64 * 1024) {
            const dim3 grid((A + na - 1) / na + (na > 1 ? ne : 0));
            if (na == 1)
                hipLaunchKernelGGL(project_small_kernel<1>, grid, dim3(256), per_atom, (hipStream_t)stream, rep, sorted_slots,
                                   type_offsets, reductors, ne, R, d, x);
            else if (na == 2)
                hipLaunchKernelGGL(project_small_kernel<2>, grid, dim3(256), 2 * per_atom, (hipStream_t)stream, rep,
                                   sorted_slots, type_offsets, reductors, ne, R, d, x);
            else
                hipLaunchKernelGGL(project_small_kernel<4>, grid, dim3(256), 4 * per_atom, (hipStream_t)stream, rep,
                                   sorted_slots, type_offsets, reductors, ne, R, d, x);
            QMLL_CHECK_LAUNCH("qmll_project_typed");
            return QMLL_OK;
        }
    }
    const int tiles = (A + PM - 1) / PM + ne;
    // the wide tile when it wastes no columns and still leaves every CU a few workgroups
    const bool wide = vec && d % 128 == 0 && (long long)tiles * (d / 128) >= 2 * 256;
    const dim3 grid(tiles, wide ? d / 128 : (d + PN - 1) / PN);
    if (wide && reductors_split) {
        const SplitLayout L = split_layout(ne, R, d);
        QMLL_REQUIRE(aligned16(reductors_split), QMLL_ERR_INVALID, "qmll_project_typed: reductors_split must be 16-byte aligned");
        const unsigned char* base = (const unsigned char*)reductors_split;
        hipLaunchKernelGGL(typed_gemm_f16_kernel, grid, dim3(PT), 0, (hipStream_t)stream, rep, R, sorted_slots,
                           (const _Float16*)base, (const int*)(base + L.fwd_bytes + L.bwd_bytes), x, d, type_offsets, ne, R, d, 1);
    } else if (wide)
        hipLaunchKernelGGL((typed_gemm_kernel<false, true, 128>), grid, dim3(PT), 0, (hipStream_t)stream, rep, R, sorted_slots,
                           reductors, (size_t)R * d, d, x, d, (const int*)nullptr, type_offsets, ne, R, d, 1);
    else if (vec)
        hipLaunchKernelGGL((typed_gemm_kernel<false, true, PN>), grid, dim3(PT), 0, (hipStream_t)stream, rep, R, sorted_slots,
                           reductors, (size_t)R * d, d, x, d, (const int*)nullptr, type_offsets, ne, R, d);
    else
        hipLaunchKernelGGL((typed_gemm_kernel<false, false, PN>), grid, dim3(PT), 0, (hipStream_t)stream, rep, R,
                           sorted_slots, reductors, (size_t)R * d, d, x, d, (const int*)nullptr, type_offsets, ne, R, d);
    QMLL_CHECK_LAUNCH("qmll_project_typed");
    return QMLL_OK;
}

extern "C" int qmll_project_typed_rows(const float* rows, const int* sorted_slots, const int* type_offsets,
                                       const float* reductors, int A, int ne, int R, int d, int group, float* x,
                                       qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && ne > 0 && R > 0 && d > 0 && group > 0, QMLL_ERR_INVALID,
                 "qmll_project_typed_rows: bad size A=%d ne=%d R=%d d=%d group=%d", A, ne, R, d, group);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(rows && sorted_slots && type_offsets && reductors && x, QMLL_ERR_INVALID,
                 "qmll_project_typed_rows: null pointer");
    QMLL_REQUIRE((long long)A * group < (1ll << 31) - PM, QMLL_ERR_INVALID,
                 "qmll_project_typed_rows: %d atoms x %d rows exceed the 32-bit row count of one launch", A, group);
    const bool vec = R % 4 == 0 && d % 4 == 0 && aligned16(rows) && aligned16(reductors);
    const long long nrows = (long long)A * group;
    const int tiles = (int)((nrows + PM - 1) / PM) + ne;
    const bool wide = vec && d % 128 == 0 && (long long)tiles * (d / 128) >= 2 * 256;
    const dim3 grid(tiles, wide ? d / 128 : (d + PN - 1) / PN);
    // the fp32 matrix instructions here: a row's result then does not depend on the rows that share its
    // tile (the half-precision kernel scales a whole chunk of the tile by one power of two), so the rows
    // of a training batch are the same however the training set is cut into batches
    if (wide)
        hipLaunchKernelGGL((typed_gemm_kernel<false, true, 128>), grid, dim3(PT), 0, (hipStream_t)stream, rows, R,
                           sorted_slots, reductors, (size_t)R * d, d, x, d, (const int*)nullptr, type_offsets, ne, R, d,
                           group);
    else if (vec)
        hipLaunchKernelGGL((typed_gemm_kernel<false, true, PN>), grid, dim3(PT), 0, (hipStream_t)stream, rows, R,
                           sorted_slots, reductors, (size_t)R * d, d, x, d, (const int*)nullptr, type_offsets, ne, R, d,
                           group);
    else
        hipLaunchKernelGGL((typed_gemm_kernel<false, false, PN>), grid, dim3(PT), 0, (hipStream_t)stream, rows, R,
                           sorted_slots, reductors, (size_t)R * d, d, x, d, (const int*)nullptr, type_offsets, ne, R, d,
                           group);
    QMLL_CHECK_LAUNCH("qmll_project_typed_rows");
    return QMLL_OK;
}

extern "C" int qmll_project_typed_backward(const float* gx, const int* sorted_slots, const int* type_offsets,
                                           const float* reductors, const void* reductors_split, const int* types, int A,
                                           int N, int ne, int R, int d, float* g_rep, qmll_stream_t stream) {
    return qmll_project_typed_backward_sums(gx, sorted_slots, type_offsets, reductors, reductors_split, types, A, N, ne, R, d,
                                            g_rep, nullptr, 0, 0, nullptr, stream);
}

extern "C" int qmll_project_typed_backward_sums(const float* gx, const int* sorted_slots, const int* type_offsets,
                                                const float* reductors, const void* reductors_split, const int* types,
                                                int A, int N, int ne, int R, int d, float* g_rep, const float* e_slots,
                                                int B, int n, float* energies, qmll_stream_t stream) {
    QMLL_REQUIRE(A >= 0 && N >= 0 && ne > 0 && R > 0 && d > 0, QMLL_ERR_INVALID,
                 "qmll_project_typed_backward: bad size A=%d N=%d ne=%d R=%d d=%d", A, N, ne, R, d);
    const bool sums = energies != nullptr && B > 0;
    QMLL_REQUIRE(!sums || (e_slots && n > 0), QMLL_ERR_INVALID, "qmll_project_typed_backward_sums: energies without e_slots");
    const bool vec = R % 4 == 0 && d % 4 == 0 && aligned16(gx) && aligned16(reductors);
    const bool small = vec && A > 0 && small_batch(A, R, d) && (size_t)8 * d * sizeof(float) <= 64 * 1024 && N <= 256 * 256;
    if (!small && ((types && N > 0) || sums)) {
        // the rows of unknown elements and the energy sums: one launch for the two
        const int zero_groups = (types && N > 0) ? (N + 255) / 256 : 0;
        const int sum_groups = sums ? (B + 255) / 256 : 0;
        QMLL_REQUIRE(g_rep || zero_groups == 0, QMLL_ERR_INVALID, "qmll_project_typed_backward: null pointer");
        hipLaunchKernelGGL(zero_untyped_rows_kernel, dim3(zero_groups + sum_groups), dim3(256), 0, (hipStream_t)stream, types,
                           N, ne, R, g_rep, zero_groups, e_slots, B, n, energies);
        QMLL_CHECK_LAUNCH("qmll_project_typed_backward");
    }
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(gx && sorted_slots && type_offsets && reductors && g_rep, QMLL_ERR_INVALID,
                 "qmll_project_typed_backward: null pointer");
    const dim3 grid((A + PM - 1) / PM + ne, (R + PN - 1) / PN);
    if (small) {
        // one launch: a workgroup per atom, one per 256 slots for the rows of unknown elements, one per 256
        // molecules for the energy sums
        const int zero_groups = (types && N > 0) ? (N + 255) / 256 : 0;
        const int sum_groups = sums ? (B + 255) / 256 : 0;
        // atoms per workgroup: one while the atoms are the only parallelism there is, more as the reductor
        // reads of all workgroups together begin to count
#define LAUNCH_BT_SMALL(NA)                                                                                         \
    {                                                                                                               \
        const int tiles = (A + (NA) - 1) / (NA) + ((NA) > 1 ? ne : 0);                                              \
        hipLaunchKernelGGL(project_bt_small_kernel<NA>, dim3(tiles + zero_groups + sum_groups), dim3(256),          \
                           sizeof(float) * (NA) * d, (hipStream_t)stream, gx, sorted_slots, type_offsets, reductors, \
                           ne, R, d, g_rep, tiles, types, N, zero_groups, e_slots, B, n, energies);                 \
    }
        if (A < 64) LAUNCH_BT_SMALL(1) else if (A < 512) LAUNCH_BT_SMALL(4) else LAUNCH_BT_SMALL(8)
#undef LAUNCH_BT_SMALL
    } else if (vec && (d == 64 || d == 128) && reductors_split) {
        // short contraction: the gradient rows stay in registers, every row is read once
        const SplitLayout L = split_layout(ne, R, d);
        QMLL_REQUIRE(aligned16(reductors_split), QMLL_ERR_INVALID,
                     "qmll_project_typed_backward: reductors_split must be 16-byte aligned");
        const unsigned char* images = (const unsigned char*)reductors_split + L.fwd_bytes;
        const dim3 g1((A + PM - 1) / PM + ne);
        if (d == 128)
            hipLaunchKernelGGL((typed_gemm_bt_rows_f16_kernel<128>), g1, dim3(PT), 0, (hipStream_t)stream, gx, images, g_rep,
                               R, sorted_slots, type_offsets, ne, R);
        else
            hipLaunchKernelGGL((typed_gemm_bt_rows_f16_kernel<64>), g1, dim3(PT), 0, (hipStream_t)stream, gx, images, g_rep,
                               R, sorted_slots, type_offsets, ne, R);
    } else if (vec)
        hipLaunchKernelGGL((typed_gemm_kernel<true, true, PN>), grid, dim3(PT), 0, (hipStream_t)stream, gx, d,
                           (const int*)nullptr, reductors, (size_t)R * d, d, g_rep, R, sorted_slots, type_offsets, ne, d, R);
    else
        hipLaunchKernelGGL((typed_gemm_kernel<true, false, PN>), grid, dim3(PT), 0, (hipStream_t)stream, gx, d,
                           (const int*)nullptr, reductors, (size_t)R * d, d, g_rep, R, sorted_slots, type_offsets, ne, d, R);
    QMLL_CHECK_LAUNCH("qmll_project_typed_backward");
    return QMLL_OK;
}
