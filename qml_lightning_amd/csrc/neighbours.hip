// Neighbour counts / lists and element types.
// Replaces qml_lightning/cuda/pairlist_kernel.cu:145-224,326-391 and
// fchl_cuda_kernel.cu:1716-1742 of the reference.
//
// One wavefront per molecule tile: lane = central atom, serial loop over the candidate
// atoms whose coordinates every lane reads at the same address (one broadcast load per
// candidate).  HBM traffic is 12 B per atom in and 4*(1+nn) B out; nothing to tile.
#include "qmll_common.h"

__device__ __forceinline__ void min_image(float& dx, float& dy, float& dz, const float* __restrict__ cell,
                                          const float* __restrict__ inv) {
    // s = inv d ; s -= round(s) ; d = cell s      (fchl_cuda_kernel.cu:16-49)
    float s0 = inv[0] * dx + inv[1] * dy + inv[2] * dz;
    float s1 = inv[3] * dx + inv[4] * dy + inv[5] * dz;
    float s2 = inv[6] * dx + inv[7] * dy + inv[8] * dz;
    s0 -= roundf(s0);
    s1 -= roundf(s1);
    s2 -= roundf(s2);
    dx = cell[0] * s0 + cell[1] * s1 + cell[2] * s2;
    dy = cell[3] * s0 + cell[4] * s1 + cell[5] * s2;
    dz = cell[6] * s0 + cell[7] * s1 + cell[8] * s2;
}

template <bool WRITE_LIST>
__global__ __launch_bounds__(64) void neighbours_kernel(const float* __restrict__ X, const int* __restrict__ natoms,
                                                         const float* __restrict__ cell,
                                                         const float* __restrict__ inv_cell, int n, int nn_max,
                                                         float rcut2, int* __restrict__ out) {
    const int m = blockIdx.x;
    const int i = blockIdx.y * 64 + threadIdx.x;
    if (i >= n) return;
    const int na = natoms[m];
    const float* Xm = X + (size_t)m * n * 3;
    const bool pbc = cell != nullptr;
    float c[9], ic[9];
    if (pbc) {
        for (int t = 0; t < 9; ++t) {
            c[t] = cell[(size_t)m * 9 + t];
            ic[t] = inv_cell[(size_t)m * 9 + t];
        }
    }
    int count = 0;
    if (i < na) {
        const float xi = Xm[i * 3 + 0], yi = Xm[i * 3 + 1], zi = Xm[i * 3 + 2];
        for (int j = 0; j < na; ++j) {
            float dx = xi - Xm[j * 3 + 0];
            float dy = yi - Xm[j * 3 + 1];
            float dz = zi - Xm[j * 3 + 2];
            if (pbc) min_image(dx, dy, dz, c, ic);
            const float r2 = dx * dx + dy * dy + dz * dz;
            if (r2 < rcut2 && r2 > 0.0f) {
                if (WRITE_LIST) {
                    if (count < nn_max) out[((size_t)m * n + i) * nn_max + count] = j;
                }
                ++count;
            }
        }
    }
    if (WRITE_LIST) {
        for (int t = (count < nn_max ? count : nn_max); t < nn_max; ++t) out[((size_t)m * n + i) * nn_max + t] = -1;
    } else {
        out[(size_t)m * n + i] = count;
    }
}

__global__ __launch_bounds__(256) void element_types_kernel(const float* __restrict__ Z, const int* __restrict__ natoms,
                                                            const float* __restrict__ species, int B, int n, int ns,
                                                            int* __restrict__ types) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)B * n) return;
    const int m = idx / n, i = idx - (size_t)m * n;
    int t = 0;
    if (i < natoms[m]) {
        const int q = (int)Z[idx];
        t = -1;
        for (int j = 0; j < ns; ++j)
            if (q == (int)species[j]) t = j;
    }
    types[idx] = t;
}

static int check_nb(const float* X, const int* natoms, const float* cell, const float* inv_cell, int B, int n,
                    const void* out) {
    QMLL_REQUIRE(B >= 0 && n >= 0, QMLL_ERR_INVALID, "neighbours: negative size B=%d n=%d", B, n);
    QMLL_REQUIRE((X && natoms && out) || B == 0 || n == 0, QMLL_ERR_INVALID, "neighbours: null pointer");
    QMLL_REQUIRE((cell == nullptr) == (inv_cell == nullptr), QMLL_ERR_INVALID,
                 "neighbours: cell and inv_cell must both be given or both be NULL");
    QMLL_REQUIRE(B <= 65535 * 1024, QMLL_ERR_INVALID, "neighbours: too many molecules (%d)", B);
    return QMLL_OK;
}

extern "C" int qmll_num_neighbours(const float* X, const int* natoms, const float* cell, const float* inv_cell, int B,
                                   int n, float rcut, int* nneigh, qmll_stream_t stream) {
    int rc = check_nb(X, natoms, cell, inv_cell, B, n, nneigh);
    if (rc) return rc;
    if (B == 0 || n == 0) return QMLL_OK;
    dim3 grid(B, (n + 63) / 64);
    hipLaunchKernelGGL(neighbours_kernel<false>, grid, dim3(64), 0, (hipStream_t)stream, X, natoms, cell, inv_cell, n, 0,
                       rcut * rcut, nneigh);
    QMLL_CHECK_LAUNCH("qmll_num_neighbours");
    return QMLL_OK;
}

extern "C" int qmll_neighbour_list(const float* X, const int* natoms, const float* cell, const float* inv_cell, int B,
                                   int n, int max_neighbours, float rcut, int* nlist, qmll_stream_t stream) {
    int rc = check_nb(X, natoms, cell, inv_cell, B, n, nlist);
    if (rc) return rc;
    QMLL_REQUIRE(max_neighbours >= 0, QMLL_ERR_INVALID, "neighbour_list: max_neighbours=%d", max_neighbours);
    if (B == 0 || n == 0 || max_neighbours == 0) return QMLL_OK;
    dim3 grid(B, (n + 63) / 64);
    hipLaunchKernelGGL(neighbours_kernel<true>, grid, dim3(64), 0, (hipStream_t)stream, X, natoms, cell, inv_cell, n,
                       max_neighbours, rcut * rcut, nlist);
    QMLL_CHECK_LAUNCH("qmll_neighbour_list");
    return QMLL_OK;
}

extern "C" int qmll_element_types(const float* Z, const int* natoms, const float* species, int B, int n, int nspecies,
                                  int* types, qmll_stream_t stream) {
    QMLL_REQUIRE(B >= 0 && n >= 0 && nspecies > 0, QMLL_ERR_INVALID, "element_types: bad size B=%d n=%d ns=%d", B, n,
                 nspecies);
    if (B == 0 || n == 0) return QMLL_OK;
    QMLL_REQUIRE(Z && natoms && species && types, QMLL_ERR_INVALID, "element_types: null pointer");
    const size_t total = (size_t)B * n;
    hipLaunchKernelGGL(element_types_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, Z,
                       natoms, species, B, n, nspecies, types);
    QMLL_CHECK_LAUNCH("qmll_element_types");
    return QMLL_OK;
}
