// FCHL19 representation, its VJP and its explicit Jacobian for gfx950.
// Replaces qml_lightning/cuda/fchl_cuda_kernel.cu:476-674 (forward), :1325-1714 (VJP),
// :676-1005 and :1007-1323 (Jacobian) of the reference.
//
// Layout: one wavefront (64 lanes, one workgroup) per central atom.  The atom's
// neighbour list is staged in LDS sorted by element, as displacement vectors d_ij = R_i - R_j
// (minimum-imaged once when a cell is given) with whatever else of a neighbour the kernel reads
// again (forward and VJP: 16-byte records written by the lane that finds the neighbour; Jacobian:
// one array per quantity); it is either read from a caller-supplied list or built in the kernel
// from the molecule's coordinates with a ballot/popcount compaction (ascending j, same rule as the
// neighbour-list kernel), so the forward/backward pair needs no host round trip for max(nneigh).
//
// Arithmetic per atom (nn neighbours): nn*nRs2 + nn(nn-1)/2*nRs3 exponentials forward;
// the kernels are VALU/transcendental bound, HBM traffic is 4R bytes out (forward) or in
// (VJP) per atom.
//
// The derivatives are written in terms of the three distances a=r_ij, b=r_ik, c=r_jk of a
// triple: every bin value T depends on positions only through (a,b,c) and
// cos_i = (a^2+b^2-c^2)/(2ab) etc., so dT = T_a da + T_b db + T_c dc with
// da/dR_i = u_ij, da/dR_j = -u_ij, db/dR_i = u_ik, db/dR_k = -u_ik, dc/dR_j = u_jk,
// dc/dR_k = -u_jk.  This is algebraically the reference's 40-term expansion; the
// degenerate-angle guard sqrt(max(1e-10, a^2 b^2 - (d_ij.d_ik)^2)) is kept.
#include <type_traits>

#include "qmll_common.h"

namespace {
// 1-ulp forms on the transcendental unit (operands here are distances and widths, far from the
// denormal range): a correctly rounded division, square root or logarithm costs ten or more
// instructions each, several times per neighbour and per triple
__device__ __forceinline__ float frcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fsqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ float frsq(float x) { return __builtin_amdgcn_rsqf(x); }
__device__ __forceinline__ float flog(float x) { return __builtin_amdgcn_logf(x) * 0.6931471805599453f; }
// floor(x / d) for 0 <= x < 1e6, 0 < d: (x + 0.5) / d is at least 0.5 / d away from an integer,
// far more than the rounding of the 1-ulp reciprocal, so the truncation is exact; five
// instructions where the integer division expands to about twenty-five
__device__ __forceinline__ int idiv_small(int x, int d) { return (int)(((float)x + 0.5f) * frcp((float)d)); }

struct FchlArgs {
    const float* X;
    const int* types;
    const float* cell;
    const float* inv_cell;
    const int* atomIDs;
    const int* molIDs;
    const int* natoms;
    const int* nlist;
    const int* nneigh;
    int nn_stride;
    int n;
    int B;
    int cap;  // capacity of the LDS neighbour arrays
    int tcap; // capacity (entries) of the forward kernel's LDS triple table
    int tpad; // extra entries for the zero padding between the table's segments
    const float* Rs2;
    const float* Rs3;
    qmll_fchl_params p;
    float gscale;  // the backward kernel returns gscale * J^T g (folded into the staged gradient row)
};

constexpr int TCH = 256;      // smallest triple table
constexpr int TCH_MAX = 1024; // largest (16 KB): beyond, element pairs are processed in chunks
constexpr float PI_F = 3.14159265358979323846f;
// three floats read from a 16-byte-aligned LDS entry with a single 12-byte instruction (a 16-byte
// read of the same entry occupies the LDS pipe a third longer)
typedef float float3v __attribute__((ext_vector_type(3)));

// LDS neighbour arrays of one central atom, sorted by element type (stable in j within a
// type); goff[e]..goff[e+1] is the slice of type e.
struct Stage {
    float* dx;
    float* dy;
    float* dz;
    float* r;
    float* fc;    // cosine cutoff at r
    float* dfc;   // its r-derivative
    int* el;
    int* j;
    int* goff;    // [ns+1]
    float* next;  // first free float after the neighbour arrays
};

constexpr int STAGE_ARRAYS = 8;   // per-neighbour arrays carved by `carve`

__device__ __forceinline__ Stage carve(float* smem, int cap, int ns) {
    Stage s;
    s.dx = smem;
    s.dy = s.dx + cap;
    s.dz = s.dy + cap;
    s.r = s.dz + cap;
    s.fc = s.r + cap;
    s.dfc = s.fc + cap;
    s.el = (int*)(s.dfc + cap);
    s.j = s.el + cap;
    s.goff = s.j + cap;
    s.next = (float*)(s.goff + ns + 1);
    return s;
}

__device__ __forceinline__ void min_image(float& dx, float& dy, float& dz, const float* c, const float* ic) {
    float s0 = ic[0] * dx + ic[1] * dy + ic[2] * dz;
    float s1 = ic[3] * dx + ic[4] * dy + ic[5] * dz;
    float s2 = ic[6] * dx + ic[7] * dy + ic[8] * dz;
    s0 -= roundf(s0);
    s1 -= roundf(s1);
    s2 -= roundf(s2);
    dx = c[0] * s0 + c[1] * s1 + c[2] * s2;
    dy = c[3] * s0 + c[4] * s1 + c[5] * s2;
    dz = c[6] * s0 + c[7] * s1 + c[8] * s2;
}


// Visit the neighbours of atom (m,i) sorted by element type; returns the neighbour count.
// goff[e]..goff[e+1] becomes the slice of type e, and emit(pos, rank, count, e, j, dx, dy, dz, r2)
// is called once per neighbour by the lane that found it: pos its place in the sorted list, rank
// its place among the `count` neighbours of its type e, j its atom index, d = R_i - R_j.
// Neighbours whose element type is negative (charge not in `species`) are dropped.  Up to 64
// candidates take a single pass; beyond, pass 0 counts per type (lane e keeps the count of type
// e) and pass 1 places each neighbour at goff[type] + its rank among the earlier ones of that type.
template <class Emit>
__device__ __forceinline__ int visit_neighbours(const FchlArgs& a, int* goff, int m, int i, int lane, Emit emit) {
    const float* Xm = a.X + (size_t)m * a.n * 3;
    const int* tm = a.types + (size_t)m * a.n;
    const int ns = a.p.nspecies;
    const bool pbc = a.cell != nullptr;
    float c[9], ic[9];
    if (pbc) {
        for (int t = 0; t < 9; ++t) {
            c[t] = a.cell[(size_t)m * 9 + t];
            ic[t] = a.inv_cell[(size_t)m * 9 + t];
        }
    }
    const float xi = Xm[i * 3 + 0], yi = Xm[i * 3 + 1], zi = Xm[i * 3 + 2];
    // atom `lane` of the molecule, fetched before the atom count is known: without a
    // neighbour list it is this lane's candidate, and the loads overlap the count's
    const int own = lane < a.n ? lane : 0;
    const float xo = Xm[own * 3 + 0], yo = Xm[own * 3 + 1], zo = Xm[own * 3 + 2];
    const int eo = tm[own];
    const float rc2 = a.p.rcut * a.p.rcut;
    const bool have_list = a.nlist != nullptr;
    int total;
    const int* li = nullptr;
    if (have_list) {
        total = a.nneigh[(size_t)m * a.n + i];
        if (total > a.nn_stride) total = a.nn_stride;
        li = a.nlist + ((size_t)m * a.n + i) * a.nn_stride;
    } else {
        total = a.natoms[m];
        if (total > a.n) total = a.n;
    }
    if (total <= QMLL_WAVE) {
        // One candidate per lane: a single pass.  The loads below depend only on the molecule
        // index, so they are issued together; the count of each type is the population of a
        // ballot, known to every lane, and a lane's slot is the running start of its type
        // plus its rank among the earlier lanes of that type.
        const int t = lane;
        const int j = have_list ? (t < total ? li[t] : -1) : t;
        const bool jok = t < total && j >= 0 && j < a.n;
        float xj = xo, yj = yo, zj = zo;
        int e = eo;
        if (have_list) {
            const int jj = jok ? j : 0;
            xj = Xm[jj * 3 + 0];
            yj = Xm[jj * 3 + 1];
            zj = Xm[jj * 3 + 2];
            e = tm[jj];
        }
        float dx = xi - xj, dy = yi - yj, dz = zi - zj;
        if (pbc) min_image(dx, dy, dz, c, ic);
        const float r2 = dx * dx + dy * dy + dz * dz;
        // a supplied list is authoritative (it may be stale on purpose, e.g. finite
        // differences with a frozen list); only the built-in search applies the cutoff
        const bool ok = jok && (have_list ? (r2 > 0.0f) : (r2 < rc2 && r2 > 0.0f)) && e >= 0 && e < ns;
        int start = 0, pos = 0, rank = 0, count = 0;
        const unsigned long long below = (1ull << lane) - 1ull;
        for (int ep = 0; ep < ns; ++ep) {
            const unsigned long long mask = __ballot(ok && e == ep);
            if (lane == 0) goff[ep] = start;
            const int cnt = __popcll(mask);
            if (e == ep) {
                rank = __popcll(mask & below);
                pos = start + rank;
                count = cnt;
            }
            start += cnt;
        }
        const int nn = start < a.cap ? start : a.cap;
        if (lane == 0) goff[ns] = nn;
        if (ok && pos < a.cap) emit(pos, rank, count, e, j, dx, dy, dz, r2);
        return nn;
    }
    int mycount = 0;   // lane e: neighbours of type e seen so far
    int nn = 0;
    for (int pass = 0; pass < 2; ++pass) {
        if (pass == 1) {
            // exclusive prefix over the type counts -> goff
            int incl = mycount;
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(incl, o, 64);
                if (lane >= o) incl += up;
            }
            if (lane < ns) goff[lane] = incl - mycount;
            nn = __shfl(incl, ns - 1, 64);
            if (nn > a.cap) nn = a.cap;
            if (lane == 0) goff[ns] = nn;
            mycount = 0;
            __syncthreads();
        }
        for (int base = 0; base < total; base += QMLL_WAVE) {
            const int t = base + lane;
            bool ok = t < total;
            int j = 0;
            float dx = 0.f, dy = 0.f, dz = 0.f, r2 = 0.f;
            int e = -1;
            if (ok) {
                j = have_list ? li[t] : t;
                ok = j >= 0 && j < a.n;
            }
            if (ok) {
                dx = xi - Xm[j * 3 + 0];
                dy = yi - Xm[j * 3 + 1];
                dz = zi - Xm[j * 3 + 2];
                if (pbc) min_image(dx, dy, dz, c, ic);
                r2 = dx * dx + dy * dy + dz * dz;
                e = tm[j];
                // a supplied list is authoritative (it may be stale on purpose, e.g. finite
                // differences with a frozen list); only the built-in search applies the cutoff
                ok = (have_list ? (r2 > 0.0f) : (r2 < rc2 && r2 > 0.0f)) && e >= 0 && e < ns;
            }
            for (int ep = 0; ep < ns; ++ep) {
                const unsigned long long mask = __ballot(ok && e == ep);
                const int before = __builtin_amdgcn_readlane(mycount, ep);
                if (pass == 1 && ok && e == ep) {
                    const int first = goff[ep];
                    const int rank = before + __popcll(mask & ((1ull << lane) - 1ull));
                    // goff of the last type's end may have been clipped to the capacity
                    if (first + rank < a.cap) emit(first + rank, rank, goff[ep + 1] - first, e, j, dx, dy, dz, r2);
                }
                if (lane == ep) mycount += __popcll(mask);
            }
        }
    }
    return nn;
}

// the cosine cutoff fc = (cos(pi r / rc) + 1) / 2 and its r-derivative from one sine / cosine pair
__device__ __forceinline__ void cutoff(float r, float inv_rc, float& fc, float& dfc) {
    float sn, cs;
    sincos_hw(r * PI_F * inv_rc, &sn, &cs);
    fc = 0.5f * (cs + 1.0f);
    dfc = -0.5f * PI_F * inv_rc * sn;
}

// the neighbour arrays of `Stage` filled by visit_neighbours
__device__ int stage_neighbours(const FchlArgs& a, const Stage& s, int m, int i, int lane) {
    const float inv_rc = frcp(a.p.rcut);
    return visit_neighbours(a, s.goff, m, i, lane,
                            [&](int pos, int, int, int e, int j, float dx, float dy, float dz, float r2) {
                                const float r = fsqrt(r2);
                                s.dx[pos] = dx;
                                s.dy[pos] = dy;
                                s.dz[pos] = dz;
                                s.r[pos] = r;
                                cutoff(r, inv_rc, s.fc[pos], s.dfc[pos]);
                                s.el[pos] = e;
                                s.j[pos] = j;
                            });
}

// 2^x and log2(x) on the transcendental unit (1 ulp)
__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float flog2(float x) { return __builtin_amdgcn_logf(x); }
constexpr float LOG2E = 1.4426950408889634f;

// row index of pair t in the list of pairs (j<k) over nn items, rows enumerated j = 0..nn-2
__device__ __forceinline__ void unrank_pair(int t, int nn, int& j, int& k) {
    const float b = (float)(2 * nn - 1);
    int jj = (int)((b - fsqrt(fmaxf(b * b - 8.0f * (float)t, 0.0f))) * 0.5f);   // first guess; corrected below
    if (jj < 0) jj = 0;
    if (jj > nn - 2) jj = nn - 2;
    // offset(j) = j (2nn - j - 1) / 2
    while (jj > 0 && (jj * (2 * nn - jj - 1)) / 2 > t) --jj;
    while (((jj + 1) * (2 * nn - jj - 2)) / 2 <= t) ++jj;
    j = jj;
    k = jj + 1 + (t - (jj * (2 * nn - jj - 1)) / 2);
}

// pair t of the list of pairs (j<k) enumerated k-major: t = k (k - 1) / 2 + j, 0 <= j < k.  No
// search and no correction step: for t in [k (k - 1) / 2, (k + 1) k / 2) the value 2 t + 1.25 lies in
// [(k - 1/2)^2 + 1, (k + 1/2)^2 - 1], so 1/2 + sqrt(2 t + 1.25) stays at least 1 / (2 k) inside
// (k, k + 1), hundreds of ulps for every t < 2^20 (k < 1449) even with a root two ulps off.
__device__ __forceinline__ void unrank_pair_kmajor(int t, int& j, int& k) {
    k = (int)(0.5f + fsqrt(fmaf(2.0f, (float)t, 1.25f)));
    j = t - (__mul24(k, k - 1) >> 1);
}

__device__ __forceinline__ int pair_offset(int ej, int ek, int ns, int nRs2, int nRs3) {
    const int p = ej < ek ? ej : ek;
    const int q = ej < ek ? ek : ej;
    return ns * nRs2 + 2 * nRs3 * (-(p * (p + 1)) / 2 + q + ns * p);   // fchl_cuda_kernel.cu:658-661
}

// geometry of one triple (central atom i, neighbours j<k in list order)
struct Triple {
    float a, b, c;           // r_ij, r_ik, r_jk
    float ci, cj, ck;        // cosines at i, j, k
    float cosT, sinT;        // cos/sin of the clamped angle at i
    float guard_inv;         // a b / sqrt(max(1e-10, a^2 b^2 - (d_ij.d_ik)^2))
    float ujk[3];            // (R_j - R_k)/c
};

__device__ __forceinline__ Triple triple_geometry(const Stage& s, int j, int k) {
    Triple t;
    const float ax = s.dx[j], ay = s.dy[j], az = s.dz[j];   // d_ij = R_i - R_j
    const float bx = s.dx[k], by = s.dy[k], bz = s.dz[k];   // d_ik
    const float cx = bx - ax, cy = by - ay, cz = bz - az;   // d_jk = R_j - R_k
    t.a = s.r[j];
    t.b = s.r[k];
    const float c2 = cx * cx + cy * cy + cz * cz;
    t.c = fsqrt(c2);
    const float ia = frcp(t.a), ib = frcp(t.b), ic = frcp(t.c);
    const float vi = ax * bx + ay * by + az * bz;           // (R_j-R_i).(R_k-R_i)
    t.ci = vi * ia * ib;
    t.ck = (cx * bx + cy * by + cz * bz) * ic * ib;         // (R_j-R_k).(R_i-R_k)
    t.cj = -(ax * cx + ay * cy + az * cz) * ia * ic;        // (R_i-R_j).(R_k-R_j)
    const float cc = fminf(1.0f, fmaxf(-1.0f, t.ci));
    t.cosT = cc;
    // a^2 b^2 - (d_ij.d_ik)^2 = |d_ij x d_ik|^2 (Lagrange): the cross product keeps full
    // relative accuracy near collinear triples, where the difference of squares cancels
    const float px = ay * bz - az * by, py = az * bx - ax * bz, pz = ax * by - ay * bx;
    const float cross2 = px * px + py * py + pz * pz;
    t.sinT = fminf(1.0f, fsqrt(cross2) * ia * ib);
    t.guard_inv = t.a * t.b * rsqrtf(fmaxf(1e-10f, cross2));
    t.ujk[0] = cx * ic;
    t.ujk[1] = cy * ic;
    t.ujk[2] = cz * ic;
    return t;
}

// ---------------------------------------------------------------------------------
// forward
//
// Atomic-free: with the neighbours sorted by element type every output block is owned by
// one loop nest.  Two-body block of type e: lanes = (neighbour sub-slot, radial bin z),
// serial over the neighbours of type e, partial sums folded across sub-slots by lane
// shuffles.  Three-body block of the type pair (p<=q): the pair's triples are evaluated
// once (lane = triple) into an LDS table (rho, K cos, K sin), then lanes = (triple
// sub-slot, radial bin l) run over the table with the bin sums in registers.  Rows go
// straight from registers to global memory.
// ---------------------------------------------------------------------------------
// (96 scalar registers: the eighth wavefront per SIMD; a SIMD has 800 of them, handed out in sixteens, and left
// alone the kernel takes 106.  The thirty-odd values that no longer fit are parked in the lanes of a vector
// register.  The backward kernel's LDS request allows no eighth wavefront, and there the cap only costs.)
__global__ __launch_bounds__(64) __attribute__((amdgpu_num_sgpr(96))) void fchl19_forward_kernel(FchlArgs a,
                                                                                                 float* __restrict__ rep) {
    extern __shared__ float smem[];
    const int lane = threadIdx.x;
    const int m = a.molIDs[blockIdx.x];
    const int i = a.atomIDs[blockIdx.x];
    if (m < 0 || m >= a.B || i < 0 || i >= a.n) return;   // malformed index: write nothing
    const int ns = a.p.nspecies, nRs2 = a.p.nRs2, nRs3 = a.p.nRs3;
    const int R = ns * nRs2 + ns * (ns + 1) * nRs3;

    // LDS: the triple table, three records per neighbour (read with one instruction each), the
    // type offsets, the radial grids, the table's segments
    float* trip = smem;                                  // [tcap + tpad][4]: sk3 rho, K cos, K sin, -
    float* recA = trip + 4 * (a.tcap + a.tpad);          // [cap][4]: d_ij, 1 / r
    float* recB = recA + 4 * a.cap;                      // [cap][4]: sk3 r / 2, fc r^-d3, element type,
                                                         //           index within the type | neighbours of the type << 16
    float* s2b = recB + 4 * a.cap;                       // [cap][4]: mu_j, log2(e) / (2 sigma_j^2), r^-d2 fc / (sigma sqrt(2pi)), -
    int* goff = (int*)(s2b + 4 * a.cap);                 // [ns+1] slices of the sorted neighbour list by type
    float* slnRs2 = (float*)(goff + ns + 1);             // [nRs2]
    float* sinvRs2 = slnRs2 + nRs2;                      // [nRs2]
    float* sRs3 = sinvRs2 + nRs2;                        // [nRs3]
    int* pbase = (int*)(sRs3 + nRs3);                    // [ns*ns] first table entry of each element pair
    int* prounds = pbase + ns * ns;                      // [ns*ns] rounds of each element pair's segment

    // Global loads that do not depend on the neighbourhood are issued first and consumed after
    // the staging, so their latency overlaps the staging's own loads.
    const float rs2v = lane < nRs2 ? a.Rs2[lane] : 1.0f;
    const float rs3v = lane < nRs3 ? a.Rs3[lane] : 0.0f;
    const float zeta2 = 0.014383766711652736f;   // 2 exp(-pi^2 / 2)
    const float k3 = a.p.eta3 * LOG2E;
    const float sk3 = fsqrt(k3);                 // exp(-eta3 (rho - Rs)^2) = exp2(-(sk3 rho - sk3 Rs)^2)
    const float inv_rc = frcp(a.p.rcut);
    // every neighbour's factors of the two-body bins and of the triples, by the lane that found it
    const int nn = visit_neighbours(
        a, goff, m, i, lane, [&](int pos, int rank, int count, int e, int, float dx, float dy, float dz, float r2) {
            const float ir = __builtin_amdgcn_rsqf(r2), r = r2 * ir;
            float fc, dfc;
            cutoff(r, inv_rc, fc, dfc);
            const float l2r = flog2(r);
            const float s2 = flog(fmaf(a.p.eta2 * ir, ir, 1.0f));
            reinterpret_cast<float4*>(s2b)[pos] = make_float4(
                fmaf(l2r, 0.6931471805599453f, -0.5f * s2),   // ln(r / sqrt(1 + eta2/r^2))
                0.5f * LOG2E * frcp(s2),
                frsq(s2) * 0.3989422804014327f * fexp2(-a.p.two_body_decay * l2r) * fc, 0.0f);
            reinterpret_cast<float4*>(recA)[pos] = make_float4(dx, dy, dz, ir);
            reinterpret_cast<float4*>(recB)[pos] = make_float4(sk3 * 0.5f * r, fc * fexp2(-a.p.three_body_decay * l2r),
                                                               __int_as_float(e), __int_as_float(rank | (count << 16)));
        });
    if (lane < nRs2) {
        slnRs2[lane] = flog(rs2v);
        sinvRs2[lane] = frcp(rs2v);
    }
    if (lane < nRs3) sRs3[lane] = rs3v;
    for (int t = lane + QMLL_WAVE; t < nRs2; t += QMLL_WAVE) {
        const float v = a.Rs2[t];
        slnRs2[t] = flog(v);
        sinvRs2[t] = frcp(v);
    }
    for (int t = lane + QMLL_WAVE; t < nRs3; t += QMLL_WAVE) sRs3[t] = a.Rs3[t];
    __syncthreads();

    float* out = rep + ((size_t)m * a.n + i) * R;

    // ---- two-body blocks ----
    {
        const int W = nRs2 < 64 ? nRs2 : 64;     // lanes per neighbour sub-slot
        const int JS = idiv_small(64, W);        // neighbour sub-slots
        const int jsub = idiv_small(lane, W), zl = lane - jsub * W;
        for (int zb = 0; zb < nRs2; zb += W) {
            const int z = zb + zl;
            const bool zok = z < nRs2 && jsub < JS;
            const float lnRs = zok ? slnRs2[z] : 0.0f;
            const float invRs = zok ? sinvRs2[z] : 0.0f;
            for (int e = 0; e < ns; ++e) {
                // the same number of rounds for every lane (the loop stays scalar and unrolls);
                // a sub-slot past the end of the type's neighbours reads a valid entry with weight 0
                const int j0 = goff[e], j1 = goff[e + 1];
                const int rounds = idiv_small(j1 - j0 + JS - 1, JS);
                float acc = 0.0f;
#pragma unroll 2
                for (int it = 0; it < rounds; ++it) {
                    const int j = j0 + jsub + it * JS;
                    const bool jok = zok && j < j1;
                    const float3v f = *reinterpret_cast<const float3v*>(s2b + 4 * (jok ? j : j0));   // one 12-byte LDS read
                    const float u = lnRs - f.x;
                    acc = fmaf(jok ? f.z : 0.0f, fexp2(-u * u * f.y), acc);
                }
                acc *= invRs;
                float tot = acc;
                for (int k = 1; k < JS; ++k) tot += __shfl(acc, zl + W * k, 64);
                if (zok && jsub == 0) out[e * nRs2 + z] = tot;
            }
        }
    }

    // ---- three-body blocks ----
    const int W3 = nRs3 < 64 ? nRs3 : 64;
    const int TS = idiv_small(64, W3);
    const int tsub = idiv_small(lane, W3), ll = lane - tsub * W3;
    constexpr int MAXLB = 4;                     // radial bins handled: up to 4 x 64

    // one table entry per triple: (sk3 rho, K cos, K sin, -) from the two neighbours' records.  With
    // a = d_ij, b = d_ik, c = b - a: cos_i cos_j cos_k = -(a.b)(a.c)(c.b) / (|a| |b| |c|)^2, the decay
    // (|a| |b| |c|)^-d3 is the product of the neighbours' factors and |c|^-d3 = exp2(-d3 log2(c.c) / 2);
    // sin_i = |a x b| / (|a| |b|) keeps full relative accuracy near collinear triples.
    const float zw3 = zeta2 * a.p.three_body_weight, hd3 = -0.5f * a.p.three_body_decay;
    auto table_entry = [&](const float4 Aj, const float4 Bj, const float4 Ak, const float4 Bk) -> float4 {
        const float cx = Ak.x - Aj.x, cy = Ak.y - Aj.y, cz = Ak.z - Aj.z;
        const float c2 = cx * cx + cy * cy + cz * cz;
        const float vi = Aj.x * Ak.x + Aj.y * Ak.y + Aj.z * Ak.z;
        const float dac = Aj.x * cx + Aj.y * cy + Aj.z * cz;
        const float dcb = cx * Ak.x + cy * Ak.y + cz * Ak.z;
        const float w = Aj.w * Ak.w;
        const float W = w * frsq(c2);
        const float px = Aj.y * Ak.z - Aj.z * Ak.y, py = Aj.z * Ak.x - Aj.x * Ak.z, pz = Aj.x * Ak.y - Aj.y * Ak.x;
        const float f = zw3 * fmaf(-3.0f * vi * dac, dcb * W * W, 1.0f) * Bj.y * Bk.y * fexp2(hd3 * flog2(c2));
        const float cosT = fminf(1.0f, fmaxf(-1.0f, vi * w));
        const float sinT = fminf(1.0f, fsqrt(px * px + py * py + pz * pz) * w);
        return make_float4(Bj.x + Bk.x, f * cosT, f * sinT, 0.0f);
    };
    const float4* rA = reinterpret_cast<const float4*>(recA);
    const float4* rB = reinterpret_cast<const float4*>(recB);
    // this lane's radial grid points, pre-scaled
    float rsl[MAXLB];
#pragma unroll
    for (int b = 0; b < MAXLB; ++b) {
        const int l = b * 64 + ll;
        rsl[b] = (b * 64 < nRs3) ? sk3 * sRs3[l < nRs3 ? l : 0] : 0.0f;
    }
    // fold the triple sub-slots and store the block of pair (p,q)
    auto store_block = [&](int sbase, const float (&accc)[MAXLB], const float (&accs)[MAXLB]) {
#pragma unroll
        for (int b = 0; b < MAXLB; ++b) {
            if (b * 64 < nRs3) {
                float tc = accc[b], tsn = accs[b];
                for (int k = 1; k < TS; ++k) {
                    tc += __shfl(accc[b], ll + W3 * k, 64);
                    tsn += __shfl(accs[b], ll + W3 * k, 64);
                }
                const int l = b * 64 + ll;
                if (tsub == 0 && l < nRs3) {
                    out[sbase + 2 * l] = tc;
                    out[sbase + 2 * l + 1] = tsn;
                }
            }
        }
    };
    const int ntrip = nn * (nn - 1) / 2;

    // The rest of the kernel, with the sub-slot count as a compile-time constant where it is one of
    // the common ones (TSC = 0: any): the table reads of a round then sit at fixed offsets from
    // one address per lane.
    auto three_body = [&](auto tsc) {
        constexpr int TSC = decltype(tsc)::value;
        const int TSv = TSC ? TSC : TS;
        // bin sums of `rounds` rounds of table entries starting at `first`, added to the
        // accumulators.  A segment is padded with zero entries to whole rounds, so every sub-slot
        // runs the same number of rounds and the loop is wavefront-uniform (scalar control, unrollable).
        auto accumulate = [&](int first, int rounds, float (&accc)[MAXLB], float (&accs)[MAXLB]) {
            const float4* src = reinterpret_cast<const float4*>(trip) + first + (tsub < TSv ? tsub : 0);
#pragma unroll
            for (int b = 0; b < MAXLB; ++b) {
                if (b * 64 < nRs3) {
                    const float rs = rsl[b];
                    float c_ = accc[b], s_ = accs[b];
#pragma unroll 4
                    for (int it = 0; it < rounds; ++it) {
                        const float3v v = *reinterpret_cast<const float3v*>(src + it * TSv);   // one 12-byte LDS read
                        const float d = v.x - rs;
                        const float e = fexp2(-d * d);
                        c_ = fmaf(e, v.y, c_);
                        s_ = fmaf(e, v.z, s_);
                    }
                    accc[b] = c_;
                    accs[b] = s_;
                }
            }
        };
        if (ntrip <= a.tcap) {
            // All triples at once (three passes of 64 lanes at 20 neighbours instead of one or
            // more per element pair): the table is ordered by element pair, pbase[p*ns+q] is
            // the first entry of pair (p<=q), prounds[p*ns+q] its length in rounds, and a triple's
            // slot follows from its position in the sorted list.
            if (ns * ns <= QMLL_WAVE) {
                // lane p*ns+q takes pair (p,q); an exclusive scan over the lanes gives the starts
                const int p = idiv_small(lane, ns), q = lane - p * ns;
                int rounds = 0, ntr = 0;
                if (lane < ns * ns && q >= p) {
                    const int np_ = goff[p + 1] - goff[p], nq = goff[q + 1] - goff[q];
                    ntr = (p == q) ? (__mul24(np_, np_ - 1) >> 1) : __mul24(np_, nq);
                    rounds = idiv_small(ntr + TSv - 1, TSv);
                }
                const int size = rounds * TSv;               // segments start on a multiple of TS
                int incl = size;
                for (int o = 1; o < ns * ns; o <<= 1) {
                    const int up = __shfl_up(incl, o, 64);
                    if (lane >= o) incl += up;
                }
                if (lane < ns * ns) {
                    pbase[lane] = incl - size;
                    prounds[lane] = rounds;
                    // the padding of the segment is zero entries: they contribute nothing
                    for (int t = incl - size + ntr; t < incl; ++t)
                        reinterpret_cast<float4*>(trip)[t] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            } else if (lane == 0) {
                int acc = 0;
                for (int p = 0; p < ns; ++p) {
                    const int np_ = goff[p + 1] - goff[p];
                    for (int q = p; q < ns; ++q) {
                        const int ntr = (p == q) ? np_ * (np_ - 1) / 2 : np_ * (goff[q + 1] - goff[q]);
                        const int rounds = idiv_small(ntr + TSv - 1, TSv);
                        pbase[p * ns + q] = acc;
                        prounds[p * ns + q] = rounds;
                        for (int t = acc + ntr; t < acc + rounds * TSv; ++t)
                            reinterpret_cast<float4*>(trip)[t] = make_float4(0.f, 0.f, 0.f, 0.f);
                        acc += rounds * TSv;
                    }
                }
            }
            __syncthreads();
            for (int tt = lane; tt < ntrip; tt += QMLL_WAVE) {
                int j, k;
                unrank_pair_kmajor(tt, j, k);
                const float4 Aj = rA[j], Ak = rA[k], Bj = rB[j], Bk = rB[k];
                const int p = __float_as_int(Bj.z), q = __float_as_int(Bk.z);   // p <= q: the list is sorted by type
                const int wj = __float_as_int(Bj.w), wk = __float_as_int(Bk.w);
                const int jl = wj & 0xffff, kl = wk & 0xffff;
                // any one-to-one numbering of a pair's triples does: k-major within one type, row by row else
                const int local = (p == q ? (__mul24(kl, kl - 1) >> 1) : __mul24(kl, wj >> 16)) + jl;
                reinterpret_cast<float4*>(trip)[pbase[__mul24(p, ns) + q] + local] = table_entry(Aj, Bj, Ak, Bk);
            }
            __syncthreads();
            for (int p = 0; p < ns; ++p) {
                for (int q = p; q < ns; ++q) {
                    float accc[MAXLB], accs[MAXLB];
#pragma unroll
                    for (int b = 0; b < MAXLB; ++b) accc[b] = accs[b] = 0.0f;
                    accumulate(pbase[p * ns + q], prounds[p * ns + q], accc, accs);
                    store_block(pair_offset(p, q, ns, nRs2, nRs3), accc, accs);
                }
            }
            return;
        }
        // more triples than the table holds: element pair by element pair, in chunks of the table
        for (int p = 0; p < ns; ++p) {
            const int op = goff[p], np_ = goff[p + 1] - op;
            for (int q = p; q < ns; ++q) {
                const int oq = goff[q], nq = goff[q + 1] - oq;
                const int ntr = (p == q) ? np_ * (np_ - 1) / 2 : np_ * nq;
                float accc[MAXLB], accs[MAXLB];
#pragma unroll
                for (int b = 0; b < MAXLB; ++b) accc[b] = accs[b] = 0.0f;
                for (int t0 = 0; t0 < ntr; t0 += a.tcap) {
                    const int nchunk = min(a.tcap, ntr - t0);
                    const int rounds = idiv_small(nchunk + TSv - 1, TSv);
                    __syncthreads();
                    for (int tt = lane; tt < nchunk; tt += QMLL_WAVE) {
                        int ja, kb;
                        if (p == q) {
                            unrank_pair(t0 + tt, np_, ja, kb);
                        } else {
                            ja = (t0 + tt) / nq;
                            kb = (t0 + tt) - ja * nq;
                        }
                        reinterpret_cast<float4*>(trip)[tt] =
                            table_entry(rA[op + ja], rB[op + ja], rA[oq + kb], rB[oq + kb]);
                    }
                    if (lane < rounds * TSv - nchunk)
                        *reinterpret_cast<float4*>(trip + (nchunk + lane) * 4) = make_float4(0.f, 0.f, 0.f, 0.f);
                    __syncthreads();
                    accumulate(0, rounds, accc, accs);
                }
                store_block(pair_offset(p, q, ns, nRs2, nRs3), accc, accs);
            }
        }
    };
    switch (TS) {
        case 1: three_body(std::integral_constant<int, 1>{}); break;
        case 2: three_body(std::integral_constant<int, 2>{}); break;
        case 3: three_body(std::integral_constant<int, 3>{}); break;
        case 4: three_body(std::integral_constant<int, 4>{}); break;
        default: three_body(std::integral_constant<int, 0>{}); break;
    }
}

// ---------------------------------------------------------------------------------
// d/dr of the two-body bin values of one neighbour, contracted or not
// ---------------------------------------------------------------------------------
struct TwoBody {
    float mu, s2, s2p, mup, pre, fc, dfc, d2_over_r;
};

__device__ __forceinline__ TwoBody two_body_setup(float r, float fc, float dfc, const qmll_fchl_params& p) {
    TwoBody t;
    const float r2 = r * r;
    t.s2 = flog(1.0f + p.eta2 * frcp(r2));
    t.mu = flog(r) - 0.5f * t.s2;
    t.s2p = -2.0f * p.eta2 * frcp(r * (r2 + p.eta2));      // d sigma^2 / dr
    t.mup = frcp(r) - 0.5f * t.s2p;                   // d mu / dr
    t.pre = frsq(t.s2) * 0.3989422804014327f * fexp2(-p.two_body_decay * flog2(r));
    t.fc = fc;
    t.dfc = dfc;
    t.d2_over_r = p.two_body_decay * frcp(r);
    return t;
}

// value and r-derivative of bin z
__device__ __forceinline__ void two_body_bin(const TwoBody& t, float lnRs, float invRs, float& val, float& dval) {
    const float u = lnRs - t.mu;
    const float inv_s2 = frcp(t.s2);
    const float Bz = t.pre * invRs * fexp2(-0.5f * LOG2E * u * u * inv_s2);
    const float Q = -0.5f * t.s2p * inv_s2 - t.d2_over_r + u * inv_s2 * (t.mup + 0.5f * u * t.s2p * inv_s2);
    val = Bz * t.fc;
    dval = Bz * (t.fc * Q + t.dfc);
}

// partial derivatives with respect to (a,b,c) of the triple's prefactor
// K = w3 (1 + 3 ci cj ck) (abc)^-d3 fc(a) fc(b), and of cos_i
struct TripleDeriv {
    float K, Ka, Kb, Kc;     // K and its partials
    float cia, cib, cic;     // partials of cos_i
};

__device__ __forceinline__ TripleDeriv triple_derivatives(const Triple& t, const qmll_fchl_params& p, float fa,
                                                          float dfa, float fb, float dfb) {
    TripleDeriv d;
    const float ia = frcp(t.a), ib = frcp(t.b), ic = frcp(t.c);
    // d cos / d distance (law of cosines)
    d.cia = ib - t.ci * ia;
    d.cib = ia - t.ci * ib;
    d.cic = -t.c * ia * ib;
    const float cja = ic - t.cj * ia, cjb = -t.b * ia * ic, cjc = ia - t.cj * ic;
    const float cka = -t.a * ib * ic, ckb = ic - t.ck * ib, ckc = ib - t.ck * ic;
    const float P = 1.0f + 3.0f * t.ci * t.cj * t.ck;
    const float Pa = 3.0f * (d.cia * t.cj * t.ck + t.ci * cja * t.ck + t.ci * t.cj * cka);
    const float Pb = 3.0f * (d.cib * t.cj * t.ck + t.ci * cjb * t.ck + t.ci * t.cj * ckb);
    const float Pc = 3.0f * (d.cic * t.cj * t.ck + t.ci * cjc * t.ck + t.ci * t.cj * ckc);
    const float dec = p.three_body_weight * fexp2(-p.three_body_decay * flog2(t.a * t.b * t.c));
    const float ksi = dec * P;
    const float ksia = dec * (Pa - p.three_body_decay * P * ia);
    const float ksib = dec * (Pb - p.three_body_decay * P * ib);
    const float ksic = dec * (Pc - p.three_body_decay * P * ic);
    d.K = ksi * fa * fb;
    d.Ka = ksia * fa * fb + ksi * dfa * fb;
    d.Kb = ksib * fa * fb + ksi * fa * dfb;
    d.Kc = ksic * fa * fb;
    return d;
}

// ---------------------------------------------------------------------------------
// VJP
// ---------------------------------------------------------------------------------
// TABLE: the force coefficients of a triple (j, k) go to a neighbour x neighbour matrix in LDS, entry
// [x][y] = (ec, coefficient of d_ix) of the triple {x, y}, and every neighbour's row is summed
// afterwards with a loop of the same length for every lane, instead of LDS atomics, which
// serialise badly here: the 64 triples of a pass share 3-4 values of j.  a.tcap is the matrix's row
// length (odd, so that rows start in different banks).
template <bool TABLE>
__global__ __launch_bounds__(64) void fchl19_vjp_kernel(FchlArgs a, const float* __restrict__ grad_rep,
                                                         float* __restrict__ grad_X) {
    extern __shared__ float smem[];
    const int lane = threadIdx.x;
    const int m = a.molIDs[blockIdx.x];
    const int i = a.atomIDs[blockIdx.x];
    if (m < 0 || m >= a.B || i < 0 || i >= a.n) return;   // malformed index: write nothing
    const int ns = a.p.nspecies, nRs2 = a.p.nRs2, nRs3 = a.p.nRs3;
    const int R2 = ns * nRs2;                        // two-body part of a representation row
    const int NE3 = (ns * (ns + 1) / 2) * nRs3;      // (element pair, radial bin) entries of its three-body part

    // [cap][4] per neighbour, read with one instruction each: (d_ij, r) and
    // (1 / r, fc, dfc / dr, element type); first in LDS, 16-byte aligned
    float* recA = smem;
    float* recB = recA + 4 * a.cap;
    float* eo = recB + 4 * a.cap;              // TABLE: [cap][tcap][2]
    float* gin3 = eo + (TABLE ? 2 * a.cap * a.tcap : 0);   // [NE3][2] incoming gradient of the three-body bins (cos, sin), see below; 8-byte aligned
    int* sj = (int*)(gin3 + 2 * NE3);          // [cap] atom index of neighbour j
    int* goff = sj + a.cap;              // [ns+1] slices of the sorted neighbour list by type
    float* sgx = (float*)(goff + ns + 1);   // [cap] gradient on neighbour j
    float* sgy = sgx + a.cap;
    float* sgz = sgy + a.cap;
    float* slnRs2 = sgz + a.cap;     // [nRs2]
    float* sRs3 = slnRs2 + nRs2;     // [nRs3] sk3 Rs3 (fast form: about the middle of the grid)
    float* sfac = sRs3 + nRs3;       // [nRs3] 2^(-u^2) of every bin (fast form)
    float* gin2 = sfac + nRs3;       // [R2] incoming gradient of the two-body bins, each divided by its Rs2
    const float4* rA = reinterpret_cast<const float4*>(recA);
    const float4* rB = reinterpret_cast<const float4*>(recB);

    // Global loads that do not depend on the neighbourhood (grid tables, the incoming gradient
    // row) are issued first and consumed after the staging, so their latency overlaps the
    // staging's own loads.
    const float* gsrc = grad_rep + ((size_t)m * a.n + i) * (R2 + 2 * NE3);
    constexpr int GREG2 = 2, GREG3 = 4;          // values / (cos, sin) pairs per lane held in registers
    float gr2[GREG2], gr3c[GREG3], gr3s[GREG3];
#pragma unroll
    for (int k = 0; k < GREG2; ++k) gr2[k] = lane + QMLL_WAVE * k < R2 ? gsrc[lane + QMLL_WAVE * k] : 0.0f;
#pragma unroll
    for (int k = 0; k < GREG3; ++k) {
        const int e = lane + QMLL_WAVE * k;
        gr3c[k] = e < NE3 ? gsrc[R2 + 2 * e] : 0.0f;
        gr3s[k] = e < NE3 ? gsrc[R2 + 2 * e + 1] : 0.0f;
    }
    const float rs2v = lane < nRs2 ? a.Rs2[lane] : 1.0f;
    const float rs3v = lane < nRs3 ? a.Rs3[lane] : 0.0f;
    for (int t = lane; t < a.cap; t += QMLL_WAVE) {
        sgx[t] = 0.0f;
        sgy[t] = 0.0f;
        sgz[t] = 0.0f;
    }
    const float inv_rc = frcp(a.p.rcut);
    const int nn = visit_neighbours(a, goff, m, i, lane,
                                    [&](int pos, int, int, int e, int j, float dx, float dy, float dz, float r2) {
                                        const float ir = __builtin_amdgcn_rsqf(r2), r = r2 * ir;
                                        float fc, dfc;
                                        cutoff(r, inv_rc, fc, dfc);
                                        reinterpret_cast<float4*>(recA)[pos] = make_float4(dx, dy, dz, r);
                                        reinterpret_cast<float4*>(recB)[pos] = make_float4(ir, fc, dfc, __int_as_float(e));
                                        sj[pos] = j;
                                    });
    const float k3 = a.p.eta3 * LOG2E;
    const float sk3 = fsqrt(k3);                       // the radial grid of the triples is kept as sk3 Rs3
    const float hfac = -2.0f * a.p.eta3 * frcp(sk3);
    // The radial factor of a triple, exp2(-(x - g_l)^2) with x = sk3 rho and g_l = sk3 Rs3_l, about the
    // middle of the grid (y = x - mid, u_l = g_l - mid): exp2(2 y u_l - y^2) 2^(-u_l^2).  The second
    // factor does not depend on the triple and goes into the staged gradient once per atom; the first
    // is one fma and the exponential per (triple, bin).  It is at most 2^(u_l^2), so the form is taken
    // only while u_l^2 <= 100 for every bin (eta3 rcut^2 up to about 270); beyond, the plain form runs.
    const float mid = 0.5f * sk3 * a.p.rcut;
    bool fast;
    {
        float um = fabsf(fmaf(sk3, rs3v, -mid));
        if (lane >= nRs3) um = 0.0f;
        for (int t = lane + QMLL_WAVE; t < nRs3; t += QMLL_WAVE) um = fmaxf(um, fabsf(fmaf(sk3, a.Rs3[t], -mid)));
        um = fmaxf(um, lane_xor<1>(um));
        um = fmaxf(um, lane_xor<2>(um));
        um = fmaxf(um, lane_xor<4>(um));
        um = fmaxf(um, lane_xor<8>(um));
        um = fmaxf(um, lane_xor<16>(um));
        um = fmaxf(um, lane_xor<32>(um));
        fast = __builtin_amdgcn_readfirstlane(__float_as_int(um)) <= __float_as_int(10.0f);
    }
    const float shift = fast ? mid : 0.0f;
    // the gradient of the two-body bins, each divided by its grid point (the bin's 1 / Rs2 factor)
#pragma unroll
    for (int k = 0; k < GREG2; ++k) {
        const int t = lane + QMLL_WAVE * k;
        if (t < R2) gin2[t] = gr2[k] * (a.gscale * frcp(a.Rs2[t - nRs2 * idiv_small(t, nRs2)]));
    }
    for (int t = lane + QMLL_WAVE * GREG2; t < R2; t += QMLL_WAVE)
        gin2[t] = gsrc[t] * (a.gscale * frcp(a.Rs2[t - nRs2 * idiv_small(t, nRs2)]));
    if (lane < nRs2) slnRs2[lane] = flog(rs2v);
    for (int t = lane + QMLL_WAVE; t < nRs2; t += QMLL_WAVE) slnRs2[t] = flog(a.Rs2[t]);
    for (int t = lane; t < nRs3; t += QMLL_WAVE) {
        const float u = fmaf(sk3, t == lane ? rs3v : a.Rs3[t], -shift);
        sRs3[t] = u;
        sfac[t] = a.gscale * (fast ? fexp2(-u * u) : 1.0f);
    }
    __syncthreads();
    // the gradient of the three-body bins per (element pair, radial bin), (cos, sin) parts, times the
    // bin's constant factor s = 2^(-u^2): with e' = exp2(2 y u - y^2) the sums over the bins of g e and
    // of g (x - g_l) e are sum (g s) e' and y sum (g s) e' - sum (g s) (u e')
    auto stage3 = [&](int e, float gc, float gs) {
        const float s_ = sfac[e - nRs3 * idiv_small(e, nRs3)];
        reinterpret_cast<float2*>(gin3)[e] = make_float2(gc * s_, gs * s_);
    };
#pragma unroll
    for (int k = 0; k < GREG3; ++k)
        if (lane + QMLL_WAVE * k < NE3) stage3(lane + QMLL_WAVE * k, gr3c[k], gr3s[k]);
    for (int e = lane + QMLL_WAVE * GREG3; e < NE3; e += QMLL_WAVE) stage3(e, gsrc[R2 + 2 * e], gsrc[R2 + 2 * e + 1]);
    if constexpr (TABLE) {
        // no triple writes the diagonal of the coefficient matrix
        for (int t = lane; t < nn; t += QMLL_WAVE) reinterpret_cast<float2*>(eo)[t * a.tcap + t] = make_float2(0.0f, 0.0f);
    }
    __syncthreads();

    float gix = 0.0f, giy = 0.0f, giz = 0.0f;

    // two-body: lanes = (bin group g, neighbour j); group g takes the bins z = g, g+G, ...
    // With u = ln Rs - mu the r-derivative of a bin is B_z (fc Q + dfc), B_z = pre / Rs exp2(-c u^2) and
    // Q a quadratic in u whose coefficients (and fc, dfc) depend on the neighbour only:
    // per bin a subtraction, the exponential and two fma for the quadratic.
    {
        const int G = (nn > 0 && nn < 64) ? idiv_small(64, nn) : 1;
        for (int base = 0; base < nn; base += QMLL_WAVE) {
            const int g = G > 1 ? idiv_small(lane, nn) : 0;
            const int j = G > 1 ? lane - g * nn : base + lane;
            const bool active = g < G && j < nn;
            float gr = 0.0f;
            float4 Aj = make_float4(0.f, 0.f, 0.f, 1.f), Bj = make_float4(1.f, 0.f, 0.f, 0.f);
            if (active) {
                Aj = rA[j];
                Bj = rB[j];
                const TwoBody tb = two_body_setup(Aj.w, Bj.y, Bj.z, a.p);
                const float inv_s2 = frcp(tb.s2);
                const float nc = -0.5f * LOG2E * inv_s2;
                const float hs = 0.5f * tb.s2p * inv_s2;
                const float q0 = fmaf(tb.fc, -hs - tb.d2_over_r, tb.dfc);
                const float q1 = tb.fc * inv_s2 * tb.mup;
                const float q2 = tb.fc * hs * inv_s2;
                const float* gz = gin2 + __float_as_int(Bj.w) * nRs2;
                for (int z = g; z < nRs2; z += G) {
                    const float u = slnRs2[z] - tb.mu;
                    const float e = fexp2(u * u * nc);
                    gr = fmaf(gz[z] * e, fmaf(fmaf(q2, u, q1), u, q0), gr);
                }
                gr *= tb.pre;
            }
            float tot = gr;
            for (int k = 1; k < G; ++k) tot += __shfl(gr, (lane + nn * k) & 63, 64);
            if (active && g == 0) {
                const float ux = Aj.x * Bj.x, uy = Aj.y * Bj.x, uz = Aj.z * Bj.x;   // dr/dR_i
                gix += tot * ux;
                giy += tot * uy;
                giz += tot * uz;
                sgx[j] -= tot * ux;   // each lane owns its own j here
                sgy[j] -= tot * uy;
                sgz[j] -= tot * uz;
            }
        }
    }
    __syncthreads();

    // three-body: lane per triple, serial over radial bins.  With a = d_ij, b = d_ik, c = b - a
    // (= R_j - R_k) and X = cos_i cos_j cos_k the partials of P = 1 + 3 X by the three distances
    // follow from the law of cosines:
    //   P_a / 3 = cos_j cos_k / |b| + cos_i cos_k / |c| - cos_i cos_j |a| / (|b| |c|) - 2 X / |a|
    // and cyclically; K = w3 P (abc)^-d3 fc(a) fc(b) and its partials share the factor
    // dec = w3 (abc)^-d3, applied once at the end together with 2 exp(-pi^2 / 2).
    const int ntrip = nn * (nn - 1) / 2;
    const float zeta2 = 0.014383766711652736f;   // 2 exp(-pi^2 / 2)
    const float d3 = a.p.three_body_decay;
    for (int tt = lane; tt < ntrip; tt += QMLL_WAVE) {
        int j, k;
        unrank_pair_kmajor(tt, j, k);                     // tt = k (k - 1) / 2 + j
        const float4 Aj = rA[j], Ak = rA[k], Bj = rB[j], Bk = rB[k];
        const float ia = Bj.x, ib = Bk.x;
        const float cx = Ak.x - Aj.x, cy = Ak.y - Aj.y, cz = Ak.z - Aj.z;
        const float c2 = cx * cx + cy * cy + cz * cz;
        const float ic = __builtin_amdgcn_rsqf(c2), c = c2 * ic;
        const float vi = Aj.x * Ak.x + Aj.y * Ak.y + Aj.z * Ak.z;
        const float dac = Aj.x * cx + Aj.y * cy + Aj.z * cz;
        const float dcb = cx * Ak.x + cy * Ak.y + cz * Ak.z;
        const float w = ia * ib, iaic = ia * ic, ibic = ib * ic;
        const float ci = vi * w, cj = -dac * iaic, ck = dcb * ibic;
        // a^2 b^2 - (d_ij.d_ik)^2 = |d_ij x d_ik|^2 (Lagrange): the cross product keeps full
        // relative accuracy near collinear triples, where the difference of squares cancels
        const float px = Aj.y * Ak.z - Aj.z * Ak.y, py = Aj.z * Ak.x - Aj.x * Ak.z, pz = Aj.x * Ak.y - Aj.y * Ak.x;
        const float cross2 = px * px + py * py + pz * pz;
        const float cosT = fminf(1.0f, fmaxf(-1.0f, ci));
        const float sinT = fminf(1.0f, fsqrt(cross2) * w);
        const float guard_inv = Aj.w * Ak.w * __builtin_amdgcn_rsqf(fmaxf(1e-10f, cross2));
        const float q1 = cj * ck, q2 = ci * ck, q3 = ci * cj;
        const float X = ci * q1, X2 = X + X;
        const float P = fmaf(3.0f, X, 1.0f);
        const float Pa3 = fmaf(q1, ib, fmaf(q2, ic, fmaf(-q3 * Aj.w, ibic, -X2 * ia)));
        const float Pb3 = fmaf(q1, ia, fmaf(q3, ic, fmaf(-q2 * Ak.w, iaic, -X2 * ib)));
        const float Pc3 = fmaf(q2, ia, fmaf(q3, ib, fmaf(-q1 * c, w, -X2 * ic)));
        const float Z = zeta2 * a.p.three_body_weight * fexp2(-d3 * flog2(Aj.w * Ak.w * c));
        const float fa = Bj.y, dfa = Bj.z, fb = Bk.y, dfb = Bk.z;
        const float F = fa * fb, d3P = d3 * P, FP = F * P;
        const float ka = fmaf(F, fmaf(3.0f, Pa3, -d3P * ia), P * dfa * fb);   // K_a / dec
        const float kb = fmaf(F, fmaf(3.0f, Pb3, -d3P * ib), P * fa * dfb);
        const float kc = F * fmaf(3.0f, Pc3, -d3P * ic);
        // the (element pair, radial bin) entries of this triple's pair: p <= q, the list is sorted by type
        const int tp = __float_as_int(Bj.w), tq = __float_as_int(Bk.w);
        const float2* g = reinterpret_cast<const float2*>(gin3) + __mul24(nRs3, __mul24(ns, tp) - (__mul24(tp, tp + 1) >> 1) + tq);
        // exp(-eta3 (rho - Rs)^2) = exp2(-(x - g_l)^2), x = sk3 rho, the grid stored pre-scaled;
        // d e / d rho = -2 eta3 (rho - Rs) e = hfac (x - g_l) e, the factor applied after the sums
        const float y = fmaf(sk3 * 0.5f, Aj.w + Ak.w, -shift);
        float Gc = 0.f, Gs = 0.f, Hc = 0.f, Hs = 0.f;
        if (fast) {
            const float y2 = y + y, ny2 = -y * y;
#pragma unroll 4
            for (int l = 0; l < nRs3; ++l) {
                const float2 gv = g[l];
                const float u = sRs3[l];
                const float e = fexp2(fmaf(y2, u, ny2));
                const float ue = u * e;
                Gc = fmaf(gv.x, e, Gc);
                Gs = fmaf(gv.y, e, Gs);
                Hc = fmaf(gv.x, ue, Hc);
                Hs = fmaf(gv.y, ue, Hs);
            }
            Hc = fmaf(y, Gc, -Hc);
            Hs = fmaf(y, Gs, -Hs);
        } else {
#pragma unroll 4
            for (int l = 0; l < nRs3; ++l) {
                const float2 gv = g[l];
                const float dl = y - sRs3[l];
                const float e = fexp2(-(dl * dl));
                const float de = dl * e;
                Gc = fmaf(gv.x, e, Gc);
                Gs = fmaf(gv.y, e, Gs);
                Hc = fmaf(gv.x, de, Hc);
                Hs = fmaf(gv.y, de, Hs);
            }
        }
        const float S0 = Gc * cosT + Gs * sinT;
        const float S1 = 0.5f * hfac * (Hc * cosT + Hs * sinT);                   // d rho/da = d rho/db = 1/2
        const float Sth = (Gc * sinT - Gs * cosT) * guard_inv;                     // multiplies d cos_i
        // d cos_i / d distance: 1/b - cos_i / a, 1/a - cos_i / b, -c / (a b)
        const float ea = Z * ia * fmaf(ka, S0, FP * fmaf(Sth, fmaf(-ci, ia, ib), S1));   // (d L / d a) / a
        const float eb = Z * ib * fmaf(kb, S0, FP * fmaf(Sth, fmaf(-ci, ib, ia), S1));
        const float ec = Z * ic * fmaf(kc, S0, -FP * Sth * c * w);
        gix = fmaf(ea, Aj.x, fmaf(eb, Ak.x, gix));
        giy = fmaf(ea, Aj.y, fmaf(eb, Ak.y, giy));
        giz = fmaf(ea, Aj.z, fmaf(eb, Ak.z, giz));
        if constexpr (TABLE) {
            // force on j: ec d_ik - (ec + ea) d_ij, on k: ec d_ij - (eb + ec) d_ik
            reinterpret_cast<float2*>(eo)[j * a.tcap + k] = make_float2(ec, ec + ea);
            reinterpret_cast<float2*>(eo)[k * a.tcap + j] = make_float2(ec, eb + ec);
        } else {
            atomicAdd(&sgx[j], fmaf(ec, cx, -ea * Aj.x));
            atomicAdd(&sgy[j], fmaf(ec, cy, -ea * Aj.y));
            atomicAdd(&sgz[j], fmaf(ec, cz, -ea * Aj.z));
            atomicAdd(&sgx[k], fmaf(-ec, cx, -eb * Ak.x));
            atomicAdd(&sgy[k], fmaf(-ec, cy, -eb * Ak.y));
            atomicAdd(&sgz[k], fmaf(-ec, cz, -eb * Ak.z));
        }
    }
    __syncthreads();
    gix = wave_sum(gix);
    giy = wave_sum(giy);
    giz = wave_sum(giz);
    float* gm = grad_X + (size_t)m * a.n * 3;
    if (lane == 0) {
        atomicAdd(&gm[i * 3 + 0], gix);
        atomicAdd(&gm[i * 3 + 1], giy);
        atomicAdd(&gm[i * 3 + 2], giz);
    }
    if constexpr (TABLE) {
        // lane = (neighbour x, component c): the force on x is sum_y ec(x,y) d_iy - d_ix sum_y own(x,y)
        // over row x of the matrix, plus what the two-body part left for x
        for (int it = lane; it < 3 * nn; it += QMLL_WAVE) {
            const int x = idiv_small(it, 3), c = it - 3 * x;
            float sum = c == 0 ? sgx[x] : (c == 1 ? sgy[x] : sgz[x]);
            float own = 0.0f;
            const float* dc = recA + c;                       // component c of d_iy at dc[4 y]
            const float2* row = reinterpret_cast<const float2*>(eo) + x * a.tcap;
#pragma unroll 4
            for (int yv = 0; yv < nn; ++yv) {
                const float2 v = row[yv];
                sum = fmaf(v.x, dc[4 * yv], sum);
                own += v.y;
            }
            atomicAdd(&gm[sj[x] * 3 + c], fmaf(-dc[4 * x], own, sum));
        }
    } else {
        for (int j = lane; j < nn; j += QMLL_WAVE) {
            const int jj = sj[j];
            atomicAdd(&gm[jj * 3 + 0], sgx[j]);
            atomicAdd(&gm[jj * 3 + 1], sgy[j]);
            atomicAdd(&gm[jj * 3 + 2], sgz[j]);
        }
    }
}

// ---------------------------------------------------------------------------------
// explicit Jacobian (and the representation itself when rep != NULL)
//
// Output-centric and atomic-free: the wavefront of central atom i produces, one target
// atom at a time (i itself, then each neighbour), the three rows jac[m,i,target,0..2,:]
// in an LDS row buffer and streams them out coalesced.  For a neighbour target only the
// triples that contain it contribute; for the self row all triples do.
// ---------------------------------------------------------------------------------
// TABLE: everything of a triple that does not depend on the radial bin (geometry, the partials of
// the angular and decay factors, the unit vectors) is computed once per triple into an LDS table
// of JT floats; the (triple, radial bin) items of every target pass then only read it.  Without
// the table each item recomputes its triple, nRs3 times over and again in the neighbour passes.
constexpr int JT = 20;   // rho, bin offset, 6 alpha, 2 beta, u_ij, u_ik, u_jk, pad
template <bool TABLE>
__global__ __launch_bounds__(64) void fchl19_jacobian_kernel(FchlArgs a, float* __restrict__ rep,
                                                              float* __restrict__ jac) {
    extern __shared__ float smem[];
    const int lane = threadIdx.x;
    const int m = a.molIDs[blockIdx.x];
    const int i = a.atomIDs[blockIdx.x];
    if (m < 0 || m >= a.B || i < 0 || i >= a.n) return;   // malformed index: write nothing
    const int ns = a.p.nspecies, nRs2 = a.p.nRs2, nRs3 = a.p.nRs3;
    const int R = ns * nRs2 + ns * (ns + 1) * nRs3;

    Stage s = carve(smem, a.cap, ns);
    float* slnRs2 = s.next;          // [nRs2]
    float* sinvRs2 = slnRs2 + nRs2;  // [nRs2]
    float* sRs3 = sinvRs2 + nRs2;    // [nRs3]
    float* row = sRs3 + nRs3;        // [3][R] rows being assembled (+ [R] value row)
    float* val = row + 3 * R;        // [R]   representation row (self pass only)
    // TABLE: [ntrip][JT], 16-byte aligned behind the rows
    float* ttab = val + R + ((4 - ((size_t)(val + R - smem) & 3)) & 3);

    for (int t = lane; t < nRs2; t += QMLL_WAVE) {
        const float v = a.Rs2[t];
        slnRs2[t] = flog(v);
        sinvRs2[t] = frcp(v);
    }
    for (int t = lane; t < nRs3; t += QMLL_WAVE) sRs3[t] = a.Rs3[t];
    const int nn = stage_neighbours(a, s, m, i, lane);
    __syncthreads();

    const float k3 = a.p.eta3 * LOG2E;
    const float zeta2 = 0.014383766711652736f;   // 2 exp(-pi^2 / 2)
    float* jbase = jac + (((size_t)m * a.n + i) * a.n) * 3 * R;

    if constexpr (TABLE) {
        // T_c = zeta2 K e cosT, T_s = zeta2 K e sinT with e = exp(-eta3 (rho - Rs_l)^2): their partials
        // with respect to the three distances are e * alpha + (de/drho) * beta, alpha and beta per triple
        const int ntrip = nn * (nn - 1) / 2;
        for (int tt = lane; tt < ntrip; tt += QMLL_WAVE) {
            int j, k;
            unrank_pair(tt, nn, j, k);
            const Triple t = triple_geometry(s, j, k);
            const TripleDeriv d = triple_derivatives(t, a.p, s.fc[j], s.dfc[j], s.fc[k], s.dfc[k]);
            const float dcos = t.sinT * t.guard_inv;       // d cosT = dcos * d cos_i
            const float dsin = -t.cosT * t.guard_inv;      // d sinT = dsin * d cos_i
            const float ia = frcp(t.a), ib = frcp(t.b);
            float4* e4 = reinterpret_cast<float4*>(ttab + (size_t)tt * JT);
            e4[0] = make_float4(0.5f * (t.a + t.b),
                                __int_as_float(pair_offset(s.el[j], s.el[k], ns, nRs2, nRs3)),
                                zeta2 * (d.Ka * t.cosT + d.K * dcos * d.cia),
                                zeta2 * (d.Kb * t.cosT + d.K * dcos * d.cib));
            e4[1] = make_float4(zeta2 * (d.Kc * t.cosT + d.K * dcos * d.cic),
                                zeta2 * (d.Ka * t.sinT + d.K * dsin * d.cia),
                                zeta2 * (d.Kb * t.sinT + d.K * dsin * d.cib),
                                zeta2 * (d.Kc * t.sinT + d.K * dsin * d.cic));
            e4[2] = make_float4(zeta2 * d.K * t.cosT, zeta2 * d.K * t.sinT, s.dx[j] * ia, s.dy[j] * ia);
            e4[3] = make_float4(s.dz[j] * ia, s.dx[k] * ib, s.dy[k] * ib, s.dz[k] * ib);
            e4[4] = make_float4(t.ujk[0], t.ujk[1], t.ujk[2], 0.0f);
        }
        __syncthreads();
    }

    // target = -1: central atom; target = 0..nn-1: neighbour at that list position
    for (int target = -1; target < nn; ++target) {
        for (int t = lane; t < 3 * R; t += QMLL_WAVE) row[t] = 0.0f;
        if (target < 0)
            for (int t = lane; t < R; t += QMLL_WAVE) val[t] = 0.0f;
        __syncthreads();

        // two-body: items (neighbour j, bin z); a neighbour target only sees its own pair
        {
            const int j0 = target < 0 ? 0 : target;
            const int j1 = target < 0 ? nn : target + 1;
            const float sign = target < 0 ? 1.0f : -1.0f;   // dr/dR_i = u_ij, dr/dR_j = -u_ij
            for (int it = lane; it < (j1 - j0) * nRs2; it += QMLL_WAVE) {
                const int jq = idiv_small(it, nRs2);
                const int j = j0 + jq;
                const int z = it - jq * nRs2;
                const float r = s.r[j];
                const TwoBody tb = two_body_setup(r, s.fc[j], s.dfc[j], a.p);
                float v, dv;
                two_body_bin(tb, slnRs2[z], sinvRs2[z], v, dv);
                const float ir = sign * dv * frcp(r);
                const int bin = s.el[j] * nRs2 + z;
                atomicAdd(&row[0 * R + bin], ir * s.dx[j]);
                atomicAdd(&row[1 * R + bin], ir * s.dy[j]);
                atomicAdd(&row[2 * R + bin], ir * s.dz[j]);
                if (target < 0) atomicAdd(&val[bin], v);
            }
        }
        // three-body with the table: owner computes.  Lanes = (triple sub-slot, radial bin l); a lane
        // sums its bin over the triples of one element pair in registers (no LDS atomics, which run
        // at one lane per clock), sub-slots are folded with shuffles, sub-slot 0 stores the bin.
        if constexpr (TABLE) {
            const int W3 = nRs3 < 64 ? nRs3 : 64;
            const int TS = idiv_small(64, W3);
            const int tsub = idiv_small(lane, W3), ll = lane - tsub * W3;
            // the triples of one block: index it -> neighbour positions j < k
            auto block = [&](int off_pair, int count, int p, int q) {
                const int op = s.goff[p], oq = s.goff[q];
                const int np_ = s.goff[p + 1] - op, nq = s.goff[q + 1] - oq;
                for (int lb = 0; lb * 64 < nRs3; ++lb) {
                    const int l = lb * 64 + ll;
                    const bool lok = l < nRs3 && tsub < TS;
                    const float rs = sRs3[lok ? l : 0];
                    float gc[3] = {0.f, 0.f, 0.f}, gs[3] = {0.f, 0.f, 0.f}, vc = 0.f, vs = 0.f;
                    for (int it = tsub; it < count && lok; it += TS) {
                        int j, k;
                        if (target < 0) {
                            if (p == q) {
                                unrank_pair(it, np_, j, k);
                                j += op;
                                k += op;
                            } else {
                                j = op + it / nq;
                                k = oq + it - (it / nq) * nq;
                            }
                        } else {   // q is the element of the other neighbour o; p that of the target
                            int o = oq + it;
                            if (p == q && o >= target) ++o;
                            j = o < target ? o : target;
                            k = o < target ? target : o;
                        }
                        const float4* e4 = reinterpret_cast<const float4*>(
                            ttab + (size_t)((j * (2 * nn - j - 1)) / 2 + (k - j - 1)) * JT);
                        const float4 q0 = e4[0], q1 = e4[1], q2 = e4[2], q3 = e4[3], q4 = e4[4];
                        const float dl = q0.x - rs;
                        const float e = fexp2(-k3 * dl * dl);
                        const float de = -a.p.eta3 * dl * e;      // (d e/d rho) * (d rho/d a)
                        const float Tca = fmaf(e, q0.z, de * q2.x), Tcb = fmaf(e, q0.w, de * q2.x), Tcc = e * q1.x;
                        const float Tsa = fmaf(e, q1.y, de * q2.y), Tsb = fmaf(e, q1.z, de * q2.y), Tsc = e * q1.w;
                        const float ua[3] = {q2.z, q2.w, q3.x};
                        const float ub[3] = {q3.y, q3.z, q3.w};
                        const float uc[3] = {q4.x, q4.y, q4.z};
                        if (target < 0) {            // d/dR_i, and the value itself
                            vc = fmaf(e, q2.x, vc);
                            vs = fmaf(e, q2.y, vs);
#pragma unroll
                            for (int x = 0; x < 3; ++x) {
                                gc[x] += Tca * ua[x] + Tcb * ub[x];
                                gs[x] += Tsa * ua[x] + Tsb * ub[x];
                            }
                        } else if (j == target) {    // d/dR_j
#pragma unroll
                            for (int x = 0; x < 3; ++x) {
                                gc[x] += -Tca * ua[x] + Tcc * uc[x];
                                gs[x] += -Tsa * ua[x] + Tsc * uc[x];
                            }
                        } else {                     // d/dR_k
#pragma unroll
                            for (int x = 0; x < 3; ++x) {
                                gc[x] += -Tcb * ub[x] - Tcc * uc[x];
                                gs[x] += -Tsb * ub[x] - Tsc * uc[x];
                            }
                        }
                    }
                    // fold the sub-slots: totals apart from the partial sums the other lanes read
                    float tc[3] = {gc[0], gc[1], gc[2]}, tsn[3] = {gs[0], gs[1], gs[2]}, tvc = vc, tvs = vs;
                    for (int kk = 1; kk < TS; ++kk) {
                        const int src = ll + W3 * kk;
#pragma unroll
                        for (int x = 0; x < 3; ++x) {
                            tc[x] += __shfl(gc[x], src, 64);
                            tsn[x] += __shfl(gs[x], src, 64);
                        }
                        tvc += __shfl(vc, src, 64);
                        tvs += __shfl(vs, src, 64);
                    }
                    if (tsub == 0 && l < nRs3) {
                        const int off = off_pair + 2 * l;
#pragma unroll
                        for (int x = 0; x < 3; ++x) {
                            row[x * R + off] = tc[x];
                            row[x * R + off + 1] = tsn[x];
                        }
                        if (target < 0) {
                            val[off] = tvc;
                            val[off + 1] = tvs;
                        }
                    }
                }
            };
            if (target < 0) {
                for (int p = 0; p < ns; ++p) {
                    const int np_ = s.goff[p + 1] - s.goff[p];
                    for (int q = p; q < ns; ++q) {
                        const int nq = s.goff[q + 1] - s.goff[q];
                        block(pair_offset(p, q, ns, nRs2, nRs3), p == q ? np_ * (np_ - 1) / 2 : np_ * nq, p, q);
                    }
                }
            } else {
                const int p = s.el[target];
                for (int q = 0; q < ns; ++q) {
                    const int nq = s.goff[q + 1] - s.goff[q];
                    block(pair_offset(p, q, ns, nRs2, nRs3), nq - (p == q ? 1 : 0), p, q);
                }
            }
        } else {
            // self: all pairs (j<k); neighbour target: the nn-1 pairs {target, other}
            const int ntr = target < 0 ? nn * (nn - 1) / 2 : nn - 1;
            for (int it = lane; it < ntr * nRs3; it += QMLL_WAVE) {
                const int tt = idiv_small(it, nRs3);
                const int l = it - tt * nRs3;
                int j, k;
                if (target < 0) {
                    unrank_pair(tt, nn, j, k);
                } else {
                    const int o = tt < target ? tt : tt + 1;
                    j = o < target ? o : target;
                    k = o < target ? target : o;
                }
                const Triple t = triple_geometry(s, j, k);
                const TripleDeriv d = triple_derivatives(t, a.p, s.fc[j], s.dfc[j], s.fc[k], s.dfc[k]);
                const float rho = 0.5f * (t.a + t.b);
                const float dl = rho - sRs3[l];
                const float e = fexp2(-k3 * dl * dl);
                const float de = -a.p.eta3 * dl * e;          // (d e/d rho) * (d rho/d a)
                // T_c = zeta2 K e cosT, T_s = zeta2 K e sinT; partials wrt a, b, c
                const float dcos = t.sinT * t.guard_inv;       // d cosT = dcos * d cos_i
                const float dsin = -t.cosT * t.guard_inv;      // d sinT = dsin * d cos_i
                float Tca, Tcb, Tcc, Tsa, Tsb, Tsc;
                {
                    const float Ke = zeta2 * d.K * e;
                    const float base_a = zeta2 * (d.Ka * e + d.K * de);
                    const float base_b = zeta2 * (d.Kb * e + d.K * de);
                    const float base_c = zeta2 * (d.Kc * e);
                    Tca = base_a * t.cosT + Ke * dcos * d.cia;
                    Tcb = base_b * t.cosT + Ke * dcos * d.cib;
                    Tcc = base_c * t.cosT + Ke * dcos * d.cic;
                    Tsa = base_a * t.sinT + Ke * dsin * d.cia;
                    Tsb = base_b * t.sinT + Ke * dsin * d.cib;
                    Tsc = base_c * t.sinT + Ke * dsin * d.cic;
                    if (target < 0) {
                        const int off = pair_offset(s.el[j], s.el[k], ns, nRs2, nRs3) + 2 * l;
                        atomicAdd(&val[off], Ke * t.cosT);
                        atomicAdd(&val[off + 1], Ke * t.sinT);
                    }
                }
                const float ia = frcp(t.a), ib = frcp(t.b);
                const float ua[3] = {s.dx[j] * ia, s.dy[j] * ia, s.dz[j] * ia};
                const float ub[3] = {s.dx[k] * ib, s.dy[k] * ib, s.dz[k] * ib};
                const int off = pair_offset(s.el[j], s.el[k], ns, nRs2, nRs3) + 2 * l;
#pragma unroll
                for (int x = 0; x < 3; ++x) {
                    float gc, gs;
                    if (target < 0) {            // d/dR_i
                        gc = Tca * ua[x] + Tcb * ub[x];
                        gs = Tsa * ua[x] + Tsb * ub[x];
                    } else if (j == target) {    // d/dR_j
                        gc = -Tca * ua[x] + Tcc * t.ujk[x];
                        gs = -Tsa * ua[x] + Tsc * t.ujk[x];
                    } else {                     // d/dR_k
                        gc = -Tcb * ub[x] - Tcc * t.ujk[x];
                        gs = -Tsb * ub[x] - Tsc * t.ujk[x];
                    }
                    atomicAdd(&row[x * R + off], gc);
                    atomicAdd(&row[x * R + off + 1], gs);
                }
            }
        }
        __syncthreads();
        const int tj = target < 0 ? i : s.j[target];
        float* dst = jbase + (size_t)tj * 3 * R;
        for (int t = lane; t < 3 * R; t += QMLL_WAVE) dst[t] = row[t];
        if (target < 0 && rep != nullptr) {
            float* out = rep + ((size_t)m * a.n + i) * R;
            for (int t = lane; t < R; t += QMLL_WAVE) out[t] = val[t];
        }
        __syncthreads();
    }
}

int fill_args(FchlArgs& a, const float* X, const int* types, const float* cell, const float* inv_cell,
              const int* atomIDs, const int* molIDs, const int* natoms, const int* nlist, const int* nneigh,
              int nn_stride, int A, int B, int n, const float* Rs2, const float* Rs3, const qmll_fchl_params* prm,
              const char* who) {
    QMLL_REQUIRE(prm != nullptr, QMLL_ERR_INVALID, "%s: null params", who);
    QMLL_REQUIRE(A >= 0 && B >= 0 && n >= 0, QMLL_ERR_INVALID, "%s: negative size A=%d B=%d n=%d", who, A, B, n);
    QMLL_REQUIRE(prm->nspecies > 0 && prm->nRs2 > 0 && prm->nRs3 > 0, QMLL_ERR_INVALID,
                 "%s: nspecies=%d nRs2=%d nRs3=%d must be positive", who, prm->nspecies, prm->nRs2, prm->nRs3);
    QMLL_REQUIRE(prm->rcut > 0.0f, QMLL_ERR_INVALID, "%s: rcut must be positive", who);
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(X && types && atomIDs && molIDs && natoms && Rs2 && Rs3, QMLL_ERR_INVALID, "%s: null pointer", who);
    QMLL_REQUIRE((cell == nullptr) == (inv_cell == nullptr), QMLL_ERR_INVALID,
                 "%s: cell and inv_cell must both be given or both be NULL", who);
    QMLL_REQUIRE((nlist == nullptr) == (nneigh == nullptr), QMLL_ERR_INVALID,
                 "%s: nlist and nneigh must both be given or both be NULL", who);
    QMLL_REQUIRE(nlist == nullptr || nn_stride > 0, QMLL_ERR_INVALID, "%s: nn_stride=%d", who, nn_stride);
    a.X = X;
    a.types = types;
    a.cell = cell;
    a.inv_cell = inv_cell;
    a.atomIDs = atomIDs;
    a.molIDs = molIDs;
    a.natoms = natoms;
    a.nlist = nlist;
    a.nneigh = nneigh;
    a.nn_stride = nn_stride;
    a.n = n;
    a.B = B;
    a.cap = nlist ? nn_stride : n;
    if (a.cap < 1) a.cap = 1;
    a.tcap = TCH;
    a.tpad = 0;
    a.Rs2 = Rs2;
    a.Rs3 = Rs3;
    a.p = *prm;
    a.gscale = 1.0f;
    return QMLL_OK;
}

constexpr size_t LDS_LIMIT = 64 * 1024;

}  // namespace

extern "C" int qmll_fchl19_forward(const float* X, const int* types, const float* cell, const float* inv_cell,
                                   const int* atomIDs, const int* molIDs, const int* natoms, const int* nlist,
                                   const int* nneigh, int nn_stride, int A, int B, int n, const float* Rs2,
                                   const float* Rs3, const qmll_fchl_params* prm, float* rep, qmll_stream_t stream) {
    FchlArgs a;
    int rc = fill_args(a, X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, nn_stride, A, B, n, Rs2, Rs3,
                       prm, "qmll_fchl19_forward");
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(rep != nullptr, QMLL_ERR_INVALID, "qmll_fchl19_forward: null output");
    QMLL_REQUIRE(prm->nRs3 <= 256, QMLL_ERR_INVALID,
                 "qmll_fchl19_forward: nRs3=%d: at most 256 three-body radial bins are supported", prm->nRs3);
    const int R = prm->nspecies * prm->nRs2 + prm->nspecies * (prm->nspecies + 1) * prm->nRs3;
    // table for every triple of a full neighbourhood when that stays small: an atom has at most cap
    // neighbours from a given list and at most max_atoms - 1 otherwise
    const long long maxnn = nlist ? a.cap : (a.cap > 1 ? a.cap - 1 : 1);
    const long long alltrip = maxnn * (maxnn - 1) / 2;
    a.tcap = alltrip <= TCH_MAX ? (int)(alltrip > 0 ? alltrip : 1) : TCH;
    // each of the ns (ns+1)/2 segments is padded to a multiple of the triple sub-slot count
    const int tsub_slots = prm->nRs3 < 64 ? 64 / prm->nRs3 : 1;
    a.tpad = prm->nspecies * (prm->nspecies + 1) / 2 * (tsub_slots - 1);
    // triple table, three per-neighbour records [cap][4], type offsets, the radial grids, the table's
    // segment starts and lengths
    const size_t lds = sizeof(float) * ((size_t)12 * a.cap + prm->nspecies + 1 + 2 * prm->nRs2 + prm->nRs3 +
                                        4 * (size_t)(a.tcap + a.tpad) + 2 * (size_t)prm->nspecies * prm->nspecies + 4);
    QMLL_REQUIRE(lds <= LDS_LIMIT, QMLL_ERR_INVALID,
                 "qmll_fchl19_forward: %zu B of LDS needed (max_atoms=%d, repsize=%d) exceeds %zu", lds, n, R, LDS_LIMIT);
    hipLaunchKernelGGL(fchl19_forward_kernel, dim3(A), dim3(64), lds, (hipStream_t)stream, a, rep);
    QMLL_CHECK_LAUNCH("qmll_fchl19_forward");
    return QMLL_OK;
}

extern "C" int qmll_fchl19_vjp(const float* X, const int* types, const float* cell, const float* inv_cell,
                               const int* atomIDs, const int* molIDs, const int* natoms, const int* nlist,
                               const int* nneigh, int nn_stride, int A, int B, int n, const float* Rs2, const float* Rs3,
                               const qmll_fchl_params* prm, const float* grad_rep, float* grad_X,
                               qmll_stream_t stream) {
    return qmll_fchl19_vjp_scaled(X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, nn_stride, A, B, n, Rs2,
                                  Rs3, prm, grad_rep, 1.0f, grad_X, stream);
}

extern "C" int qmll_fchl19_vjp_scaled(const float* X, const int* types, const float* cell, const float* inv_cell,
                                      const int* atomIDs, const int* molIDs, const int* natoms, const int* nlist,
                                      const int* nneigh, int nn_stride, int A, int B, int n, const float* Rs2,
                                      const float* Rs3, const qmll_fchl_params* prm, const float* grad_rep, float scale,
                                      float* grad_X, qmll_stream_t stream) {
    FchlArgs a;
    int rc = fill_args(a, X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, nn_stride, A, B, n, Rs2, Rs3,
                       prm, "qmll_fchl19_vjp");
    if (rc) return rc;
    a.gscale = scale;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(grad_rep && grad_X, QMLL_ERR_INVALID, "qmll_fchl19_vjp: null gradient pointer");
    const int R = prm->nspecies * prm->nRs2 + prm->nspecies * (prm->nspecies + 1) * prm->nRs3;
    // two records [cap][4], atom indices, neighbour gradients [3][cap], type offsets, grids, the bins' constant
    // factors, the gradient row
    size_t lds = sizeof(float) * ((size_t)12 * a.cap + prm->nspecies + 1 + prm->nRs2 + 2 * prm->nRs3 + R);
    QMLL_REQUIRE(lds <= LDS_LIMIT, QMLL_ERR_INVALID,
                 "qmll_fchl19_vjp: %zu B of LDS needed (max_atoms=%d, repsize=%d) exceeds %zu", lds, n, R, LDS_LIMIT);
    // neighbour x neighbour coefficient matrix (two floats per entry, rows of odd length) while it stays small;
    // LDS atomics beyond
    a.tcap = a.cap | 1;
    const size_t table = sizeof(float) * 2 * (size_t)a.cap * a.tcap;
    if (table <= 24 * 1024 && lds + table <= LDS_LIMIT) {
        lds += table;
        hipLaunchKernelGGL(fchl19_vjp_kernel<true>, dim3(A), dim3(64), lds, (hipStream_t)stream, a, grad_rep, grad_X);
    } else {
        hipLaunchKernelGGL(fchl19_vjp_kernel<false>, dim3(A), dim3(64), lds, (hipStream_t)stream, a, grad_rep, grad_X);
    }
    QMLL_CHECK_LAUNCH("qmll_fchl19_vjp");
    return QMLL_OK;
}

extern "C" int qmll_fchl19_jacobian(const float* X, const int* types, const float* cell, const float* inv_cell,
                                    const int* atomIDs, const int* molIDs, const int* natoms, const int* nlist,
                                    const int* nneigh, int nn_stride, int A, int B, int n, const float* Rs2,
                                    const float* Rs3, const qmll_fchl_params* prm, float* rep, float* jac,
                                    qmll_stream_t stream) {
    FchlArgs a;
    int rc = fill_args(a, X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, nn_stride, A, B, n, Rs2, Rs3,
                       prm, "qmll_fchl19_jacobian");
    if (rc) return rc;
    if (A == 0) return QMLL_OK;
    QMLL_REQUIRE(jac != nullptr, QMLL_ERR_INVALID, "qmll_fchl19_jacobian: null output");
    const int R = prm->nspecies * prm->nRs2 + prm->nspecies * (prm->nspecies + 1) * prm->nRs3;
    size_t lds = sizeof(float) * ((size_t)STAGE_ARRAYS * a.cap + prm->nspecies + 1 + 2 * prm->nRs2 + prm->nRs3 + 4 * (size_t)R);
    QMLL_REQUIRE(lds <= LDS_LIMIT, QMLL_ERR_INVALID,
                 "qmll_fchl19_jacobian: %zu B of LDS needed (max_atoms=%d, repsize=%d) exceeds %zu", lds, n, R,
                 LDS_LIMIT);
    // per-triple table while it fits: an atom has at most cap neighbours from a given list and at
    // most max_atoms - 1 otherwise
    const size_t maxnn = nlist ? (size_t)a.cap : (size_t)(a.cap > 1 ? a.cap - 1 : 1);
    const size_t table = sizeof(float) * (JT * (maxnn * (maxnn - 1) / 2) + 4);
    if (lds + table <= LDS_LIMIT) {
        lds += table;
        hipLaunchKernelGGL(fchl19_jacobian_kernel<true>, dim3(A), dim3(64), lds, (hipStream_t)stream, a, rep, jac);
    } else {
        hipLaunchKernelGGL(fchl19_jacobian_kernel<false>, dim3(A), dim3(64), lds, (hipStream_t)stream, a, rep, jac);
    }
    QMLL_CHECK_LAUNCH("qmll_fchl19_jacobian");
    return QMLL_OK;
}
