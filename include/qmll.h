/*
 * libqmll -- C ABI of the MI355X (gfx950) kernels behind the QML-Lightning hot path:
 * FCHL19 representation (+ Jacobian / VJP), SORF (sign diagonal . fast Walsh-Hadamard
 * stacks), cos features and their derivatives, RFF features, and the Z^T Z / Z^T y
 * accumulation.
 *
 * Conventions for every entry point
 *   - all pointers are DEVICE pointers of the current HIP device unless marked "host";
 *     tensors are dense row-major with the shapes written next to them;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work is only
 *     enqueued: nothing here allocates, frees, synchronises or throws;
 *   - the return value is QMLL_OK or a negative QMLL_ERR_* code; qmll_last_error() gives
 *     the message of the calling thread's last failure;
 *   - shapes are validated on the host before any launch; a bad argument never reaches
 *     a kernel.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the
 * reference tree, nickjbrowning/qml-lightning).
 */
#ifndef QMLL_H
#define QMLL_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QMLL_OK 0
#define QMLL_ERR_INVALID (-1)   /* bad shape / null pointer / unsupported size */
#define QMLL_ERR_LAUNCH (-2)    /* HIP refused the launch */
#define QMLL_ERR_NOT_POW2 (-3)  /* "input size must be power of 2." (hadamard_kernel.cu:730) */

typedef void* qmll_stream_t;

/* FCHL19 hyper-parameters as FCHLCuda hands them to its kernels
 * (qml_lightning/representations/FCHL.py:25-40): three_body_weight already includes
 * sqrt(eta3/pi). */
typedef struct qmll_fchl_params {
    int nspecies;
    int nRs2;
    int nRs3;
    float eta2;
    float eta3;
    float two_body_decay;
    float three_body_weight;
    float three_body_decay;
    float rcut;
} qmll_fchl_params;

int qmll_version(void);
const char* qmll_last_error(void);

/* ---- neighbours and element types ------------------------------------------------ */

/* Replaces pairlist_gpu.get_num_neighbours_gpu (qml_lightning/cuda/pairlist_cuda.cpp:21-40,
 * kernel pairlist_kernel.cu:145-224).  X f32 [B,n,3], natoms i32 [B], cell/inv_cell f32
 * [B,3,3] or NULL (no periodic images) -> nneigh i32 [B,n] (every slot written; padded
 * atoms get 0).  j counts for i when 0 < |d_ij|^2 < rcut^2. */
int qmll_num_neighbours(const float* X, const int* natoms, const float* cell, const float* inv_cell,
                        int B, int n, float rcut, int* nneigh, qmll_stream_t stream);

/* Replaces pairlist_gpu.get_neighbour_list_gpu (pairlist_cuda.cpp:42-65, kernel
 * pairlist_kernel.cu:326-391).  -> nlist i32 [B,n,max_neighbours], ascending j, unused
 * slots -1 (every slot written).  An atom with more than max_neighbours neighbours keeps
 * the first max_neighbours of them. */
int qmll_neighbour_list(const float* X, const int* natoms, const float* cell, const float* inv_cell,
                        int B, int n, int max_neighbours, float rcut, int* nlist, qmll_stream_t stream);

/* Replaces fchl_gpu.get_element_types_gpu (qml_lightning/cuda/fchl_cuda.cpp:36-62, kernel
 * fchl_cuda_kernel.cu:1716-1742).  Z f32 [B,n] charges, species f32 [nspecies] ->
 * types i32 [B,n]: index of int(charge) in species, -1 if absent, 0 for padded slots. */
int qmll_element_types(const float* Z, const int* natoms, const float* species, int B, int n, int nspecies,
                       int* types, qmll_stream_t stream);

/* ---- FCHL19 ---------------------------------------------------------------------- */

/* Replaces fchl_gpu.get_fchl_representation / FCHLCuda (fchl_cuda.cpp:64-95, launcher
 * fchl_cuda_kernel.cu:1804-1846, kernel :476-674).  One wavefront per entry of
 * atomIDs/molIDs (i32 [A], one per real atom).  nlist i32 [B,n,nn_stride] + nneigh i32
 * [B,n] may both be NULL: the kernel then builds each atom's neighbour list itself in LDS
 * (same rule as qmll_neighbour_list), which removes the host sync on max(nneigh).
 * rep f32 [B,n,R], R = ns*nRs2 + ns*(ns+1)*nRs3: rows of the listed atoms are
 * overwritten; rows of padded slots are left untouched (the caller zero-fills, as the
 * reference wrapper does at fchl_cuda.cpp:83). */
int qmll_fchl19_forward(const float* X, const int* types, const float* cell, const float* inv_cell,
                        const int* atomIDs, const int* molIDs, const int* natoms,
                        const int* nlist, const int* nneigh, int nn_stride,
                        int A, int B, int n, const float* Rs2, const float* Rs3,
                        const qmll_fchl_params* prm, float* rep, qmll_stream_t stream);

/* Replaces fchl_gpu.fchl_backwards / FCHLBackwardsCuda (fchl_cuda.cpp:169-202, launcher
 * fchl_cuda_kernel.cu:1885-1926, kernel :1325-1714): grad_X[m,j,:] += sum_{i,f}
 * grad_rep[m,i,f] d rep[m,i,f]/d X[m,j,:].  grad_X f32 [B,n,3] is accumulated with
 * atomics and must be zero-filled by the caller (reference: fchl_cuda.cpp:196). */
int qmll_fchl19_vjp(const float* X, const int* types, const float* cell, const float* inv_cell,
                    const int* atomIDs, const int* molIDs, const int* natoms,
                    const int* nlist, const int* nneigh, int nn_stride,
                    int A, int B, int n, const float* Rs2, const float* Rs3,
                    const qmll_fchl_params* prm, const float* grad_rep, float* grad_X,
                    qmll_stream_t stream);

/* The same with the result scaled: grad_X += scale * J^T grad_rep at no cost (the factor goes into
 * the gradient row as it is staged).  scale = -1 turns dE/dX into forces in the kernel that forms
 * them (the reference negates the gradient in a separate elementwise pass,
 * qml_lightning/models/hadamard_features.py:156-162). */
int qmll_fchl19_vjp_scaled(const float* X, const int* types, const float* cell, const float* inv_cell,
                           const int* atomIDs, const int* molIDs, const int* natoms, const int* nlist,
                           const int* nneigh, int nn_stride, int A, int B, int n, const float* Rs2, const float* Rs3,
                           const qmll_fchl_params* prm, const float* grad_rep, float scale, float* grad_X,
                           qmll_stream_t stream);

/* Replaces fchl_gpu.get_fchl_and_derivative / FCHLRepresentationAndDerivativeCuda and
 * FCHLDerivativeCuda (fchl_cuda.cpp:97-167, launchers fchl_cuda_kernel.cu:1848-1883,
 * 1928-1964, kernels :676-1005, :1007-1323).  jac f32 [B,n,n,3,R] with
 * jac[m,i,j,x,f] = d rep[m,i,f]/d X[m,j,x]: for every listed atom i the rows of i itself
 * and of its neighbours are overwritten in full; all other rows are left untouched (the
 * caller zero-fills, reference: fchl_cuda.cpp:187).  rep may be NULL (Jacobian only). */
int qmll_fchl19_jacobian(const float* X, const int* types, const float* cell, const float* inv_cell,
                         const int* atomIDs, const int* molIDs, const int* natoms,
                         const int* nlist, const int* nneigh, int nn_stride,
                         int A, int B, int n, const float* Rs2, const float* Rs3,
                         const qmll_fchl_params* prm, float* rep, float* jac, qmll_stream_t stream);

/* ---- SORF ------------------------------------------------------------------------ */

/* Replaces sorf_gpu.hadamard_transform_gpu / hadamard_gpu and sorf_matrix_gpu /
 * compute_sorf_matrix (qml_lightning/cuda/hadamard_cuda.cpp:47-56, 72-87; kernels
 * hadamard_kernel.cu:5-102, 424-539).  x f32 [A,d], D f32 [T,S,d] (+-1) ->
 * out f32 [A,S,d] (== [A,S*d]) = normalisation * prod_m (H/sqrt(d) diag(D[m,s])) x.
 * d must be a power of two in [2, 2048] (QMLL_ERR_NOT_POW2 otherwise). */
int qmll_sorf_forward(const float* x, const float* D, int A, int d, int S, int T, float normalisation,
                      float* out, qmll_stream_t stream);

/* Replaces sorf_gpu.hadamard_transform_backwards_gpu / hadamard_backwards_gpu
 * (hadamard_cuda.cpp:58-70; kernel hadamard_kernel.cu:204-312).  g f32 [A,S,d] ->
 * gx f32 [A,d], the adjoint of qmll_sorf_forward summed over stacks (overwritten). */
int qmll_sorf_adjoint(const float* g, const float* D, int A, int d, int S, int T, float normalisation,
                      float* gx, qmll_stream_t stream);

/* Segment table of a molecule-major atom list, the form in which the reference builds
 * batch_indexes (torch.where(Z == e)[0], hadamard_features.py:101-107; ordering in
 * kernel.py:143-149).  mol_index i32 [A] -> seg i32 [nmol+2], zero-filled by the caller:
 * seg[m] = first atom of molecule m (seg[nmol] = A); seg[nmol+1] becomes non-zero when
 * mol_index is not ascending or leaves [0,nmol), in which case the table must not be used
 * (the feature kernels below check the flag on the device, no host round trip). */
int qmll_segment_offsets(const int* mol_index, int A, int nmol, int* seg, qmll_stream_t stream);

/* Replaces sorf_gpu.CosFeaturesCUDA / cos_features_gpu (hadamard_cuda.cpp:23-32; kernel
 * hadamard_kernel.cu:778-800).  coeffs f32 [A,F], bias f32 [F], mol_index i32 [A]
 * (row of Zf each atom adds to, values in [0,nmol)) -> Zf f32 [nmol,F] +=
 * sqrt(2/F) cos(coeffs+bias), into caller-zeroed memory.  seg: NULL, or the table from
 * qmll_segment_offsets for the same mol_index: each molecule's atoms are then summed in
 * registers in atom order and added once (deterministic, no atomics); without a table, or
 * with one flagged invalid, partial sums are added with atomics in any order. */
int qmll_cos_features_f32(const float* coeffs, const float* bias, const int* mol_index, const int* seg, int A, int F,
                          int nmol, float* Zf, qmll_stream_t stream);

/* Replaces sorf_gpu.compute_hadamard_features / compute_molecular_featurization
 * (hadamard_cuda.cpp:89-93; kernel hadamard_kernel.cu:541-563): same as above but every
 * fp32 feature value is widened and accumulated into Zf f64 [nmol,F] (in place). */
int qmll_cos_features_f64(const float* coeffs, const float* bias, const int* mol_index, const int* seg, int A, int F,
                          int nmol, double* Zf, qmll_stream_t stream);

/* Replaces sorf_gpu.CosDerivativeFeaturesCUDA / cos_derivative_features_gpu
 * (hadamard_cuda.cpp:34-45; kernel hadamard_kernel.cu:816-839).  gZ f32 [nmol,F] ->
 * gc f32 [A,F] = gZ[mol(a),f] * -sin(coeffs+bias) * sqrt(2/F) (overwritten). */
int qmll_cos_features_backward(const float* gZ, const float* coeffs, const float* bias, const int* mol_index,
                               int A, int F, int nmol, float* gc, qmll_stream_t stream);

/* Replaces sorf_gpu.compute_partial_feature_derivatives (hadamard_cuda.cpp:95-109, kernel
 * hadamard_kernel.cu:565-585): out f64 [A,F] = +sin(coeffs+bias) * sqrt(2/F), each value
 * computed in fp32 and widened. */
int qmll_sin_coeffs_f64(const float* coeffs, const float* bias, int A, int F, double* out, qmll_stream_t stream);

/* Replaces sorf_gpu.compute_molecular_featurization_derivative (hadamard_cuda.cpp:95-109,
 * launcher hadamard_kernel.cu:905-932, kernel :587-717).  cos_derivs f64 [A,F] (from
 * qmll_sin_coeffs_f64), input_derivative f32 [A,n,3,d] (projected Jacobian rows of the A
 * atoms), D f32 [T,S,d] -> G f64 [nmol,n,3,F] +=
 * normalisation * cos_derivs[a,s*d+p] * (prod_m (H/sqrt(d) diag(D[m,s])) u)[p].
 * Two ways to say which molecule an atom belongs to:
 *   mol_index i32 [A] (any order, seg_offsets NULL): fp64 atomics, as the reference does;
 *   seg_offsets i32 [nmol+1] (atoms molecule-major, atoms seg[m]..seg[m+1] belong to m):
 *   atomic-free, each G element read-modify-written once, fixed summation order. */
int qmll_derivative_features(const double* cos_derivs, double normalisation, const int* mol_index,
                             const int* seg_offsets, const float* input_derivative, const float* D,
                             int A, int n, int d, int S, int T, int nmol, double* G, qmll_stream_t stream);

/* One element's inputs of qmll_derivative_features_typed: sine coefficients f64 [A_e, S*d], projected
 * Jacobian rows f32 [A_e, n, 3, d], sign diagonals f32 [T, S, d], and the first atom of each molecule
 * in the element's molecule-major atom list, i32 [nmol + 1] (all device pointers). */
typedef struct {
    const double* cos_derivs;
    const float* input_derivative;
    const float* D;
    const int* seg_offsets;
} qmll_df_element;

/* qmll_derivative_features for every element of the batch in ONE launch (the loop over elements of
 * calculate_features, qml_lightning/models/hadamard_features.py:66-80, around
 * compute_molecular_featurization_derivative, cuda/hadamard_kernel.cu:587-717): G f64 [nmol, n, 3, S*d]
 * += the force-feature rows of all `ne` elements (host array `elements`, ne <= 8), each G element read
 * and written once; with overwrite != 0, G = those rows (never read, so it need not be cleared first:
 * the reference's loop starts from torch.zeros, kernel.py:134-137).  64 <= d <= 256. */
int qmll_derivative_features_typed(const qmll_df_element* elements, int ne, double normalisation, int n, int d, int S,
                                   int T, int nmol, int overwrite, double* G, qmll_stream_t stream);

/* Fused predict path for one element: SORF (T = ntransforms) + cos features + energy
 * contraction + the gradient with respect to the projected representation, without ever
 * materialising the [A,F] coefficients.  The result equals the chain
 * get_SORF_coefficients -> get_cos_features -> matmul(Z, alpha) and its autograd
 * backward (qml_lightning/models/hadamard_features.py:113-121, torchscript/SORF.cpp:74-136)
 * for d(sum E)/dE = 1.
 *   x f32 [A,d], D f32 [T,S,d], bias f32 [S*d], alpha f32 [S*d],
 *   out_index i32 [A] or NULL (slot of e_atom each atom writes; NULL = a)
 *   -> e_atom[out_index[a]] = sum_f sqrt(2/F) cos(c[a,f]+b[f]) alpha[f]  (overwritten, no atomics;
 *      the molecular energy is the sum of its atoms' slots)
 *   -> gx f32 [A,d] = d e_atom[a] / d x[a,:]  (overwritten; NULL = energies only) */
int qmll_sorf_energy_fused(const float* x, const float* D, const float* bias, const float* alpha,
                           const int* out_index, int A, int d, int S, int T, float normalisation,
                           float* e_atom, float* gx, qmll_stream_t stream);

/* All elements in one launch (no counterpart in the reference, which loops over elements
 * on the host and gathers each element's atoms with boolean masks,
 * qml_lightning/models/hadamard_features.py:99-119).  x_all f32 [N, ne*d]: row = atom slot
 * (molecule-major, padded slots included), one d-wide block per element type holding that
 * slot's representation projected with the element's reductor; types i32 [N] (as from
 * qmll_element_types, -1 = element not in the model); atom_slots i32 [A]: slots of the real
 * atoms; D f32 [ne,T,S,d]; bias f32 [ne,S*d]; alpha f32 [S*d].
 *   -> e_slots[slot] = energy contribution of the atom in that slot (only listed slots are
 *      written; the caller zero-fills the rest)
 *   -> gx_all f32 [N, ne*d]: block types[slot] of a listed slot = d e_slots[slot] / d x_all
 *      (other blocks untouched: the caller zero-fills; NULL = energies only) */
int qmll_sorf_energy_typed(const float* x_all, const int* types, const int* atom_slots, const float* D,
                           const float* bias, const float* alpha, int A, int N, int ne, int d, int S, int T,
                           float normalisation, float* e_slots, float* gx_all, qmll_stream_t stream);

/* ---- element-sorted projection ---------------------------------------------------- */
/* The three entry points below replace, for all elements of a batch at once, the
 * per-element loop `sub = rep[Z == e]; sub = matmul(sub, reductors[e])` of
 * qml_lightning/models/hadamard_features.py:99-108 (projection:
 * qml_lightning/representations/dimensionality_reduction.py:47-72) and its autograd
 * transpose; the fused energy kernel then consumes the compact, element-sorted rows. */

/* Stable counting sort of the real atoms by element type.  types i32 [N] per atom slot (as
 * from qmll_element_types), slots i32 [A] = slot of each real atom.
 *   -> sorted_slots i32 [A]: slots ordered by type (original order kept within a type);
 *      atoms whose type is outside [0,ne) are left out and the tail is filled with 0
 *   -> type_offsets i32 [ne+1]: atoms of type t are sorted_slots[type_offsets[t] ..
 *      type_offsets[t+1])
 * workspace: device memory of at least qmll_sort_by_type_workspace(A, ne) bytes. ne <= 32. */
size_t qmll_sort_by_type_workspace(int A, int ne);
int qmll_sort_by_type(const int* types, const int* slots, int A, int ne, void* workspace, size_t workspace_bytes,
                      int* sorted_slots, int* type_offsets, qmll_stream_t stream);

/* qmll_sort_by_type for the listed atoms of a padded batch: slot of atom a = molIDs[a] * n +
 * atomIDs[a] (the index the reference builds as torch.where(Z == e) over the [B, n] charges,
 * models/hadamard_features.py:99-107).  atomIDs, molIDs i32 [A], types i32 [B * n].  Up to 1024
 * atoms the whole sort is one launch and needs no workspace (qmll_sort_atoms_workspace returns 0);
 * beyond, the slots are written to the workspace and qmll_sort_by_type runs on them. */
size_t qmll_sort_atoms_workspace(int A, int ne);
int qmll_sort_atoms_by_type(const int* types, const int* atomIDs, const int* molIDs, int n, int A, int ne,
                            void* workspace, size_t workspace_bytes, int* sorted_slots, int* type_offsets,
                            qmll_stream_t stream);

/* qmll_sort_by_type for callers that cannot allocate device memory or carry a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose wrappers allocate with torch::zeros on every call).
 * Same inputs, outputs and results as qmll_sort_by_type; the per-workgroup counters live in a
 * device array built into the library (QMLL_SORT_NOALLOC_MAX_COUNTS ints = 512 KiB, held on
 * every GPU the library runs on until the process ends), so ceil(A/256)*ne must not exceed
 * QMLL_SORT_NOALLOC_MAX_COUNTS (QMLL_ERR_INVALID otherwise).  Calls no hipMalloc / hipFree.
 * All calls on one GPU share that array: two calls that overlap on one GPU (different
 * streams or host threads) race; calls on one stream are ordered and safe.  The first call
 * on a device looks the array's address up (hipGetSymbolAddress): make it outside capture. */
#define QMLL_SORT_NOALLOC_MAX_COUNTS 131072
int qmll_sort_by_type_noalloc(const int* types, const int* slots, int A, int ne, int* sorted_slots,
                              int* type_offsets, qmll_stream_t stream);

/* Everything the fused predict chain needs before its first compute kernel, for a padded batch
 * (Z f32 [B,n], natoms i32 [B], atomIDs / molIDs i32 [A]):
 *   types i32 [B,n]      <- qmll_element_types(Z, natoms, species[nspecies])
 *   sort_types i32 [B,n] <- the same by model_species[ne], the element list of the MODEL (its reductor /
 *                           Dmat / bias rows; qml_lightning/models/hadamard_features.py:99-107 selects
 *                           atoms over self.elements); model_species NULL: the model goes by `species`
 *                           (ne = nspecies) and sort_types is not written
 *   sorted_slots i32 [A], type_offsets i32 [ne+1] <- qmll_sort_atoms_by_type by that index
 *   zero f32 [zero_count] <- 0 (the arrays the chain accumulates into)
 * in ONE launch for up to 4096 listed atoms (65 536 slots, 262 144 floats to clear), else as the
 * separate kernels.  workspace: as for qmll_sort_atoms_by_type (none up to 1024 atoms; not used up to
 * 4096). */
int qmll_prepare_batch(const float* Z, const int* natoms, const float* species, int nspecies, const float* model_species,
                       int ne, const int* atomIDs, const int* molIDs, int B, int n, int A, void* workspace,
                       size_t workspace_bytes, int* types, int* sort_types, int* sorted_slots, int* type_offsets,
                       float* zero, size_t zero_count, qmll_stream_t stream);

/* The projection matrices ("reductors", f32 [ne,R,d], qml_lightning/models/kernel.py:28) are constants
 * of a model.  For large batches the two projections below multiply on the fp16 matrix cores with
 * every fp32 operand as two fp16 parts behind power-of-two scales (fp32 accumulation): the
 * reductors are prepared for that ONCE, here, in the layouts the kernels keep in LDS (forward: per
 * element, 32-row chunk and 128-column block; transposed: per element and 32 rows of U), so that
 * no workgroup repeats the split.  qmll_reductor_presplit_bytes: size of the prepared form (0 when
 * no kernel would use one: R must be a multiple of 4, d 64 or a multiple of 128).  The caller owns
 * the buffer (16-byte aligned) and refreshes it when the reductors change. */
size_t qmll_reductor_presplit_bytes(int ne, int R, int d);
int qmll_reductor_presplit(const float* reductors, int ne, int R, int d, void* reductors_split, size_t reductors_split_bytes,
                           qmll_stream_t stream);

/* x f32 [A,d]: row a = rep[sorted_slots[a], :] . reductors[type of a]  (rep f32 [N,R],
 * reductors f32 [ne,R,d]); rows at and beyond type_offsets[ne] are not written.
 * reductors_split: the prepared form from qmll_reductor_presplit, or NULL.  With it, batches from
 * about 65 000 atoms on (at d = 128) take the fp16 matrix-core kernel, whose results differ from the
 * fp32 kernels' in the last bits (1.7e-7 of the row's largest entry against fp64; fp32 matrix
 * instructions: 7.9e-7) and where a row's rounding depends on the largest entry among the 32 rows
 * that share its wavefront: a molecule's projection can change in the last bit with the batch it
 * is in.  The shared scale comes from the largest FINITE entry: a row of rep holding an infinity or a
 * NaN comes out non-finite (not necessarily the values the fp32 kernels give) and leaves the rows
 * beside it as they are.  Without the prepared form every batch takes the fp32 kernels. */
int qmll_project_typed(const float* rep, const int* sorted_slots, const int* type_offsets, const float* reductors,
                       const void* reductors_split, int A, int ne, int R, int d, float* x, qmll_stream_t stream);

/* The same product for `group` rows per atom: rows f32 [N*group, R] holds rows
 * slot*group ... slot*group + group - 1 for every slot, x f32 [A*group, d] receives
 * x[a*group + g, :] = rows[sorted_slots[a]*group + g, :] . reductors[type of a].  With
 * group = 3n and rows = the FCHL19 Jacobian [N, n, 3, R] this is the projection of the
 * derivative rows of every element in one launch, in place of the per-element
 * index_select + torch.matmul of the reference (qml_lightning/models/kernel.py:143-160,
 * representations/dimensionality_reduction.py:61-72); the rows of element t are
 * x[type_offsets[t]*group : type_offsets[t+1]*group].  A*group must stay below 2^31 - 128. */
int qmll_project_typed_rows(const float* rows, const int* sorted_slots, const int* type_offsets,
                            const float* reductors, int A, int ne, int R, int d, int group, float* x,
                            qmll_stream_t stream);

/* Transpose of qmll_project_typed: g_rep[sorted_slots[a], :] = gx[a, :] . reductors[type]^T
 * (g_rep f32 [N,R]).  Rows of slots that are not in the sorted list are not written, except
 * that with types != NULL (i32 [N]) the rows of slots whose type is outside [0,ne) are set
 * to zero.  reductors_split as for qmll_project_typed (NULL = fp32 kernels only); the fp16
 * matrix-core kernel (d = 64 or 128, batches beyond the small-batch kernels) scales the 32 gradient
 * rows of a wavefront by one power of two (of their largest finite entry: a non-finite gradient row
 * spoils its own result only) and every row of U by its own. */
int qmll_project_typed_backward(const float* gx, const int* sorted_slots, const int* type_offsets,
                                const float* reductors, const void* reductors_split, const int* types, int A, int N,
                                int ne, int R, int d, float* g_rep, qmll_stream_t stream);

/* qmll_project_typed_backward and, with energies != NULL, the per-molecule energies of a padded batch
 * as well: energies[m] = sum_i e_slots[m*n + i] (e_slots f32 [B*n] as written by
 * qmll_sorf_energy_sorted / qmll_rff_energy_sorted into a zero-filled array; the index_add of
 * qml_lightning/models/hadamard_features.py:119-121).  The two are independent; for small batches they
 * share one launch (a single molecule's predict step is a chain of short dependent launches, and each
 * one less counts), for large ones the sum is a launch of its own.  With A = 0 (and N = 0) only the
 * sums are formed; they add a molecule's slots in ascending order, the same in both cases. */
int qmll_project_typed_backward_sums(const float* gx, const int* sorted_slots, const int* type_offsets,
                                     const float* reductors, const void* reductors_split, const int* types, int A, int N,
                                     int ne, int R, int d, float* g_rep, const float* e_slots, int B, int n,
                                     float* energies, qmll_stream_t stream);

/* qmll_sorf_energy_typed on compact element-sorted rows: x f32 [A,d] as written by
 * qmll_project_typed, D f32 [ne,T,S,d], bias f32 [ne,S*d], alpha f32 [S*d].
 *   -> e_slots[sorted_slots[a]] = energy contribution of atom a (a < type_offsets[ne];
 *      the caller zero-fills the rest)
 *   -> gx f32 [A,d] = d e / d x  (rows beyond type_offsets[ne] set to zero; NULL = energies
 *      only)
 * bias_absmax: device pointer to ONE float, an upper bound on |bias| over all elements (a constant
 * of the model, e.g. max |bias| computed once), or NULL.  The kernel takes sine and cosine from the
 * transcendental unit, whose own range reduction ends at 256 revolutions, and takes whole
 * revolutions off larger arguments first; with the bound it decides once per atom, from
 * sum |x| and the bound, that no argument can be that large (5 % faster at 16 384 features),
 * without it every stack inspects its arguments.  Results are the same either way. */
int qmll_sorf_energy_sorted(const float* x, const int* type_offsets, const int* sorted_slots, const float* D,
                            const float* bias, const float* alpha, const float* bias_absmax, int A, int ne, int d, int S,
                            int T, float normalisation, float* e_slots, float* gx, qmll_stream_t stream);

/* ---- RFF ------------------------------------------------------------------------- */

/* Replaces rff_gpu.get_rff / compute_rff (qml_lightning/cuda/random_features.cpp:11-20,
 * kernel random_features_kernel.cu:5-41).  x f32 [A,d], W f64 [d,F], b f64 [F],
 * mol_index i32 [A] -> Zf f64 [nmol,F] += sqrt(2/F) cos(x.W + b) (fp64 arithmetic). */
int qmll_rff_features(const float* x, const double* W, const double* b, const int* mol_index,
                      int A, int d, int F, int nmol, double* Zf, qmll_stream_t stream);

/* Replaces rff_gpu.get_rff_derivatives / compute_rff_derivatives (random_features.cpp:22-33,
 * kernel random_features_kernel.cu:43-94).  grad f32 [A,n,3,d] -> G f64 [nmol,n,3,F] +=
 * sqrt(2/F) sin(x.W+b)_f * (grad[a,j,c,:].W)_f.
 * The molecule of an atom is given as for qmll_derivative_features: mol_index i32 [A] (any
 * order, fp64 atomics) or seg_offsets i32 [nmol+1] (atoms molecule-major); with seg_offsets
 * and d in {64,128,256} the products run on the fp64 matrix cores, atomic-free.  One of
 * the two may be NULL (mol_index only when that matrix-core route applies). */
int qmll_rff_derivative_features(const float* x, const float* grad, const double* W, const double* b,
                                 const int* mol_index, const int* seg_offsets, int A, int n, int d, int F,
                                 int nmol, double* G, qmll_stream_t stream);

/* W f32 [ne,d,F] of a RandomFourrierFeaturesModel (qml_lightning/models/random_features.py:42-55) is
 * a constant of the model: it is split ONCE into the form the fused predict kernel multiplies with
 * (per element and 32-feature chunk: the chunk scaled by a power of two of its own, every entry as two
 * fp16 parts, in the two layouts the kernel's matrix instructions read, laid out byte for byte as
 * the kernel keeps it in LDS) so that no workgroup repeats the split.  d is 64 or 128, F a multiple
 * of 32.  qmll_rff_presplit_bytes: size of that form in bytes (0 for unsupported sizes); the caller
 * owns the buffer (16-byte aligned) and refreshes it when W changes. */
size_t qmll_rff_presplit_bytes(int ne, int d, int F);
int qmll_rff_presplit(const float* W, int ne, int d, int F, void* W_split, size_t W_split_bytes, qmll_stream_t stream);

/* Fused RFF predict path on element-sorted rows (x f32 [A,d] from qmll_project_typed).
 * Replaces, for all elements at once, the loop body of the reference's TorchScript forward
 * (qml_lightning/models/random_features.py:88-102: matmul(sub, W[e]) + b, cos, index_add,
 * matmul(Ztest, alpha)) and its autograd transpose; the [atoms,F] feature matrix is never
 * written.  W_split: W [ne,d,F] as prepared by qmll_rff_presplit, b f32 [ne,F], alpha f32 [F];
 * d is 64 or 128, F a multiple of 32.
 *   -> e_slots[sorted_slots[a]] = sqrt(2/F) sum_f alpha_f cos(x_a . W_t[:,f] + b_t[f])
 *      (only atoms a < type_offsets[ne]; e_slots must arrive zero-filled: the launch may
 *      split the features in parts that add into it)
 *   -> gx f32 [A,d] = d e / d x (rows beyond type_offsets[ne] zero; NULL = energies only)
 * The products run on the fp16 matrix cores with every fp32 operand as two fp16 parts behind a
 * power-of-two scale (x per 32 atoms, W per chunk, alpha per launch part) and fp32 accumulation:
 * a row's rounding depends on the largest finite entry among the 32 rows that share its wavefront;
 * a row of x holding an infinity or a NaN gives a non-finite energy and gradient for its own atom
 * only, non-finite entries of W or alpha make every result non-finite (not necessarily the values
 * fp32 arithmetic gives). */
int qmll_rff_energy_sorted(const float* x, const int* type_offsets, const int* sorted_slots, const void* W_split,
                           const float* b, const float* alpha, int A, int ne, int d, int F, float* e_slots,
                           float* gx, qmll_stream_t stream);

/* ---- Gram ------------------------------------------------------------------------ */

/* Replaces the Gram accumulation of BaseKernel.build_Z_components
 * (qml_lightning/models/kernel.py:190-192: ZTZ += Z^T Z, ZtrainY += Z^T y, both fp64).
 * Z f64 [M,F] row-major (lda = F), y f64 [M] or NULL -> ZTZ f64 [F,F] += Z^T Z (both
 * triangles written), ZTy f64 [F] += Z^T y.  fp64 MFMA. */
int qmll_gram_f64(const double* Z, const double* y, int M, int F, double* ZTZ, double* ZTy, qmll_stream_t stream);

/* qmll_gram_f64 without its last pass: only the tiles (128 x 128) on or above the diagonal of
 * ZTZ are accumulated; the strictly lower tiles are left as they are.  For a caller that
 * accumulates several row batches (the loop of build_Z_components, kernel.py:93-192): add
 * every batch with this entry, then call qmll_gram_mirror_f64 once. */
int qmll_gram_upper_f64(const double* Z, const double* y, int M, int F, double* ZTZ, double* ZTy,
                        qmll_stream_t stream);

/* qmll_gram_upper_f64 with a device workspace of qmll_gram_workspace_bytes() bytes (same part of
 * kernel.py:190-192).  The tiles run in rounds of one per workgroup slot; when the last round is
 * less than half full (64 of 8256 tiles at F = 16 384) its tiles are cut into row ranges that fill
 * the slots, the partial tiles go to the workspace and are added in a fixed order, so the result
 * stays deterministic (it differs from qmll_gram_upper_f64 by the rounding of that regrouping).
 * With workspace NULL, fewer bytes, fewer than 2048 rows or a well-filled last round it is
 * qmll_gram_upper_f64.  The number of slots, and with it whether and how the last tiles are cut, follows
 * from the device's CU count (hipDeviceAttributeMultiprocessorCount): results are reproducible
 * from run to run on one device model, and equal up to that regrouping's rounding (1e-16 relative)
 * between device models or between calls with and without a workspace. */
size_t qmll_gram_workspace_bytes(void);
int qmll_gram_upper_ws_f64(const double* Z, const double* y, int M, int F, double* ZTZ, double* ZTy,
                           double* workspace, size_t workspace_bytes, qmll_stream_t stream);

/* ZTZ[j,i] = ZTZ[i,j] for the tiles strictly above the diagonal: completes a matrix built with
 * qmll_gram_upper_f64 (both triangles bit-identical). */
int qmll_gram_mirror_f64(double* ZTZ, int F, qmll_stream_t stream);

/* ---- regularised solve: replaces torch.linalg.solve(ZTZ + lambda I, ZtrainY) of
 * qml_lightning/models/kernel.py:226-234 (LU there; the matrix is symmetric positive definite) ---- */

/* Bytes of device workspace qmll_cholesky_f64 / qmll_cholesky_solve_f64 need for an F x F matrix. */
size_t qmll_cholesky_workspace_bytes(int F);

/* In-place fp64 Cholesky factorisation A = U^T U of the F x F matrix A (row-major, row stride ld
 * doubles, ld even).  Reads only elements on or above the diagonal; on exit they hold U.  Below
 * the diagonal, the lower halves of the 128 x 128 diagonal tiles are overwritten with junk, the
 * rest is untouched.  workspace (qmll_cholesky_workspace_bytes(F), 16-byte aligned) receives the
 * inverses of the 128 x 128 diagonal blocks of U and must be passed unchanged to
 * qmll_cholesky_solve_f64.
 * info (device int, zeroed by the caller): 0 on success, else 1 + the index of the first pivot
 * that is not positive; U is then unusable.  When F is a multiple of 128 (and A 16-byte aligned) a
 * panel of 512 rows and the trailing update of the panel before it are one launch whose workgroups
 * wait for one another through flags in the workspace; every such wait is bounded, and one that
 * runs out (never seen) leaves info = -1, which callers treat like a failed pivot.  The tile products
 * add into the trailing matrix with hardware fp64 atomic adds, which need A in ordinary device memory
 * (hipMalloc; what torch allocates), not in host-mapped or managed memory. */
int qmll_cholesky_f64(double* A, int F, long long ld, void* workspace, int* info, qmll_stream_t stream);

/* b <- (U^T U)^-1 b for one right-hand side b[F], U and workspace from qmll_cholesky_f64.  One launch per
 * direction, a workgroup per 128-row block; the blocks wait for one another's results with bounded waits,
 * and one that runs out (never seen) leaves NaN in b rather than a wrong number.  Calls that share a
 * workspace must not overlap. */
int qmll_cholesky_solve_f64(const double* U, int F, long long ld, void* workspace, double* b, qmll_stream_t stream);

/* Feature-tiled variant (kernel.py:172-181, ntiles > 1): ZTZ_tile f64 [f1-f0, F] +=
 * Z[:, f0:f1]^T Z, ZTy f64 [F] (rows f0..f1 updated) += Z[:, f0:f1]^T y. */
int qmll_gram_tile_f64(const double* Z, const double* y, int M, int F, int f0, int f1, double* ZTZ_tile, double* ZTy,
                       qmll_stream_t stream);

/* Replaces utils_gpu.matmul_and_reduce (qml_lightning/cuda/utils_cuda.cpp:26-33, kernel
 * utils_kernel.cu:70-129): C f64 [Ar,Bc] += (double)(A f32 [Ar,K] . B f32 [K,Bc]) with the
 * K-sum carried in fp32 with Kahan compensation. */
int qmll_matmul_and_reduce(const float* A, const float* B, int Ar, int K, int Bc, double* C, qmll_stream_t stream);

/* ---- measured ceilings of the device (no counterpart in the reference; the benchmark divides
 * each kernel's rate by these next to the nominal peaks) ------------------------------------- */

/* dst[0..nfloats) = value with plain 16-byte stores; dst = src with plain 16-byte loads and stores
 * (nfloats a multiple of 4, pointers 16-byte aligned).  The copy is also the known-size reference
 * for scaling a profiler's FETCH_SIZE / WRITE_SIZE counters. */
int qmll_probe_fill(float* dst, size_t nfloats, float value, qmll_stream_t stream);
int qmll_probe_copy(const float* src, float* dst, size_t nfloats, qmll_stream_t stream);

/* A loop of `iters` rounds of independent instructions on every SIMD of the chip: which = 0
 * v_mfma_f64_16x16x4_f64, 1 v_mfma_f32_32x32x2_f32, 2 v_exp_f32, 3 v_mfma_f32_32x32x16_f16;
 * blocks_per_cu (1..16) workgroups of four wavefronts per compute unit, i.e. that many wavefronts
 * per SIMD.  out: device scratch of qmll_probe_out_bytes() bytes.  Returns the number of operations
 * the launch performs (flop, or exponentials for which = 2), to be divided by the measured
 * duration; negative on error. */
size_t qmll_probe_out_bytes(void);
double qmll_probe_rate(int which, int iters, int blocks_per_cu, void* out, qmll_stream_t stream);

/* Straight-line loops of the instruction classes the fused SORF kernel issues, on independent
 * registers: mix = 0 128 plain fp32, 1 128 DPP fmac, 2 128 v_sin_f32, 3 the per-stack mix of the
 * fused kernel at 128 components (82 plain + 64 DPP + 16 transcendental).
 * Returns wavefront-iterations per SIMD (blocks_per_cu x iters), so
 * duration x clock / that = SIMD clocks per iteration; negative on error. */
double qmll_probe_mix(int mix, int iters, int blocks_per_cu, void* out, qmll_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* QMLL_H */
