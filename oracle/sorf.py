"""CPU oracle (test infrastructure, never the product path): SORF / cos features /
derivative features / Gram / RFF in fp64 NumPy.

Follows (paths relative to the reference tree):
  * fast Walsh-Hadamard butterflies .... qml_lightning/cuda/hadamard_kernel.cu:32-90
  * SORF coefficients .................. qml_lightning/cuda/hadamard_kernel.cu:5-102, 424-539
  * SORF adjoint ....................... qml_lightning/cuda/hadamard_kernel.cu:204-312
  * cos features (+ f64 accumulate) .... qml_lightning/cuda/hadamard_kernel.cu:541-563, 778-800
  * cos-feature backward ............... qml_lightning/cuda/hadamard_kernel.cu:816-839
  * sin coefficients ................... qml_lightning/cuda/hadamard_kernel.cu:565-585
  * derivative features ................ qml_lightning/cuda/hadamard_kernel.cu:587-717
  * model-level feature assembly ....... qml_lightning/models/hadamard_features.py:66-121
  * regularised solve .................. qml_lightning/models/kernel.py:226-234
  * Gram accumulation, targets ......... qml_lightning/models/kernel.py:118-192
  * fp32-Kahan -> fp64 product ......... qml_lightning/cuda/utils_kernel.cu:70-119
  * RFF features / derivative .......... qml_lightning/cuda/random_features_kernel.cu:5-94,
                                         qml_lightning/models/random_features.py:38,54-55,98
  * PCA projection ..................... qml_lightning/representations/dimensionality_reduction.py:58,72

Pinned by: the reference's aspirin known-answer vector (SORF T=1, cos features, their
backward, Z.alpha), the closed form scipy.linalg.hadamard(d)/sqrt(d), <Ax,y> = <x,A^T y>,
finite differences of Z in fp64 and G.alpha == forces (tests/test_oracle_sorf.py).
ntransforms > 1 and the RFF functions are pinned by closed forms only: the reference
holds no vector for them (its RFF model file is absent).
"""
import numpy as np


def fwht(v):
    """Unnormalised Walsh-Hadamard transform along the last axis, natural (Sylvester)
    order, by the reference's butterflies: one radix-2 stage at stride 1 when log2(d) is
    odd, then radix-4 stages (a radix-4 stage at stride s is the radix-2 stages at 2s and s)
    (hadamard_kernel.cu:32-83)."""
    v = np.array(v, dtype=np.float64, copy=True)
    d = v.shape[-1]
    log2d = int(round(np.log2(d)))
    if (1 << log2d) != d:
        raise RuntimeError("input size must be power of 2.")   # hadamard_kernel.cu:730
    stride = 1
    if log2d & 1:
        a = v[..., 0::2].copy()
        b = v[..., 1::2].copy()
        v[..., 0::2] = a + b
        v[..., 1::2] = a - b
        stride <<= 1
    while stride <= d >> 2:
        pos = np.arange(d // 4)
        lo = pos & (stride - 1)
        i0 = ((pos - lo) << 2) + lo
        i1, i2, i3 = i0 + stride, i0 + 2 * stride, i0 + 3 * stride
        D0, D1, D2, D3 = v[..., i0], v[..., i1], v[..., i2], v[..., i3]
        A0, A2 = D0 + D2, D0 - D2
        A1, A3 = D1 + D3, D1 - D3
        v[..., i0] = A0 + A1
        v[..., i1] = A0 - A1
        v[..., i2] = A2 + A3
        v[..., i3] = A2 - A3
        stride <<= 2
    return v


def sorf_coefficients(x, D, normalisation):
    """out[a,s,:] = normalisation * prod_{m<T} (H/sqrt(d) diag(D[m,s])) x[a]
    (hadamard_kernel.cu:19-100).  x [A,d], D [T,S,d] -> [A,S,d]."""
    x = np.asarray(x, dtype=np.float64)
    D = np.asarray(D, dtype=np.float64)
    T, S, d = D.shape
    normh = 1.0 / 2.0 ** (np.log2(d) / 2.0)
    s = np.repeat(x[:, None, :], S, axis=1)
    for m in range(T):
        s = normh * fwht(D[m][None, :, :] * s)
    return normalisation * s


def sorf_adjoint(g, D, normalisation):
    """Adjoint of sorf_coefficients summed over stacks (hadamard_kernel.cu:225-311):
    for m = T-1..0: s = D[m,s] * normh * FWHT(s).  g [A,S,d] -> [A,d]."""
    s = np.asarray(g, dtype=np.float64)
    D = np.asarray(D, dtype=np.float64)
    T, S, d = D.shape
    normh = 1.0 / 2.0 ** (np.log2(d) / 2.0)
    for m in range(T - 1, -1, -1):
        s = D[m][None, :, :] * normh * fwht(s)
    return normalisation * s.sum(axis=1)


def cos_features(coeffs, bias, mol_index, nmol):
    """Z[mol(a),f] += sqrt(2/F) cos(c[a,f]+b[f]) (hadamard_kernel.cu:558-562, 795-799)."""
    coeffs = np.asarray(coeffs, dtype=np.float64)
    F = coeffs.shape[1]
    Z = np.zeros((nmol, F))
    np.add.at(Z, np.asarray(mol_index), np.cos(coeffs + np.asarray(bias, dtype=np.float64)[None, :]) * np.sqrt(2.0 / F))
    return Z


def cos_features_backward(gZ, coeffs, bias, mol_index):
    """g_c[a,f] = g_Z[mol(a),f] * -sin(c+b) * sqrt(2/F) (hadamard_kernel.cu:834-838)."""
    coeffs = np.asarray(coeffs, dtype=np.float64)
    F = coeffs.shape[1]
    return np.asarray(gZ, dtype=np.float64)[np.asarray(mol_index)] * -np.sin(coeffs + np.asarray(bias, dtype=np.float64)[None, :]) * np.sqrt(2.0 / F)


def sin_coeffs(coeffs, bias):
    """s[a,f] = +sin(c+b) sqrt(2/F) (hadamard_kernel.cu:580-584)."""
    coeffs = np.asarray(coeffs, dtype=np.float64)
    F = coeffs.shape[1]
    return np.sin(coeffs + np.asarray(bias, dtype=np.float64)[None, :]) * np.sqrt(2.0 / F)


def derivative_features(cos_derivs, normalisation, mol_index, input_derivative, D, nmol):
    """G[mol(a),j,x,s*d+p] += normalisation * cos_derivs[a,s*d+p] * (chain_s u)[p],
    u = input_derivative[a,j,x,:], chain_s = prod_m (H/sqrt(d) diag(D[m,s]))
    (hadamard_kernel.cu:616-715).  input_derivative [A,n,3,d] -> G [nmol,n,3,S*d]."""
    u = np.asarray(input_derivative, dtype=np.float64)
    D = np.asarray(D, dtype=np.float64)
    A, n, _, d = u.shape
    T, S, _ = D.shape
    normc = 1.0 / 2.0 ** (np.log2(d) / 2.0)
    G = np.zeros((nmol, n, 3, S * d))
    cd = np.asarray(cos_derivs, dtype=np.float64).reshape(A, S, d)
    for a in range(A):
        v = np.repeat(u[a][:, :, None, :], S, axis=2)          # [n,3,S,d]
        for m in range(T):
            v = normc * fwht(D[m][None, None, :, :] * v)
        G[mol_index[a]] += (normalisation * cd[a][None, None, :, :] * v).reshape(n, 3, S * d)
    return G


def project(rep_rows, reductor):
    """rep @ U (dimensionality_reduction.py:58); works for [A,R] and [A,n,3,R] (:72)."""
    return np.asarray(rep_rows, dtype=np.float64) @ np.asarray(reductor, dtype=np.float64)


def hadamard_model_features(rep, charges, elements, reductors, Dmat, bias, sigma, jac=None):
    """Molecular feature matrix Z [B,F] and, when `jac` [B,n,n,3,R] is given, the force
    feature tensor G [B,n,3,F] assembled per element exactly like
    HadamardFeaturesModel.calculate_features inside BaseKernel.build_Z_components
    (hadamard_features.py:66-80, kernel.py:141-162)."""
    rep = np.asarray(rep, dtype=np.float64)
    B, n, R = rep.shape
    T, S, d = np.asarray(Dmat[0]).shape
    F = S * d
    Z = np.zeros((B, F))
    G = np.zeros((B, n, 3, F)) if jac is not None else None
    norm = np.sqrt(d) / sigma
    q = np.asarray(charges).astype(np.int64)
    for ei, e in enumerate(elements):
        mask = q == int(e)
        if not mask.any():
            continue
        mol_index = np.nonzero(mask)[0]
        sub = project(rep[mask], reductors[ei])
        coeffs = sorf_coefficients(sub, Dmat[ei], norm).reshape(len(sub), F)
        Z += cos_features(coeffs, bias[ei], mol_index, B)
        if jac is not None:
            sg = project(np.asarray(jac, dtype=np.float64)[mask], reductors[ei])     # [A_e,n,3,d]
            G += derivative_features(sin_coeffs(coeffs, bias[ei]), norm, mol_index, sg, Dmat[ei], B)
    return Z, G


def training_rows(Z, G, E=None, F=None):
    """Stack the rows and targets the way build_Z_components does (kernel.py:118-124,
    164-170): B energy rows then B*n*3 force rows; energy rows zeroed when E is None."""
    B = Z.shape[0]
    Zrows = Z.copy()
    if E is None:
        Zrows[:] = 0.0
    if F is not None:
        Zrows = np.concatenate([Zrows, G.reshape(-1, G.shape[-1])], axis=0)
    if E is not None and F is None:
        y = np.asarray(E, dtype=np.float64)[:, None]
    elif E is None:
        y = np.concatenate([np.zeros((B, 1)), np.asarray(F, dtype=np.float64).reshape(-1, 1)], axis=0)
    else:
        y = np.concatenate([np.asarray(E, dtype=np.float64)[:, None], np.asarray(F, dtype=np.float64).reshape(-1, 1)], axis=0)
    return Zrows, y


def gram(Zrows, y):
    """ZTZ = Z^T Z, ZTy = Z^T y in fp64 (kernel.py:190-192)."""
    return Zrows.T @ Zrows, Zrows.T @ y


def regularised_solve(ZTZ, ZTy, llambda):
    """alpha of the regularised normal equations, the way train() gets it: lambda added to the
    diagonal of Z^T Z, then a general (LU) solve (qml_lightning/models/kernel.py:226-234).
    Pinned by the identity it solves: tests check the residual and the agreement with a Cholesky
    factorisation of the same matrix."""
    A = np.array(ZTZ, dtype=np.float64, copy=True)
    A[np.diag_indices_from(A)] += llambda
    return np.linalg.solve(A, np.asarray(ZTy, dtype=np.float64))


def matmul_and_reduce(A32, B32, C64, block=16):
    """C += double(float(A) @ float(B)) with the inner sum carried in fp32 with Kahan
    compensation (utils_kernel.cu:104-117).  The reference walks K in zero-padded tiles of
    16 (utils_kernel.cu:90-101), and a zero product still applies the pending compensation
    (y = fma(0, 0, -c)), so the padded steps are part of the arithmetic and are kept.
    Small sizes only (Python loop over K)."""
    A32 = np.asarray(A32, dtype=np.float32)
    B32 = np.asarray(B32, dtype=np.float32)
    K = A32.shape[1]
    Kpad = -(-K // block) * block
    s = np.zeros((A32.shape[0], B32.shape[1]), dtype=np.float32)
    c = np.zeros_like(s)
    for k in range(Kpad):
        if k < K:
            prod = A32[:, k:k + 1].astype(np.float64) * B32[k:k + 1, :].astype(np.float64)   # exact in fp64
        else:
            prod = np.zeros(s.shape)
        # fma(a, b, -c): one rounding of the exact a*b - c
        yv = (prod - c.astype(np.float64)).astype(np.float32)
        t = (s + yv).astype(np.float32)
        c = ((t - s).astype(np.float32) - yv).astype(np.float32)
        s = t
    C64 += s.astype(np.float64)
    return C64


def rff_features(x, W, b, mol_index, nmol):
    """Z[mol(a),f] += sqrt(2/F) cos(x[a].W[:,f] + b[f]) (random_features_kernel.cu:28-40)."""
    x = np.asarray(x, dtype=np.float64)
    W = np.asarray(W, dtype=np.float64)
    F = W.shape[1]
    Z = np.zeros((nmol, F))
    np.add.at(Z, np.asarray(mol_index), np.sqrt(2.0 / F) * np.cos(x @ W + np.asarray(b, dtype=np.float64)[None, :]))
    return Z


def rff_derivative_features(x, grad, W, b, mol_index, nmol):
    """G[mol(a),j,c,f] += sqrt(2/F) sin(x[a].W+b)_f * (grad[a,j,c,:].W)_f
    (random_features_kernel.cu:71-92)."""
    x = np.asarray(x, dtype=np.float64)
    W = np.asarray(W, dtype=np.float64)
    grad = np.asarray(grad, dtype=np.float64)
    F = W.shape[1]
    A, n = grad.shape[0], grad.shape[1]
    G = np.zeros((nmol, n, 3, F))
    fd = np.sqrt(2.0 / F) * np.sin(x @ W + np.asarray(b, dtype=np.float64)[None, :])     # [A,F]
    np.add.at(G, np.asarray(mol_index), fd[:, None, None, :] * (grad @ W))
    return G
