"""CPU oracle (test infrastructure, never the product path): FCHL19 in fp64 NumPy.

A restatement of the reference's CUDA arithmetic, formula by formula, so the HIP
kernels can be checked against it.  Only tests, the smoke check and the CPU-baseline
leg of the benchmark may import this module.

Follows (paths relative to the reference tree):
  * neighbour count / list ........ qml_lightning/cuda/pairlist_kernel.cu:145-224, 326-391
  * minimum image ................. qml_lightning/cuda/fchl_cuda_kernel.cu:16-49
  * element types ................. qml_lightning/cuda/fchl_cuda_kernel.cu:1716-1742
  * cosine cutoff + derivative .... qml_lightning/cuda/fchl_cuda_kernel.cu:51-98
  * log-normal radial derivative .. qml_lightning/cuda/fchl_cuda_kernel.cu:154-170
  * forward representation ........ qml_lightning/cuda/fchl_cuda_kernel.cu:570-673
  * explicit Jacobian ............. qml_lightning/cuda/fchl_cuda_kernel.cu:768-1004
  * VJP (backward) ................ qml_lightning/cuda/fchl_cuda_kernel.cu:1438-1713
  * hyper-parameter tensors ....... qml_lightning/representations/FCHL.py:18-42

Pinned by: the reference's aspirin known-answer vector (forward + VJP, end to end),
central finite differences of the forward (Jacobian), the translation sum rule,
permutation / rotation invariance and hand-computed 3-atom cases
(tests/test_oracle_fchl.py).  The minimum-image branch is pinned by a brute-force
27-image search only; the reference holds no vector for it.
"""
import numpy as np


class FCHLParams:
    """Hyper-parameters exactly as FCHLCuda hands them to its kernels
    (qml_lightning/representations/FCHL.py:18-42): three_body_weight already carries
    sqrt(eta3/pi); Rs2/Rs3 are linspace(0, rcut, n+1)[1:]."""

    def __init__(self, species, rcut=6.0, nRs2=24, nRs3=20, eta2=0.32, eta3=2.7,
                 two_body_decay=1.8, three_body_weight=13.4, three_body_decay=0.57,
                 raw_three_body_weight=None, Rs2=None, Rs3=None):
        self.species = np.asarray(species, dtype=np.float64)
        self.nspecies = len(self.species)
        self.rcut = float(rcut)
        self.eta2 = float(eta2)
        self.eta3 = float(eta3)
        self.two_body_decay = float(two_body_decay)
        if raw_three_body_weight is not None:
            self.three_body_weight = float(raw_three_body_weight)
        else:
            self.three_body_weight = float(np.sqrt(eta3 / np.pi) * three_body_weight)
        self.three_body_decay = float(three_body_decay)
        self.Rs2 = (np.linspace(0.0, rcut, nRs2 + 1)[1:] if Rs2 is None
                    else np.asarray(Rs2, dtype=np.float64))
        self.Rs3 = (np.linspace(0.0, rcut, nRs3 + 1)[1:] if Rs3 is None
                    else np.asarray(Rs3, dtype=np.float64))
        self.nRs2 = len(self.Rs2)
        self.nRs3 = len(self.Rs3)
        ns = self.nspecies
        self.repsize = ns * self.nRs2 + ns * (ns + 1) * self.nRs3


def pbc_drij(d, cell, inv_cell):
    """General minimum image (fchl_cuda_kernel.cu:16-49): s = inv_cell d,
    s -= round(s), d = cell s.  `d` is [..., 3]."""
    s = np.einsum("mk,...k->...m", inv_cell, d)
    s = s - np.round(s)
    return np.einsum("mk,...k->...m", cell, s)


def neighbours(X, natoms, rcut, cell=None, inv_cell=None):
    """Counts [B,n] and ascending-j lists [B,n,nn] padded with -1
    (pairlist_kernel.cu:202-219, 372-390): j is a neighbour of i when
    0 < |d_ij|^2 < rcut^2, with d_ij minimum-imaged if a cell is given."""
    X = np.asarray(X, dtype=np.float64)
    B, n, _ = X.shape
    counts = np.zeros((B, n), dtype=np.int32)
    lists = []
    for m in range(B):
        na = int(natoms[m])
        d = X[m, :na, None, :] - X[m, None, :na, :]
        if cell is not None and len(cell) > 0:
            d = pbc_drij(d, np.asarray(cell[m], dtype=np.float64), np.asarray(inv_cell[m], dtype=np.float64))
        r2 = (d * d).sum(-1)
        mask = (r2 < rcut * rcut) & (r2 > 0)
        counts[m, :na] = mask.sum(1)
        lists.append(mask)
    nn = int(counts.max()) if counts.size else 0
    nlist = -np.ones((B, n, nn), dtype=np.int32)
    for m in range(B):
        mask = lists[m]
        for i in range(mask.shape[0]):
            js = np.nonzero(mask[i])[0]
            nlist[m, i, :len(js)] = js
    return counts, nlist


def element_types(Z, natoms, species):
    """Index of int(charge) in `species`, -1 if absent (fchl_cuda_kernel.cu:1726-1740);
    padded slots keep 0 like the reference's zero-initialised output."""
    Z = np.asarray(Z)
    B, n = Z.shape
    out = np.zeros((B, n), dtype=np.int32)
    for m in range(B):
        for i in range(int(natoms[m])):
            q = int(Z[m, i])
            idx = -1
            for j, s in enumerate(species):
                if q == s:
                    idx = j
            out[m, i] = idx
    return out


def _cut(r, rcut):
    return 0.5 * (np.cos(r * np.pi / rcut) + 1.0)          # fchl_cuda_kernel.cu:57


def _dcut(r, rcut):
    return -0.5 * np.sin(r * np.pi / rcut) * np.pi / rcut  # fchl_cuda_kernel.cu:81


def _disp(X, m, i, js, cell, inv_cell):
    d = X[m, i][None, :] - X[m, js]                         # ri - rj  (:574-576)
    if cell is not None and len(cell) > 0:
        d = pbc_drij(d, np.asarray(cell[m], dtype=np.float64), np.asarray(inv_cell[m], dtype=np.float64))
    return d


def _pair_offset(p, q, ns, nRs2, nRs3):
    # fchl_cuda_kernel.cu:658-661
    return ns * nRs2 + nRs3 * 2 * (-(p * (p + 1)) // 2 + q + ns * p)


def forward(X, types, atomIDs, molIDs, nlist, nneigh, prm, cell=None, inv_cell=None):
    """rep [B,n,R] (fchl_cuda_kernel.cu:570-673)."""
    X = np.asarray(X, dtype=np.float64)
    B, n, _ = X.shape
    ns, nRs2, nRs3 = prm.nspecies, prm.nRs2, prm.nRs3
    rep = np.zeros((B, n, prm.repsize))
    zeta = np.exp(-np.pi ** 2 * 0.5)
    lnRs2 = np.log(prm.Rs2)
    for i, m in zip(atomIDs, molIDs):
        nn = int(nneigh[m, i])
        js = nlist[m, i, :nn]
        if nn == 0:
            continue
        d = _disp(X, m, i, js, cell, inv_cell)              # drij, [nn,3]
        r = np.sqrt((d * d).sum(-1))
        el = types[m, js]
        # two-body (:586-603)
        scaling = 1.0 / r ** prm.two_body_decay
        fc = _cut(r, prm.rcut)
        mu = np.log(r / np.sqrt(1.0 + prm.eta2 / r ** 2))
        sigma = np.sqrt(np.log(1.0 + prm.eta2 / r ** 2))
        radial = (1.0 / (sigma[:, None] * np.sqrt(2 * np.pi) * prm.Rs2[None, :])
                  * np.exp(-(lnRs2[None, :] - mu[:, None]) ** 2 / (2.0 * sigma[:, None] ** 2))
                  * scaling[:, None] * fc[:, None])
        for a in range(nn):
            rep[m, i, el[a] * nRs2:(el[a] + 1) * nRs2] += radial[a]
        if nn < 2:
            continue
        # three-body over list positions j<k (:605-672)
        ja, ka = np.triu_indices(nn, 1)
        dij, dik = d[ja], d[ka]
        djk = dik - dij                                      # = rj - rk (:617-619)
        rij, rik = r[ja], r[ka]
        rjk = np.sqrt((djk * djk).sum(-1))
        cos_i = ((-dij) * (-dik)).sum(-1) / (rij * rik)      # (drji, drki)   :647
        cos_k = (djk * dik).sum(-1) / (rjk * rik)            # (drjk, drik)   :649
        cos_j = (dij * (-djk)).sum(-1) / (rij * rjk)         # (drij, drkj)   :651
        angle = np.arccos(np.clip(cos_i, -1.0, 1.0))         # :251-261
        ksi3 = prm.three_body_weight * (1.0 + 3.0 * cos_i * cos_j * cos_k) / (rij * rik * rjk) ** prm.three_body_decay
        cos_a = zeta * 2.0 * np.cos(angle)
        sin_a = zeta * 2.0 * np.sin(angle)
        p = np.minimum(el[ja], el[ka])
        q = np.maximum(el[ja], el[ka])
        s = _pair_offset(p, q, ns, nRs2, nRs3)
        rad = (np.exp(-prm.eta3 * (0.5 * (rij + rik)[:, None] - prm.Rs3[None, :]) ** 2)
               * (fc[ja] * fc[ka])[:, None])
        vc = rad * (cos_a * ksi3)[:, None]
        vs = rad * (sin_a * ksi3)[:, None]
        idx = s[:, None] + 2 * np.arange(nRs3)[None, :]
        np.add.at(rep[m, i], idx, vc)
        np.add.at(rep[m, i], idx + 1, vs)
    return rep


def _lognormal_dradial(dx, r, eta, Rs):
    """get_radial_derivative_distribution, log-normal branch
    (fchl_cuda_kernel.cu:154-170).  dx [nn,3], r [nn], Rs [nz] -> [nn,3,nz]."""
    mu = np.log(r / np.sqrt(1.0 + eta / r ** 2))
    sigma = np.sqrt(np.log(1.0 + eta / r ** 2))
    sigma2 = sigma ** 2
    sigma4 = sigma ** 4
    lnRs = np.log(Rs)
    exp_ln = np.exp(-(lnRs[None, :] - mu[:, None]) ** 2 / sigma2[:, None] * 0.5)      # [nn,nz]
    r2 = r ** 2
    dsigma = dx * (eta * (1.0 / ((eta + r2) * r * np.sqrt(np.log((eta + r2) / r2)))))[:, None]   # [nn,3]
    dmu = -dx * ((2 * eta + r2) / ((eta + r2) * r))[:, None]
    mml = (mu[:, None] - lnRs[None, :])                                                # [nn,nz]
    pref = np.sqrt(2.0) / (2 * np.sqrt(np.pi) * Rs[None, :] * sigma4[:, None])         # [nn,nz]
    out = (pref[:, None, :]
           * (((mml[:, None, :] * dsigma[:, :, None] - sigma[:, None, None] * dmu[:, :, None]) * mml[:, None, :])
              - sigma2[:, None, None] * dsigma[:, :, None])
           * exp_ln[:, None, :])
    return out


def jacobian(X, types, atomIDs, molIDs, nlist, nneigh, prm, cell=None, inv_cell=None):
    """grad [B,n,n,3,R] with grad[m,i,j,x,f] = d rep[m,i,f] / d X[m,j,x]
    (fchl_cuda_kernel.cu:768-1004, all terms kept as the reference writes them)."""
    X = np.asarray(X, dtype=np.float64)
    B, n, _ = X.shape
    ns, nRs2, nRs3 = prm.nspecies, prm.nRs2, prm.nRs3
    R = prm.repsize
    grad = np.zeros((B, n, n, 3, R))
    zeta = np.exp(-np.pi ** 2 * 0.5)
    lnRs2 = np.log(prm.Rs2)
    invcut = 1.0 / prm.rcut
    w3 = prm.three_body_weight
    d3 = prm.three_body_decay
    larr = np.arange(nRs3)
    for i, m in zip(atomIDs, molIDs):
        nn = int(nneigh[m, i])
        js = nlist[m, i, :nn]
        if nn == 0:
            continue
        d = _disp(X, m, i, js, cell, inv_cell)
        r2 = (d * d).sum(-1)
        r = np.sqrt(r2)
        el = types[m, js]
        scaling = 1.0 / r ** prm.two_body_decay
        fc = _cut(r, prm.rcut)
        mu = np.log(r / np.sqrt(1.0 + prm.eta2 / r ** 2))
        sigma = np.sqrt(np.log(1.0 + prm.eta2 / r ** 2))
        dcut = _dcut(r, prm.rcut)
        dscal = -prm.two_body_decay / r ** (prm.two_body_decay + 1.0)
        radial = (1.0 / (sigma[:, None] * np.sqrt(2.0 * np.pi) * prm.Rs2[None, :])
                  * np.exp(-(lnRs2[None, :] - mu[:, None]) ** 2 / (2.0 * sigma[:, None] ** 2)))   # [nn,nz]
        dx = d / r[:, None]                                                                      # [nn,3]
        dradial = _lognormal_dradial(dx, r, prm.eta2, prm.Rs2)                                   # [nn,3,nz]
        dcutx = dcut[:, None] * -dx
        dscalx = dscal[:, None] * -dx
        deriv = (dradial * (scaling * fc)[:, None, None]
                 + radial[:, None, :] * dscalx[:, :, None] * fc[:, None, None]
                 + radial[:, None, :] * scaling[:, None, None] * dcutx[:, :, None])              # :821
        for a in range(nn):
            sl = slice(el[a] * nRs2, (el[a] + 1) * nRs2)
            grad[m, i, i, :, sl] += -deriv[a]                                                    # :823
            grad[m, i, js[a], :, sl] += deriv[a]                                                 # :824
        if nn < 2:
            continue
        ja, ka = np.triu_indices(nn, 1)
        drij, drik = d[ja], d[ka]
        drjk = drik - drij
        drji, drki, drkj = -drij, -drik, -drjk
        rij2, rik2 = r2[ja], r2[ka]
        rij, rik = r[ja], r[ka]
        rjk2 = (drjk * drjk).sum(-1)
        rjk = np.sqrt(rjk2)
        invrij, invrik, invrjk = 1.0 / rij, 1.0 / rik, 1.0 / rjk
        invrij2, invrik2, invrjk2 = invrij ** 2, invrik ** 2, invrjk ** 2
        rcutij, rcutik = fc[ja], fc[ka]
        cos_i = (drji * drki).sum(-1) * invrij * invrik
        cos_k = (drjk * drik).sum(-1) * invrjk * invrik
        cos_j = (drij * drkj).sum(-1) * invrij * invrjk
        angle = np.arccos(np.clip(cos_i, -1.0, 1.0))
        cos_angle = zeta * 2.0 * np.cos(angle)
        sin_angle = zeta * 2.0 * np.sin(angle)
        invr_atm = (invrij * invrjk * invrik) ** d3
        atm = (1.0 + 3.0 * cos_i * cos_j * cos_k) * invr_atm * w3
        p = np.minimum(el[ja], el[ka])
        q = np.maximum(el[ja], el[ka])
        s = _pair_offset(p, q, ns, nRs2, nRs3)
        vi = (drji * drki).sum(-1)
        vj = (drkj * drij).sum(-1)
        vk = (drik * drjk).sum(-1)
        guard = np.sqrt(np.maximum(1e-10, rij2 * rik2 - vi * vi))                                # :911
        dcos_angle = zeta * 2.0 * np.sin(angle) / guard
        dsin_angle = -zeta * 2.0 * np.cos(angle) / guard
        atm_i = (3.0 * cos_j * cos_k) * invr_atm * invrij * invrik
        atm_j = (3.0 * cos_k * cos_i) * invr_atm * invrij * invrjk
        atm_k = (3.0 * cos_i * cos_j) * invr_atm * invrjk * invrik
        a_, c_ = drji, drki                                                                      # b = 0
        col = lambda v: v[:, None]
        d_radial_d_j = (-a_) * col(invrij)
        d_radial_d_k = (-c_) * col(invrik)
        d_radial_d_i = -(d_radial_d_j + d_radial_d_k)
        d_angular_d_j = c_ + col(vi) * ((-a_) * col(invrij2))
        d_angular_d_k = a_ + col(vi) * ((-c_) * col(invrik2))
        d_angular_d_i = -(d_angular_d_j + d_angular_d_k)
        d_ijdecay = -np.pi * (-a_) * col(np.sin(np.pi * rij * invcut) * 0.5 * invrij * invcut)
        d_ikdecay = -np.pi * (-c_) * col(np.sin(np.pi * rik * invcut) * 0.5 * invrik * invcut)
        d_atm_ii = -a_ - c_ - col(vi) * ((-a_) * col(invrij2) + (-c_) * col(invrik2))
        d_atm_ij = c_ - a_ - col(vj) * (-a_) * col(invrij2)
        d_atm_ik = a_ - c_ - col(vk) * (-c_) * col(invrik2)
        d_atm_ji = c_ - col(vi) * a_ * col(invrij2)
        d_atm_jj = 2 * a_ - c_ - col(vj) * (a_ * col(invrij2) + (a_ - c_) * col(invrjk2))
        d_atm_jk = -c_ - col(vk) * (a_ - c_) * col(invrjk2)
        d_atm_ki = a_ - col(vi) * c_ * col(invrik2)
        d_atm_kj = -a_ - col(vj) * (c_ - a_) * col(invrjk2)
        d_atm_kk = 2 * c_ - a_ - col(vk) * ((c_ - a_) * col(invrjk2) + c_ * col(invrik2))
        ex = col(atm * d3 / w3)
        d_atm_extra_i = (a_ * col(invrij2) + c_ * col(invrik2)) * ex
        d_atm_extra_j = ((-a_) * col(invrij2) + (c_ - a_) * col(invrjk2)) * ex
        d_atm_extra_k = ((a_ - c_) * col(invrjk2) + (-c_) * col(invrik2)) * ex
        ravg = 0.5 * (rij + rik)
        radial3 = np.exp(-prm.eta3 * (ravg[:, None] - prm.Rs3[None, :]) ** 2)                   # [nt,nl]
        d_radial = radial3 * prm.eta3 * (ravg[:, None] - prm.Rs3[None, :])

        A3 = lambda v: v[:, :, None]      # [nt,3] -> [nt,3,1]
        T1 = lambda v: v[:, None, None]   # [nt]   -> [nt,1,1]
        Lr = radial3[:, None, :]          # [nt,1,nl]
        Ld = d_radial[:, None, :]
        rc = T1(rcutij * rcutik)

        def term(ang, dang, d_ang_vec, d_rad_vec, atm_mix, decay):
            return (T1(dang) * A3(d_ang_vec) * Lr * T1(atm) * rc
                    + T1(ang) * Ld * A3(d_rad_vec) * T1(atm) * rc
                    + T1(ang) * Lr * A3(atm_mix) * w3 * rc
                    + T1(ang) * Lr * A3(decay) * T1(atm))

        mix_i = col(atm_i) * d_atm_ii + col(atm_j) * d_atm_ij + col(atm_k) * d_atm_ik + d_atm_extra_i
        mix_j = col(atm_i) * d_atm_ji + col(atm_j) * d_atm_jj + col(atm_k) * d_atm_jk + d_atm_extra_j
        mix_k = col(atm_i) * d_atm_ki + col(atm_j) * d_atm_kj + col(atm_k) * d_atm_kk + d_atm_extra_k
        dec_i = d_ijdecay * col(rcutik) + col(rcutij) * d_ikdecay
        dec_j = -d_ijdecay * col(rcutik)
        dec_k = -col(rcutij) * d_ikdecay
        out = {}
        for name, dav, drv, mix, dec in (("i", d_angular_d_i, d_radial_d_i, mix_i, dec_i),
                                         ("j", d_angular_d_j, d_radial_d_j, mix_j, dec_j),
                                         ("k", d_angular_d_k, d_radial_d_k, mix_k, dec_k)):
            out[name] = (term(cos_angle, dcos_angle, dav, drv, mix, dec),
                         term(sin_angle, dsin_angle, dav, drv, mix, dec))    # each [nt,3,nl]
        idx = s[:, None] + 2 * larr[None, :]                                   # [nt,nl]
        gi = grad[m, i]                                                        # [n,3,R]
        nt = len(ja)
        for t in range(nt):
            jj, kk = js[ja[t]], js[ka[t]]
            gi[i][:, idx[t]] += out["i"][0][t]
            gi[i][:, idx[t] + 1] += out["i"][1][t]
            gi[jj][:, idx[t]] += out["j"][0][t]
            gi[jj][:, idx[t] + 1] += out["j"][1][t]
            gi[kk][:, idx[t]] += out["k"][0][t]
            gi[kk][:, idx[t] + 1] += out["k"][1][t]
    return grad


def vjp(grad_in, X, types, atomIDs, molIDs, nlist, nneigh, prm, cell=None, inv_cell=None):
    """grad_X [B,n,3] = sum_{i,f} grad_in[m,i,f] * d rep[m,i,f]/dX[m,:,:].
    The reference's backward kernel (fchl_cuda_kernel.cu:1438-1713) evaluates exactly the
    Jacobian terms of :768-1004 and contracts them with grad_in on the fly; here the
    contraction is done on the explicit Jacobian of `jacobian`."""
    J = jacobian(X, types, atomIDs, molIDs, nlist, nneigh, prm, cell, inv_cell)
    return np.einsum("mif,mijxf->mjx", np.asarray(grad_in, dtype=np.float64), J)
