"""Seeded randomized sweeps against the oracle over shapes the fixed cases do not hold:
24 FCHL19 configurations (1-5 species, 1-45 atoms, 1-39 two-body and 1-29 three-body bins,
cutoffs 2-8 A, with and without a given neighbour list) and 12 model configurations (projected
dimension 8-256, 1-8 stacks, 1-3 transforms, both predict routes and the training Gram matrix).
Every configuration is printed before it runs; the sweep stops at the first failure.
QMLL_SWEEP_SEED=<int> in the environment draws another set of configurations (the default set is
what the suite pins)."""
import os

import numpy as np
import pytest
import torch

from oracle import fchl19
from oracle import model as omodel
from oracle import sorf as osorf
from tests import helpers
from tests.test_gpu_kernels import REL_EF, REL_REP, close, dev, gpu_prm, make_batch, oracle_prm, t32, ti32

pytestmark = pytest.mark.gpu

ELEMS = [1, 6, 7, 8, 9, 16, 17]
SEED_SHIFT = int(os.environ.get("QMLL_SWEEP_SEED", "0"))


def test_fchl19_randomized_configurations_vs_oracle():
    from qml_lightning_amd import ops
    rng = np.random.default_rng(20240 + 1000 * SEED_SHIFT)
    done = 0
    while done < 24:
        ns = int(rng.integers(1, 6))
        species = sorted(rng.choice(ELEMS, ns, replace=False).tolist())
        nmol = int(rng.integers(1, 4))
        kw = dict(nRs2=int(rng.integers(1, 40)), nRs3=int(rng.integers(1, 30)), rcut=float(rng.uniform(2.0, 8.0)),
                  eta2=float(rng.uniform(0.1, 1.0)), eta3=float(rng.uniform(0.5, 4.0)),
                  two_body_decay=float(rng.uniform(1.0, 3.0)), three_body_decay=float(rng.uniform(0.3, 1.0)),
                  three_body_weight=float(rng.uniform(5, 20)))
        coords, charges = [], []
        big = done % 8 == 7                              # every eighth configuration: one large molecule
        for _ in range(1 if big else nmol):
            na = int(rng.integers(31, 46)) if big else int(rng.integers(1, 31))
            coords.append(helpers.random_geometry(rng, na, max(3.0, (na * 8.0) ** (1 / 3)), 0.9))
            charges.append(rng.choice(species, na))
        print("fchl sweep %d: species=%s atoms=%s %s" % (done, species, [len(c) for c in coords],
              {k: (round(v, 3) if isinstance(v, float) else v) for k, v in kw.items()}), flush=True)
        prm = oracle_prm(species, **kw)
        X, Z, aid, mid, nat = make_batch(coords, charges)
        cnt, nl = fchl19.neighbours(X, nat, prm.rcut)
        ty = fchl19.element_types(Z, nat, prm.species)
        rep = fchl19.forward(X, ty, aid, mid, nl, cnt, prm)
        J = fchl19.jacobian(X, ty, aid, mid, nl, cnt, prm)
        g = rng.normal(size=rep.shape)
        v = np.einsum("mif,mijxf->mjx", g, J)
        args = (t32(X), ti32(ty), None, None, ti32(aid), ti32(mid), ti32(nat), t32(prm.Rs2), t32(prm.Rs3), gpu_prm(prm))
        for with_list in (False, True):
            lists = {}
            if with_list:
                lists = dict(nlist=ti32(nl if nl.shape[-1] else np.zeros(nl.shape[:-1] + (1,), np.int32)), nneigh=ti32(cnt))
            tag = "sweep %d list=%s " % (done, with_list)
            close(ops.fchl_forward(*args, **lists), rep, REL_REP, tag + "rep")
            if np.abs(v).max() > 0:
                close(ops.fchl_vjp(t32(g), *args, **lists), v, REL_EF, tag + "vjp")
            g_rep, g_J = ops.fchl_jacobian(*args, **lists)
            close(g_rep, rep, REL_REP, tag + "rep of the jacobian kernel")
            if np.abs(J).max() > 0:
                close(g_J, J, REL_REP, tag + "jacobian")
        done += 1


def test_model_randomized_configurations_vs_oracle():
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rng = np.random.default_rng(20241 + 1000 * SEED_SHIFT)
    dims = [8, 16, 32, 64, 128, 256]
    done = 0
    while done < 12:
        ns = int(rng.integers(1, 5))
        species = sorted(rng.choice(ELEMS[:5], ns, replace=False).tolist())
        nmol = int(rng.integers(1, 7))
        npcas = dims[done % 6]                          # every projected dimension twice
        S, T = int(rng.integers(1, 9)), int(rng.integers(1, 4))
        kw = dict(nRs2=int(rng.integers(6, 26)), nRs3=int(rng.integers(4, 22)), rcut=float(rng.uniform(3.0, 7.0)))
        rep = FCHLCuda(species=np.array(species), **kw)
        if rep.get_repsize() < npcas:                   # fewer representation entries than components
            continue
        coords, charges = [], []
        for _ in range(nmol):
            na = int(rng.integers(1, 24))
            coords.append(helpers.random_geometry(rng, na, max(3.0, (na * 8.0) ** (1 / 3)), 0.9))
            charges.append(rng.choice(species, na))
        sigma = float(np.float32(rng.uniform(1.5, 6.0)))
        print("model sweep %d: species=%s atoms=%s npcas=%d S=%d T=%d sigma=%.3f %s"
              % (done, species, [len(c) for c in coords], npcas, S, T, sigma, kw), flush=True)
        red, D, bias, alpha = helpers.model_weights(ns, rep.get_repsize(), npcas, S, T, seed=100 + done)
        D64 = D.astype(np.float64)
        prm = oracle_prm(species, **kw)
        X, Z, aid, mid, nat = make_batch(coords, charges)
        a32 = alpha.astype(np.float32).astype(np.float64)
        E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D64, bias, a32, sigma)
        for fused in (True, False):
            m = HadamardFeaturesModel(rep=rep, elements=np.array(species), ntransforms=T, sigma=sigma, llambda=1e-5,
                                      npcas=npcas, nstacks=S, nbatch_train=3, nbatch_test=4, fused=fused)
            m.reductors, m.Dmat, m.bias = t32(red), t32(D), t32(bias)
            m.alpha = torch.tensor(alpha, device=dev())
            m.is_trained = True
            e, f = m.predict_opt(t32(X), t32(Z), ti32(aid), ti32(mid), ti32(nat))
            # a molecule's energy is a sum of natoms * F terms sqrt(2/F) alpha_f cos(.) that can cancel (one
            # molecule with a few features: |E| a thousandth of the sum of |terms|); fp32 rounds every term, so
            # besides the relative bound the comparison allows four roundings of that sum of magnitudes
            terms = np.sqrt(2.0 / alpha.size) * np.abs(alpha).sum() * max(len(c) for c in coords)
            err = np.abs(e.detach().double().cpu().numpy() - E).max()
            assert err <= REL_EF * np.abs(E).max() + 4 * 2.0 ** -24 * terms, \
                "sweep %d fused=%s energies: max abs err %.3e, |E| max %.3e, sum of |terms| %.3e" % (
                    done, fused, err, np.abs(E).max(), terms)
            if np.abs(F).max() > 0:
                close(f, F, REL_EF, "sweep %d fused=%s forces" % (done, fused))
        # training rows through build_Z_components (batches of 3 molecules) against the oracle's rows
        Et = rng.normal(size=nmol)
        Ft = [rng.normal(size=(len(c), 3)) for c in coords]
        rows, ys = [], []
        for i in range(0, nmol, 3):
            Xb, Zb, ab, mb, nb_ = make_batch(coords[i:i + 3], charges[i:i + 3])
            Fb = np.zeros((len(nb_), Xb.shape[1], 3))
            for k, fo in enumerate(Ft[i:i + 3]):
                Fb[k, :len(fo)] = fo
            r, y = omodel.sorf_training_rows(Xb, Zb, ab, mb, nb_, prm, species, red, D64, bias, sigma, E=Et[i:i + 3], F=Fb)
            rows.append(r)
            ys.append(y)
        ZTZ_ref, ZTy_ref = osorf.gram(np.concatenate(rows), np.concatenate(ys))
        ZTZ, ZTy = m.build_Z_components([np.asarray(c, dtype=np.float32) for c in coords], charges, E=Et, F=Ft,
                                        print_info=False)
        close(ZTZ, ZTZ_ref, 2e-5, "sweep %d ZTZ" % done)      # products of 1e-5-accurate features
        close(ZTy, ZTy_ref, 2e-5, "sweep %d ZTy" % done)
        done += 1
