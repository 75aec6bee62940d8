"""GPU parity: every C-ABI kernel of libqmll against the fp64 oracle on the same seeded
inputs.  Tolerances (stated by the task): 1e-5 relative on representations and features,
1e-4 relative on energies and forces; "relative" is measured against the largest
magnitude of the reference tensor (max-norm), which is how a mixed rtol/atol check such as
the reference's own `np.isclose(..., rtol=1e-4, atol=1e-4)` behaves on O(1..100) data."""
import numpy as np
import pytest
import torch

from oracle import fchl19, model, sorf
from tests import helpers

pytestmark = pytest.mark.gpu

REL_REP = 1e-5
REL_EF = 1e-4


def dev():
    return torch.device("cuda:0")


def close(got, ref, rel, what=""):
    got = got.detach().double().cpu().numpy() if torch.is_tensor(got) else np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = max(np.abs(ref).max(), 1e-30)
    err = np.abs(got - ref).max()
    assert err <= rel * scale, "%s: max abs err %.3e vs scale %.3e (rel %.2e > %.1e)" % (what, err, scale, err / scale, rel)


def t32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=dev())


def ti32(a):
    return torch.tensor(np.asarray(a), dtype=torch.int32, device=dev())


def make_batch(coords, charges):
    """fp32-rounded batch for both sides."""
    coords = [np.asarray(c, dtype=np.float32).astype(np.float64) for c in coords]
    X, Z, aid, mid, nat = model.format_batch(coords, charges)
    return X, Z, aid, mid, nat


def gpu_prm(prm):
    from qml_lightning_amd import ops
    return ops.FchlParams(prm.nspecies, prm.nRs2, prm.nRs3, prm.eta2, prm.eta3, prm.two_body_decay,
                          prm.three_body_weight, prm.three_body_decay, prm.rcut)


def oracle_prm(species, **kw):
    """Oracle parameters whose scalars are exactly the fp32 values the GPU side receives."""
    p = fchl19.FCHLParams(species, **kw)
    for k in ("eta2", "eta3", "two_body_decay", "three_body_weight", "three_body_decay", "rcut"):
        setattr(p, k, float(np.float32(getattr(p, k))))
    p.Rs2 = p.Rs2.astype(np.float32).astype(np.float64)
    p.Rs3 = p.Rs3.astype(np.float32).astype(np.float64)
    return p


CASES = {
    "benzene_c1": lambda: (helpers.benzene_batch(3, 0), [1, 6], {}),
    "aspirin_c2": lambda: (helpers.fixed_composition_batch(helpers.ASPIRIN, 3, 1), [1, 6, 8], {}),
    "ragged_c3": lambda: (helpers.ragged_batch(12, 2), [1, 6, 7, 8, 9], {}),
    "flexible_c4": lambda: (helpers.fixed_composition_batch(helpers.C12H12N2O, 2, 3, sigma=0.15), [1, 6, 7, 8], {}),
    # 40 atoms: more neighbours than the backward kernel's per-triple table holds (its other path)
    "big_molecule": lambda: (helpers.fixed_composition_batch(np.array([6] * 14 + [1] * 20 + [8] * 6), 1, 11, box=8.0),
                             [1, 6, 8], {}),
    # 72 atoms, up to 60 neighbours: more candidates than one wavefront pass stages and more
    # triples (1770) than the forward kernel's table holds (its chunked path)
    "many_atoms": lambda: (helpers.fixed_composition_batch(np.array([6] * 26 + [1] * 36 + [8] * 10), 1, 12, box=9.0),
                           [1, 6, 8], {}),
    "short_cutoff": lambda: (helpers.fixed_composition_batch(helpers.ASPIRIN, 2, 5), [1, 6, 8],
                             {"rcut": 3.1, "nRs2": 7, "nRs3": 5}),
    # more radial bins than a wavefront has lanes: several bin blocks per lane, one triple per round
    "many_bins": lambda: (helpers.fixed_composition_batch(helpers.ASPIRIN, 2, 6), [1, 6, 8], {"nRs2": 80, "nRs3": 70}),
    # 33 to 64 three-body bins: one triple per round, one bin block
    "forty_bins": lambda: (helpers.fixed_composition_batch(helpers.ASPIRIN, 1, 7), [1, 6, 8], {"nRs2": 33, "nRs3": 40}),
    # narrow three-body Gaussians: sqrt(eta3 log2 e) rcut / 2 = 12.5 is beyond what the backward kernel's
    # form about the middle of the grid takes (10), so its plain radial loop runs
    "sharp_radial": lambda: (helpers.fixed_composition_batch(helpers.ASPIRIN, 2, 8), [1, 6, 8], {"eta3": 12.0}),
}


@pytest.mark.parametrize("case", list(CASES))
def test_neighbours_and_types(case):
    from qml_lightning_amd import ops
    (coords, charges), species, kw = CASES[case]()
    prm = oracle_prm(species, **kw)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    cnt, nl = fchl19.neighbours(X, nat, prm.rcut)
    g_cnt = ops.num_neighbours(t32(X), ti32(nat), prm.rcut)
    assert (g_cnt.cpu().numpy() == cnt).all()           # integer work: bit exact
    g_nl = ops.neighbour_list(t32(X), ti32(nat), int(cnt.max()), prm.rcut)
    assert (g_nl.cpu().numpy() == nl).all()
    ty = fchl19.element_types(Z, nat, prm.species)
    g_ty = ops.element_types(t32(X), t32(Z), ti32(nat), t32(prm.species))
    assert (g_ty.cpu().numpy() == ty).all()


def test_element_types_unknown_species_is_minus_one():
    from qml_lightning_amd import ops
    Z = t32([[6, 9, 1, 0]])
    ty = ops.element_types(torch.zeros(1, 4, 3, device=dev()), Z, ti32([3]), t32([1, 6]))
    assert ty.cpu().tolist() == [[1, -1, 0, 0]]


@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("with_list", [False, True])
def test_fchl_forward_vjp_jacobian(case, with_list):
    from qml_lightning_amd import ops
    (coords, charges), species, kw = CASES[case]()
    prm = oracle_prm(species, **kw)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    cnt, nl = fchl19.neighbours(X, nat, prm.rcut)
    ty = fchl19.element_types(Z, nat, prm.species)
    rep = fchl19.forward(X, ty, aid, mid, nl, cnt, prm)
    J = fchl19.jacobian(X, ty, aid, mid, nl, cnt, prm)
    g = np.random.default_rng(7).normal(size=rep.shape)
    v = np.einsum("mif,mijxf->mjx", g, J)

    gp = gpu_prm(prm)
    lists = dict(nlist=ti32(nl), nneigh=ti32(cnt)) if with_list else {}
    args = (t32(X), ti32(ty), None, None, ti32(aid), ti32(mid), ti32(nat), t32(prm.Rs2), t32(prm.Rs3), gp)
    g_rep = ops.fchl_forward(*args, **lists)
    close(g_rep, rep, REL_REP, "rep")
    # padded slots stay exactly zero
    for m in range(len(nat)):
        assert (g_rep[m, nat[m]:] == 0).all()
    g_v = ops.fchl_vjp(t32(g), *args, **lists)
    close(g_v, v, REL_EF, "vjp")
    g_rep2, g_J = ops.fchl_jacobian(*args, **lists)
    close(g_rep2, rep, REL_REP, "rep from jacobian kernel")
    close(g_J, J, REL_REP, "jacobian")


def test_fchl_periodic_cell():
    from qml_lightning_amd import ops
    prm = oracle_prm([1, 8], nRs2=6, nRs3=4, rcut=2.4)
    rng = np.random.default_rng(8)
    cellm = np.array([[5.0, 0.0, 0.0], [0.5, 5.2, 0.0], [0.2, 0.3, 4.9]]).T.astype(np.float32).astype(np.float64)
    inv = np.linalg.inv(cellm).astype(np.float32).astype(np.float64)
    coords = [helpers.random_geometry(rng, 6, 4.8, 1.2), helpers.random_geometry(rng, 5, 4.8, 1.2)]
    ch = [np.array([8, 1, 1, 8, 1, 1]), np.array([8, 1, 1, 1, 8])]
    X, Z, aid, mid, nat = make_batch(coords, ch)
    cell = np.stack([cellm, cellm])
    icell = np.stack([inv, inv])
    cnt, nl = fchl19.neighbours(X, nat, prm.rcut, cell, icell)
    ty = fchl19.element_types(Z, nat, prm.species)
    rep = fchl19.forward(X, ty, aid, mid, nl, cnt, prm, cell, icell)
    J = fchl19.jacobian(X, ty, aid, mid, nl, cnt, prm, cell, icell)
    g_cnt = ops.num_neighbours(t32(X), ti32(nat), prm.rcut, t32(cell), t32(icell))
    assert (g_cnt.cpu().numpy() == cnt).all()
    g_nl = ops.neighbour_list(t32(X), ti32(nat), int(cnt.max()), prm.rcut, t32(cell), t32(icell))
    assert (g_nl.cpu().numpy() == nl).all()
    args = (t32(X), ti32(ty), t32(cell), t32(icell), ti32(aid), ti32(mid), ti32(nat), t32(prm.Rs2), t32(prm.Rs3),
            gpu_prm(prm))
    close(ops.fchl_forward(*args), rep, REL_REP, "pbc rep")
    g = np.random.default_rng(1).normal(size=rep.shape)
    close(ops.fchl_vjp(t32(g), *args), np.einsum("mif,mijxf->mjx", g, J), REL_EF, "pbc vjp")
    close(ops.fchl_jacobian(*args)[1], J, REL_REP, "pbc jacobian")


def test_fchl_forward_refuses_more_radial_bins_than_it_handles():
    from qml_lightning_amd import ops
    prm = oracle_prm([1, 6], nRs3=300)
    args = (t32(np.zeros((1, 2, 3))), ti32([[1, 0]]), None, None, ti32([0, 1]), ti32([0, 0]), ti32([2]), t32(prm.Rs2),
            t32(prm.Rs3), gpu_prm(prm))
    with pytest.raises(RuntimeError, match="nRs3"):
        ops.fchl_forward(*args)


def test_fchl_single_atom_and_empty_batch():
    from qml_lightning_amd import ops
    prm = oracle_prm([1, 6])
    args = (t32(np.zeros((1, 1, 3))), ti32([[1]]), None, None, ti32([0]), ti32([0]), ti32([1]), t32(prm.Rs2),
            t32(prm.Rs3), gpu_prm(prm))
    rep = ops.fchl_forward(*args)
    assert rep.shape == (1, 1, prm.repsize) and (rep == 0).all()
    empty = (torch.zeros(0, 4, 3, device=dev()), torch.zeros(0, 4, dtype=torch.int32, device=dev()), None, None,
             ti32([]), ti32([]), ti32([]), t32(prm.Rs2), t32(prm.Rs3), gpu_prm(prm))
    assert ops.fchl_forward(*empty).shape == (0, 4, prm.repsize)


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("d", [2, 8, 32, 64, 128, 256, 512, 1024])
@pytest.mark.parametrize("T", [1, 2])
def test_sorf_forward_and_adjoint(d, T):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d + T)
    A, S = 9, 5
    x = rng.normal(size=(A, d)).astype(np.float32)
    D = np.where(rng.uniform(-1, 1, (T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    norm = float(np.float32(np.sqrt(d) / 2.0))
    c = sorf.sorf_coefficients(x, D, norm)
    close(ops.sorf_forward(t32(x), t32(D), norm, T), c, REL_REP, "sorf forward")
    y = rng.normal(size=(A, S, d)).astype(np.float32)
    close(ops.sorf_adjoint(t32(y), t32(D), norm, T), sorf.sorf_adjoint(y, D, norm), REL_REP, "sorf adjoint")


def test_sorf_many_stacks_full_size():
    """npcas 128 x nstacks 128 (16384 features) and 256 x 128 (32768), the benchmark shapes."""
    from qml_lightning_amd import ops
    for d, S in ((128, 128), (256, 128)):
        rng = np.random.default_rng(S)
        x = rng.normal(size=(4, d)).astype(np.float32)
        D = np.where(rng.uniform(-1, 1, (1, S, d)) > 0, 1.0, -1.0).astype(np.float32)
        close(ops.sorf_forward(t32(x), t32(D), 5.65, 1), sorf.sorf_coefficients(x, D, np.float32(5.65)), REL_REP)


def test_sorf_rejects_non_power_of_two():
    from qml_lightning_amd import ops
    with pytest.raises(RuntimeError, match="power of 2"):
        ops.sorf_forward(torch.zeros(2, 12, device=dev()), torch.ones(1, 2, 12, device=dev()), 1.0, 1)


def test_ops_reject_cpu_tensors():
    from qml_lightning_amd import ops
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ops.sorf_forward(torch.zeros(2, 8), torch.ones(1, 2, 8), 1.0, 1)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ops.num_neighbours(torch.zeros(1, 2, 3), torch.ones(1, dtype=torch.int32), 2.0)


@pytest.mark.parametrize("scale", [1.0, 30.0, 3000.0])
def test_cos_features_forward_backward_sin(scale):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(3)
    A, F, nmol = 70, 600, 9
    c = (rng.normal(size=(A, F)) * scale).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, F).astype(np.float32)
    idx = np.sort(rng.integers(0, nmol, A)).astype(np.int32)
    # the argument the kernel sees is the fp32 sum c+b
    carg = (c + b[None, :]).astype(np.float32).astype(np.float64)
    zero_b = np.zeros(F)
    Zref = sorf.cos_features(carg, zero_b, idx, nmol)
    close(ops.cos_features(t32(c), t32(b), nmol, ti32(idx)), Zref, REL_REP, "cos features f32")
    Z64 = torch.ones(nmol, F, dtype=torch.float64, device=dev())
    ops.cos_features(t32(c), t32(b), nmol, ti32(idx), out=Z64)
    close(Z64 - 1.0, Zref, REL_REP, "cos features f64 accumulate")
    g = rng.normal(size=(nmol, F)).astype(np.float32)
    close(ops.cos_features_backward(t32(g), t32(c), t32(b), nmol, ti32(idx)),
          sorf.cos_features_backward(g, carg, zero_b, idx), REL_REP, "cos backward")
    out = torch.empty(A, F, dtype=torch.float64, device=dev())
    close(ops.sin_coeffs(t32(c), t32(b), out), sorf.sin_coeffs(carg, zero_b), REL_REP, "sin coeffs")


@pytest.mark.parametrize("F", [64, 63, 1030])
def test_cos_features_unsorted_molecule_index(F):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(4)
    A, nmol = 50, 7
    c = rng.normal(size=(A, F)).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, F).astype(np.float32)
    idx = rng.integers(0, nmol, A).astype(np.int32)
    carg = (c + b[None, :]).astype(np.float32).astype(np.float64)
    close(ops.cos_features(t32(c), t32(b), nmol, ti32(idx)), sorf.cos_features(carg, np.zeros(F), idx, nmol), REL_REP)
    g = rng.normal(size=(nmol, F)).astype(np.float32)
    close(ops.cos_features_backward(t32(g), t32(c), t32(b), nmol, ti32(idx)),
          sorf.cos_features_backward(g, carg, np.zeros(F), idx), REL_REP, "cos backward, odd sizes")
    out = torch.empty(A, F, dtype=torch.float64, device=dev())
    close(ops.sin_coeffs(t32(c), t32(b), out), sorf.sin_coeffs(carg, np.zeros(F)), REL_REP, "sin coeffs, odd sizes")


def test_segment_offsets_table_and_validity_flag():
    """Segment table of an ascending molecule index (== numpy searchsorted); the flag in the
    last entry is raised for an index that is not ascending or leaves [0, nmol)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(8)
    for nmol, A in ((1, 5), (7, 40), (300, 2500), (50, 3)):       # the last: mostly empty molecules
        idx = np.sort(rng.integers(0, nmol, A)).astype(np.int32)
        seg = ops.segment_offsets(ti32(idx), nmol).cpu().numpy()
        assert seg[nmol + 1] == 0
        assert (seg[:nmol + 1] == np.searchsorted(idx, np.arange(nmol + 1), side="left")).all()
    idx = np.array([0, 1, 1, 3, 2, 4], dtype=np.int32)            # not ascending
    assert ops.segment_offsets(ti32(idx), 5).cpu().numpy()[6] != 0
    idx = np.array([0, 1, 5], dtype=np.int32)                     # 5 is outside [0, 5)
    assert ops.segment_offsets(ti32(idx), 5).cpu().numpy()[6] != 0
    idx = np.array([-1, 0, 1], dtype=np.int32)
    assert ops.segment_offsets(ti32(idx), 5).cpu().numpy()[6] != 0


@pytest.mark.parametrize("d,S,T", [(16, 3, 1), (128, 8, 1), (64, 4, 2), (256, 4, 1)])
def test_derivative_features(d, S, T):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d)
    A, n, nmol = 11, 5, 4
    u = rng.normal(size=(A, n, 3, d)).astype(np.float32)
    u[2, 3] = 0.0                                    # a target that is not a neighbour
    D = np.where(rng.uniform(-1, 1, (T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    cd = rng.normal(size=(A, S * d))
    idx = np.sort(rng.integers(0, nmol, A)).astype(np.int32)
    norm = 2.5
    ref = sorf.derivative_features(cd, norm, idx, u, D, nmol)
    for molecule_major in (False, True):
        G = torch.ones(nmol, n, 3, S * d, dtype=torch.float64, device=dev())      # accumulates in place
        ops.derivative_features(torch.tensor(cd, device=dev()), norm, t32(D), t32(u), ti32(idx), G,
                                molecule_major=molecule_major)
        close(G - 1.0, ref, REL_REP, "derivative features, molecule_major=%s" % molecule_major)


@pytest.mark.parametrize("d,S,T,ne", [(64, 5, 2, 3), (128, 17, 1, 3), (128, 8, 1, 1), (256, 6, 1, 5), (128, 4, 3, 8)])
def test_derivative_features_all_elements_in_one_launch(d, S, T, ne):
    """The typed entry (every element of the batch in one launch) against the oracle summed over the
    elements, with molecules that lack an element, more atoms in a molecule than one pass holds,
    rows that are not neighbours, and G either holding earlier contributions (add) or garbage
    (overwrite)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d + S + ne)
    n, nmol = 7, 6
    norm = 1.75
    ref = np.zeros((nmol, n, 3, S * d))
    items = []
    for e in range(ne):
        A = int(rng.integers(1, 30)) if e else 23          # the first element: up to 23 atoms in few molecules
        idx = np.sort(rng.integers(0, nmol if e else 2, A)).astype(np.int32)
        u = rng.normal(size=(A, n, 3, d)).astype(np.float32)
        u[rng.integers(0, A), rng.integers(0, n)] = 0.0
        D = np.where(rng.uniform(-1, 1, (T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
        cd = rng.normal(size=(A, S * d))
        ref += sorf.derivative_features(cd, norm, idx, u, D, nmol)
        items.append((torch.tensor(cd, device=dev()), t32(D), t32(u), ti32(idx)))
    G = torch.full((nmol, n, 3, S * d), 0.5, dtype=torch.float64, device=dev())
    ops.derivative_features_typed(items, norm, G)
    close(G - 0.5, ref, REL_REP, "typed derivative features")
    G = torch.full((nmol, n, 3, S * d), float("nan"), dtype=torch.float64, device=dev())
    ops.derivative_features_typed(items, norm, G, overwrite=True)
    close(G, ref, REL_REP, "typed derivative features, overwrite")
    ops.derivative_features_typed([], norm, G, overwrite=True)
    assert float(G.abs().max()) == 0.0
    with pytest.raises(RuntimeError):
        ops.derivative_features_typed(items * 9, norm, G)          # more than 8 elements


@pytest.mark.parametrize("d,S,T", [(8, 3, 1), (64, 5, 2), (128, 16, 1), (128, 9, 2), (128, 5, 3), (256, 8, 1), (256, 6, 2),
                                   (512, 4, 1), (512, 3, 2)])
def test_fused_energy_matches_two_op_chain(d, S, T):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d + S)
    A = 13
    F = S * d
    x = rng.normal(size=(A, d)).astype(np.float32)
    D = np.where(rng.uniform(-1, 1, (T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, F).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    norm = float(np.float32(np.sqrt(d) / 2.0))
    c = sorf.sorf_coefficients(x, D, norm).reshape(A, F)
    e_ref = (np.sqrt(2.0 / F) * np.cos(c + b) * alpha).sum(1)
    gc = -np.sqrt(2.0 / F) * np.sin(c + b) * alpha
    gx_ref = sorf.sorf_adjoint(gc.reshape(A, S, d), D, norm)
    perm = rng.permutation(A + 3)[:A].astype(np.int32)
    e_slots = torch.zeros(A + 3, device=dev())
    gx = ops.sorf_energy_fused(t32(x), t32(D), t32(b), t32(alpha), ti32(perm), norm, T, e_slots)
    close(e_slots[torch.tensor(perm.astype(np.int64), device=dev())], e_ref, REL_EF, "fused energy")
    close(gx, gx_ref, REL_EF, "fused gradient")
    e2 = torch.zeros(A, device=dev())
    assert ops.sorf_energy_fused(t32(x), t32(D), t32(b), t32(alpha), None, norm, T, e2, with_grad=False) is None
    close(e2, e_ref, REL_EF, "fused energy only")


@pytest.mark.parametrize("d", [64, 128, 256])
def test_fused_energy_large_arguments(d):
    """Arguments of hundreds to tens of thousands of radians (beyond the range the sine / cosine
    unit reduces itself).  A one-hot input makes the transform exact in fp32 (every coefficient is
    +-x_k times the scale), so the fp32 argument the kernel forms is known: one rounding of
    x * (scale / 2 pi), one fused multiply-add with the bias, in revolutions.  Energies and
    gradients must match the fp64 cosine / sine of exactly that argument."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d)
    S = 5
    F = S * d
    norm = np.float32(8.0)
    # the kernel's scale is normalisation * 2^(-log2(d) / 2) in fp32 (the transform itself is unnormalised)
    scale = np.float32(norm * np.float32(2.0 ** (-0.5 * np.log2(d))))
    mags = (np.array([0.1, 8.0, 56.0, 320.0, 1280.0, 7200.0, 36000.0]) / scale).astype(np.float32)   # coefficients in radians
    A = len(mags)
    hot = rng.integers(0, d, A)
    x = np.zeros((A, d), dtype=np.float32)
    x[np.arange(A), hot] = mags * np.where(rng.uniform(size=A) > 0.5, 1, -1)
    D = np.where(rng.uniform(-1, 1, (1, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, F).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    inv2pi = np.float32(0.15915494309189535)
    xs = np.float32(scale * inv2pi)
    from scipy.linalg import hadamard
    H = hadamard(d).astype(np.float64)
    u = np.zeros((A, F))
    for a_ in range(A):
        w32 = np.float32(x[a_, hot[a_]] * xs)                                    # one rounding
        for s_ in range(S):
            w = H[:, hot[a_]] * float(D[0, s_, hot[a_]]) * float(w32)            # exact: +-w32
            u[a_, s_ * d:(s_ + 1) * d] = (w + b[s_ * d:(s_ + 1) * d].astype(np.float64) * float(inv2pi)).astype(np.float32)
    arg = 2.0 * np.pi * u
    assert np.abs(arg).max() > 32000 and (np.abs(arg).max(axis=1) < 7.0).any()
    nf = np.sqrt(2.0 / F)
    e_ref = (nf * np.cos(arg) * alpha).sum(1)
    gc = -nf * np.sin(arg) * alpha
    gx_ref = sorf.sorf_adjoint(gc.reshape(A, S, d), D, float(norm))
    e = torch.zeros(A, device=dev())
    gx = ops.sorf_energy_fused(t32(x), t32(D), t32(b), t32(alpha), None, float(norm), 1, e)
    e_scale = nf * np.abs(alpha).sum()                 # what the per-atom sums are made of
    assert np.abs(e.double().cpu().numpy() - e_ref).max() <= 2e-6 * e_scale
    for a_ in range(A):                                # per atom: the gradient scales differ by orders of magnitude
        close(gx[a_], gx_ref[a_], REL_EF, "fused gradient, |arg| up to %.0f" % np.abs(arg[a_]).max())


@pytest.mark.parametrize("bias_scale", [1.0, 500.0])
def test_sorted_fused_energy_with_the_bias_bound_equals_the_checked_form(bias_scale):
    """The element-sorted entry gets the largest |bias| and decides once per atom, from sum |x| and that
    bound, whether any argument can leave the range the sine / cosine unit reduces itself; the
    unsorted entry inspects every argument.  Atoms with small and with huge coefficients side by side
    (the decision is per wavefront of four atoms), and a bias of thousands of radians: same results."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(11)
    d, S, A = 128, 6, 37
    F = S * d
    x = rng.normal(size=(A, d)).astype(np.float32)
    x[5] *= 400.0                      # arguments of thousands of radians in the middle of a tile
    x[20:24] *= 3000.0                 # a whole wavefront beyond the range
    x[30] = 0.0
    D = np.where(rng.uniform(-1, 1, (1, 1, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = (rng.uniform(0, 2 * np.pi, (1, F)) * bias_scale).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    types = np.zeros(A, dtype=np.int32)
    ss, off = ops.sort_by_type(ti32(types), ti32(np.arange(A, dtype=np.int32)), 1)
    e_ref = torch.zeros(A, device=dev())
    g_ref = ops.sorf_energy_fused(t32(x), t32(D[0]), t32(b[0]), t32(alpha), None, 2.5, 1, e_ref)
    e, g = ops.sorf_energy_sorted(t32(x), off, ss, t32(D), t32(b), t32(alpha), 2.5, 1, A)
    # the two entries run the same arithmetic per atom (the compiler may contract the two instances of
    # the stack differently: last bits); only the decision differs
    assert (e - e_ref).abs().max() <= 1e-6 * e_ref.abs().max()
    for a_ in range(A):                # per atom: the gradient scales differ by orders of magnitude
        assert (g[a_] - g_ref[a_]).abs().max() <= 2e-6 * g_ref[a_].abs().max() + 1e-30, a_


def test_typed_fused_energy_matches_per_element_calls():
    """All elements in one launch == one fused call per element (slots, padded rows, unknown types)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(9)
    ne, d, S, T, N = 3, 64, 6, 1, 40
    F = S * d
    x_all = rng.normal(size=(N, ne * d)).astype(np.float32)
    types = rng.integers(-1, ne, N).astype(np.int32)              # -1: element not in the model
    slots = np.sort(rng.choice(N, size=29, replace=False)).astype(np.int32)   # the rest are padding
    D = np.where(rng.uniform(-1, 1, (ne, T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, (ne, F)).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    norm = 3.0
    e, gx = ops.sorf_energy_typed(t32(x_all), ti32(types), ti32(slots), t32(D), t32(b), t32(alpha), norm, T)
    e_ref = np.zeros(N)
    g_ref = np.zeros((N, ne * d))
    for s_ in slots:
        t_ = types[s_]
        if t_ < 0:
            continue
        xs = x_all[s_, t_ * d:(t_ + 1) * d][None, :]
        c = sorf.sorf_coefficients(xs, D[t_], norm).reshape(1, F)
        e_ref[s_] = (np.sqrt(2.0 / F) * np.cos(c + b[t_]) * alpha).sum()
        gc = -np.sqrt(2.0 / F) * np.sin(c + b[t_]) * alpha
        g_ref[s_, t_ * d:(t_ + 1) * d] = sorf.sorf_adjoint(gc.reshape(1, S, d), D[t_], norm)[0]
    close(e, e_ref, REL_EF, "typed energies")
    close(gx, g_ref, REL_EF, "typed gradients")


@pytest.mark.parametrize("A,N,ne", [(0, 4, 3), (1, 1, 1), (255, 300, 2), (256, 256, 5), (1000, 1400, 4),
                                    (70001, 70001, 3)])
def test_sort_by_type_is_a_stable_counting_sort(A, N, ne):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(A + ne)
    types = rng.integers(-1, ne + 1, N).astype(np.int32)     # -1 and ne: elements the model does not know
    slots = np.sort(rng.choice(N, size=A, replace=False)).astype(np.int32)
    got_slots, got_off = ops.sort_by_type(ti32(types), ti32(slots), ne)
    t_atoms = types[slots]
    known = (t_atoms >= 0) & (t_atoms < ne)
    order = np.argsort(t_atoms[known], kind="stable")
    ref = slots[known][order]
    off = np.concatenate([[0], np.cumsum(np.bincount(t_atoms[known], minlength=ne))])
    assert np.array_equal(got_off.cpu().numpy(), off)
    got = got_slots.cpu().numpy()
    assert np.array_equal(got[:len(ref)], ref)
    assert (got[len(ref):] == 0).all()


@pytest.mark.parametrize("B,n,ne", [(1, 21, 3), (0, 5, 2), (48, 21, 3), (49, 21, 3), (300, 29, 5), (4, 1, 1)])
def test_sort_atoms_by_type_equals_the_sort_of_their_slots(B, n, ne):
    """The sort that builds slot = molIDs * n + atomIDs itself (one launch up to 1024 atoms, the slots
    through the workspace beyond) against `sort_by_type` of the explicit slots, on ragged batches with
    elements the model does not know."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(B * 31 + n)
    counts = rng.integers(1, n + 1, B)
    aid = np.concatenate([np.arange(c) for c in counts]).astype(np.int32) if B else np.zeros(0, np.int32)
    mid = np.repeat(np.arange(B), counts).astype(np.int32)
    types = rng.integers(-1, ne + 1, B * n).astype(np.int32) if B else np.zeros(0, np.int32)
    got_s, got_o = ops.sort_atoms_by_type(ti32(types), ti32(aid), ti32(mid), n, ne)
    ref_s, ref_o = ops.sort_by_type(ti32(types), ti32(mid * n + aid), ne)
    assert torch.equal(got_o, ref_o)
    total = int(ref_o[-1].item())
    assert torch.equal(got_s[:total], ref_s[:total]) and (got_s[total:] == 0).all()


@pytest.mark.parametrize("R,d,ne,N,A", [(312, 128, 3, 500, 500), (75, 64, 2, 90, 61), (720, 256, 5, 700, 523),
                                        (10, 8, 1, 5, 3), (496, 256, 4, 130, 130),
                                        # small batches: one workgroup per atom instead of matrix tiles
                                        (312, 128, 3, 100, 100), (312, 128, 3, 140, 128), (312, 128, 3, 1300, 1201),
                                        (312, 64, 2, 40, 21), (720, 256, 5, 60, 33), (76, 20, 2, 30, 17),
                                        (312, 128, 3, 3000, 2900), (312, 64, 3, 2600, 2500), (312, 128, 3, 1300, 1260),
                                        # the last size the small kernels take (eight atoms per workgroup), and
                                        # large enough for the matrix tiles at 128 and 64 components (rows in
                                        # registers in the transpose); 720 x 256: four atoms per workgroup fit in LDS
                                        (312, 128, 3, 4200, 4096), (312, 128, 3, 5000, 4900), (312, 64, 3, 4600, 4500),
                                        (720, 256, 5, 1100, 1000), (720, 256, 5, 1300, 1200)])
def test_project_typed_forward_and_backward(R, d, ne, N, A):
    """Element-sorted projection against fp64 matmul, both directions: gathered rows, tiles that end
    inside a type, R not a multiple of 4, unknown elements; the matrix-core kernels and the
    one-workgroup-per-atom kernels of small batches."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(R + d)
    rep = rng.normal(size=(N, R)).astype(np.float32)
    red = rng.normal(size=(ne, R, d)).astype(np.float32)
    types = rng.integers(0, ne, N).astype(np.int32)
    types[rng.choice(N, size=max(1, N // 20), replace=False)] = -1
    slots = np.sort(rng.choice(N, size=A, replace=False)).astype(np.int32)
    ss, off = ops.sort_by_type(ti32(types), ti32(slots), ne)
    x = ops.project_typed(t32(rep), ss, off, t32(red))
    ssn = ss.cpu().numpy()
    total = int(off[-1].item())
    x_ref = np.stack([rep[s_].astype(np.float64) @ red[types[s_]].astype(np.float64) for s_ in ssn[:total]]) \
        if total else np.zeros((0, d))
    close(x[:total], x_ref, REL_REP, "projection")
    gx = rng.normal(size=(A, d)).astype(np.float32)
    g = ops.project_typed_backward(t32(gx), ss, off, t32(red), ti32(types), N)
    g_ref = np.zeros((N, R))
    for a_, s_ in enumerate(ssn[:total]):
        g_ref[s_] = gx[a_].astype(np.float64) @ red[types[s_]].astype(np.float64).T
    close(g, g_ref, REL_REP, "projection transpose")
    # unlisted and unknown rows are exactly zero
    mask = np.ones(N, bool)
    mask[ssn[:total]] = False
    assert (g.cpu().numpy()[mask] == 0).all()


@pytest.mark.parametrize("R,d,ne,N,A,group", [(312, 128, 3, 80, 61, 63), (53, 20, 2, 40, 40, 7), (312, 128, 3, 600, 600, 9),
                                               (64, 256, 4, 30, 17, 36)])
def test_project_typed_rows_projects_a_group_of_rows_per_atom(R, d, ne, N, A, group):
    """`group` rows per slot (the 3n derivative rows of an atom) through the typed product, against
    fp64 matmul of each atom's rows with its element's matrix: tiles that start and end inside an atom's
    group and inside a type, an element without atoms, unknown elements, R not a multiple of 4."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(R + d + group)
    rows = rng.normal(size=(N * group, R)).astype(np.float32)
    red = rng.normal(size=(ne, R, d)).astype(np.float32)
    types = rng.integers(0, ne, N).astype(np.int32)
    if ne > 2:
        types[types == 1] = 0                      # no atom of element 1
    types[rng.choice(N, size=max(1, N // 20), replace=False)] = -1
    slots = np.sort(rng.choice(N, size=A, replace=False)).astype(np.int32)
    ss, off = ops.sort_by_type(ti32(types), ti32(slots), ne)
    x = ops.project_typed_rows(t32(rows), ss, off, t32(red), group)
    assert tuple(x.shape) == (A * group, d)
    ssn, total = ss.cpu().numpy(), int(off[-1].item())
    assert total > 0
    r3 = rows.reshape(N, group, R).astype(np.float64)
    x_ref = np.concatenate([r3[s_] @ red[types[s_]].astype(np.float64) for s_ in ssn[:total]])
    close(x[:total * group], x_ref, REL_REP, "projection of grouped rows")
    # group = 1 is the plain projection
    x1 = ops.project_typed_rows(t32(rows[:N]), ss, off, t32(red), 1)
    close(x1[:total], ops.project_typed(t32(rows[:N]), ss, off, t32(red))[:total].double().cpu().numpy(), REL_REP,
          "one row per atom")


@pytest.mark.parametrize("rscale,uscale", [(1.0, 1.0), (1e-6, 1e3), (3e4, 1e-4), (1e10, 1e-12), (1e-36, 1.0), (0.0, 1.0)])
def test_projection_on_the_fp16_matrix_cores_over_operand_scales(rscale, uscale):
    """The projection of a large batch and the transposed projection multiply on the fp16 matrix cores with
    every fp32 operand split in two fp16 parts behind powers of two (per chunk of the tile, per wavefront,
    per row of the matrix): operands far outside fp16's range, rows that are small beside their tile's
    largest, an operand whose power of two would not be a float, a zero operand; against fp64 at fp32
    accuracy (2e-6 of the largest entry)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(11)
    R, d, ne, N = 312, 128, 2, 66000          # 516 tiles of 128 rows: the large-batch kernel
    rep = torch.randn(N, R, device=dev(), generator=torch.Generator(device=dev()).manual_seed(3)) * rscale
    rep[::7] *= 1e-3                           # rows that are small beside the others of their tile
    rep[5::11, 100:] = 0.0
    red = (rng.normal(size=(ne, R, d)) * uscale).astype(np.float32)
    red[1, :, 64:] *= 1e-2
    types = torch.tensor(rng.integers(0, ne, N).astype(np.int32), device=dev())
    ss, off = ops.sort_by_type(types, torch.arange(N, dtype=torch.int32, device=dev()), ne)
    x = ops.project_typed(rep, ss, off, t32(red))
    pick = torch.tensor(rng.choice(N, size=3000, replace=False), device=dev())
    ssl = ss.long()[pick]
    U = torch.tensor(red, device=dev()).double()[types.long()[ssl]]
    x_ref = torch.einsum('ar,ard->ad', rep[ssl].double(), U)
    scale = float(x_ref.abs().max())
    assert float((x[pick].double() - x_ref).abs().max()) <= 2e-6 * max(scale, 1e-300)
    # rows small beside their tile's largest keep their own accuracy down to 2^-17 of it
    small = (ssl % 7 == 0)
    if rscale > 1e-30 and bool(small.any()):      # below, the small rows are fp32 subnormals
        ref_s = x_ref[small]
        assert float((x[pick][small].double() - ref_s).abs().max()) <= 1e-5 * float(ref_s.abs().max())
    gx = torch.randn(N, d, device=dev(), generator=torch.Generator(device=dev()).manual_seed(4)) * rscale
    g = ops.project_typed_backward(gx, ss, off, t32(red), types, N)
    g_ref = torch.einsum('ad,ard->ar', gx[pick].double(), U)
    assert float((g[ssl].double() - g_ref).abs().max()) <= 2e-6 * max(float(g_ref.abs().max()), 1e-300)


@pytest.mark.parametrize("T,S,d", [(1, 6, 64), (2, 6, 64), (1, 64, 128), (1, 70, 64), (2, 64, 64)])
def test_sorted_fused_energy_matches_per_atom_oracle(T, S, d):
    """Element-sorted rows through the fused kernel: energies land in the atoms' slots, the
    gradient stays in sorted order, rows past the last known atom give zero.  From 64 stacks on, a
    batch this small runs with sixteen wavefronts per workgroup sharing out the stacks."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(19)
    ne, N, A = 3, 50, 37
    F = S * d
    types = rng.integers(-1, ne, N).astype(np.int32)
    slots = np.sort(rng.choice(N, size=A, replace=False)).astype(np.int32)
    ss, off = ops.sort_by_type(ti32(types), ti32(slots), ne)
    ssn, total = ss.cpu().numpy(), int(off[-1].item())
    x = rng.normal(size=(A, d)).astype(np.float32)
    D = np.where(rng.uniform(-1, 1, (ne, T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, (ne, F)).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    norm = 3.0
    e, gx = ops.sorf_energy_sorted(t32(x), off, ss, t32(D), t32(b), t32(alpha), norm, T, N)
    e_ref = np.zeros(N)
    g_ref = np.zeros((A, d))
    for a_ in range(total):
        t_ = types[ssn[a_]]
        c = sorf.sorf_coefficients(x[a_][None, :], D[t_], norm).reshape(1, F)
        e_ref[ssn[a_]] = (np.sqrt(2.0 / F) * np.cos(c + b[t_]) * alpha).sum()
        gc = -np.sqrt(2.0 / F) * np.sin(c + b[t_]) * alpha
        g_ref[a_] = sorf.sorf_adjoint(gc.reshape(1, S, d), D[t_], norm)[0]
    close(e, e_ref, REL_EF, "sorted energies")
    close(gx, g_ref, REL_EF, "sorted gradients")
    assert (gx[total:] == 0).all()
    e2, g2 = ops.sorf_energy_sorted(t32(x), off, ss, t32(D), t32(b), t32(alpha), norm, T, N, with_grad=False)
    assert g2 is None
    close(e2, e_ref, REL_EF, "sorted energies only")


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("M,F", [(37, 24), (300, 128), (1000, 384), (513, 200), (40, 2176), (33, 3000), (20, 4224),
                                 (18, 1100), (25, 8200)])
def test_gram_matches_fp64_matmul(M, F):
    """Widths from one tile to 65 tiles per edge: whole super-tiles per XCD, left-over super-tiles shared
    row by row (4 of 36 at F = 8200), left-over diagonal super-tiles dealt tile by tile, partial tiles."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(M)
    Zr = rng.normal(size=(M, F))
    y = rng.normal(size=(M, 1))
    ZTZ0 = rng.normal(size=(F, F))
    ZTZ0 = ZTZ0 + ZTZ0.T
    ZTy0 = rng.normal(size=(F, 1))
    ZTZ = torch.tensor(ZTZ0, device=dev())
    ZTy = torch.tensor(ZTy0, device=dev())
    ops.gram(torch.tensor(Zr, device=dev()), torch.tensor(y, device=dev()), ZTZ, ZTy)
    close(ZTZ, ZTZ0 + Zr.T @ Zr, 1e-13, "ZTZ")           # fp64 arithmetic: only summation order differs
    close(ZTy, ZTy0 + Zr.T @ y, 1e-13, "ZTy")
    assert torch.equal(ZTZ, ZTZ.T)                         # both triangles come from one accumulator
    # feature-tiled build equals the untiled one
    nt = 3
    nsub = int(np.ceil(F / nt))
    full = torch.zeros(F, F, dtype=torch.float64, device=dev())
    zty = torch.zeros(F, 1, dtype=torch.float64, device=dev())
    for t in range(nt):
        lo, hi = t * nsub, min(F, (t + 1) * nsub)
        tile = torch.zeros(hi - lo, F, dtype=torch.float64, device=dev())
        ops.gram(torch.tensor(Zr, device=dev()), torch.tensor(y, device=dev()), tile, zty, f0=lo, f1=hi)
        full[lo:hi] = tile
    close(full, Zr.T @ Zr, 1e-13, "tiled ZTZ")
    close(zty, Zr.T @ y, 1e-13, "tiled ZTy")


@pytest.mark.parametrize("F", [200, 384])
def test_gram_upper_batches_then_one_mirror(F):
    """Two row batches added with the upper-tile entry and mirrored once equal two full calls bit for bit."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(F)
    batches = [torch.tensor(rng.normal(size=(m, F)), device=dev()) for m in (130, 77)]
    ys = [torch.tensor(rng.normal(size=(b.shape[0], 1)), device=dev()) for b in batches]
    full = torch.zeros(F, F, dtype=torch.float64, device=dev())
    fy = torch.zeros(F, 1, dtype=torch.float64, device=dev())
    up = torch.full((F, F), 7.0, dtype=torch.float64, device=dev()).tril(-128).contiguous()   # junk below the tiles
    uy = torch.zeros(F, 1, dtype=torch.float64, device=dev())
    for b, y in zip(batches, ys):
        ops.gram(b, y, full, fy)
        ops.gram(b, y, up, uy, mirror=False)
    lower_tiles = torch.ones(F, F, device=dev()).tril(-1).bool() & \
        ((torch.arange(F, device=dev())[:, None] // 128) > (torch.arange(F, device=dev())[None, :] // 128))
    assert (up[lower_tiles] == 7.0).sum() > 0              # untouched until mirrored
    ops.gram_mirror(up)
    assert torch.equal(up, full) and torch.equal(uy, fy)
    ref = sum(b.cpu().numpy().T @ b.cpu().numpy() for b in batches)
    close(up, ref, 1e-13, "batched ZTZ")


@pytest.mark.parametrize("F,M", [(4096, 2500), (4100, 2100)])
def test_gram_with_workspace_splits_the_last_round_of_tiles(F, M):
    """More tiles than workgroup slots and a sparsely filled last round (528 tiles at F = 4096, 561
    at 4100 where every load is bounds-checked): with a workspace the last tiles are cut into row ranges
    whose partial tiles are added in a fixed order.  Against fp64 matmul, against the entry without a
    workspace (equal up to the regrouping of the sums), bit-equal from call to call, accumulating onto
    what is already there, and untouched below the diagonal tiles."""
    from qml_lightning_amd import _lib
    from qml_lightning_amd.ops import _ptr, _stream
    L = _lib.lib()
    g = torch.Generator(device="cpu").manual_seed(F)
    Z = torch.randn(M, F, dtype=torch.float64, generator=g).to(dev())
    y = torch.randn(M, dtype=torch.float64, generator=g).to(dev())
    ws = torch.empty(int(L.qmll_gram_workspace_bytes()) // 8, dtype=torch.float64, device=dev())
    ws.fill_(float("nan"))                       # whatever the workspace holds must not matter

    def run(with_ws, start):
        C = torch.full((F, F), start, dtype=torch.float64, device=dev())
        zy = torch.zeros(F, dtype=torch.float64, device=dev())
        if with_ws:
            rc = L.qmll_gram_upper_ws_f64(_ptr(Z), _ptr(y), M, F, _ptr(C), _ptr(zy), _ptr(ws), ws.numel() * 8, _stream())
        else:
            rc = L.qmll_gram_upper_f64(_ptr(Z), _ptr(y), M, F, _ptr(C), _ptr(zy), _stream())
        assert rc == 0, _lib.last_error()
        return C, zy
    plain, zy0 = run(False, 0.0)
    split, zy1 = run(True, 0.0)
    again, _ = run(True, 0.0)
    assert torch.equal(split, again)
    zy_ref = torch.matmul(Z.T, y)                # Z^T y adds its row blocks with fp64 atomics: equal to rounding
    assert (zy0 - zy_ref).abs().max() <= 1e-13 * zy_ref.abs().max() and (zy1 - zy_ref).abs().max() <= 1e-13 * zy_ref.abs().max()
    ref = torch.matmul(Z.T, Z)
    tiles = torch.arange(F, device=dev()) // 128
    upper = tiles[:, None] <= tiles[None, :]
    scale = ref.abs().max().item()
    assert (split - ref)[upper].abs().max().item() <= 1e-13 * scale
    assert (split - plain)[upper].abs().max().item() <= 1e-13 * scale
    assert not torch.equal(split, plain)         # the split did run: the last tiles are summed in another grouping
    assert (split[~upper] == 0).all()
    onto, _ = run(True, 3.0)                     # accumulates: C += Z^T Z on the tiles it owns
    assert (onto - 3.0 - ref)[upper].abs().max().item() <= 1e-13 * scale and (onto[~upper] == 3.0).all()
    # too small a workspace, or none: the ordinary launch, bit-equal to the entry without one
    C = torch.zeros(F, F, dtype=torch.float64, device=dev())
    assert L.qmll_gram_upper_ws_f64(_ptr(Z), None, M, F, _ptr(C), None, _ptr(ws), 1024, _stream()) == 0
    assert torch.equal(C, plain)


# multiples of 128 take the one-launch-per-panel route (one, two and several panels), the others a launch per step
@pytest.mark.parametrize("F", [6, 100, 128, 300, 384, 640, 1064, 1536, 2176])
def test_cholesky_solve_matches_lapack(F):
    """(Z^T Z + lambda I) x = b by the library's blocked Cholesky against numpy's LU solve (the
    reference's route, kernel.py:231) and numpy's factor; conditioning as in training (few rows
    more than features, small lambda)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(F)
    Zr = rng.normal(size=(F + 20, F))
    A = Zr.T @ Zr + 1e-6 * np.eye(F)
    b = rng.normal(size=(F, 1))
    At = torch.tensor(A, device=dev())
    keep = At.clone()
    x, info = ops.cholesky_solve_spd(At, torch.tensor(b, device=dev()))
    assert int(info.item()) == 0
    assert torch.equal(At, keep)                                   # the input is left alone
    x_ref = sorf.regularised_solve(Zr.T @ Zr, b, 1e-6)             # the reference's LU route
    resid = np.abs(A @ x.cpu().numpy() - b).max()
    resid_ref = np.abs(A @ x_ref - b).max()
    assert resid <= 10 * resid_ref + 1e-9, (resid, resid_ref)
    assert np.abs(x.cpu().numpy() - x_ref).max() <= 1e-6 * np.abs(x_ref).max() * max(1.0, np.linalg.cond(A) * 1e-9)
    # the factor itself: in place, upper triangle = chol(A)^T
    U = At.clone()
    work = torch.empty(int(ops._lib.lib().qmll_cholesky_workspace_bytes(F)) // 8 + 1, dtype=torch.float64, device=dev())
    info2 = torch.zeros(1, dtype=torch.int32, device=dev())
    ops.check(ops._lib.lib().qmll_cholesky_f64(ops._ptr(U), F, F, ops._ptr(work), ops._ptr(info2), ops._stream()), "chol")
    Uref = np.linalg.cholesky(A).T
    got = np.triu(U.cpu().numpy())
    assert np.abs(got - Uref).max() <= 1e-9 * np.abs(Uref).max()
    assert int(info2.item()) == 0


@pytest.mark.parametrize("llambda", [1e-11, 1e-10])
@pytest.mark.parametrize("kind", ["fewer_rows", "smooth_columns"])
def test_regularised_solve_of_a_numerically_rank_deficient_gram_matrix(kind, llambda):
    """The shipped default is lambda = 1e-11 (HadamardFeaturesModel), where Z^T Z + lambda I has a
    condition number near 1 / eps: fewer rows than features (exactly rank deficient before lambda)
    and smooth, strongly correlated columns.  BaseKernel._solve_spd (blocked Cholesky with
    explicitly inverted diagonal blocks, LU when a pivot is not positive) must leave a residual
    no worse than ten times that of the reference's LU route (kernel.py:231) on the same matrix."""
    from qml_lightning_amd.models.kernel import BaseKernel
    rng = np.random.default_rng(17)
    F = 700
    if kind == "fewer_rows":
        Zr = rng.normal(size=(F // 2, F))
    else:
        t = np.linspace(0.0, 1.0, F)[None, :]
        Zr = np.cos(rng.uniform(0.5, 3.0, (F + 50, 1)) * t + rng.uniform(0, 6.28, (F + 50, 1)))
    A = Zr.T @ Zr
    b = Zr.T @ rng.normal(size=(Zr.shape[0], 1))
    A[np.diag_indices(F)] += llambda
    x = BaseKernel._solve_spd(torch.tensor(A, device=dev()), torch.tensor(b, device=dev())).cpu().numpy()
    x_lu = np.linalg.solve(A, b)
    resid = np.abs(A @ x - b).max()
    resid_lu = np.abs(A @ x_lu - b).max()
    print("%s lambda %.0e: cond %.1e, residual %.2e (LU %.2e), |x| %.2e" % (kind, llambda, np.linalg.cond(A), resid,
                                                                           resid_lu, np.abs(x).max()))
    assert np.isfinite(x).all()
    assert resid <= 10 * resid_lu + 1e-12 * np.abs(b).max(), (resid, resid_lu)


def test_solve_falls_back_to_lu_when_a_pivot_is_not_positive():
    """A symmetric matrix that rounding has left indefinite: the Cholesky route reports the pivot
    and _solve_spd returns the LU solution."""
    from qml_lightning_amd.models.kernel import BaseKernel
    rng = np.random.default_rng(6)
    F = 300
    Q, _ = np.linalg.qr(rng.normal(size=(F, F)))
    w = np.linspace(1.0, 2.0, F)
    w[123] = -1e-3                                          # one slightly negative eigenvalue
    A = (Q * w) @ Q.T
    A = 0.5 * (A + A.T)
    b = rng.normal(size=(F, 1))
    x = BaseKernel._solve_spd(torch.tensor(A, device=dev()), torch.tensor(b, device=dev())).cpu().numpy()
    assert np.abs(A @ x - b).max() <= 1e-9 * np.abs(x).max()


def test_triangular_solves_hand_a_nan_on_instead_of_waiting_for_it():
    """The blocks of the two solve launches hand their results on as the values themselves, with one NaN bit
    pattern meaning "not yet".  A right-hand side that holds NaNs, that very pattern among them, must come back
    as NaNs, not hang a consumer."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(12)
    F = 640
    Zr = rng.normal(size=(F + 20, F))
    A = torch.tensor(Zr.T @ Zr + 1e-6 * np.eye(F), device=dev())
    b = rng.normal(size=(F, 1))
    b[7, 0] = np.nan
    b[300, 0] = np.frombuffer(np.uint64(0x7FF8C0DEC0DE0001).tobytes(), dtype=np.float64)[0]
    x, info = ops.cholesky_solve_spd(A, torch.tensor(b, device=dev()))
    assert int(info.item()) == 0
    assert torch.isnan(x).all()                      # block 0 is poisoned, and every later block takes it in
    # and the same matrix with a clean right-hand side right after
    b2 = rng.normal(size=(F, 1))
    x2, _ = ops.cholesky_solve_spd(A, torch.tensor(b2, device=dev()))
    assert np.abs(A.cpu().numpy() @ x2.cpu().numpy() - b2).max() <= 1e-7 * np.abs(b2).max()


@pytest.mark.parametrize("F", [300, 640])
def test_solve_in_the_matrix_itself_and_its_restoration_for_lu(F):
    """train() lets _solve_spd use up Z^T Z: the same solution as from a copy when the matrix is positive
    definite; when a pivot fails, the matrix is put together again (diagonal tiles kept aside, the rest from
    the lower triangle) and LU solves the original system."""
    from qml_lightning_amd.models.kernel import BaseKernel
    rng = np.random.default_rng(F)
    Zr = rng.normal(size=(F + 20, F))
    A = Zr.T @ Zr + 1e-6 * np.eye(F)
    b = rng.normal(size=(F, 1))
    bt = torch.tensor(b, device=dev())
    x_copy = BaseKernel._solve_spd(torch.tensor(A, device=dev()), bt)
    x_used = BaseKernel._solve_spd(torch.tensor(A, device=dev()), bt, overwrite_a=True)
    assert torch.equal(x_copy, x_used)
    Q, _ = np.linalg.qr(rng.normal(size=(F, F)))
    w = np.linspace(1.0, 2.0, F)
    w[F // 2] = -1e-3                                       # one slightly negative eigenvalue
    Ai = (Q * w) @ Q.T
    Ai = 0.5 * (Ai + Ai.T)
    At = torch.tensor(Ai, device=dev())
    x = BaseKernel._solve_spd(At, bt, overwrite_a=True).cpu().numpy()
    assert np.abs(Ai @ x - b).max() <= 1e-9 * np.abs(x).max()
    assert torch.equal(At, torch.tensor(Ai, device=dev()))  # restored exactly


def test_cholesky_in_place_on_a_strided_view():
    """overwrite_a=True factors inside a wider buffer (row stride 700 for a 300 x 300 matrix) and
    touches nothing outside the matrix."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(9)
    F, W = 300, 700
    Zr = rng.normal(size=(F + 20, F))
    A = Zr.T @ Zr + 1e-6 * np.eye(F)
    b = rng.normal(size=(F, 1))
    big = torch.full((F + 3, W), 5.0, dtype=torch.float64, device=dev())
    view = big[1:F + 1, 100:100 + F]
    view.copy_(torch.tensor(A, device=dev()))
    x, info = ops.cholesky_solve_spd(view, torch.tensor(b, device=dev()), overwrite_a=True)
    assert int(info.item()) == 0
    assert np.abs(A @ x.cpu().numpy() - b).max() <= 1e-7 * np.abs(b).max()
    assert np.abs(np.triu(view.cpu().numpy()) - np.linalg.cholesky(A).T).max() <= 1e-9 * np.abs(A).max() ** 0.5
    outside = big.clone()
    outside[1:F + 1, 100:100 + F] = 5.0
    assert (outside == 5.0).all()


@pytest.mark.parametrize("F,bad", [(200, 150), (256, 150), (1152, 3), (1152, 300), (1152, 700), (1152, 1151)])
def test_cholesky_reports_a_matrix_that_is_not_positive_definite(F, bad):
    """On both routes (a launch per step; one launch per panel, where the other workgroups of the panel
    and every later launch must leave without waiting for the block that failed)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(5)
    Zr = rng.normal(size=(F + 20, F))
    A = Zr.T @ Zr
    A[bad, bad] = -1.0                                             # this pivot cannot be positive
    x, info = ops.cholesky_solve_spd(torch.tensor(A, device=dev()), torch.zeros(F, 1, dtype=torch.float64, device=dev()))
    assert int(info.item()) == bad + 1


def test_matmul_and_reduce_is_the_reference_kahan_sum():
    from qml_lightning_amd import ops
    rng = np.random.default_rng(3)
    A = rng.normal(size=(40, 150)).astype(np.float32)
    Bm = rng.normal(size=(150, 33)).astype(np.float32)
    C0 = rng.normal(size=(40, 33))
    ref = sorf.matmul_and_reduce(A, Bm, C0.copy())
    C = torch.tensor(C0, device=dev())
    ops.matmul_and_reduce(t32(A), t32(Bm), C)
    # same operations in the same order; the oracle rounds a*b-c to fp64 before fp32, which
    # can differ from the single rounding of a hardware fma by one fp32 ulp in rare ties
    got = C.cpu().numpy()
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()
    assert (got == ref).mean() > 0.99


@pytest.mark.parametrize("d,F", [(16, 40), (128, 700)])
def test_rff_features_and_derivatives(d, F):
    from qml_lightning_amd import ops
    rng = np.random.default_rng(F)
    A, n, nmol = 19, 6, 5
    x = rng.normal(size=(A, d)).astype(np.float32)
    grad = rng.normal(size=(A, n, 3, d)).astype(np.float32)
    grad[1, 2] = 0.0
    W = rng.normal(size=(d, F)) / 8.0
    b = rng.uniform(0, 2 * np.pi, F)
    idx = np.sort(rng.integers(0, nmol, A)).astype(np.int32)
    Zf = torch.zeros(nmol, F, dtype=torch.float64, device=dev())
    ops.rff_features(t32(x), torch.tensor(W, device=dev()), torch.tensor(b, device=dev()), ti32(idx), Zf)
    close(Zf, sorf.rff_features(x, W, b, idx, nmol), 1e-12, "rff features")
    G = torch.zeros(nmol, n, 3, F, dtype=torch.float64, device=dev())
    ops.rff_derivative_features(t32(x), t32(grad), torch.tensor(W, device=dev()), torch.tensor(b, device=dev()),
                                ti32(idx), G)
    close(G, sorf.rff_derivative_features(x, grad, W, b, idx, nmol), 1e-12, "rff derivative features")


@pytest.mark.parametrize("d,F,ne,A", [(64, 64, 1, 5), (128, 192, 3, 300), (64, 640, 2, 131)])
def test_rff_energy_sorted_kernel(d, F, ne, A):
    """Fused x.W + b -> cos -> alpha contraction and its gradient on element-sorted rows."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d + F)
    N = A + 9
    types = rng.integers(0, ne, N).astype(np.int32)
    types[rng.choice(N, size=3, replace=False)] = -1
    slots = np.sort(rng.choice(N, size=A, replace=False)).astype(np.int32)
    ss, off = ops.sort_by_type(ti32(types), ti32(slots), ne)
    ssn, total = ss.cpu().numpy(), int(off[-1].item())
    x = rng.normal(size=(A, d)).astype(np.float32)
    W = (rng.normal(size=(ne, d, F)) / 8.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, (ne, F)).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    e, gx = ops.rff_energy_sorted(t32(x), off, ss, t32(W), t32(b), t32(alpha), N)
    e_ref = np.zeros(N)
    g_ref = np.zeros((A, d))
    nf = np.sqrt(2.0 / F)
    for a_ in range(total):
        t_ = types[ssn[a_]]
        arg = x[a_].astype(np.float64) @ W[t_].astype(np.float64) + b[t_]
        e_ref[ssn[a_]] = nf * (alpha * np.cos(arg)).sum()
        g_ref[a_] = -nf * W[t_].astype(np.float64) @ (alpha * np.sin(arg))
    close(e, e_ref, REL_EF, "fused rff energies")
    close(gx, g_ref, REL_EF, "fused rff gradient")
    assert (gx[total:] == 0).all()
    e2, g2 = ops.rff_energy_sorted(t32(x), off, ss, t32(W), t32(b), t32(alpha), N, with_grad=False)
    assert g2 is None
    close(e2, e_ref, REL_EF, "fused rff energies only")


@pytest.mark.parametrize("wscale,ascale,xscale", [(0.125, 1.0, 1.0), (1e-3, 1e4, 1.0), (1e-4, 1e20, 1.0), (0.125, 1e-6, 1.0),
                                                  (125.0, 1e-20, 1e-3), (2e-6, 1.0, 6e4), (0.125, 1.0, 0.0)])
def test_rff_energy_sorted_kernel_over_operand_scales(wscale, ascale, xscale):
    """The fused kernel multiplies on the fp16 matrix cores with every fp32 operand split in two fp16
    parts behind a power-of-two scale of its own (x per wavefront, alpha per workgroup, W per chunk of 32
    features): W, alpha and x far outside fp16's range, one feature with a tie between two fp16 values,
    and an all-zero x, against fp64 at fp32 accuracy (5e-6 of the largest entry; arguments up to ~15; an
    operand part lost to fp16's range or a split that mixes two roundings costs 1e-5 to 1e-3)."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(7)
    d, F, A, ne = 128, 1056, 150, 1
    types = np.zeros(A, dtype=np.int32)
    ss, off = ops.sort_by_type(ti32(types), ti32(np.arange(A, dtype=np.int32)), ne)
    x = (rng.normal(size=(A, d)) * xscale).astype(np.float32)
    W = (rng.normal(size=(ne, d, F)) * wscale).astype(np.float32)
    W[0, :, 40:72] *= 1e-3                                    # a chunk of small entries beside the others
    b = rng.uniform(0, 2 * np.pi, (ne, F)).astype(np.float32)
    alpha = (rng.normal(size=F) * ascale).astype(np.float32)
    alpha[5] = 0.0
    e, gx = ops.rff_energy_sorted(t32(x), off, ss, t32(W), t32(b), t32(alpha), A)
    arg = x.astype(np.float64) @ W[0].astype(np.float64) + b[0]
    nf = np.sqrt(2.0 / F)
    e_ref = nf * np.cos(arg) @ alpha.astype(np.float64)
    g_ref = -nf * (np.sin(arg) * alpha.astype(np.float64)) @ W[0].astype(np.float64).T
    assert np.abs(arg).max() < 40
    close(e, e_ref, 5e-6, "fused rff energies")
    close(gx, g_ref, 5e-6, "fused rff gradient")


@pytest.mark.parametrize("d,F,n", [(64, 200, 6), (128, 704, 21), (128, 130, 29), (256, 64, 9), (16, 40, 6)])
def test_rff_derivatives_molecule_major(d, F, n):
    """Matrix-core route (segments instead of a molecule index); accumulates onto G;
    molecule 2 is left without atoms; n = 29 needs two row groups; d = 16 falls back."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(d + F + n)
    A, nmol = 23, 6
    x = rng.normal(size=(A, d)).astype(np.float32)
    grad = rng.normal(size=(A, n, 3, d)).astype(np.float32)
    grad[1, 2] = 0.0
    W = rng.normal(size=(d, F)) / 8.0
    b = rng.uniform(0, 2 * np.pi, F)
    idx = np.sort(rng.choice([0, 1, 3, 4, 5], A)).astype(np.int32)
    G0 = rng.normal(size=(nmol, n, 3, F))
    G = torch.tensor(G0, device=dev())
    ops.rff_derivative_features(t32(x), t32(grad), torch.tensor(W, device=dev()), torch.tensor(b, device=dev()),
                                ti32(idx), G, molecule_major=True)
    close(G, G0 + sorf.rff_derivative_features(x, grad, W, b, idx, nmol), 1e-12, "rff derivative features (segments)")


def test_prepared_model_constants_follow_their_tensors():
    """W of the RFF kernel and the reductors of the large-batch projections are split once and the
    split form is kept per tensor: an in-place update (version counter), a new tensor and a tensor
    that dies must each be noticed."""
    import gc
    from qml_lightning_amd import ops
    g = torch.Generator(device=dev()).manual_seed(5)
    A, d, F, R, ne = 2304, 128, 256, 312, 2
    x = torch.randn(A, d, device=dev(), generator=g)
    W = torch.randn(ne, d, F, device=dev(), generator=g) / 8
    b = torch.rand(ne, F, device=dev(), generator=g) * 6.28
    alpha = torch.randn(F, device=dev(), generator=g)
    types = torch.arange(A, device=dev(), dtype=torch.int32) % ne
    ss, off = ops.sort_by_type(types, torch.arange(A, device=dev(), dtype=torch.int32), ne)

    def rff_ref(Wt):
        t = types.long()[ss.long()]
        arg = torch.einsum('ak,akf->af', x.double(), Wt.double()[t]) + b.double()[t]
        return (2.0 / F) ** 0.5 * (torch.cos(arg) * alpha.double()).sum(dim=1)
    e0, _ = ops.rff_energy_sorted(x, off, ss, W, b, alpha, A)
    close(e0[ss.long()], rff_ref(W).cpu().numpy(), REL_EF, "first use")
    nkeys = len(ops._PRESPLIT)
    e0b, _ = ops.rff_energy_sorted(x, off, ss, W, b, alpha, A)
    assert len(ops._PRESPLIT) == nkeys                # no second split
    assert (e0 - e0b).abs().max() <= 1e-6 * e0.abs().max()     # the feature parts add with fp32 atomics
    W.mul_(0.5)                                       # in place: same object, same address, new version
    e1, _ = ops.rff_energy_sorted(x, off, ss, W, b, alpha, A)
    close(e1[ss.long()], rff_ref(W).cpu().numpy(), REL_EF, "after an in-place update")
    W2 = W * 3.0
    e2, _ = ops.rff_energy_sorted(x, off, ss, W2, b, alpha, A)
    close(e2[ss.long()], rff_ref(W2).cpu().numpy(), REL_EF, "another tensor")
    del W2
    gc.collect()
    assert len(ops._PRESPLIT) == nkeys                # the dead tensor's entry is gone

    rep = torch.randn(A, R, device=dev(), generator=g)
    red = torch.randn(ne, R, d, device=dev(), generator=g)
    gx = torch.randn(A, d, device=dev(), generator=g)

    def bwd_ref(U):
        return torch.einsum('ad,ard->ar', gx.double(), U.double()[types.long()[ss.long()]])
    for scale in (1.0, -0.25):
        if scale != 1.0:
            red.mul_(scale)
        gr = ops.project_typed_backward(gx, ss, off, red, types, A)      # beyond the small-batch kernels: prepared form
        close(gr[ss.long()], bwd_ref(red).cpu().numpy(), REL_REP, "transposed projection, reductors x %g" % scale)
        xs = ops.project_typed(rep, ss, off, red)
        ref = torch.einsum('ar,ard->ad', rep[ss.long()].double(), red.double()[types.long()[ss.long()]])
        close(xs, ref.cpu().numpy(), REL_REP, "projection, reductors x %g" % scale)


def test_a_non_finite_row_spoils_only_itself_in_the_fp16_matrix_core_kernels():
    """The projection kernels on the fp16 matrix cores and the fused RFF kernel scale the 32 rows of a
    wavefront by one power of two taken from their largest FINITE entry: a row holding an infinity (or
    a NaN) comes out non-finite, the rows beside it are unchanged."""
    from qml_lightning_amd import ops
    g = torch.Generator(device=dev()).manual_seed(9)
    A, R, d, ne, F = 2304, 312, 128, 2, 256
    types = torch.arange(A, device=dev(), dtype=torch.int32) % ne
    ss, off = ops.sort_by_type(types, torch.arange(A, device=dev(), dtype=torch.int32), ne)
    red = torch.randn(ne, R, d, device=dev(), generator=g)
    gx = torch.randn(A, d, device=dev(), generator=g)
    clean = ops.project_typed_backward(gx, ss, off, red, types, A)
    bad = gx.clone()
    bad[7, 3] = float("inf")
    bad[40, 100] = float("nan")
    out = ops.project_typed_backward(bad, ss, off, red, types, A)
    rows = ss.long()
    hit = torch.zeros(A, dtype=torch.bool, device=dev())
    hit[rows[7]] = hit[rows[40]] = True
    assert not torch.isfinite(out[hit]).all(dim=1).any()
    assert torch.equal(out[~hit], clean[~hit])
    x = torch.randn(A, d, device=dev(), generator=g)
    W = torch.randn(ne, d, F, device=dev(), generator=g) / 8
    b = torch.rand(ne, F, device=dev(), generator=g) * 6.28
    alpha = torch.randn(F, device=dev(), generator=g)
    e0, g0 = ops.rff_energy_sorted(x, off, ss, W, b, alpha, A)
    xb = x.clone()
    xb[11, 5] = float("inf")
    e1, g1 = ops.rff_energy_sorted(xb, off, ss, W, b, alpha, A)
    keep = torch.ones(A, dtype=torch.bool, device=dev())
    keep[11] = False
    assert not torch.isfinite(g1[11]).all()
    assert (g1[keep] - g0[keep]).abs().max() <= 1e-6 * g0.abs().max()      # feature parts add with fp32 atomics
    slot_keep = torch.ones(A, dtype=torch.bool, device=dev())
    slot_keep[rows[11]] = False
    assert (e1[slot_keep] - e0[slot_keep]).abs().max() <= 1e-6 * e0.abs().max()


def test_batch_preparation_of_few_atoms_among_many_padded_slots():
    """700 listed atoms (no sort workspace is asked for up to 1024) in 70 000 slots (more than the
    one-workgroup form takes): the general form without a workspace."""
    from qml_lightning_amd import ops
    B, n = 700, 100
    rng = np.random.default_rng(2)
    Z = np.zeros((B, n), np.float32)
    Z[:, 0] = rng.choice([1.0, 6.0, 8.0], size=B)
    t = lambda a: torch.tensor(a, device=dev())
    counts = t(np.ones(B, np.int32))
    ai, mi = t(np.zeros(B, np.int32)), t(np.arange(B, dtype=np.int32))
    species = t(np.array([1.0, 6.0, 8.0], np.float32))
    types, stypes, ss, off, zero = ops.prepare_batch(t(Z), counts, species, ai, mi, None, 4 * B * n)
    want = ops.element_types(torch.zeros(B, n, 3, device=dev()), t(Z), counts, species)
    assert torch.equal(types, want) and stypes is types
    want_ss, want_off = ops.sort_atoms_by_type(want, ai, mi, n, 3)
    assert torch.equal(off, want_off) and torch.equal(ss, want_ss)
    assert zero.shape[0] == 4 * B * n and not zero.any()


@pytest.mark.parametrize("nmol,model_list", [(1, None), (40, None), (40, [8.0, 1.0]), (300, [6.0, 9.0, 1.0]), (0, None)])
def test_batch_preparation_in_one_call_equals_the_separate_kernels(nmol, model_list):
    """qmll_prepare_batch (element indices by the representation's and by the model's species, the
    sort of the listed atoms, the zero fill; one launch up to 1024 atoms) against qmll_element_types,
    qmll_sort_atoms_by_type and a fill: bit-exact, ragged molecules with padding, a model list that is a
    subset / permutation of the species and leaves some atoms without an element."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(nmol + 5)
    n = 23
    counts = rng.integers(1, n + 1, size=nmol).astype(np.int32)
    Z = np.zeros((nmol, n), np.float32)
    for m in range(nmol):
        Z[m, :counts[m]] = rng.choice([1.0, 6.0, 8.0, 7.0], size=counts[m])          # 7: in no list
    atomIDs = np.concatenate([np.arange(c) for c in counts]).astype(np.int32) if nmol else np.zeros(0, np.int32)
    molIDs = np.repeat(np.arange(nmol), counts).astype(np.int32)
    t = lambda a: torch.tensor(a, device=dev())
    Zt, ct, ai, mi = t(Z), t(counts), t(atomIDs), t(molIDs)
    species = t(np.array([1.0, 6.0, 8.0], np.float32))
    msp = t(np.array(model_list, np.float32)) if model_list else None
    nz = 4 * nmol * n
    types, stypes, ss, off, zero = ops.prepare_batch(Zt, ct, species, ai, mi, msp, nz)
    X0 = torch.zeros(nmol, n, 3, device=dev())
    want_types = ops.element_types(X0, Zt, ct, species) if nmol else types
    assert torch.equal(types, want_types.view(nmol, n))
    want_st = ops.element_types(X0, Zt, ct, msp).view(nmol, n) if (msp is not None and nmol) else want_types.view(nmol, n)
    assert torch.equal(stypes, want_st)
    ne = len(model_list) if model_list else 3
    want_ss, want_off = ops.sort_atoms_by_type(want_st, ai, mi, n, ne)
    assert torch.equal(off, want_off)
    last = int(off[-1])
    assert torch.equal(ss[:last], want_ss[:last])
    assert zero.shape[0] == nz and not zero.any()


def test_transposed_projection_with_the_energy_sums_in_the_same_call():
    """qmll_project_typed_backward_sums against qmll_project_typed_backward and a row sum, on both sides
    of the small-batch switch; rows of atoms whose element the model does not hold come out zero."""
    from qml_lightning_amd import ops
    g = torch.Generator(device=dev()).manual_seed(3)
    for B, n in ((1, 21), (10, 21), (48, 21), (400, 21)):      # one, four, eight atoms per workgroup; the tiled kernel
        N = B * n
        types = torch.randint(-1, 3, (N,), device=dev(), generator=g, dtype=torch.int32)
        slots = torch.arange(N, device=dev(), dtype=torch.int32)
        ss, off = ops.sort_by_type(types, slots, 3)
        red = torch.randn(3, 312, 128, device=dev(), generator=g)
        gx = torch.randn(N, 128, device=dev(), generator=g)
        e_slots = torch.randn(N, device=dev(), generator=g)
        want = ops.project_typed_backward(gx, ss, off, red, types, N)
        got, energies = ops.project_typed_backward_sums(gx, ss, off, red, types, N, e_slots, B, n)
        assert torch.equal(got, want)
        assert not got[types < 0].any()
        ref = e_slots.view(B, n).double().sum(1)
        assert (energies.double() - ref).abs().max() <= 1e-6 * ref.abs().max()


def test_fused_energy_agrees_across_the_stack_sharing_switch():
    """Up to 1536 atoms a workgroup of the fused kernel runs sixteen wavefronts that share out the stacks,
    beyond that four: the same atoms evaluated in a batch on either side of the switch give the same
    energies and gradient rows (the stacks are summed in another order: last bits), and a sample of them
    matches the oracle."""
    from qml_lightning_amd import ops
    rng = np.random.default_rng(23)
    ne, d, S = 3, 128, 64
    F = S * d
    A_big = 1800
    x = rng.normal(size=(A_big, d)).astype(np.float32)
    types = (np.arange(A_big) % ne).astype(np.int32)
    D = np.where(rng.uniform(-1, 1, (ne, 1, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, (ne, F)).astype(np.float32)
    alpha = rng.normal(size=F).astype(np.float32)
    out = {}
    for A in (1536, A_big):
        ss, off = ops.sort_by_type(ti32(types[:A]), ti32(np.arange(A, dtype=np.int32)), ne)
        xs = t32(x[:A])[ss.long()]                      # rows in sorted order
        e, gx = ops.sorf_energy_sorted(xs, off, ss, t32(D), t32(b), t32(alpha), 3.0, 1, A)
        g = torch.empty_like(gx)
        g[ss.long()] = gx                               # back to atom order
        out[A] = (e, g)
    e0, g0 = out[1536]
    e1, g1 = out[A_big]
    assert (e0 - e1[:1536]).abs().max() <= 2e-6 * e1.abs().max()
    assert (g0 - g1[:1536]).abs().max() <= 2e-6 * g1.abs().max()
    for a_ in (0, 700, 1535):
        t_ = types[a_]
        c = sorf.sorf_coefficients(x[a_][None, :], D[t_], 3.0).reshape(1, F)
        e_ref = (np.sqrt(2.0 / F) * np.cos(c + b[t_]) * alpha).sum()
        gc = -np.sqrt(2.0 / F) * np.sin(c + b[t_]) * alpha
        g_ref = sorf.sorf_adjoint(gc.reshape(1, S, d), D[t_], 3.0)[0]
        assert abs(float(e0[a_]) - e_ref) <= REL_EF * float(e1.abs().max())
        assert np.abs(g0[a_].cpu().numpy() - g_ref).max() <= REL_EF * float(g1.abs().max())
