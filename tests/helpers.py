"""Shared synthetic inputs for the parity tests (seeded, deterministic)."""
import numpy as np

from oracle import fchl19


def kat_params(d):
    return fchl19.FCHLParams(d["species"], rcut=float(d["rcut"]), eta2=float(d["eta2"]), eta3=float(d["eta3"]),
                             two_body_decay=float(d["two_body_decay"]),
                             raw_three_body_weight=float(d["three_body_weight"]),
                             three_body_decay=float(d["three_body_decay"]), Rs2=d["Rs2"], Rs3=d["Rs3"])


def random_geometry(rng, natoms, box, min_sep):
    """Rejection-sample `natoms` points uniform in a cube of side `box` with pairwise
    separation >= min_sep."""
    pts = []
    while len(pts) < natoms:
        p = rng.uniform(0, box, 3)
        if all(np.linalg.norm(p - q) >= min_sep for q in pts):
            pts.append(p)
    return np.array(pts)


def benzene_batch(ncopies=4, seed=0):
    """BASELINE config 1: C6H6, C ring 1.39 A, H ring 2.47 A, + N(0,0.05) noise."""
    rng = np.random.default_rng(seed)
    ang = np.arange(6) * np.pi / 3
    base = np.concatenate([np.stack([1.39 * np.cos(ang), 1.39 * np.sin(ang), 0 * ang], 1),
                           np.stack([2.47 * np.cos(ang), 2.47 * np.sin(ang), 0 * ang], 1)])
    charges = np.array([6] * 6 + [1] * 6)
    coords = [base + rng.normal(0, 0.05, base.shape) for _ in range(ncopies)]
    return coords, [charges] * ncopies


def fixed_composition_batch(charges, ncopies, seed, box=7.0, min_sep=1.0, sigma=0.05):
    """BASELINE configs 2/4/5: one base geometry in a cube, Gaussian displaced copies."""
    rng = np.random.default_rng(seed)
    charges = np.asarray(charges)
    base = random_geometry(rng, len(charges), box, min_sep)
    coords = [base + rng.normal(0, sigma, base.shape) for _ in range(ncopies)]
    return coords, [charges] * ncopies


ASPIRIN = np.array([6] * 9 + [1] * 8 + [8] * 4)            # C9H8O4
C12H12N2O = np.array([6] * 12 + [1] * 12 + [7] * 2 + [8])


def ragged_batch(nmol, seed=2, nmin=3, nmax=29):
    """BASELINE config 3: atom counts uniform in [nmin,nmax]; heavy atoms (<= 9) from
    C/N/O/F with p = .7/.12/.15/.03, H fills the rest up to 1.8x the heavy count."""
    rng = np.random.default_rng(seed)
    coords, charges = [], []
    for _ in range(nmol):
        n = int(rng.integers(nmin, nmax + 1))
        h = min(9, max(1, int(np.ceil(n / 2.8))))
        while h + int(round(1.8 * h)) < n and h < 9:
            h += 1
        nh = n - h
        if nh < 0:
            h, nh = n, 0
        heavy = rng.choice([6, 7, 8, 9], size=h, p=[0.7, 0.12, 0.15, 0.03])
        q = np.concatenate([heavy, np.ones(nh, dtype=np.int64)]).astype(np.int64)
        box = max(3.0, 1.6 * n ** (1.0 / 3.0) + 1.0)
        coords.append(random_geometry(rng, n, box, 0.95))
        charges.append(q)
    return coords, charges


def model_weights(nelements, repsize, npcas, nstacks, ntransforms=1, seed=10):
    """Reductors = orthonormalised Gaussian [ne,R,d]; D = +-1; bias U(0,2pi); alpha N(0,1)."""
    rng = np.random.default_rng(seed)
    red = np.zeros((nelements, repsize, npcas), dtype=np.float32)
    for e in range(nelements):
        qm, _ = np.linalg.qr(rng.normal(size=(repsize, npcas)))
        red[e] = qm.astype(np.float32)
    rng = np.random.default_rng(seed + 1)
    D = np.where(rng.uniform(-1, 1, (nelements, ntransforms, nstacks, npcas)) > 0, 1.0, -1.0).astype(np.float32)
    rng = np.random.default_rng(seed + 2)
    bias = (rng.uniform(0, 1, (nelements, nstacks * npcas)) * 2 * np.pi).astype(np.float32)
    rng = np.random.default_rng(seed + 3)
    alpha = rng.normal(size=nstacks * npcas)
    return red, D, bias, alpha
