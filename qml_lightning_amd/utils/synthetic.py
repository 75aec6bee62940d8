"""Seeded synthetic molecules and model weights of the benchmark configurations
(no dataset is needed or downloaded)."""
import numpy as np

ASPIRIN = np.array([6] * 9 + [1] * 8 + [8] * 4)            # C9H8O4, 21 atoms
C12H12N2O = np.array([6] * 12 + [1] * 12 + [7] * 2 + [8])   # 27 atoms


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
    """C6H6: C ring 1.39 A, H ring 2.47 A, planar, + N(0, 0.05 A) noise per coordinate."""
    rng = np.random.default_rng(seed)
    ang = np.arange(6) * np.pi / 3
    base = np.concatenate([np.stack([1.39 * np.cos(ang), 1.39 * np.sin(ang), 0 * ang], 1),
                           np.stack([2.47 * np.cos(ang), 2.47 * np.sin(ang), 0 * ang], 1)])
    charges = np.array([6] * 6 + [1] * 6)
    coords = [base + rng.normal(0, 0.05, base.shape) for _ in range(ncopies)]
    return coords, [charges] * ncopies


def fixed_composition_batch(charges, ncopies, seed, box=7.0, min_sep=1.0, sigma=0.05):
    """One base geometry in a cube (pairwise separation >= min_sep), Gaussian displaced copies."""
    rng = np.random.default_rng(seed)
    charges = np.asarray(charges)
    base = random_geometry(rng, len(charges), box, min_sep)
    coords = [base + rng.normal(0, sigma, base.shape) for _ in range(ncopies)]
    return coords, [charges] * ncopies


def ragged_batch(nmol, seed=2, nmin=3, nmax=29):
    """Atom counts uniform in [nmin,nmax]; heavy atoms (<= 9) from C/N/O/F with
    p = .7/.12/.15/.03, H fills the rest (about 1.8 x the heavy count)."""
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
    """Reductors = orthonormalised Gaussian [ne,R,d] (QR); D = +-1 [ne,T,S,d]; bias U(0,2pi)
    [ne,S*d]; alpha N(0,1) [S*d] (fp64)."""
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
