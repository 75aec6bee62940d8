"""Benchmark of the QML-Lightning hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = energies + forces (FCHL19 -> PCA projection -> SORF -> cos features -> E, and
-dE/dX; `model.energies_and_forces`, the body of the reference-shaped `predict_opt`; the
differentiable `forward` + `autograd.grad` route of a TorchScript caller is timed beside
it) for the 4096-molecule C9H8O4 batch of the benchmark's second configuration (21 atoms,
species {1,6,8}, npcas 128, nstacks 128 = 16384 features, fp32), inputs resident in HBM.
Prints one JSON line: molecules/s, the per-kernel rooflines measured with HIP events on
the launch stream, the time to build Z^T Z / Z^T y for 1000 such molecules with forces,
and the fp64 CPU oracle timed on the host cores for the same workload (bounded sample).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

SPECIES = [1, 6, 8]
NPCAS, NSTACKS, SIGMA = 128, 128, 2.0
NMOL_PREDICT, NMOL_TRAIN = 4096, 1000
HBM_PEAK_GBS = 8000.0
FP32_PEAK_TFLOPS = 157.3
FP16_PEAK_TFLOPS = 2500.0         # dense v_mfma_f32_32x32x16_f16
FP64_PEAK_TFLOPS = 78.6


def cpu_baseline_worker(args):
    """Energy + forces of a few molecules with the fp64 oracle (one process)."""
    coords, charges, weights = args
    from oracle import fchl19, model as omodel
    red, D, bias, alpha = weights
    prm = fchl19.FCHLParams(SPECIES)
    X, Z, aid, mid, nat = omodel.format_batch(coords, charges)
    E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, SPECIES, red, D.astype(np.float64), bias, alpha,
                                        SIGMA)
    return E, F


def cpu_config1_worker(args):
    """Configuration 1 (the CPU-reference configuration): energies + forces of C6H6 copies, fp64 oracle."""
    coords, charges, weights = args
    from oracle import fchl19, model as omodel
    red, D, bias, alpha = weights
    prm = fchl19.FCHLParams([1, 6])
    X, Z, aid, mid, nat = omodel.format_batch(coords, charges)
    return omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, [1, 6], red, D.astype(np.float64), bias, alpha, SIGMA)[:2]


def cpu_config1(cores):
    """The whole of configuration 1 on the host: 100 noisy C6H6, npcas 64, nstacks 8, fp64."""
    import multiprocessing as mp
    from qml_lightning_amd.utils import synthetic
    coords, charges = synthetic.benzene_batch(100, seed=0)
    coords = [c.astype(np.float32).astype(np.float64) for c in coords]      # the values the GPU side receives
    red, D, bias, alpha = synthetic.model_weights(2, 2 * 24 + 2 * 3 * 20, 64, 8)
    weights = (red, D, bias, alpha.astype(np.float32).astype(np.float64))
    chunks = [(coords[i::cores], charges[i::cores], weights) for i in range(cores)]
    ctx = mp.get_context("fork")
    with ctx.Pool(cores) as pool:
        pool.map(cpu_config1_worker, [(c[0][:1], c[1][:1], c[2]) for c in chunks])      # import + warm
        t0 = time.perf_counter()
        res = pool.map(cpu_config1_worker, chunks)
        dt = time.perf_counter() - t0
    E = np.zeros(100)
    F = np.zeros((100, 12, 3))
    for i, (e, f) in enumerate(res):
        E[i::cores], F[i::cores] = e, f
    return {"seconds": dt, "E": E, "F": F, "cores": cores}


def cpu_baseline(coords, charges, weights, nsample, cores):
    """The oracle ("port") on `cores` host processes over the first `nsample` molecules."""
    import multiprocessing as mp
    chunks = [(coords[i::cores][:], charges[i::cores][:], weights) for i in range(cores)]
    chunks = [(c[0][:(nsample + cores - 1) // cores], c[1][:(nsample + cores - 1) // cores], c[2]) for c in chunks]
    n = sum(len(c[0]) for c in chunks)
    ctx = mp.get_context("fork")          # forked before anything touches the GPU
    with ctx.Pool(cores) as pool:
        pool.map(cpu_baseline_worker, [(c[0][:1], c[1][:1], c[2]) for c in chunks])   # import + warm
        t0 = time.perf_counter()
        out = pool.map(cpu_baseline_worker, chunks)
        dt = time.perf_counter() - t0
    return n / dt, n, dt, out, chunks


def bench_solve(torch, ops, timed, ZTZ, ZTy, F):
    """(Z^T Z + lambda I) alpha = Z^T y on the matrix just built: the library's blocked Cholesky,
    with the torch (rocSOLVER) factorisation of the same matrix beside it."""
    ZTZ.diagonal().add_(1e-5)
    t_solve = timed(lambda: ops.cholesky_solve_spd(ZTZ, ZTy), iters=2)
    xs, info = ops.cholesky_solve_spd(ZTZ, ZTy)
    resid = float((ZTZ @ xs - ZTy).abs().max() / ZTy.abs().max())

    def torch_route():
        L, _ = torch.linalg.cholesky_ex(ZTZ)
        return torch.cholesky_solve(ZTy, L)
    t_torch = timed(torch_route, iters=2)
    # what train() runs: the factorisation in Z^T Z itself (the matrix is not needed again), the diagonal
    # tiles kept aside for the LU fallback; the copy this benchmark needs is made outside the timed region
    from qml_lightning_amd.models.kernel import BaseKernel
    t_used = 0.0
    for _ in range(2):
        work = ZTZ.clone()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        x_used = BaseKernel._solve_spd(work, ZTy, overwrite_a=True)
        e.record()
        torch.cuda.synchronize()
        t_used = s.elapsed_time(e) * 1e-3
        del work
    return {"solve_seconds": t_solve, "solve_TFLOPs": F ** 3 / 3.0 / t_solve / 1e12, "solve_info": int(info.item()),
            "solve_relative_residual": resid, "solve_seconds_torch_cholesky": t_torch,
            "solve_includes": "copy of Z^T Z + Cholesky factorisation + two triangular solves",
            "solve_seconds_in_place": t_used, "solve_in_place_equal": bool(torch.equal(x_used, xs)),
            "solve_in_place_includes": "what train() runs: 16 MB of diagonal tiles kept aside, the factorisation "
                                       "in Z^T Z itself, two triangular solves, the read-back of info"}


def other_configs(torch, dev):
    """Short measurements of the other benchmark configurations (1, 3, 4, 5) with the
    same step definition; reported under "other_configs", never as `value`."""
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    from qml_lightning_amd.utils import synthetic

    def sorf_model(species, npcas, nstacks, nbatch_train):
        rep = FCHLCuda(species=np.array(species))
        m = HadamardFeaturesModel(rep=rep, elements=np.array(species), ntransforms=1, sigma=SIGMA, llambda=1e-5,
                                  npcas=npcas, nstacks=nstacks, nbatch_train=nbatch_train, nbatch_test=1 << 20)
        red, D, bias, alpha = synthetic.model_weights(len(species), rep.get_repsize(), npcas, nstacks)
        m.reductors, m.Dmat, m.bias = (torch.tensor(v, device=dev) for v in (red, D, bias))
        m.alpha = torch.tensor(alpha, device=dev)
        m.is_trained = True
        return m

    def predict_rate(model, coords, charges, forces, steps=5, warm=2):
        data = model.format_data([c.astype(np.float32) for c in coords], charges)
        X, Z = data['coordinates'], data['charges']
        aid, mid, nat = data['atomIDs'], data['molIDs'], data['natom_counts']

        def step():
            return model.energies_and_forces(X, Z, aid, mid, nat, forces=forces)
        for _ in range(warm):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        return {"molecules": len(coords), "atoms": int(aid.shape[0]), "ms_per_step": dt * 1e3,
                "molecules_per_s": len(coords) / dt, "outputs": "energies + forces" if forces else "energies"}

    def ztz_seconds(model, coords, charges, natoms):
        rng = np.random.default_rng(14)
        nm = len(coords)
        Et = rng.normal(size=nm)
        Ft = [rng.normal(size=(natoms, 3)) for _ in range(nm)]
        model.build_Z_components(coords[:16], charges[:16], E=Et[:16], F=Ft[:16], print_info=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ZTZ, ZTy = model.build_Z_components(coords, charges, E=Et, F=Ft, print_info=False)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        M, Fn = nm * (1 + 3 * natoms), model.nfeatures()
        return {"ztz_seconds": dt, "ztz_molecules": nm, "ztz_rows": M, "ztz_features": Fn,
                "ztz_TFLOPs_whole_build": (float(M) * Fn * (Fn + 1)) / dt / 1e12}

    out = {}
    # config 1: 100 noisy C6H6, npcas 64 x nstacks 8
    coords, charges = synthetic.benzene_batch(100, seed=0)
    m1 = sorf_model([1, 6], 64, 8, 64)
    out["config1_c6h6_100"] = predict_rate(m1, coords, charges, True, steps=50, warm=10)
    d1 = m1.format_data([c.astype(np.float32) for c in coords], charges)
    e1, f1 = m1.energies_and_forces(d1['coordinates'], d1['charges'], d1['atomIDs'], d1['molIDs'], d1['natom_counts'])
    out["config1_c6h6_100"]["_E"] = e1.double().cpu().numpy()
    out["config1_c6h6_100"]["_F"] = f1.double().cpu().numpy()
    # config 3: 8192 ragged molecules (3..29 atoms, H C N O F), npcas 128 x nstacks 64, energies only
    coords, charges = synthetic.ragged_batch(8192, seed=2)
    out["config3_ragged_8192"] = predict_rate(sorf_model([1, 6, 7, 8, 9], 128, 64, 64), coords, charges, False)
    # config 4: C12H12N2O (27 atoms), npcas 256 x nstacks 128 = 32768 features: fp64 Gram on 500, predict on 1548
    coords, charges = synthetic.fixed_composition_batch(synthetic.C12H12N2O, 2048, seed=3, sigma=0.15)
    m4 = sorf_model([1, 6, 7, 8], 256, 128, 250)
    r4 = predict_rate(m4, coords[500:], charges[500:], True)
    r4.update(ztz_seconds(m4, [c.astype(np.float32) for c in coords[:500]], charges[:500], 27))
    out["config4_c12h12n2o"] = r4
    del m4
    torch.cuda.empty_cache()
    # config 5: random Fourier features, 32768 features, projected dimension 128, C9H8O4 batch;
    # W = N(0,1)/(2 sigma^2) as the reference samples it; SORF at the same feature count beside it
    coords, charges = synthetic.fixed_composition_batch(synthetic.ASPIRIN, NMOL_PREDICT, seed=1)
    np.random.seed(15)
    rep = FCHLCuda(species=np.array(SPECIES))
    m5 = RandomFourrierFeaturesModel(rep=rep, elements=np.array(SPECIES), sigma=SIGMA, llambda=1e-5, npcas=128,
                                     nstacks=256, nbatch_train=500, nbatch_test=1 << 20)
    red, _, _, alpha = synthetic.model_weights(len(SPECIES), rep.get_repsize(), 128, 256)
    m5.reductors = torch.tensor(red, device=dev)
    m5.alpha = torch.tensor(alpha, device=dev)
    m5.is_trained = True
    r5 = predict_rate(m5, coords, charges, True)
    # the fused RFF kernel of that step alone (HIP events on the launch stream), against the pipe it runs on
    from qml_lightning_amd import ops
    d5 = m5.format_data([c.astype(np.float32) for c in coords], charges)
    prm5 = ops.make_params(len(SPECIES), rep.Rs2, rep.Rs3, rep.eta2, rep.eta3, rep.two_body_decay, rep.three_body_weight,
                           rep.three_body_decay, rep.rcut)
    t5 = ops.element_types(d5['coordinates'], d5['charges'], d5['natom_counts'], rep.species)
    rep5 = ops.fchl_forward(d5['coordinates'], t5, None, None, d5['atomIDs'], d5['molIDs'], d5['natom_counts'], rep.Rs2,
                            rep.Rs3, prm5)
    B5, n5 = d5['charges'].shape
    ss5, off5 = ops.sort_atoms_by_type(t5, d5['atomIDs'], d5['molIDs'], n5, len(SPECIES))
    x5 = ops.project_typed(rep5.view(B5 * n5, -1), ss5, off5, m5.reductors)
    a5 = m5.alpha.float()
    for _ in range(2):
        ops.rff_energy_sorted(x5, off5, ss5, m5.W, m5.b, a5, B5 * n5)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(5):
        ops.rff_energy_sorted(x5, off5, ss5, m5.W, m5.b, a5, B5 * n5)
    ev1.record()
    torch.cuda.synchronize()
    t_rff = ev0.elapsed_time(ev1) / 5 * 1e-3
    fl5 = 4.0 * x5.shape[0] * x5.shape[1] * m5.nfeatures()          # x.W and its transpose product
    r5["rff_energy_sorted_kernel"] = {
        "seconds": t_rff, "bound": "mfma",
        "pipe": "fp16 matrix cores (v_mfma_f32_32x32x16_f16), fp32 operands split in two fp16 parts (W once per model, x and "
                "the sine factors in the kernel), fp32 accumulation",
        "TFLOPs": fl5 / t_rff / 1e12, "executed_TFLOPs": 3.0 * fl5 / t_rff / 1e12, "peak_TFLOPs": FP16_PEAK_TFLOPS,
        "frac": 3.0 * fl5 / t_rff / 1e12 / FP16_PEAK_TFLOPS}
    del d5, rep5, x5
    r5.update(ztz_seconds(m5, [c.astype(np.float32) for c in coords[:NMOL_TRAIN]], charges[:NMOL_TRAIN], 21))
    out["config5_rff_32768"] = r5
    del m5
    torch.cuda.empty_cache()
    out["config5_sorf_32768"] = predict_rate(sorf_model(SPECIES, 128, 256, 500), coords, charges, True)
    # one C9H8O4 molecule with the config-2 model: the latency of the step's chain of dependent launches,
    # eager, through forward + autograd.grad, and replayed from a captured HIP graph (each replay checked)
    m2 = sorf_model(SPECIES, NPCAS, NSTACKS, 500)
    out["c9h8o4_48_molecules"] = predict_rate(m2, coords[:48], charges[:48], True, steps=200, warm=20)   # 1008 atoms
    one = predict_rate(m2, coords[:1], charges[:1], True, steps=200, warm=20)
    data = m2.format_data([coords[0].astype(np.float32)], charges[:1])
    X, Z = data['coordinates'], data['charges']
    aid, mid, nat = data['atomIDs'], data['molIDs'], data['natom_counts']

    def autograd_step():
        Xg = X.detach().requires_grad_(True)
        E = m2.forward(Xg, Z, aid, mid, nat)
        return E, torch.autograd.grad(-E.sum(), Xg)[0]
    for _ in range(20):
        autograd_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(200):
        autograd_step()
    torch.cuda.synchronize()
    one["autograd_ms_per_step"] = (time.perf_counter() - t0) / 200 * 1e3
    Xs = X.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            m2.energies_and_forces(Xs, Z, aid, mid, nat, forces=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        Eg, Fg = m2.energies_and_forces(Xs, Z, aid, mid, nat, forces=True)
    ok = True
    for it in range(4):      # replays with changed inputs, eager work and synchronisations between them
        Xp = X + 0.01 * it
        Ee, Fe = m2.energies_and_forces(Xp, Z, aid, mid, nat, forces=True)
        torch.cuda.synchronize()
        Xs.copy_(Xp)
        graph.replay()
        torch.cuda.synchronize()
        ok = ok and bool(torch.equal(Eg, Ee)) and bool((Fg - Fe).abs().max() <= 1e-5 * Fe.abs().max())
    for _ in range(20):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(200):
        graph.replay()
    torch.cuda.synchronize()
    one["graph_replay_ms_per_step"] = (time.perf_counter() - t0) / 200 * 1e3
    one["graph_replays_match_eager"] = ok
    out["one_molecule_c9h8o4"] = one
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train", action="store_true", help="skip the Z^T Z build measurement")
    ap.add_argument("--no-solve", action="store_true", help="skip the regularised solve after the Z^T Z build")
    ap.add_argument("--cpu-sample", type=int, default=1024)
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short measurements of configurations 1, 3, 4 and 5")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a plain 1 GiB read + 1 GiB write elementwise kernel (reference point for "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; run with --gpus 1 (molecules shard trivially across GPUs, "
              "but no multi-GPU figure is produced here)", file=sys.stderr)
        sys.exit(2)

    import torch
    import qml_lightning_amd  # noqa: F401
    from qml_lightning_amd import ops
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    from qml_lightning_amd.utils import synthetic

    # ---- workload (configuration 2) ---------------------------------------------------------
    coords, charges = synthetic.fixed_composition_batch(synthetic.ASPIRIN, NMOL_PREDICT, seed=1)
    coords = [c.astype(np.float32) for c in coords]
    nrep = len(SPECIES) * 24 + len(SPECIES) * (len(SPECIES) + 1) * 20
    red, D, bias, alpha = synthetic.model_weights(len(SPECIES), nrep, NPCAS, NSTACKS)

    # ---- CPU baseline first: its worker processes are forked before the GPU is initialised --
    cpu = None
    cpu_c1 = None
    if not args.no_cpu_baseline:
        cores = min(os.cpu_count() or 1, 16)
        cpu_c1 = cpu_config1(cores)
        c64 = [c.astype(np.float64) for c in coords[:args.cpu_sample]]
        cpu = cpu_baseline(c64, charges[:args.cpu_sample], (red, D, bias, alpha.astype(np.float32).astype(np.float64)),
                           args.cpu_sample, cores) + (cores,)

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    rep = FCHLCuda(species=np.array(SPECIES))
    model = HadamardFeaturesModel(rep=rep, elements=np.array(SPECIES), ntransforms=1, sigma=SIGMA, llambda=1e-5,
                                  npcas=NPCAS, nstacks=NSTACKS, nbatch_train=500, nbatch_test=NMOL_PREDICT, fused=True)
    assert rep.get_repsize() == nrep
    model.reductors = torch.tensor(red, device=dev)
    model.Dmat = torch.tensor(D, device=dev)
    model.bias = torch.tensor(bias, device=dev)
    model.alpha = torch.tensor(alpha, device=dev)
    model.is_trained = True
    data = model.format_data(coords, charges)
    X, Z = data['coordinates'], data['charges']
    aid, mid, nat = data['atomIDs'], data['molIDs'], data['natom_counts']
    B, n = Z.shape
    A = int(aid.shape[0])
    F = NPCAS * NSTACKS
    R = rep.get_repsize()

    if args.calibration_copy:
        # a plain copy of known size (1 GiB read, 1 GiB written): the reference point for the
        # FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this script
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            ops.check(ops._lib.lib().qmll_probe_copy(ops._ptr(src), ops._ptr(dst), src.numel(), ops._stream()), "copy")
        del src, dst
        torch.cuda.synchronize()
    # ceilings measured on this very device (a few ms each), next to the nominal ones
    from qml_lightning_amd.utils import peaks as peaks_mod
    peaks = peaks_mod.measure()
    peaks["nominal"] = dict(peaks_mod.NOMINAL)
    # what a wavefront instruction of each class costs a SIMD, and the per-stack instruction mix of the
    # fused SORF kernel next to the same mix with its in-row butterfly stages on the matrix pipe
    mixes = peaks_mod.instruction_mixes()
    best = {k: min(v.values()) for k, v in mixes.items()}
    instruction_mixes = {
        "ns_per_wavefront_iteration_per_simd": {k: {w: t * 1e9 for w, t in v.items()} for k, v in mixes.items()},
        "ns_per_instruction": {"plain_fp32": best["plain_fp32_x128"] / 128 * 1e9, "dpp_fmac": best["dpp_fmac_x128"] / 128 * 1e9,
                               "transcendental": best["transcendental_x128"] / 128 * 1e9},
        "fused_kernel_stack_ns": best["fused_kernel_stack"] * 1e9,
        "note": "one iteration of fused_kernel_stack = 82 plain + 64 DPP + 16 transcendental wavefront instructions = one "
                "stack of four atoms at 128 components",
    }
    torch.cuda.empty_cache()

    def step():
        return model.energies_and_forces(X, Z, aid, mid, nat)

    def step_autograd():
        Xg = X.detach().requires_grad_(True)
        Ea = model.forward(Xg, Z, aid, mid, nat)
        Fa, = torch.autograd.grad(-Ea.sum(), Xg)
        return Ea, Fa

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        E, Fr = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = B * args.steps / dt
    # the same step through forward + autograd.grad (the route of a TorchScript caller)
    for _ in range(args.warmup):
        step_autograd()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        Ea, Fa = step_autograd()
    torch.cuda.synchronize()
    ms_autograd = (time.perf_counter() - t0) / args.steps * 1e3
    autograd_route = {"ms_per_step": ms_autograd, "molecules_per_s": B / ms_autograd * 1e3,
                      "max_abs_diff_energy": float((Ea.detach() - E).abs().max()),
                      "max_abs_diff_force": float((Fa - Fr).abs().max())}

    # the same step through the reference's two-operator contract (get_SORF_coefficients +
    # get_cos_features with autograd, the only operators a model file saved by the reference calls):
    # the [atoms, features] coefficient array goes through HBM four times
    model.fused = False
    for _ in range(2):
        step_autograd()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        E2, F2 = step_autograd()
    torch.cuda.synchronize()
    ms_two_op = (time.perf_counter() - t0) / 5 * 1e3
    # GPU time of the same step as the sum of its kernels' durations (one profiled step): what the
    # route costs when the host keeps up; the difference to the wall time is host time
    kernel_sum_ms = None
    try:
        from torch.profiler import ProfilerActivity, profile
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            step_autograd()
            torch.cuda.synchronize()
        kernel_sum_ms = sum(ev.self_device_time_total for ev in prof.key_averages()) / 1e3
    except Exception as exc:      # the profiler is optional; the wall time stands on its own
        kernel_sum_ms = None
        print("bench.py: two-op kernel sum not measured: %r" % (exc,), file=sys.stderr)
    model.fused = True
    two_op_route = {"ms_per_step": ms_two_op, "molecules_per_s": B / ms_two_op * 1e3,
                    "kernel_sum_ms": kernel_sum_ms,
                    "gpu_share_of_wall": (kernel_sum_ms / ms_two_op) if kernel_sum_ms else None,
                    "max_abs_diff_energy": float((E2.detach() - E).abs().max()),
                    "max_abs_diff_force": float((F2 - Fr).abs().max()),
                    "hbm_bytes_per_step_algorithmic": float(A) * (20.0 * F + 8.0 * NPCAS)}
    del E2, F2
    torch.cuda.empty_cache()

    # the same batch handed over as host arrays (lists of numpy coordinates / charges): batch
    # formatting on the host, upload over PCIe, predict, results left on the device
    model.predict(coords[:64], charges[:64], n, forces=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        model.predict(coords, charges, n, forces=True)
    torch.cuda.synchronize()
    ms_host = (time.perf_counter() - t0) / 3 * 1e3
    from_host = {"ms_per_step": ms_host, "molecules_per_s": B / ms_host * 1e3,
                 "includes": "format_data on the host + host-to-device copies + predict; never the headline value"}
    # the same batch as ONE zero-padded host array pair: two uploads, indices built on the device
    Xpad = np.stack(coords).astype(np.float32)
    Qpad = np.stack(charges).astype(np.float32)
    model.predict(Xpad[:64], Qpad[:64], n, forces=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        model.predict(Xpad, Qpad, n, forces=True)
    torch.cuda.synchronize()
    ms_pad = (time.perf_counter() - t0) / 3 * 1e3
    from_host["padded_arrays_ms_per_step"] = ms_pad
    from_host["padded_arrays_molecules_per_s"] = B / ms_pad * 1e3

    # ---- per-kernel timing with HIP events on the launch stream ----------------------------
    def timed(fn, iters=5):
        fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(iters):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / iters * 1e-3

    prm = ops.make_params(len(SPECIES), rep.Rs2, rep.Rs3, rep.eta2, rep.eta3, rep.two_body_decay,
                          rep.three_body_weight, rep.three_body_decay, rep.rcut)
    types = ops.element_types(X, Z, nat, rep.species)
    fargs = (X, types, None, None, aid, mid, nat, rep.Rs2, rep.Rs3, prm)
    rep_t = ops.fchl_forward(*fargs)
    g_rep = torch.randn_like(rep_t)
    t_fwd = timed(lambda: ops.fchl_forward(*fargs))
    t_vjp = timed(lambda: ops.fchl_vjp(g_rep, *fargs))
    nn = n - 1                                              # every atom of the 7 A box is within rcut 6
    exp_fwd = A * (nn * 24 + nn * (nn - 1) // 2 * 20)
    kernels = {}
    kernels["fchl19_forward"] = {"seconds": t_fwd, "bound": "valu", "exp_per_s": exp_fwd / t_fwd,
                                 "hbm_GBs": A * R * 4 / t_fwd / 1e9}
    kernels["fchl19_vjp"] = {"seconds": t_vjp, "bound": "valu", "exp_per_s": exp_fwd / t_vjp,
                             "hbm_GBs": A * R * 4 / t_vjp / 1e9}

    flat_rep = rep_t.view(B * n, R)
    alpha32 = model.alpha.float()
    norm = float(np.sqrt(NPCAS) / SIGMA)
    t_fused = 0.0
    t_sorf = t_cos = t_cosb = t_adj = 0.0
    big = {"atoms": 0}          # the launches of the element with the most atoms: what the profiler's per-launch bytes refer to
    for ei, e in enumerate(SPECIES):
        idx = model._element_index(data, data['charges'], e)
        sub = torch.matmul(flat_rep.index_select(0, idx), model.reductors[ei])
        Ae = sub.shape[0]
        # the reference's two-op contract, kernel by kernel (coefficients materialised)
        molidx = torch.div(idx, n, rounding_mode='floor').to(torch.int32)
        te_sorf = timed(lambda: ops.sorf_forward(sub, model.Dmat[ei], norm, 1))
        coeffs = ops.sorf_forward(sub, model.Dmat[ei], norm, 1).view(Ae, F)
        te_cos = timed(lambda: ops.cos_features(coeffs, model.bias[ei], B, molidx))
        gZ = alpha32[None, :].expand(B, F).contiguous()
        te_cosb = timed(lambda: ops.cos_features_backward(gZ, coeffs, model.bias[ei], B, molidx))
        gc = ops.cos_features_backward(gZ, coeffs, model.bias[ei], B, molidx).view(Ae, NSTACKS, NPCAS)
        te_adj = timed(lambda: ops.sorf_adjoint(gc, model.Dmat[ei], norm, 1))
        del coeffs, gc
        t_sorf, t_cos, t_cosb, t_adj = t_sorf + te_sorf, t_cos + te_cos, t_cosb + te_cosb, t_adj + te_adj
        if Ae > big["atoms"]:
            big = {"atoms": Ae, "element": int(e), "sorf": te_sorf, "cos": te_cos, "cosb": te_cosb, "adj": te_adj}
    d = NPCAS
    log2d = int(np.log2(d))
    # the predict step's own launches: sort by element, projection (and its transpose), fused kernel
    ne = len(SPECIES)
    slots = mid * n + aid
    tflat = types.view(-1)
    ss, off = ops.sort_by_type(tflat, slots, ne)
    x_sorted = ops.project_typed(flat_rep, ss, off, model.reductors)
    gx_sorted = torch.randn_like(x_sorted)
    t_sort = timed(lambda: ops.sort_by_type(tflat, slots, ne))
    t_proj = timed(lambda: ops.project_typed(flat_rep, ss, off, model.reductors))
    t_projb = timed(lambda: ops.project_typed_backward(gx_sorted, ss, off, model.reductors, tflat, B * n))
    t_fused = timed(lambda: ops.sorf_energy_sorted(x_sorted, off, ss, model.Dmat, model.bias, alpha32, norm, 1, B * n))
    proj_flops = 2.0 * A * R * d
    kernels["sort_by_type"] = {"seconds": t_sort, "bound": "latency"}
    # Both projections multiply fp32 operands split into two fp16 parts: three v_mfma_f32_32x32x16_f16 per
    # product term (hi.hi + hi.lo + lo.hi).  `TFLOPs` counts the algorithmic 2.R.d per atom, `executed_TFLOPs`
    # the three-fold matrix work the fp16 pipe does, and `frac` divides THAT by the fp16 peak; the split
    # itself is vector work, so the kernels sit well below either ceiling (`mfma_busy` in profiles/).
    for key, tk in (("project_typed", t_proj), ("project_typed_backward", t_projb)):
        kernels[key] = {"seconds": tk, "bound": "mfma", "pipe": "fp16 matrix cores (v_mfma_f32_32x32x16_f16), fp32 operands "
                        "split in two fp16 parts, fp32 accumulation; the splits run on the vector unit",
                        "TFLOPs": proj_flops / tk / 1e12, "executed_TFLOPs": 3.0 * proj_flops / tk / 1e12,
                        "peak_TFLOPs": FP16_PEAK_TFLOPS, "frac": 3.0 * proj_flops / tk / 1e12 / FP16_PEAK_TFLOPS,
                        "algorithmic_bytes": float(A * 4 * (R + d)), "GBs": A * 4 * (R + d) / tk / 1e9,
                        "frac_hbm": A * 4 * (R + d) / tk / 1e9 / HBM_PEAK_GBS}
    # fused kernel, algorithmic flops per atom: forward+adjoint butterflies 2*F*log2(d), D multiplies 2F,
    # scale+bias FMA 2F, one sin and one cos per feature 2F, energy FMA 2F, alpha*norm*sin 2F
    fused_flops = A * F * (2 * log2d + 10)
    # 162 vector instructions per wavefront and stack in the kernel's main loop at d = 128 (8 coefficients
    # per lane; counted in its ISA): 82 plain fp32, 64 DPP butterflies, 8 v_sin_f32 + 8 v_cos_f32
    kernels["sorf_energy_fused"] = {"seconds": t_fused, "bound": "valu", "TFLOPs": fused_flops / t_fused / 1e12,
                                    "sincos_per_s": A * F / t_fused,
                                    "valu_wave_instr_per_s": 162.0 / 8.0 * A * F / 64 / t_fused}
    # the two-operator contract, kernel by kernel: `seconds` and the bytes are those of ONE launch, the
    # element with the most atoms (the launch the profiler's per-dispatch counters describe);
    # `seconds_all_elements` sums the launches of the three elements of one step
    Ab = big["atoms"]
    for key, tk, tall, nbytes in (("sorf_forward", "sorf", t_sorf, Ab * (4 * d + 4 * F)),
                                  ("cos_features_f32", "cos", t_cos, Ab * 4 * F + B * 8 * F),
                                  ("cos_features_backward", "cosb", t_cosb, Ab * 8 * F),
                                  ("sorf_adjoint", "adj", t_adj, Ab * (4 * F + 4 * d))):
        kernels[key] = {"seconds": big[tk], "bound": "hbm", "atoms": Ab, "element": big["element"],
                        "algorithmic_bytes": float(nbytes), "GBs": nbytes / big[tk] / 1e9,
                        "frac": nbytes / big[tk] / 1e9 / HBM_PEAK_GBS, "seconds_all_elements": tall}

    # ---- Z^T Z / Z^T y for 1000 molecules with forces --------------------------------------
    train = {}
    if not args.no_train:
        rng = np.random.default_rng(14)
        tc, tq = coords[:NMOL_TRAIN], charges[:NMOL_TRAIN]
        Et = rng.normal(size=NMOL_TRAIN)
        Ft = [rng.normal(size=(21, 3)) for _ in range(NMOL_TRAIN)]
        model.build_Z_components(tc[:64], tq[:64], E=Et[:64], F=Ft[:64], print_info=False)   # warm-up
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for b0 in range(0, NMOL_TRAIN, 500):                 # the host formatting the build repeats per batch
            model.format_data(tc[b0:b0 + 500], tq[b0:b0 + 500], E=Et[b0:b0 + 500], F=Ft[b0:b0 + 500])
        torch.cuda.synchronize()
        t_format = time.perf_counter() - t0
        t0 = time.perf_counter()
        ZTZ, ZTy = model.build_Z_components(tc, tq, E=Et, F=Ft, print_info=False)
        torch.cuda.synchronize()
        t_build = time.perf_counter() - t0
        # the same training set handed over as zero-padded arrays (X [N,n,3], Q [N,n], E [N], F [N,n,3]):
        # the formatter then uploads the arrays as they are and everything else happens on the device
        Xp = np.ascontiguousarray(np.stack(tc), dtype=np.float32)
        Qp = np.ascontiguousarray(np.stack(tq), dtype=np.float32)
        Fp = np.stack(Ft)
        model.format_data(Xp[:64], Qp[:64], E=Et[:64], F=Fp[:64])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for b0 in range(0, NMOL_TRAIN, 500):
            model.format_data(Xp[b0:b0 + 500], Qp[b0:b0 + 500], E=Et[b0:b0 + 500], F=Fp[b0:b0 + 500])
        torch.cuda.synchronize()
        t_format_padded = time.perf_counter() - t0
        t0 = time.perf_counter()
        ZTZp, ZTyp = model.build_Z_components(Xp, Qp, E=Et, F=Fp, print_info=False)
        torch.cuda.synchronize()
        t_build_padded = time.perf_counter() - t0
        padded_equal = bool(torch.equal(ZTZp, ZTZ))
        del ZTZp, ZTyp
        # one 500-molecule batch of that build, phase by phase (each timed alone, so their sum exceeds the
        # batch's share of the build, where the host runs ahead of the device)
        bd = model.format_data(tc[:500], tq[:500], E=Et[:500], F=Ft[:500])
        t_rep = timed(lambda: model.rep.get_representation_and_derivative(
            bd['coordinates'], bd['charges'], bd['atomIDs'], bd['molIDs'], bd['natom_counts'], bd['cells'], bd['inv_cells']), iters=3)
        t_proj = timed(lambda: model._batch_projected(bd, True), iters=3)
        proj = model._batch_projected(bd, True)
        t_rows = timed(lambda: model._rows_from_projected(proj, True), iters=3)
        brow = model._rows_from_projected(proj, True)
        btar = model._targets(bd, 500, True, True)
        bz = torch.zeros(F, F, dtype=torch.float64, device=dev)
        by = torch.zeros(F, 1, dtype=torch.float64, device=dev)
        t_bgram = timed(lambda: ops.gram(brow, btar, bz, by, mirror=False), iters=2)
        batch_phases = {"molecules": 500, "rows": int(brow.shape[0]), "format_data_ms": t_format / (NMOL_TRAIN / 500) * 1e3,
                        "representation_and_jacobian_ms": t_rep * 1e3, "projection_of_all_rows_ms": (t_proj - t_rep) * 1e3,
                        "feature_rows_ms": t_rows * 1e3, "gram_ms": t_bgram * 1e3}
        del bd, proj, brow, btar, bz, by
        # the step after the build: (Z^T Z + lambda I) alpha = Z^T y by the library's blocked
        # Cholesky, with the torch (rocSOLVER) factorisation of the same matrix beside it
        solve = {}
        if not args.no_solve:
            solve = bench_solve(torch, ops, timed, ZTZ, ZTy, F)
        del ZTZ, ZTy
        # the Gram kernel alone, at the full training shape
        M = NMOL_TRAIN * (1 + 3 * n)
        rows = torch.randn(M, F, dtype=torch.float64, device=dev)
        yv = torch.randn(M, 1, dtype=torch.float64, device=dev)
        ZTZ = torch.zeros(F, F, dtype=torch.float64, device=dev)
        ZTy = torch.zeros(F, 1, dtype=torch.float64, device=dev)
        t_gram = timed(lambda: ops.gram(rows, yv, ZTZ, ZTy), iters=2)
        gram_flops = float(M) * F * (F + 1) + 2.0 * M * F
        kernels["gram_f64"] = {"seconds": t_gram, "bound": "mfma", "TFLOPs": gram_flops / t_gram / 1e12,
                               "frac": gram_flops / t_gram / 1e12 / FP64_PEAK_TFLOPS}
        # half the width: 64 x 64 tiles, whose 28 strictly-upper super-tiles do not divide by the 8 XCDs
        rows_h = rows[:32000, :F // 2].contiguous()
        ZTZ_h = torch.zeros(F // 2, F // 2, dtype=torch.float64, device=dev)
        t_gram_h = timed(lambda: ops.gram(rows_h, None, ZTZ_h, None), iters=3)
        fl_h = 32000.0 * (F // 2) * (F // 2 + 1)
        kernels["gram_f64_half_width"] = {"seconds": t_gram_h, "bound": "mfma", "rows": 32000, "features": F // 2,
                                          "TFLOPs": fl_h / t_gram_h / 1e12, "frac": fl_h / t_gram_h / 1e12 / FP64_PEAK_TFLOPS}
        del rows_h, ZTZ_h
        train = {"ztz_seconds": t_build, "ztz_molecules": NMOL_TRAIN, "ztz_rows": M, "ztz_features": F,
                 "ztz_includes": "host format_data + FCHL19 Jacobian + projection + SORF rows + Gram, 500 molecules per batch",
                 "ztz_seconds_excluding_format_data": t_build - t_format, "format_data_seconds": t_format,
                 "gram_kernel_seconds": t_gram, "one_batch_phases": batch_phases,
                 "from_padded_arrays": {"ztz_seconds": t_build_padded, "format_data_seconds": t_format_padded,
                                        "ztz_bit_equal_to_list_route": padded_equal}}
        train.update(solve)
        if solve:
            kernels["cholesky_solve_f64"] = {"seconds": solve["solve_seconds"], "bound": "mfma",
                                             "TFLOPs": solve["solve_TFLOPs"],
                                             "frac": solve["solve_TFLOPs"] / FP64_PEAK_TFLOPS}
        del rows, yv, ZTZ, ZTy

    # HBM-side bytes per launch come from separate rocprofv3 --pmc runs of this script (they
    # cannot be read from inside it); the committed summary is attached when present
    traffic = {}
    tpath = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath))
    for k in kernels:
        if k in traffic:
            kernels[k]["traffic_bytes"] = traffic[k]["read_bytes"] + traffic[k]["written_bytes"]

    # every fraction against the ceiling measured on this device as well as the nominal one
    exp_nominal = 1024 * 64 / 8.0 * 2.4e9           # 1024 SIMDs, one 64-lane v_exp_f32 per 8 clocks (a quarter of the plain fp32 rate)
    for k, v in kernels.items():
        if v["bound"] == "hbm" and "GBs" in v:
            v["frac_of_measured"] = v["GBs"] / max(peaks["hbm_fill_GBs"], peaks["hbm_copy_GBs"])
        elif v["bound"] == "mfma":
            if "executed_TFLOPs" in v:          # split-fp16 products: executed matrix work over the measured fp16 rate
                v["frac_of_measured"] = v["executed_TFLOPs"] / peaks["mfma_f16_TFLOPs"]
                v["frac_hbm_of_measured"] = v["GBs"] / max(peaks["hbm_fill_GBs"], peaks["hbm_copy_GBs"])
            else:
                v["frac_of_measured"] = v["TFLOPs"] / peaks["mfma_f64_TFLOPs"]
        elif "exp_per_s" in v:
            v["frac"] = v["exp_per_s"] / exp_nominal
            v["frac_of_measured"] = v["exp_per_s"] / peaks["exp_per_s"]
    kernels["sorf_energy_fused"]["frac"] = kernels["sorf_energy_fused"]["TFLOPs"] / FP32_PEAK_TFLOPS
    # a wavefront of the fused kernel carries four atoms through one stack per iteration: its time per
    # wavefront-stack per SIMD against the bare instruction mix of such an iteration (probe kernel)
    wave_stacks_per_simd = (A / 4.0) * NSTACKS / 1024.0
    kernels["sorf_energy_fused"]["ns_per_wavefront_stack_per_simd"] = t_fused / wave_stacks_per_simd * 1e9
    kernels["sorf_energy_fused"]["instruction_mix_ns"] = instruction_mixes["fused_kernel_stack_ns"]
    kernels["sorf_energy_fused"]["frac_of_instruction_mix"] = (
        instruction_mixes["fused_kernel_stack_ns"] / kernels["sorf_energy_fused"]["ns_per_wavefront_stack_per_simd"])
    kernels["sorf_energy_fused"]["sincos_frac_of_measured_exp_rate"] = (
        2.0 * kernels["sorf_energy_fused"]["sincos_per_s"] / peaks["exp_per_s"])
    dominant = max(("fchl19_forward", "fchl19_vjp", "sorf_energy_fused"), key=lambda k: kernels[k]["seconds"])
    if dominant == "sorf_energy_fused":
        roofline = {"kernel": dominant, "bound": "valu", "achieved": kernels[dominant]["TFLOPs"],
                    "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": kernels[dominant]["TFLOPs"] / FP32_PEAK_TFLOPS,
                    "frac_of_instruction_mix": kernels[dominant]["frac_of_instruction_mix"],
                    "traffic": kernels[dominant].get("traffic_bytes"),
                    "note": "fused FWHT+sincos kernel: neither HBM nor MFMA bounds it (8d bytes per atom, no "
                            "contraction); it is bound by vector instruction issue.  Algorithmic flops count one "
                            "flop per sin and per cos and per butterfly add, while a butterfly across lanes issues "
                            "at half rate and v_sin/v_cos at quarter rate, none of them an FMA, so the fraction of "
                            "the fp32 FMA peak understates it: frac_of_instruction_mix is the time a probe kernel needs for the "
                            "bare instruction mix of one wavefront-stack (82 plain + 64 DPP + 16 transcendental, independent "
                            "registers, no memory access) over the kernel's own time per wavefront-stack, both measured in this run; "
                            "traffic = bytes per launch from profiles/pmc_traffic.json"}
    else:
        roofline = {"kernel": dominant, "bound": "valu", "achieved": kernels[dominant]["exp_per_s"] / 1e12,
                    "peak": exp_nominal / 1e12, "unit": "Texp/s", "frac": kernels[dominant]["exp_per_s"] / exp_nominal,
                    "frac_of_measured": kernels[dominant]["frac_of_measured"], "traffic": None}

    out = {
        "metric": "molecules/s (FCHL19+SORF energy+force predict); Z^T Z build time, 16384 feats",
        "value": value, "unit": "molecules/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 (projection/RFF products: split-fp16 operands, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "config 2: 4096 x C9H8O4 (21 atoms), species {1,6,8}, FCHL19 rcut 6 "
                               "nRs2 24 nRs3 20, SORF npcas 128 x nstacks 128 = 16384 features, energies + forces",
                   "molecules_per_step": B, "atoms_per_step": A},
        "roofline": roofline,
        "peaks_measured": peaks,
        "instruction_mixes": instruction_mixes,
        "autograd_route": autograd_route,
        "two_op_route": two_op_route,
        "from_host_arrays": from_host,
        "kernels": kernels,
        "step_kernels_sum_ms": 1e3 * sum(kernels[k]["seconds"] for k in ("fchl19_forward", "sort_by_type", "project_typed",
                                                                        "sorf_energy_fused", "project_typed_backward",
                                                                        "fchl19_vjp")),
        "step_kernels_sum_note": "the step's kernels timed one at a time (several launches of one kernel in a row between two "
                                 "HIP events); inside the step they overlap at their boundaries (a kernel's last workgroups "
                                 "run beside the next kernel's first) and run at the clock of the whole step, so this sum "
                                 "exceeds ms_per_step, which is the measured quantity",
    }
    out.update(train)
    if "gram_f64" in kernels:
        g = kernels["gram_f64"]
        out["roofline_ztz"] = {"kernel": "gram_f64", "bound": "mfma", "achieved": g["TFLOPs"], "peak": FP64_PEAK_TFLOPS,
                               "unit": "TFLOP/s", "frac": g["frac"], "frac_of_measured": g["frac_of_measured"],
                               "peak_measured": peaks["mfma_f64_TFLOPs"], "traffic": g.get("traffic_bytes")}
    if not args.no_other_configs:
        torch.cuda.empty_cache()
        try:
            out["other_configs"] = other_configs(torch, dev)
        except Exception as exc:   # the headline line must survive a failure here
            out["other_configs"] = {"error": repr(exc)}

    c1 = out.get("other_configs", {}).get("config1_c6h6_100")
    E1 = c1.pop("_E", None) if isinstance(c1, dict) else None
    F1 = c1.pop("_F", None) if isinstance(c1, dict) else None
    if cpu_c1 is not None:
        # configuration 1 is the CPU-reference configuration: the oracle on all of it, and the GPU
        # result of the same 100 molecules checked against it
        out["cpu_baseline_c1"] = {"value": 100.0 / cpu_c1["seconds"], "unit": "molecules/s", "cores": cpu_c1["cores"],
                                  "kind": "port", "seconds": cpu_c1["seconds"],
                                  "sample": "configuration 1 in full: 100 noisy C6H6 (12 atoms), species {1,6}, npcas 64 x "
                                            "nstacks 8 = 512 features, energies + forces, fp64 NumPy oracle"}
        if E1 is not None:
            out["cpu_baseline_c1"]["gpu_molecules_per_s"] = c1["molecules_per_s"]
            out["parity_vs_oracle_c1"] = {
                "energy_rel_err": float(np.abs(E1 - cpu_c1["E"]).max() / np.abs(cpu_c1["E"]).max()),
                "force_rel_err": float(np.abs(F1 - cpu_c1["F"]).max() / np.abs(cpu_c1["F"]).max()), "molecules": 100}
    if cpu is not None:
        rate, nsamp, secs, res, chunks, cores = cpu
        # the sample doubles as a parity check of this very run
        Eg = E.detach().double().cpu().numpy()
        Fg = Fr.double().cpu().numpy()
        e_err = f_err = 0.0
        e_scale = f_scale = 1e-30
        for ci, (Ec, Fc) in enumerate(res):
            ids = list(range(ci, args.cpu_sample, cores))[:len(Ec)]
            e_err = max(e_err, np.abs(Eg[ids] - Ec).max())
            f_err = max(f_err, np.abs(Fg[ids] - Fc).max())
            e_scale = max(e_scale, np.abs(Ec).max())
            f_scale = max(f_scale, np.abs(Fc).max())
        out["cpu_baseline"] = {"value": rate, "unit": "molecules/s", "cores": cores, "kind": "port",
                               "sample": "%d molecules of the same batch, energies + forces, fp64 NumPy oracle, "
                                         "%d processes, %.1f s" % (nsamp, cores, secs)}
        out["parity_vs_oracle"] = {"energy_rel_err": e_err / e_scale, "force_rel_err": f_err / f_scale,
                                   "molecules": nsamp}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
