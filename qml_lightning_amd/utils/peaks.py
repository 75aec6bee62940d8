"""Measured ceilings of the GPU the library runs on, next to the nominal ones: fill and copy
bandwidth, fp64 / fp32 / fp16 matrix-core rate, transcendental rate.  Each probe is a few milliseconds
of the library's own probe kernels, timed with HIP events on the current stream."""
import ctypes

import torch

from .. import _lib
from ..ops import _ptr, _stream

NOMINAL = {"hbm_GBs": 8000.0, "mfma_f64_TFLOPs": 78.6, "mfma_f32_TFLOPs": 157.3, "mfma_f16_TFLOPs": 2500.0}


def _timed(fn, iters):
    fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters * 1e-3


def measure(nbytes=1 << 30, device="cuda:0"):
    """{'hbm_fill_GBs', 'hbm_copy_GBs' (bytes read + written), 'mfma_f64_TFLOPs',
    'mfma_f32_TFLOPs', 'mfma_f16_TFLOPs', 'exp_per_s'} of the current device."""
    L = _lib.lib()
    n = nbytes // 4
    src = torch.empty(n, dtype=torch.float32, device=device)
    dst = torch.empty(n, dtype=torch.float32, device=device)

    def fill():
        _lib.check(L.qmll_probe_fill(_ptr(src), n, 1.0, _stream()), "qmll_probe_fill")

    def copy():
        _lib.check(L.qmll_probe_copy(_ptr(src), _ptr(dst), n, _stream()), "qmll_probe_copy")

    out = {"hbm_fill_GBs": nbytes / _timed(fill, 10) / 1e9, "hbm_copy_GBs": 2.0 * nbytes / _timed(copy, 10) / 1e9}
    del src, dst
    scratch = torch.empty(int(L.qmll_probe_out_bytes()) // 8, dtype=torch.float64, device=device)
    # the best over 1, 2, 4 and 8 wavefronts per SIMD (the rate a loop of nothing but matrix or
    # transcendental instructions holds depends on how many wavefronts issue them)
    for key, which, iters, scale in (("mfma_f64_TFLOPs", 0, 1000, 1e12), ("mfma_f32_TFLOPs", 1, 4000, 1e12),
                                     ("mfma_f16_TFLOPs", 3, 4000, 1e12), ("exp_per_s", 2, 4000, 1.0)):
        best = 0.0
        for per_cu in (1, 2, 4, 8):
            ops = [0.0]

            def run():
                ops[0] = float(L.qmll_probe_rate(which, iters, per_cu, _ptr(scratch), _stream()))
                if ops[0] < 0:
                    _lib.check(-1, "qmll_probe_rate")
            t = _timed(run, 2)
            best = max(best, ops[0] / t / scale)
            out.setdefault(key + "_by_wavefronts_per_simd", {})[str(per_cu)] = ops[0] / t / scale
        out[key] = best
    return out


MIXES = ("plain_fp32_x128", "dpp_fmac_x128", "transcendental_x128", "fused_kernel_stack")


def instruction_mixes(device="cuda:0", iters=2000):
    """Seconds per wavefront-iteration per SIMD of each instruction mix of the library's probe
    (see qmll_probe_mix), at 1, 2, 4 and 8 wavefronts per SIMD: {'name': {'1': s, ...}}.  Times a
    clock frequency these are SIMD clocks per iteration; the ratios between mixes need no clock."""
    L = _lib.lib()
    scratch = torch.empty(int(L.qmll_probe_out_bytes()) // 8, dtype=torch.float64, device=device)
    out = {}
    for mix, name in enumerate(MIXES):
        out[name] = {}
        for per_cu in (1, 2, 4, 8):
            units = [0.0]

            def run():
                units[0] = float(L.qmll_probe_mix(mix, iters, per_cu, _ptr(scratch), _stream()))
                if units[0] < 0:
                    _lib.check(-1, "qmll_probe_mix")
            t = _timed(run, 2)
            out[name][str(per_cu)] = t / units[0]
    return out


if __name__ == "__main__":
    # python -m qml_lightning_amd.utils.peaks [mixes|peaks]: one JSON line (what a profiler run of the
    # probe kernels is pointed at)
    import json
    import sys
    import qml_lightning_amd  # noqa: F401
    what = sys.argv[1] if len(sys.argv) > 1 else "both"
    out = {}
    if what in ("peaks", "both"):
        out["peaks"] = measure()
    if what in ("mixes", "both"):
        out["instruction_mixes_seconds_per_wavefront_iteration"] = instruction_mixes()
    print(json.dumps(out))
