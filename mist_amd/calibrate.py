"""Hardware-parameter calibration on one MI355X: the single-GPU part of the reference's
``mist/tools/profile_interference.py`` (measurement) and ``mist/tools/optimize.py`` (fitting).

The reference times a half-precision matmul, an all-gather, a host-to-device copy and a
device-to-host copy issued together on four streams over a grid of sizes, then fits

* ``gpu_gpu_comm_params`` (32 values) from the all-gather-only cases,
* ``cpu_gpu_comm_params`` / ``gpu_cpu_comm_params`` ((GB/s, s) each) from the copy-only cases,
* ``interference_model_params`` (28 factors) from the overlapped cases, mask by mask.

With one GPU there is no all-gather: this module measures the (compute, host-to-device,
device-to-host) part of the grid, writes the reference's result-file schema (so either side's
fitter reads either side's file) and fits what those cases determine: both copy models and the
9 interference factors of the masks without the GPU-to-GPU resource.  The other 19 factors and
the 32 collective parameters are reported as not measured.

Measurement uses torch for the matmul, the pinned host buffers and the streams, as the
reference does; every stream keeps the default priority.
"""
from __future__ import annotations

import argparse
import json
import time
from itertools import product
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .stage_inputs import THREE_CASE_MASKS, TWO_CASE_MASKS, interference_factor_table

COMPUTE_M = 4096          # profile_interference.py:119-123
COMPUTE_K = 4096
MB = 1024 ** 2
BASE_TIME_MSEC = 3
RATIOS = (0, 1, 2, 3, 4)
UP_BOUND = 50             # optimize.py:19, upper bound of an interference factor
ONLY_COMM_MBYTES = tuple(32 * n for n in range(2, 17))  # profile_interference.py:368

# Which of the 28 factors the cases without a GPU-to-GPU transfer determine: index ranges in the
# parameter vector [4-way (4) | 3-way (4 masks x 3) | 2-way (6 masks x 2)].
RESOURCES = ("compute", "gpu_gpu", "cpu_to_gpu", "gpu_to_cpu")


def mask_slice(mask: Sequence[bool]) -> slice:
    """Positions of a mask's factors in the 28-vector (optimize.py:1125-1159)."""
    mask = tuple(bool(m) for m in mask)
    n = sum(mask)
    if n == 4:
        return slice(0, 4)
    if n == 3:
        start = 4 + 3 * THREE_CASE_MASKS.index(mask)
        return slice(start, start + 3)
    if n == 2:
        start = 16 + 2 * TWO_CASE_MASKS.index(mask)
        return slice(start, start + 2)
    raise ValueError(f"a mask needs 2 to 4 resources, got {mask}")


SINGLE_GPU_MASKS = tuple(m for m in TWO_CASE_MASKS + THREE_CASE_MASKS if not m[1])


# ------------------------------------------------------------------------------ models (host)
def cpu_gpu_latency(gbytes, params) -> np.ndarray:
    """optimize.py:465-470: ``gbytes / k + b``, 0 for an empty transfer."""
    k, b = params
    gbytes = np.asarray(gbytes, dtype=np.float64)
    return np.where(gbytes == 0, 0.0, gbytes / k + b)


def interference_estimate(C, G2G, C2G, G2C, params) -> np.ndarray:
    """optimize.py:1012-1079: total time of the four resources running together.  Mask by mask
    (4-way, 3-way, 2-way), rows whose non-zero pattern equals the mask overlap for
    ``min(x * f)`` and keep ``(x * f - overlap) / f`` of each resource; what is left at the end
    runs alone."""
    X = np.stack(np.broadcast_arrays(
        *[np.atleast_1d(np.asarray(a, dtype=np.float64)) for a in (C, G2G, C2G, G2C)]), axis=1).copy()
    out = np.zeros(X.shape[0])
    table = interference_factor_table(params)
    masks = [(True,) * 4] + list(THREE_CASE_MASKS) + list(TWO_CASE_MASKS)
    for mask, factors in zip(masks, table):
        mask = np.array(mask)
        nonzero = np.logical_not(np.isclose(X, 0))
        rows = np.where(np.all(nonzero == mask, axis=1))[0]
        if len(rows) == 0:
            continue
        scaled = X[rows] * factors
        overlap = scaled[:, mask].min(axis=1)
        left = (scaled - overlap[:, None]) / factors
        X[np.ix_(rows, np.where(mask)[0])] = left[:, mask]
        out[rows] += overlap
    return out + X.sum(axis=1)


# ------------------------------------------------------------------------------ result files
def case_name(n: int, g2g: int, c2g: int, g2c: int, world: int = 1, intra: int = 1, inter: int = 1) -> str:
    """profile_interference.py:166."""
    return (f"N_{n}-M_{COMPUTE_M}-K_{COMPUTE_K}-G2G_{g2g}-C2G_{c2g}-G2C_{g2c}-"
            f"W_{world}-Intra_{intra}-Inter_{inter}")


def _seconds(text) -> float:
    """optimize.py:26-33."""
    if isinstance(text, (int, float)):
        return float(text)
    if "ms" in text:
        return float(text.replace("ms", "")) / 1000
    if "s" in text:
        return float(text.replace("s", ""))
    return float(text)


def preprocess_data(cases: Dict[str, dict]):
    """optimize.py:36-102 on the cases of one device: arrays (latency s, compute_n, compute-only
    latency s, G2G GB, C2G GB, G2C GB, intra, inter).  Cases noisier than std/mean 0.1 are
    skipped; the compute latency of a case is the measured latency of its compute-only case."""
    cols: List[List[float]] = [[] for _ in range(8)]
    for value in cases.values():
        latency = _seconds(value["latency"])
        latency = latency if latency > 1e-5 else 0.0
        if float(value["std/mean"]) > 0.1:
            continue
        n = int(value["compute_n"])
        world, intra, inter = (int(value[k]) for k in ("world_size", "intra_group_size", "inter_group_size"))
        alone = case_name(n, 0, 0, 0, world, intra, inter)
        if alone in cases:
            compute = _seconds(cases[alone]["latency"])
            compute = compute if compute > 1e-5 else 0.0
        elif n == 0:
            compute = 0.0
        else:
            raise ValueError(f"Entry {alone} not found in the data")
        row = (latency, n, compute, int(value["gpu_to_gpu_mbytes"]) / 1024,
               int(value["cpu_to_gpu_mbytes"]) / 1024, int(value["gpu_to_cpu_mbytes"]) / 1024, intra, inter)
        for col, v in zip(cols, row):
            col.append(v)
    return tuple(np.array(c, dtype=np.float64) for c in cols)


# ------------------------------------------------------------------------------ fitting
def fit_cpu_gpu_params(data) -> Tuple[np.ndarray, np.ndarray]:
    """optimize.py:473-549: least squares of ``gbytes / k + b`` over the copy-only cases of each
    direction with ``k >= 0.1`` GB/s and ``b >= 0``.  The reference hands this to
    ``scipy.optimize.minimize`` from (6 GB/s, 0 s); on second-scale latencies its default
    tolerances end the search far from the minimum.  The model is linear in ``(1 / k, b)``, so
    the same objective is minimised in closed form here.  Returns (c2g, g2c) params."""
    L, N, C, G2G, C2G, G2C, _, _ = data
    out = []
    for own, other in ((C2G, G2C), (G2C, C2G)):
        pick = (own != 0) & (N == 0) & (G2G == 0) & (other == 0)
        if not pick.any():
            raise ValueError("no copy-only cases in the data")
        lat, gb = L[pick], own[pick]
        design = np.stack([gb, np.ones_like(gb)], axis=1)
        (slope, offset), *_ = np.linalg.lstsq(design, lat, rcond=None)
        if offset < 0 or len(gb) == 1:  # bound b >= 0 active: best slope through the origin
            slope, offset = float(gb @ lat / (gb @ gb)), 0.0
        slope = min(max(slope, 1e-12), 1.0 / 0.1)  # k >= 0.1
        if slope == 1.0 / 0.1:
            offset = max(float(np.mean(lat - gb * slope)), 0.0)
        out.append(np.array([1.0 / slope, offset]))
    return out[0], out[1]


def interference_fitting_data(data, c2g_params, g2c_params, g2g_latency=None, remove_outliers=True):
    """optimize.py:105-180: per case the standalone latency of each resource (measured for the
    matmul, modelled for the transfers); cases with a single resource carry no interference
    and are dropped, and so are cases slower than running everything back to back."""
    L, _, C, G2G, C2G, G2C, _, _ = data
    g2g_lat = np.zeros_like(L) if g2g_latency is None else np.asarray(g2g_latency, dtype=np.float64)
    if g2g_latency is None and np.any(G2G != 0):
        raise ValueError("cases with a GPU-to-GPU transfer need its modelled latency")
    c2g_lat, g2c_lat = cpu_gpu_latency(C2G, c2g_params), cpu_gpu_latency(G2C, g2c_params)
    zeros = sum(np.isclose(x, 0).astype(int) for x in (C, g2g_lat, c2g_lat, g2c_lat))
    keep = zeros < 3
    if remove_outliers:
        keep &= L <= C + g2g_lat + c2g_lat + g2c_lat
    return L[keep], C[keep], g2g_lat[keep], c2g_lat[keep], g2c_lat[keep]


def fit_interference(fit_data, masks=SINGLE_GPU_MASKS) -> Tuple[np.ndarray, Dict[tuple, dict]]:
    """optimize.py:1162-1240, mask by mask: the cases whose resources are exactly the mask's
    determine that mask's factors (least squares on the total time, bounds [1, UP_BOUND]; the
    reference starts one L-BFGS-B run at the number of resources).  Deviation: the reference fits
    a three-resource mask with every two-resource factor at 1 (``fit(*mask)`` passes no
    defaults) although the model it then evaluates peels the remaining pair with the fitted
    two-resource factors; here a mask is fitted with the factors found so far in place, so the
    fitted model is the evaluated one.  Factors of masks that are not fitted stay 1.  Returns the
    28-vector and per mask ``{"params", "cases", "mean_error"}``."""
    from scipy.optimize import minimize

    L, C, G2G, C2G, G2C = fit_data
    X = np.stack([C, G2G, C2G, G2C], axis=1)
    nonzero = np.logical_not(np.isclose(X, 0))
    params = np.ones(28)
    report: Dict[tuple, dict] = {}
    for mask in masks:
        mask = tuple(bool(m) for m in mask)
        rows = np.where(np.all(nonzero == np.array(mask), axis=1))[0]
        n = sum(mask)
        where = mask_slice(mask)
        if len(rows) == 0:
            # optimize.py:1184-1186 returns the resource count as every factor of such a mask
            params[where] = float(n)
            report[mask] = dict(params=[float(n)] * n, cases=0, mean_error=float("nan"))
            continue

        def predict(p, rows=rows, where=where):
            full = params.copy()  # the masks fitted so far (two resources before three)
            full[where] = p
            return interference_estimate(C[rows], G2G[rows], C2G[rows], G2C[rows], full)

        # the reference's objective (sum of squared errors in seconds); expressed in
        # milliseconds so that the optimiser's default tolerances mean something, and started
        # from a few points because the model is only piecewise smooth
        loss = lambda p, rows=rows: float(np.sum((1e3 * (L[rows] - predict(p))) ** 2))
        best = None
        for start in (float(n), 1.0, 1.5, 2.5):
            result = minimize(loss, [start] * n, bounds=[(1.0, UP_BOUND)] * n, method="L-BFGS-B",
                              options=dict(ftol=1e-14, gtol=1e-10, maxiter=500))
            polished = minimize(loss, result.x, method="Nelder-Mead",
                                bounds=[(1.0, UP_BOUND)] * n, options=dict(xatol=1e-6, fatol=1e-14))
            for r in (result, polished):
                if best is None or r.fun < best.fun:
                    best = r
        params[where] = best.x
        err = np.abs(L[rows] - predict(best.x)) / L[rows]
        report[mask] = dict(params=[float(v) for v in best.x], cases=int(len(rows)),
                            mean_error=float(err.mean()))
    return params, report


def fit(cases: Dict[str, dict]) -> dict:
    """Everything the cases of one device determine, as a dict with the hardware-section names."""
    data = preprocess_data(cases)
    c2g, g2c = fit_cpu_gpu_params(data)
    has_g2g = bool(np.any(data[3] != 0))
    if has_g2g:
        raise NotImplementedError(
            "the data holds GPU-to-GPU cases: fitting the 32 collective parameters is not part of "
            "the single-GPU calibration")
    fit_data = interference_fitting_data(data, c2g, g2c)
    params, report = fit_interference(fit_data)
    L, C, G2G, C2G, G2C = fit_data
    err = np.abs(L - interference_estimate(C, G2G, C2G, G2C, params)) / L if len(L) else np.array([])
    return dict(
        cpu_gpu_comm_params=[float(v) for v in c2g],
        gpu_cpu_comm_params=[float(v) for v in g2c],
        interference_model_params=[float(v) for v in params],
        fitted_interference_indices=sorted(
            i for m in SINGLE_GPU_MASKS if report[m]["cases"] for i in range(*mask_slice(m).indices(28))),
        not_measured=["gpu_gpu_comm_params (32 values: needs a collective between GPUs)",
                      "interference factors of the 7 masks with a GPU-to-GPU transfer (19 values)"],
        masks={"+".join(r for r, on in zip(RESOURCES, m) if on): v for m, v in report.items()},
        cases=int(len(data[0])), overlapped_cases=int(len(L)),
        mean_error=float(err.mean()) if len(err) else float("nan"),
    )


# ------------------------------------------------------------------------------ measurement
def _round_up(x: float, v: int = 8) -> int:
    return int(-(-x // v) * v)  # profile_interference.py:77-78


def sweep(compute_tflops: float, copy_gbps: float, overlap: bool = True):
    """The reference's grid without its GPU-to-GPU axis (profile_interference.py:367-412):
    copy-only cases of 64..512 MB, and the product of sizes that take 0, 3, 6, 9, 12 ms alone at
    the given reference rates."""
    n_cand, mb_cand = [], []
    for ratio in RATIOS:
        sec = BASE_TIME_MSEC * ratio * 1e-3
        n_cand.append(_round_up(sec / (COMPUTE_M * COMPUTE_K / (compute_tflops * 1e12))))
        mb_cand.append(_round_up(sec / (1.0 / (copy_gbps * 1024))))
    choices = set()
    for mb in ONLY_COMM_MBYTES:
        choices.add((0, mb, 0))
        choices.add((0, 0, mb))
    if overlap:
        for n, c2g, g2c in product(n_cand, mb_cand, mb_cand):
            if n or c2g or g2c:
                choices.add((n, c2g, g2c))
    return sorted(choices, key=lambda c: -(c[1] + c[2]))


class Bench:
    """Buffers and streams of the measurement, allocated once for the largest case."""

    def __init__(self, device: str, max_n: int, max_mb: int):
        import torch

        self.torch, self.device = torch, torch.device(device)
        dtype = torch.float16
        self.streams = [torch.cuda.Stream(self.device) for _ in range(3)]  # compute, c2g, g2c
        numel = max(max_mb, 1) * MB // 2
        self.host_src = torch.empty(numel, dtype=dtype, pin_memory=True).normal_()
        self.dev_dst = torch.zeros(numel, dtype=dtype, device=self.device)
        self.dev_src = torch.zeros(numel, dtype=dtype, device=self.device)
        self.host_dst = torch.empty(numel, dtype=dtype, pin_memory=True)
        self.mat_a = torch.ones((max(max_n, 8), COMPUTE_K), dtype=dtype, device=self.device)
        self.mat_b = torch.ones((COMPUTE_K, COMPUTE_M), dtype=dtype, device=self.device)
        self.mat_out = torch.zeros((max(max_n, 8), COMPUTE_M), dtype=dtype, device=self.device)

    def run(self, n: int, c2g_mb: int, g2c_mb: int) -> None:
        torch = self.torch
        if g2c_mb > 0:
            with torch.cuda.stream(self.streams[2]):
                k = g2c_mb * MB // 2
                self.host_dst[:k].copy_(self.dev_src[:k], non_blocking=True)
        if c2g_mb > 0:
            with torch.cuda.stream(self.streams[1]):
                k = c2g_mb * MB // 2
                self.dev_dst[:k].copy_(self.host_src[:k], non_blocking=True)
        if n > 0:
            with torch.no_grad(), torch.cuda.stream(self.streams[0]):
                torch.matmul(self.mat_a[:n], self.mat_b, out=self.mat_out[:n])

    def time(self, n: int, c2g_mb: int, g2c_mb: int, warmup: int = 20, number: int = 10) -> np.ndarray:
        """Wall time of ``number`` issues, each between two device synchronisations."""
        torch = self.torch
        for _ in range(warmup):  # mist/utils/common.py:191-231: every issue is synchronised
            self.run(n, c2g_mb, g2c_mb)
            torch.cuda.synchronize(self.device)
        costs = []
        for _ in range(number):
            start = time.perf_counter()
            self.run(n, c2g_mb, g2c_mb)
            torch.cuda.synchronize(self.device)
            costs.append(time.perf_counter() - start)
        return np.array(costs)


def measure(device: str = "cuda:0", compute_tflops: Optional[float] = None,
            copy_gbps: Optional[float] = None, overlap: bool = True, warmup: int = 20,
            number: int = 10, progress=None) -> Dict[str, dict]:
    """Runs the sweep and returns the cases in the reference's result schema
    (profile_interference.py:310-331).  The two reference rates that size the sweep are measured
    first (a 8192-row matmul, a 256 MB copy) unless given."""
    probe = Bench(device, 8192, 256)
    if compute_tflops is None:
        t = probe.time(8192, 0, 0, 5, 5).mean()
        compute_tflops = 8192 * COMPUTE_M * COMPUTE_K / t / 1e12
    if copy_gbps is None:
        copy_gbps = 0.25 / probe.time(0, 256, 0, 3, 5).mean()
    del probe
    choices = sweep(compute_tflops, copy_gbps, overlap)
    bench = Bench(device, max(c[0] for c in choices), max(max(c[1], c[2]) for c in choices))
    cases: Dict[str, dict] = {}
    for i, (n, c2g, g2c) in enumerate(choices):
        costs = bench.time(n, c2g, g2c, warmup, number)
        mean, std = float(costs.mean()), float(costs.std())
        cases[case_name(n, 0, c2g, g2c)] = {
            "compute_n": str(n), "compute_m": str(COMPUTE_M), "compute_k": str(COMPUTE_K),
            "gpu_to_gpu_mbytes": "0", "cpu_to_gpu_mbytes": str(c2g), "gpu_to_cpu_mbytes": str(g2c),
            "latency": f"{mean * 1e3:.4f} ms", "std": f"{std * 1e3:.4f} ms", "std/mean": f"{std / mean:.4f}",
            "world_size": "1", "intra_group_size": "1", "inter_group_size": "1",
            "gflops": f"{n * COMPUTE_M * COMPUTE_K / (mean * 1e9):.2f} GFLOPS",
            "g2g_bandwidth": "0.00 GB/s", "c2g_bandwidth": f"{c2g / 1024 / mean:.2f} GB/s",
            "g2c_bandwidth": f"{g2c / 1024 / mean:.2f} GB/s",
        }
        if progress is not None and i % 20 == 0:
            progress(i, len(choices))
    return cases


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("--output", default=None, help="result file to write (reference schema)")
    parser.add_argument("--input", default=None, help="fit an existing result file instead of measuring")
    parser.add_argument("--device", default="cuda:0")
    parser.add_argument("--only-comm", action="store_true", help="copy-only cases, no overlap grid")
    args = parser.parse_args(argv)
    if args.input:
        with open(args.input) as f:
            results = json.load(f)
        name, cases = next(iter(results.items()))
    else:
        import torch

        name = torch.cuda.get_device_name(args.device).lower().replace(" ", "-")
        cases = measure(args.device, overlap=not args.only_comm,
                        progress=lambda i, n: print(f"case {i} of {n}", flush=True))
        if args.output:
            with open(args.output, "w") as f:
                json.dump({name: cases}, f, indent=1)
    fitted = fit(cases)
    print(json.dumps({name: fitted}, indent=1))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
