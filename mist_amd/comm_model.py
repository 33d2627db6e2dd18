"""Host-side scalar forms of the reference's alpha-beta communication models.

Used only to build per-(micro-batch, tp) input tables (tensor-parallel collective extras inside
the op latencies, pre/post layer collectives); the per-candidate evaluation runs in the HIP
kernels.  Follows mist/tools/optimize.py:201-303 (GPU<->GPU) and :459-470 (CPU<->GPU).
"""
from __future__ import annotations

from typing import Optional, Sequence

OP_FACTORS = {"all_reduce": 2.1, "all_gather": 1.0, "reduce_scatter": 1.1, "none": 0.0}


def _table_index(size: float) -> int:
    # optimize.py:277-297: 1,2,4,8 -> 0..3, anything above 8 -> 3.
    if size == 1:
        return 0
    if size == 2:
        return 1
    if size == 4:
        return 2
    if size >= 8:
        return 3
    raise ValueError(f"communication group size {size} is not one of 1, 2, 4, >=8")


def gpu_gpu_comm_latency(
    op_name: str,
    gbytes: float,
    inter_size: Optional[float],
    intra_size: Optional[float],
    gpu_gpu_comm_params: Sequence[float],
) -> float:
    """optimize.py:201-254. ``gpu_gpu_comm_params`` is the flat 32-vector
    [(k GB/s, b s) for inter in 1,2,4,8 for intra in 1,2,4,8]."""
    if len(gpu_gpu_comm_params) != 32:
        raise ValueError(f"Invalid size of gpu_gpu_comm_params: {len(gpu_gpu_comm_params)}")
    gbytes = float(gbytes)
    if op_name == "p2p":
        assert inter_size is None or intra_size is None
        if inter_size is not None:
            bandwidth = gpu_gpu_comm_params[(1 * 4 + 0) * 2]
        else:
            bandwidth = gpu_gpu_comm_params[(0 * 4 + 1) * 2]
        return gbytes / bandwidth
    if op_name not in OP_FACTORS:
        raise ValueError(f"Invalid op_name: {op_name}")
    intra = 1.0 if intra_size is None else float(intra_size)
    inter = 1.0 if inter_size is None else float(inter_size)
    ngpu = intra * inter
    if gbytes < 1e-5 or ngpu == 1:
        lat = 0.0
    else:
        cell = (_table_index(inter) * 4 + _table_index(intra)) * 2
        k = gpu_gpu_comm_params[cell]
        b = gpu_gpu_comm_params[cell + 1]
        lat = gbytes / k * (ngpu - 1) / ngpu + b
    return lat * OP_FACTORS[op_name]


def cpu_gpu_comm_latency(gbytes: float, params: Sequence[float]) -> float:
    """optimize.py:459-470."""
    k, b = params
    gbytes = float(gbytes)
    return 0.0 if gbytes == 0 else gbytes / k + b
