"""Oracle (test infrastructure): alpha-beta communication latency models, vectorised numpy.

Restates mist/tools/optimize.py:201-303 (``predict_gpu_gpu_comm_latency`` +
``_compute_comm_latency_impl``) and :459-470 (``predict_cpu_gpu_comm_latency``).

Pinned by: closed form; special cases ``n == 1 -> 0``, ``gbytes < 1e-5 -> 0``,
``all_reduce == 2.1 * all_gather``, ``reduce_scatter == 1.1 * all_gather``
(tests/test_oracle_models.py).
"""
import numpy as np

_FACTOR = {"all_reduce": 2.1, "all_gather": 1.0, "reduce_scatter": 1.1, "none": 0.0}


def _size_index(size):
    """optimize.py:277-297. Sizes other than 1, 2, 4, 8, >8 leave the index unset in the
    reference's compiled loop; they are rejected here."""
    size = np.asarray(size)
    idx = np.full(size.shape, -1, dtype=np.int64)
    idx[size == 1] = 0
    idx[size == 2] = 1
    idx[size == 4] = 2
    idx[size >= 8] = 3
    return idx


def gpu_gpu_only_latency(gbytes, intra_size, inter_size, params):
    """optimize.py:257-347: ``GB / k * (n - 1) / n + b`` per element, 0 where ``GB < 1e-5`` or
    ``n == 1``; (k, b) = params[idx(inter), idx(intra)]."""
    intra_size = 1 if intra_size is None else intra_size
    inter_size = 1 if inter_size is None else inter_size
    gbytes = np.atleast_1d(np.asarray(gbytes, dtype=np.float64))
    intra = np.atleast_1d(np.asarray(intra_size))
    inter = np.atleast_1d(np.asarray(inter_size))
    n = max(gbytes.size, intra.size, inter.size)
    gbytes = np.broadcast_to(gbytes, (n,))
    intra = np.broadcast_to(intra, (n,))
    inter = np.broadcast_to(inter, (n,))
    params = np.asarray(params, dtype=np.float64)
    assert params.size == 32, params.size
    params = params.reshape(4, 4, 2)
    ngpu = intra * inter
    zero = (gbytes < 1e-5) | (ngpu == 1)
    ii = _size_index(intra)
    oi = _size_index(inter)
    if np.any((~zero) & ((ii < 0) | (oi < 0))):
        raise ValueError("communication group size not in {1, 2, 4, >=8}")
    k = params[np.maximum(oi, 0), np.maximum(ii, 0), 0]
    b = params[np.maximum(oi, 0), np.maximum(ii, 0), 1]
    with np.errstate(divide="ignore", invalid="ignore"):
        lat = gbytes / k * (ngpu - 1) / ngpu + b
    return np.where(zero, 0.0, lat)


def gpu_gpu_comm_latency(op_name, gbytes, intra_size, inter_size, gpu_gpu_comm_params):
    """optimize.py:201-254."""
    if op_name not in ("p2p", "all_reduce", "all_gather", "reduce_scatter", "none"):
        raise ValueError(f"Invalid op_name: {op_name}")
    params = np.asarray(gpu_gpu_comm_params, dtype=np.float64)
    if params.size != 32:
        raise ValueError(f"Invalid size of gpu_gpu_comm_params: {params.size}")
    params = params.reshape(4, 4, 2)
    if op_name == "p2p":
        assert inter_size is None or intra_size is None
        if inter_size is not None:
            size, bandwidth = inter_size, params[1, 0][0]
        else:
            size, bandwidth = intra_size, params[0, 1][0]
        assert np.all(np.asarray(size) == 1), size
        return gbytes / bandwidth
    comm = gpu_gpu_only_latency(gbytes, intra_size, inter_size, params)
    return comm * _FACTOR[op_name]


def cpu_gpu_comm_latency(gbytes, params):
    """optimize.py:459-470: ``GB / k + b``, 0 where ``GB == 0``."""
    k, b = params
    gbytes = np.asarray(gbytes, dtype=np.float64)
    lat = gbytes / k + b
    return np.where(gbytes == 0, 0, lat)
