"""The entry point that allocates nothing, ``mist_dp_run_static``, against ``mist_dp_run``: same
DP instances through both, every output (stage count, sum, running maximum, back-pointers) equal
bit for bit; two calls in a row, the second smaller, so that what the first left in the shared
built-in scratch cannot leak into the second."""
import ctypes

import numpy as np
import pytest

from util import tiny_plan

pytestmark = pytest.mark.gpu


def _runner():
    from mist_amd.inter_tuning import _DpRunner
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates

    cfg, tables = tiny_plan(1, layers=7, hardware__num_nodes=2, hardware__num_gpus_per_node=4,
                            training__global_batch_size=32, hardware__memory_capacity=8.0)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, L, meshes, Gs, 1, cfg, sample_size=1).tune()
    return _DpRunner(res, L, hw.num_nodes * hw.num_gpus_per_node, meshes, 0), len(Gs)


def _both(runner, g_index, tmax, mode, want_argmin=True):
    """(outputs of mist_dp_run, outputs of mist_dp_run_static) for the same instances.  The
    static call must leave the driver's free device memory as it found it (the first call on a
    device, which resolves the address of the built-in array and loads the code object, is made
    before the reading)."""
    import torch

    from mist_amd import _lib
    from mist_amd.inter_tuning import _stream

    lib, fam, dev = runner.lib, runner.families[0], runner.device
    n = len(tmax)
    shape = ctypes.c_void_p(fam.shape.ctypes.data)
    d_tmax = torch.from_numpy(np.asarray(tmax, dtype=np.float32)).to(dev)
    d_g = torch.from_numpy(np.asarray(g_index, dtype=np.int32)).to(dev)
    outs = []
    for static in (False, True):
        best_s = torch.full((n,), -7, dtype=torch.int32, device=dev)
        best_sum = torch.full((n,), -7.0, dtype=torch.float32, device=dev)
        stage_max = torch.full((n,), -7.0, dtype=torch.float32, device=dev)
        argmin = (torch.full((n, fam.S_max + 1, fam.L + 1, fam.D + 1, 4), -1, dtype=torch.int32, device=dev)
                  if want_argmin else torch.zeros(1, dtype=torch.int32, device=dev))
        args = [shape, ctypes.byref(fam.costs_struct), d_tmax.data_ptr(), d_g.data_ptr(), n, mode,
                best_s.data_ptr(), best_sum.data_ptr(), stage_max.data_ptr(),
                argmin.data_ptr() if want_argmin else None]
        if static:
            _lib.check(lib.mist_dp_run_static(*args, _stream(dev)), "mist_dp_run_static (warm-up)")
            torch.cuda.synchronize(dev)
            if want_argmin:
                argmin.fill_(-1)
            torch.cuda.synchronize(dev)
            free_before = torch.cuda.mem_get_info(dev)[0]  # the driver's view: sees any hipMalloc
            torch_before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
            _lib.check(lib.mist_dp_run_static(*args, _stream(dev)), "mist_dp_run_static")
            torch.cuda.synchronize(dev)
            assert torch.cuda.mem_get_info(dev)[0] == free_before
            assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == torch_before
        else:
            scratch = torch.empty(lib.mist_dp_scratch_floats(shape, n), dtype=torch.float32, device=dev)
            _lib.check(lib.mist_dp_run(*args, scratch.data_ptr(), _stream(dev)), "mist_dp_run")
        torch.cuda.synchronize(dev)
        outs.append([t.cpu().numpy() for t in (best_s, best_sum, stage_max, argmin)])
    return outs


def test_static_scratch_run_equals_run_with_caller_scratch():
    from mist_amd import _lib

    runner, n_g = _runner()
    finite = np.concatenate([runner.cost[v].cpu().numpy().ravel() for v in range(3)])
    finite = finite[np.isfinite(finite)]
    assert len(finite) > 50
    rng = np.random.default_rng(5)
    n_feasible = 0
    for n in (40, 7):  # the second call is smaller than the first
        tmax = rng.choice(finite, size=n).astype(np.float32)
        tmax[0] = np.float32(finite.max())  # everything admissible: certainly feasible
        g_index = rng.integers(0, n_g, size=n).astype(np.int32)
        for mode in (_lib.DP_THRESHOLD, _lib.DP_BOTTLENECK):
            want, got = _both(runner, g_index, tmax, mode)
            for name, w, g in zip(("best_s", "best_sum", "stage_max", "argmin"), want, got):
                assert np.array_equal(w.view(np.int32), g.view(np.int32)), (n, mode, name)
            n_feasible += int((want[0] >= 0).sum())
            assert not np.any(want[0] == -7)
    assert n_feasible > 10


def test_static_scratch_at_its_size_limit():
    """The largest batch of the 80-layer, 256-device shape the built-in array holds (49 instances;
    50 are rejected), against ``mist_dp_run`` with caller scratch."""
    from mist_amd import _lib
    from mist_amd.inter_tuning import _DpRunner
    from mist_amd.intra_tuning import IntraStageTuner
    from mist_amd.search_space import _get_device_mesh_candidates, _get_grad_accumu_steps_candidates
    from util import load_plan

    cfg, tables = load_plan(5)
    hw, L = cfg.hardware, cfg.model.num_hidden_layers
    meshes = _get_device_mesh_candidates(hw.num_nodes, hw.num_gpus_per_node, False)
    Gs = _get_grad_accumu_steps_candidates(cfg.training.global_batch_size)
    res = IntraStageTuner(tables, L, meshes, Gs, 8, cfg, sample_size=1).tune()
    runner = _DpRunner(res, L, hw.num_nodes * hw.num_gpus_per_node, meshes, 0)
    fam, lib = runner.families[0], runner.lib
    shape = ctypes.c_void_p(fam.shape.ctypes.data)
    limit = lib.mist_dp_static_scratch_floats()
    assert lib.mist_dp_scratch_floats(shape, 50) > limit >= lib.mist_dp_scratch_floats(shape, 49)
    g = len(Gs) - 2
    _, bott, _ = runner.run(np.array([g], dtype=np.int32), np.zeros(1, dtype=np.float32), _lib.DP_BOTTLENECK)
    assert np.isfinite(bott[0])
    tmax = (np.float32(bott[0]) * np.linspace(0.97, 1.3, 49)).astype(np.float32)
    want, got = _both(runner, np.full(49, g, dtype=np.int32), tmax, _lib.DP_THRESHOLD, want_argmin=False)
    for name, w, gt in zip(("best_s", "best_sum", "stage_max"), want, got):
        assert np.array_equal(w.view(np.int32), gt.view(np.int32)), name
    assert (want[0] >= 0).sum() >= 40 and (want[0] < 0).sum() >= 1
    import torch

    dev = runner.device
    d_t = torch.zeros(50, dtype=torch.float32, device=dev)
    d_g = torch.zeros(50, dtype=torch.int32, device=dev)
    out = torch.zeros(50, dtype=torch.int32, device=dev)
    outf = torch.zeros(2, 50, dtype=torch.float32, device=dev)
    from mist_amd.inter_tuning import _stream

    rc = lib.mist_dp_run_static(shape, ctypes.byref(fam.costs_struct), d_t.data_ptr(), d_g.data_ptr(), 50,
                                _lib.DP_THRESHOLD, out.data_ptr(), outf[0].data_ptr(), outf[1].data_ptr(),
                                None, _stream(dev))
    assert rc == -1 and b"built-in scratch holds" in lib.mist_last_error()
