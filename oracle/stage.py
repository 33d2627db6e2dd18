"""Oracle (test infrastructure): per-stage latency + memory model and its reduction.

Numpy restatement of ``batched_tune_best_latency_for_stage`` / ``batched_stage_analyze`` with
``get_best_solution=True`` (mist/analyzer/batched_module_analyzer.py:581-3144) and of
``get_concrete_latency_exec`` (:259-414).  The traced ``LayerInfo`` objects of the reference are
replaced by a ``tables`` provider with accessor methods (see mist_amd/layer_tables.py for the
mapping to the reference helpers); everything else keeps the reference's operation order, dtypes
and rounding points (float64 everywhere; stable / delta latencies rounded to float32 at
:2212-2213) so that results can be compared bit for bit.

Pinned by (tests/test_oracle_stage.py): algebraic invariants (monotone peaks in l and p,
non-increasing in the offload ratios; interference factors 1 -> latency terms reduce to max();
G == 1 -> delta == 0), the index/cost consistency of the reduction against ``np.argmin``, the
reference's documented quirks (cells never written), and a scalar re-derivation of single
cells.  No reference-held golden values exist for this function.
"""
import numpy as np

from .comm import cpu_gpu_comm_latency, gpu_gpu_comm_latency
from .interference import interference_one_group
from .pareto import sample_pareto_frontier
from .search_space import create_search_space

BATCH_SIZE_CANDIDATES = (1, 2, 4)  # batched_module_analyzer.py:53 (the module constant, :870)

MEM_INF = 1e12
GB = 1 << 30
MB = 1 << 20
VARIANTS = ("base", "with_pre", "with_post", "no_pp")


def latency_exec_single(tables, kind, b, tp, inter_size, intra_size, grad_accum_steps):
    """``_single_get_concrete_latency_exec`` (:324-414): sum of op latencies with the
    ``bwd > 2.3 * fwd -> 2 * fwd`` clamp, the ``fwd < 5e-5 or bwd < 1e-4`` drop and the
    gradient-accumulation term ``ga * (G - 1) / G``."""
    fwd_sum = bwd_sum = efwd_sum = ebwd_sum = 0
    for fwd, bwd, efwd, ebwd in tables.op_profiles(kind, int(b), int(tp), inter_size, intra_size):
        if bwd != 0 and bwd > 2.3 * fwd:
            bwd = fwd * 2
        fwd += efwd
        bwd += ebwd
        if fwd < 5e-5 or bwd < 1e-4:
            continue
        fwd_sum += fwd
        bwd_sum += bwd
        efwd_sum += efwd
        ebwd_sum += ebwd
    for ga in tables.grad_accum_profiles(kind, int(b), int(tp)):
        bwd_sum += ga * (grad_accum_steps - 1) / grad_accum_steps
    return fwd_sum, bwd_sum, efwd_sum, ebwd_sum


def latency_exec(tables, kind, b, tp, inter_size, intra_size, grad_accum_steps):
    """``get_concrete_latency_exec`` (:259-321): per-element evaluation, four (N,) arrays."""
    b = np.atleast_1d(np.asarray(b))
    tp = np.atleast_1d(np.asarray(tp))
    inter_size = np.broadcast_to(np.asarray(inter_size), b.shape)
    intra_size = np.broadcast_to(np.asarray(intra_size), b.shape)
    cache = {}
    out = np.empty((b.shape[0], 4), dtype=np.float64)
    for i in range(b.shape[0]):
        key = (float(b[i]), float(tp[i]), float(inter_size[i]), float(intra_size[i]))
        if key not in cache:
            cache[key] = latency_exec_single(tables, kind, *key, grad_accum_steps)
        out[i] = cache[key]
    return out[:, 0], out[:, 1], out[:, 2], out[:, 3]


def _arr(x):
    """``_convert_to_np_array`` (:848-852)."""
    if isinstance(x, np.ndarray) and x.ndim > 0:
        return x
    return np.array([x])


def pre_post_strategy_fields(config, num_nodes, num_gpus_per_node, analysis_rows=None):
    """:777-845: (dp, tp, wre, gre, ore, wo, go, oo, ac) of the pre/post layers.  The tuning path
    reads ``config.tuning.pre_post_strategy``; the analysis path (``analysis_rows`` = the
    strategy rows) reads ``config.strategy.pre_post_strategy`` and also knows ``tuned``."""
    if analysis_rows is None:
        strategy = config.tuning.pre_post_strategy
    else:
        strategy = config.strategy.pre_post_strategy
        if strategy == "tuned":  # :789-799
            r = analysis_rows
            return r[:, 1], r[:, 2], r[:, 3], r[:, 4], r[:, 5], 0.0, 0.0, 0.0, 0.0
    if strategy == "preset":
        # The reference reads ``config.strategy.pre_post_strategy_array`` here (:801-809).
        a = config.strategy.pre_post_strategy_array
        return a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], a[9]
    if strategy == "dp":
        return num_nodes * num_gpus_per_node, 1, False, False, True, 0.0, 0.0, 0.0, 0.0
    if strategy in ("intra-node-tp-with-ore", "intra-node-tp-without-ore"):
        ore = strategy == "intra-node-tp-with-ore"
        return num_nodes, num_gpus_per_node, False, True, ore, 0.0, 0.0, 0.0, 0.0
    raise NotImplementedError(f"pre_post_strategy: {strategy}")


def batched_stage_analyze(
    tables,
    config,
    pre_saved_micro_batches_candidates,
    num_layers_candidates,
    num_ckpt_layers_candidates,
    num_nodes,
    num_gpus_per_node,
    gradient_accumulation_steps,
    stage_strategies,
    sample_size,
    debug=None,
    analysis=None,
    inner="numpy",
    threads=0,
):
    """:687-3144 with ``get_best_solution=True``.

    ``inner="c"`` runs the loops over (ckpt layers, pre-saved micro-batches) and the argmin scan
    through oracle/stage_loop.c instead of the numpy statements below: the same expressions
    cell by cell, bit-equal tables (tests/test_oracle_stage_c.py), two orders of magnitude
    faster on the large plans.  Everything up to the loops is the numpy code either way.

    ``analysis`` (a list of four dicts) additionally receives what the ``get_best_solution=False``
    path returns (:2788-2803, 2876-2892, 2980-2996, 3063-3079): per variant and ``(p, l, c)`` the
    per-row arrays ``latency`` (incl. twice the p2p latency of the layer output, :1298-1308,
    except for the pre-and-post variant), ``mem_fwd_peak``, ``mem_bwd_peak`` and the stable /
    delta latency of that variant (the ``****latency_*`` entries, :2550-2567), unmasked.

    Returns four tuples ``(costs_stable, costs_delta, solutions, indices)`` for the variants
    base / with_pre / with_post / no_pp; ``indices`` (row index into ``stage_strategies``, -1
    where nothing is feasible or the cell is never written) is an addition for comparisons.
    ``debug`` (a dict) receives the row-invariant intermediate arrays when given."""
    rows = np.asarray(stage_strategies, dtype=np.float64).reshape(-1, 10)
    if rows.size == 0:
        raise ValueError("stage_strategies is empty")
    G = gradient_accumulation_steps
    hw = config.hardware
    P = max(pre_saved_micro_batches_candidates)
    Lmax = max(num_layers_candidates)
    Cmax = max(num_ckpt_layers_candidates)
    S = sample_size
    F = rows.shape[1]

    def full(shape, dtype=np.float64, value=np.inf):
        return np.full(shape, value, dtype=dtype)

    costs_stable = full((P + 1, Lmax, Cmax + 1, S))
    costs_stable_pre = full((P + 1, Lmax, Cmax + 1, S))
    costs_stable_post = full((Lmax, Cmax + 1, S))
    costs_stable_nopp = full((Cmax + 1, S))
    costs_delta = full((P + 1, Lmax, Cmax + 1, S))
    costs_delta_pre = full((P + 1, Lmax, Cmax + 1, S))
    costs_delta_post = full((Lmax, Cmax + 1, S))
    costs_delta_nopp = full((Cmax + 1, S))
    solutions = full((P + 1, Lmax, Cmax + 1, S, F))
    solutions_pre = full((P + 1, Lmax, Cmax + 1, S, F))
    solutions_post = full((Lmax, Cmax + 1, S, F))
    solutions_nopp = full((Cmax + 1, S, F))
    idx_base = full((P + 1, Lmax, Cmax + 1, S), np.int64, -1)
    idx_pre = full((P + 1, Lmax, Cmax + 1, S), np.int64, -1)
    idx_post = full((Lmax, Cmax + 1, S), np.int64, -1)
    idx_nopp = full((Cmax + 1, S), np.int64, -1)

    def gpu_gpu(op_name, mbytes, inter_size, intra_size):
        return gpu_gpu_comm_latency(
            op_name, mbytes / 1024, intra_size, inter_size, hw.gpu_gpu_comm_params
        )

    def cpu_to_gpu(mbytes):
        return cpu_gpu_comm_latency(mbytes / 1024, hw.cpu_gpu_comm_params)

    def gpu_to_cpu(mbytes):
        return cpu_gpu_comm_latency(mbytes / 1024, hw.gpu_cpu_comm_params)

    # ------------------------------------------------------------------ pre / post layers (:777-1138)
    (pp_dp, pp_tp, pp_wre, pp_gre, pp_ore, pp_wo, pp_go, pp_oo, pp_ac) = [
        _arr(v) for v in pre_post_strategy_fields(
            config, num_nodes, num_gpus_per_node, rows if analysis is not None else None)
    ]
    pp_b = config.training.global_batch_size // G // pp_dp
    if analysis is not None and pp_b.size == 1 and not 1 <= int(pp_b[0]) <= max(BATCH_SIZE_CANDIDATES):
        return None  # :868-880: the analysis path returns its (empty) dicts here

    def full_states(kind, item, tp):
        return np.atleast_1d(tables.mem_full_states(kind, item, np.asarray(tp, dtype=np.float64)))

    def partial(full_, shard, ratio):
        return full_ / shard * (1 - ratio)  # :143-153

    pre_W = full_states("pre", "weights", pp_tp)
    pre_G = full_states("pre", "grads", pp_tp)
    pre_O = full_states("pre", "opts", pp_tp)
    pre_states = (
        partial(pre_W, np.where(pp_wre, pp_dp, 1), pp_wo)
        + partial(pre_G, np.where(pp_gre, pp_dp, 1), pp_go)
        + partial(pre_O, np.where(pp_ore, pp_dp, 1), pp_oo)
    )
    f64 = lambda a: np.asarray(a).astype(np.float64)
    pre_saved = np.atleast_1d(tables.mem_saved("pre", False, f64(pp_b), f64(pp_tp)))
    pre_states_and_saved = pre_states + pre_saved
    post_W = full_states("post", "weights", pp_tp)
    post_G = full_states("post", "grads", pp_tp)
    post_O = full_states("post", "opts", pp_tp)
    post_pO = partial(post_O, np.where(pp_ore, pp_dp, 1), pp_oo)
    post_states = post_W + post_G + post_pO
    post_fwd_peak = np.atleast_1d(tables.mem_peak("post", "fwd", f64(pp_b), f64(pp_tp), None))
    post_bwd_peak = np.atleast_1d(tables.mem_peak("post", "bwd", f64(pp_b), f64(pp_tp)))
    post_output = np.atleast_1d(tables.mem_output("post", f64(pp_b), f64(pp_tp)))

    pp_tp_inter = np.where(pp_tp > num_gpus_per_node, pp_tp // num_gpus_per_node, 1)
    pp_tp_intra = np.where(pp_tp > num_gpus_per_node, num_gpus_per_node, pp_tp)
    pre_fwd, pre_bwd, _, _ = latency_exec(tables, "pre", pp_b, pp_tp, pp_tp_inter, pp_tp_intra, G)
    post_fwd, post_bwd, _, _ = latency_exec(
        tables, "post", pp_b, pp_tp, pp_tp_inter, pp_tp_intra, G
    )
    pp_dp_kwargs = dict(
        inter_size=np.where(pp_dp > num_nodes, num_nodes, pp_dp),
        intra_size=np.where(pp_dp > num_nodes, pp_dp // num_nodes, 1),
    )
    pre_AG = np.where(pp_dp == 1, 0, gpu_gpu("all_gather", pre_W, **pp_dp_kwargs))
    post_AG = np.where(pp_dp == 1, 0, gpu_gpu("all_gather", post_W, **pp_dp_kwargs))
    pre_RS = np.where(pp_dp == 1, 0, gpu_gpu("reduce_scatter", pre_G, **pp_dp_kwargs))
    post_RS = np.where(pp_dp == 1, 0, gpu_gpu("reduce_scatter", post_G, **pp_dp_kwargs))

    # ------------------------------------------------------------------ block layer rows (:1144-1408)
    b, dp, tp = rows[:, 0], rows[:, 1], rows[:, 2]
    wre, gre, ore = rows[:, 3], rows[:, 4], rows[:, 5]
    wo, go, oo, ao = rows[:, 6], rows[:, 7], rows[:, 8], rows[:, 9]
    wre_size = np.where(wre == 1, dp, 1)
    gre_size = np.where(gre == 1, dp, 1)
    ore_size = np.where(ore == 1, dp, 1)

    frag = 0.0
    if "hidden_size" in config.model and "max_sequence_length" in config.training:
        frag += max(0, config.model.hidden_size / 2048 - 1) * 0.005
        frag += max(0, config.training.max_sequence_length / 2048 - 1) * 0.045
    mf = np.ones_like(b, dtype=float)
    mf += frag
    mf += np.where(wo > 0, 0.025, 0)
    mf += np.where(go > 0, 0.025, 0)
    mf += np.where(oo > 0, 0.03, 0)
    mf += np.where(ao > 0, 0.04, 0)
    mf += np.where(wre, 0.025, 0)
    mf += np.where(gre, 0.025, 0)
    mf += np.where(tp > 1, 0.04, 0)
    mf += np.where(b >= 4, 0.01, 0)
    mf_pp = mf + 0.025

    gcb = 0
    if not config.model.use_flash_attn:
        gcb += (
            2
            * b
            * config.model.num_attention_heads
            / tp
            * (config.training.max_sequence_length**2)
            / (1024**2)
        )

    W = np.atleast_1d(tables.mem_full_states("block", "weights", tp))
    Gr = np.atleast_1d(tables.mem_full_states("block", "grads", tp))
    O = np.atleast_1d(tables.mem_full_states("block", "opts", tp))
    pW = partial(W, wre_size, wo)
    pG = partial(Gr, gre_size, go)
    pO = partial(O, ore_size, oo)
    raw_ck = np.atleast_1d(tables.mem_saved("block", True, b, tp))
    S_ck = raw_ck * (1 - ao)
    D_ck = raw_ck * ao
    raw_nock = np.atleast_1d(tables.mem_saved("block", False, b, tp))
    S_nock = raw_nock * (1 - ao)
    D_nock = raw_nock * ao
    fwd_peak_nock = np.atleast_1d(tables.mem_peak("block", "fwd", b, tp, False))
    bwd_peak = np.atleast_1d(tables.mem_peak("block", "bwd", b, tp))
    out = np.atleast_1d(tables.mem_output("block", b, tp))

    dp_kwargs = dict(
        inter_size=np.where(dp > num_nodes, num_nodes, dp),
        intra_size=np.where(dp > num_nodes, dp // num_nodes, 1),
    )
    tp_inter = np.where(tp > num_gpus_per_node, tp // num_gpus_per_node, 1)
    tp_intra = np.where(tp > num_gpus_per_node, num_gpus_per_node, tp)
    exec_fwd, exec_bwd_nock, extra_fwd, extra_bwd = latency_exec(
        tables, "block", b, tp, tp_inter, tp_intra, G
    )
    ag_saved_ck = np.array([0.0])  # PARTITION_SAVED_TENSORS is False (:1250,1355-1356)
    exec_bwd_ck = exec_fwd + exec_bwd_nock

    so_W = gpu_to_cpu(W / wre_size * wo)
    si_W = cpu_to_gpu(W / wre_size * wo)
    so_G = gpu_to_cpu(Gr / gre_size * go)
    si_G = cpu_to_gpu(Gr / gre_size * go)
    so_O = gpu_to_cpu(O / ore_size * oo)
    si_O = cpu_to_gpu(O / ore_size * oo)
    so_A_ck = gpu_to_cpu(raw_ck * ao)
    si_A_ck = cpu_to_gpu(raw_ck * ao)
    so_A_nock = gpu_to_cpu(raw_nock * ao)
    si_A_nock = cpu_to_gpu(raw_nock * ao)
    AG_w = gpu_gpu("all_gather", W, **dp_kwargs)
    RS_g = gpu_gpu("reduce_scatter", Gr, **dp_kwargs)
    AR_g = gpu_gpu("all_reduce", Gr, **dp_kwargs)

    zeros = np.zeros_like(exec_fwd)
    adv = config.enable_advanced_opt_in_first_block
    params = hw.interference_model_params

    def I(exec_, g2g, g2c, c2g):  # get_layer_critical_latency (:1413-1422)
        return interference_one_group(C=exec_, G2G=g2g, C2G=c2g, G2C=g2c, params=params)

    # ------------------------------------------------------------------ forward phases (:1432-1621)
    g2c_F1 = so_O + so_W
    c2g_F1 = si_O + si_G
    g2g_F1 = AG_w * ore
    g2c_Fn = np.zeros_like(so_W)
    c2g_Fn = si_W
    g2g_Fn = AG_w * wre
    E_f = exec_fwd - extra_fwd
    fwd = {}
    for ph, g2g, g2c, c2g, pre_g2g, pre_c2g in (
        ("F1", g2g_F1, g2c_F1, c2g_F1, g2g_F1, c2g_F1 if adv else zeros),
        ("Fn", g2g_Fn, g2c_Fn, c2g_Fn, g2g_Fn if adv else zeros, c2g_Fn if adv else zeros),
    ):
        first = I(E_f, g2g, zeros, c2g) + extra_fwd
        extra_pre = I(zeros, pre_g2g, zeros, pre_c2g)
        for k, so_A in (("nock", so_A_nock), ("ck", so_A_ck)):
            fwd[ph, k] = dict(
                layer=I(E_f, g2g, g2c + so_A, c2g) + extra_fwd,
                first=first,
                last=I(E_f, zeros, g2c + so_A, zeros) + extra_fwd,
                extra_pre=extra_pre,
                extra_post=I(zeros, zeros, g2c + so_A, zeros),
            )

    # ------------------------------------------------------------------ backward phases (:1646-1902)
    g2c_B = so_G
    c2g_B = si_W + si_G
    g2g_BL = AG_w * wre + RS_g * ore + AR_g * (1 - ore)
    g2g_Bn = AG_w * wre + RS_g * gre
    extra_fb = extra_fwd + extra_bwd
    bwd = {}
    for ph, g2g in (("BL", g2g_BL), ("Bn", g2g_Bn)):
        for k, E, extra, si_A in (
            ("nock", exec_bwd_nock - extra_bwd, extra_bwd, si_A_nock),
            ("ck", exec_bwd_ck - extra_fb, extra_fb, si_A_ck),
        ):
            if ph == "BL":
                # :1702-1703 (without ckpt) and :1759-1763 (with ckpt) differ in form.
                if k == "nock":
                    red = RS_g * ore + AR_g * (1 - ore)
                else:
                    red = np.where(ore == 1, RS_g, AR_g)
            else:
                red = RS_g * gre
            g2g_layer = g2g if k == "nock" else g2g + ag_saved_ck
            bwd[ph, k] = dict(
                layer=I(E, g2g_layer, g2c_B, c2g_B + si_A) + extra,
                last=I(E, AG_w * wre, zeros, c2g_B + si_A) + extra,
                first=I(E, red, g2c_B if adv else zeros, zeros) + extra,
                extra_pre=I(zeros, AG_w * wre, zeros, c2g_B + si_A),
                extra_post=I(zeros, red, g2c_B if adv else zeros, zeros),
            )

    # ------------------------------------------------------------------ combinations (:1910-2028)
    def families(fph, bph, k):
        f_, b_ = fwd[fph, k], bwd[bph, k]
        return (
            f_["layer"] + b_["layer"],
            f_["extra_pre"] + b_["extra_post"] + f_["first"] + b_["first"],
            f_["extra_post"] + b_["extra_pre"] + f_["last"] + b_["last"],
        )

    lat = {}
    for k in ("nock", "ck"):
        if G == 1:
            s_layer, s_first, s_last = families("F1", "BL", k)
            d_layer = d_first = d_last = 0
        else:
            s_layer, s_first, s_last = families("Fn", "Bn", k)
            d_layer = fwd["F1", k]["layer"] + bwd["BL", k]["layer"] - s_layer
            d_first = (
                fwd["F1", k]["extra_pre"]
                + bwd["BL", k]["extra_post"]
                + fwd["F1", k]["first"]
                + bwd["BL", k]["first"]
                - s_first
            )
            d_last = (
                fwd["F1", k]["extra_post"]
                + bwd["BL", k]["extra_pre"]
                + fwd["F1", k]["last"]
                + bwd["BL", k]["last"]
                - s_last
            )
        lat[k] = dict(
            s_layer=s_layer, s_first=s_first, s_last=s_last,
            d_layer=d_layer, d_first=d_first, d_last=d_last,
        )

    # ------------------------------------------------------------------ module-level memory (:2062-2162)
    num_layers = np.array(num_layers_candidates)[:, np.newaxis]
    n = num_layers.shape[0]
    lm2 = np.maximum(num_layers - 2, 0)
    lm1 = np.maximum(num_layers - 1, 0)
    wbuf_on = np.logical_or.reduce(
        (wre_size > 1, np.broadcast_to(pp_wre, wre_size.shape) == 1, wo > 0)
    )
    gbuf_on = np.logical_or.reduce(
        (gre_size > 1, np.broadcast_to(pp_gre, gre_size.shape) == 1, go > 0)
    )
    Wbuf = np.where(
        wbuf_on,
        np.maximum.reduce(
            (np.broadcast_to(pre_W, W.shape), np.broadcast_to(post_W, W.shape), W)
        ),
        0,
    )
    Gbuf = np.where(
        gbuf_on,
        np.maximum.reduce(
            (np.broadcast_to(pre_G, Gr.shape), np.broadcast_to(post_G, Gr.shape), Gr)
        ),
        0,
    )
    fwd_states = 2 * (Wbuf + Gbuf) + O // ore_size + num_layers * (pW + pG) + lm1 * pO
    bwd_states = 2 * (Wbuf + Gbuf) + num_layers * (pW + pG + pO)

    so_A_sel = {True: so_A_ck, False: so_A_nock}
    extra_pre_Bn_ck = bwd["Bn", "ck"]["extra_pre"]
    # Row-invariant pieces of the post-layer overlap terms (:2251-2292).
    ovw = {
        k: np.maximum(exec_fwd - g2c_Fn - so_A_sel[k == "ck"], 0) for k in ("ck", "nock")
    }
    nAG = {k: np.maximum(post_AG - ovw[k], 0) for k in ("ck", "nock")}
    ovg = {
        "ck": np.maximum(exec_bwd_ck - AG_w * wre - c2g_B - si_A_ck, 0),
        "nock": np.maximum(exec_bwd_nock - AG_w * wre - c2g_B - si_A_nock, 0),
    }
    nRS = {k: np.maximum(post_RS - ovg[k], 0) for k in ("ck", "nock")}
    opb = np.maximum(post_bwd - extra_pre_Bn_ck, 0)

    if debug is not None:
        debug.update(
            mf=mf, gcb=gcb, pW=pW, pG=pG, pO=pO, S_ck=S_ck, S_nock=S_nock, D_ck=D_ck,
            D_nock=D_nock, Wbuf=Wbuf, Gbuf=Gbuf, T0=2 * (Wbuf + Gbuf) + O // ore_size,
            T1=2 * (Wbuf + Gbuf), pWG=pW + pG, pWGO=pW + pG + pO,
            fwd_peak_nock=np.broadcast_to(fwd_peak_nock, b.shape),
            bwd_peak=np.broadcast_to(bwd_peak, b.shape), out=np.broadcast_to(out, b.shape),
            lat=lat, fwd=fwd, bwd=bwd, nAG=nAG, nRS=nRS, opb=opb, RD=raw_nock - S_nock,
            AG_w=AG_w, RS_g=RS_g, AR_g=AR_g, so_W=so_W, si_W=si_W, so_G=so_G, si_G=si_G,
            so_O=so_O, si_O=si_O, so_A_ck=so_A_ck, si_A_ck=si_A_ck, so_A_nock=so_A_nock,
            si_A_nock=si_A_nock, exec_fwd=exec_fwd, exec_bwd_nock=exec_bwd_nock,
            extra_fwd=extra_fwd, extra_bwd=extra_bwd,
            pre=dict(states=pre_states, saved=pre_saved, fwd=pre_fwd, bwd=pre_bwd, AG=pre_AG,
                     RS=pre_RS, W=pre_W, G=pre_G),
            post=dict(states=post_states, fwd_peak=post_fwd_peak, bwd_peak=post_bwd_peak,
                      output=post_output, fwd=post_fwd, bwd=post_bwd, AG=post_AG, RS=post_RS,
                      W=post_W, G=post_G),
        )

    def get_latencies(num_ckpt):  # :2165-2216
        no_ckpt = num_ckpt == 0
        all_ckpt = num_ckpt == num_layers
        n_ck = np.clip(num_ckpt - 1, 0, lm2)
        n_nock = lm2 - n_ck
        stable = (
            n_ck * lat["ck"]["s_layer"]
            + n_nock * lat["nock"]["s_layer"]
            + np.where(all_ckpt, lat["ck"]["s_first"], lat["nock"]["s_first"])
            + np.where(no_ckpt, lat["nock"]["s_last"], lat["ck"]["s_last"])
        )
        delta = (
            n_ck * lat["ck"]["d_layer"]
            + n_nock * lat["nock"]["d_layer"]
            + np.where(all_ckpt, lat["ck"]["d_first"], lat["nock"]["d_first"])
            + np.where(no_ckpt, lat["nock"]["d_last"], lat["ck"]["d_last"])
        )
        delta = np.broadcast_to(delta, stable.shape)
        return stable.astype(np.float32), delta.astype(np.float32)

    cap = hw.memory_capacity * GB / MB
    ar_n = np.arange(n)[:, None]
    if analysis is not None:
        across_nodes = num_gpus_per_node == hw.num_gpus_per_node  # :1299
        p2p = gpu_gpu("p2p", out, inter_size=1 if across_nodes else None,
                      intra_size=None if across_nodes else 1) * 2

    extra_of_c = {}  # get_extra_info (:2401-2749) of the current c, per layer index

    def record(variant, p, c, stable_v, delta_v, latency_v, fwd, bwd):
        for i, l in enumerate(num_layers_candidates):
            analysis[variant][(p, l, c)] = {
                "latency": np.broadcast_to(latency_v, stable_v.shape)[i],
                "mem_fwd_peak": np.broadcast_to(fwd, stable_v.shape)[i],
                "mem_bwd_peak": np.broadcast_to(bwd, stable_v.shape)[i],
                "latency_stable": stable_v[i],
                "latency_delta": np.broadcast_to(delta_v, stable_v.shape)[i],
                "extra_info": extra_of_c.get(i),
            }

    def row0(x):
        """First (in the analysis path: only) row of a per-row quantity as a python float."""
        return float(np.asarray(x, dtype=np.float64).reshape(-1)[0])

    def extra_info(i, c, variants, mod_saved):
        """The debugging entries of the reference's result dictionaries for layer index ``i``
        (get_extra_info, :2401-2749; its per-row arrays are indexed there with the layer index,
        which only works with one candidate: here they are the given row's values).
        ``variants`` = ((stable, delta), ...) of base / with_pre / with_post / with_pre_and_post."""
        k_last = "ck" if c > 0 else "nock"
        e = {
            "*****memory_factor": row0(mf),
            "*****mem_per_full_weight_buffer": row0(Wbuf),
            "*****mem_per_full_grad_buffer": row0(Gbuf),
            "****non_overlapped_post_weights_all_gather_latency": row0(nAG[k_last]),
            "****non_overlapped_post_grad_sync_latency": row0(nRS[k_last]),
            "****overlapped_post_bwd_latency": row0(opb),
        }
        ck_name = {"nock": "without_ckpt", "ck": "with_ckpt"}
        for k in ("nock", "ck"):
            for ph, mb in (("F1", "first"), ("Fn", "not_first")):
                f_ = fwd[ph, k]
                e[f"****latency_first_layer_critical_fwd_{mb}_micro_batch_{ck_name[k]}"] = row0(f_["first"])
                e[f"****latency_last_layer_critical_fwd_{mb}_micro_batch_{ck_name[k]}"] = row0(f_["last"])
                e[f"****latency_extra_pre_fwd_{mb}_micro_batch_{ck_name[k]}"] = row0(f_["extra_pre"])
                e[f"****latency_extra_post_fwd_{mb}_micro_batch_{ck_name[k]}"] = row0(f_["extra_post"])
                stars = "**" if k == "nock" else "*"
                e[f"{stars}_latency_layer_critical_fwd_{mb}_micro_batch_{ck_name[k]}"] = row0(f_["layer"])
            for ph, mb in (("BL", "last"), ("Bn", "not_last")):
                b_ = bwd[ph, k]
                e[f"****latency_last_layer_critical_bwd_{mb}_micro_batch_{ck_name[k]}"] = row0(b_["last"])
                e[f"****latency_first_layer_critical_bwd_{mb}_micro_batch_{ck_name[k]}"] = row0(b_["first"])
                e[f"****latency_extra_pre_bwd_{mb}_micro_batch_{ck_name[k]}"] = row0(b_["extra_pre"])
                e[f"****latency_extra_post_bwd_{mb}_micro_batch_{ck_name[k]}"] = row0(b_["extra_post"])
                stars = "**" if k == "nock" else "*"
                e[f"{stars}_latency_layer_critical_bwd_{mb}_micro_batch_{ck_name[k]}"] = row0(b_["layer"])
            e[f"****latency_layer_critical_stable_{ck_name[k]}"] = row0(lat[k]["s_layer"])
            e[f"****latency_layer_critical_delta_{ck_name[k]}"] = row0(lat[k]["d_layer"])
            e[f"****latency_pre_fwd_and_post_bwd_and_first_layer_stable_{ck_name[k]}"] = row0(lat[k]["s_first"])
            e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_stable_{ck_name[k]}"] = row0(lat[k]["s_last"])
            e[f"****latency_pre_fwd_and_post_bwd_and_first_layer_delta_{ck_name[k]}"] = row0(lat[k]["d_first"])
            e[f"****latency_post_fwd_and_pre_bwd_and_last_layer_delta_{ck_name[k]}"] = row0(lat[k]["d_last"])
        for (stable_v, delta_v), suffix in zip(variants, ("", "_with_pre", "_with_post", "_with_pre_and_post")):
            e["****latency_stable" + suffix] = row0(np.asarray(stable_v)[i])
            e["****latency_delta" + suffix] = row0(np.broadcast_to(delta_v, np.asarray(stable_v).shape)[i])
        # pre / post layers (:1069-1138)
        pre_AR = gpu_gpu("all_reduce", pre_G, **pp_dp_kwargs)
        post_AR = gpu_gpu("all_reduce", post_G, **pp_dp_kwargs)
        amortized = lambda flag, v: np.where(flag == 1, v, v / G)
        e.update({
            "_latency_pre_fwd_latency": row0(pre_fwd),
            "_latency_pre_bwd_latency": row0(pre_bwd),
            "_latency_pre_weights_all_gather_latency": row0(pre_AG),
            "_latency_pre_weights_all_gather_latency_amortized": row0(amortized(pp_wre, pre_AG)),
            "_latency_pre_grad_sync_latency": row0(pre_RS),
            "_latency_pre_grad_sync_amortized": row0(np.where(pp_ore == 0, pre_AR / G, amortized(pp_gre, pre_RS))),
            "_latency_post_fwd_latency": row0(post_fwd),
            "_latency_post_bwd_latency": row0(post_bwd),
            "_latentcy_post_weights_all_gather_latency_amortized": row0(amortized(pp_wre, post_AG)),
            "_latency_post_grad_sync_amortized": row0(np.where(pp_ore == 0, post_AR / G, amortized(pp_gre, post_RS))),
            "_latency_post_grad_sync_latency": row0(post_RS),
            "_latency_post_weights_all_gather_latency": row0(post_AG),
            "_latency_layer_exec_fwd": row0(exec_fwd),
            "_latency_layer_exec_bwd_without_ckpt": row0(exec_bwd_nock),
            "_latency_layer_exec_bwd_with_ckpt": row0(exec_bwd_ck),
            "_latency_layer_gpu_to_cpu_fwd_first_micro_batch_exclude_act": row0(g2c_F1),
            "_latency_layer_cpu_to_gpu_fwd_first_micro_batch_exclude_act": row0(c2g_F1),
            "_latency_layer_gpu_gpu_fwd_first_micro_batch_exclude_act": row0(g2g_F1),
            "_latency_layer_gpu_to_cpu_fwd_not_first_micro_batch_exclude_act": row0(g2c_Fn),
            "_latency_layer_cpu_to_gpu_fwd_not_first_micro_batch_exclude_act": row0(c2g_Fn),
            "_latency_layer_gpu_gpu_fwd_not_first_micro_batch_exclude_act": row0(g2g_Fn),
            "_latency_layer_gpu_to_cpu_bwd_last_micro_batch_exclude_act": row0(g2c_B),
            "_latency_layer_cpu_to_gpu_bwd_last_micro_batch_exclude_act": row0(c2g_B),
            "_latency_layer_gpu_gpu_bwd_last_micro_batch_exclude_act": row0(g2g_BL),
            "_latency_layer_gpu_to_cpu_bwd_not_last_micro_batch_exclude_act": row0(g2c_B),
            "_latency_layer_cpu_to_gpu_bwd_not_last_micro_batch_exclude_act": row0(c2g_B),
            "_latency_layer_gpu_gpu_bwd_not_last_micro_batch_exclude_act": row0(g2g_Bn),
            "_latency_layer_swap_out_weights": row0(so_W),
            "_latency_layer_swap_in_weights": row0(si_W),
            "_latency_layer_all_gather_weights": row0(AG_w),
            "_latency_layer_swap_in_grads": row0(si_G),
            "_latency_layer_swap_in_activations_with_ckpt": row0(si_A_ck),
            "_latency_layer_swap_in_activations_without_ckpt": row0(si_A_nock),
            "_latency_layer_swap_out_grads": row0(so_G),
            "_latency_layer_swap_out_activations_with_ckpt": row0(so_A_ck),
            "_latency_layer_swap_out_activations_without_ckpt": row0(so_A_nock),
            "_latency_layer_reduce_scatter_grads": row0(RS_g),
            "_latency_layer_bwd_all_gather_saved_with_ckpt": row0(ag_saved_ck),
            "_latency_p2p_output": row0(p2p),
            "_mem_layer_full_weights": row0(W),
            "_mem_layer_full_grads": row0(Gr),
            "_mem_layer_full_opts": row0(O),
            "_mem_layer_partial_weights": row0(pW),
            "_mem_layer_partial_grads": row0(pG),
            "_mem_layer_partial_opts": row0(pO),
            "_mem_layer_saved_with_ckpt": row0(S_ck),
            "_mem_layer_saved_without_ckpt": row0(S_nock),
            "_mem_raw_layer_saved_with_ckpt": row0(raw_ck),
            "_mem_raw_layer_saved_without_ckpt": row0(raw_nock),
            "_mem_layer_fwd_peak_with_ckpt": row0(tables.mem_peak("block", "fwd", b, tp, True)),
            "_mem_layer_fwd_peak_without_ckpt": row0(fwd_peak_nock),
            "_mem_layer_bwd_peak": row0(bwd_peak),
            "_mem_layer_output": row0(out),
            "_mem_module_fwd_saved": row0(np.asarray(mod_saved)[i]),
            "_mem_pre_layer_full_weights": row0(pre_W),
            "_mem_pre_layer_full_grads": row0(pre_G),
            "_mem_pre_layer_full_opts": row0(pre_O),
            "_mem_pre_layer_saved_without_ckpt": row0(pre_saved),
            "_mem_pre_layer_states": row0(pre_states),
            "_mem_post_layer_full_weights": row0(post_W),
            "_mem_post_layer_full_grads": row0(post_G),
            "_mem_post_layer_full_opts": row0(post_O),
            "_mem_post_layer_saved_without_ckpt": row0(tables.mem_saved("post", False, f64(pp_b), f64(pp_tp))),
            "_mem_post_layer_states": row0(post_states),
            "_mem_post_layer_fwd_peak": row0(post_fwd_peak),
            "_mem_post_layer_bwd_peak": row0(post_bwd_peak),
            "_mem_post_layer_output": row0(post_output),
            "_mem_module_fwd_states": row0(np.asarray(fwd_states)[i]),
            "_mem_module_bwd_states": row0(np.asarray(bwd_states)[i]),
        })
        return e

    def reduce_and_gather(x, y_num, mask):
        """:2813-2824: indices, gathered stable / delta / rows with -1 -> inf."""
        indices = sample_pareto_frontier(x, y_num / G, S, mask=mask)
        sel_s = x[ar_n, indices].astype(np.float64)
        sel_d = y_num[ar_n, indices].astype(np.float64)
        sel_sol = rows[indices]
        sel_s[indices == -1] = np.inf
        sel_d[indices == -1] = np.inf
        sel_sol[indices == -1] = np.inf
        return indices, sel_s, sel_d, sel_sol

    if inner in ("c", "c-fused"):  # "c-fused": the argmin objective as one fused multiply-add
        assert analysis is None, "the C loops cover the tuning path only"
        assert list(pre_saved_micro_batches_candidates) == list(range(P + 1))
        assert list(num_layers_candidates) == list(range(1, Lmax + 1))
        assert list(num_ckpt_layers_candidates) == list(range(Cmax + 1))
        from . import stage_c
        from .pareto import alpha_ratios

        res = stage_c.run(
            rows.shape[0], Lmax, Cmax, P + 1, S, G, alpha_ratios(S),
            lat=lat,
            mem=dict(T0=2 * (Wbuf + Gbuf) + O // ore_size, T1=2 * (Wbuf + Gbuf), pWG=pW + pG,
                     pO=pO, pWGO=pW + pG + pO, S_ck=S_ck, S_nock=S_nock, D_ck=D_ck, D_nock=D_nock,
                     fwd_peak=fwd_peak_nock, bwd_peak=bwd_peak, out=out, gcb=gcb, mf=mf,
                     RD=raw_nock - S_nock),
            post=dict(nAG=nAG, nRS=nRS, opb=opb),
            scalars=dict(
                pre_fwd=pre_fwd, pre_bwd=pre_bwd, W1=np.where(pp_wre == 1, pre_AG, 0),
                W2=np.where(pp_gre == 1, pre_RS, 0), W1d=np.where(pp_wre == 1, 0, pre_AG),
                W2d=np.where(pp_gre == 1, 0, pre_RS), post_fwd=post_fwd, pre_saved=pre_saved,
                pre_states=pre_states, pre_states_and_saved=pre_states_and_saved,
                post_states=post_states, post_fwd_peak=post_fwd_peak,
                post_bwd_peak=post_bwd_peak, post_output=post_output),
            pp_wre=int(np.asarray(pp_wre).reshape(-1)[0] == 1),
            pp_gre=int(np.asarray(pp_gre).reshape(-1)[0] == 1), cap=cap, threads=threads,
            fused=inner == "c-fused")
        out_tuples = []
        for stable_t, delta_t, idx_t in res:
            sol_t = rows[idx_t]  # :2819-2824: gather, then -1 -> inf
            sol_t[idx_t == -1] = np.inf
            out_tuples.append((stable_t, delta_t, sol_t, idx_t))
        return tuple(out_tuples)

    for c in num_ckpt_layers_candidates:
        valid_l = c <= num_layers.flatten()
        c_eq_l = c == num_layers
        c_eq_0 = c == 0
        last_ck = c > 0
        stable, delta = get_latencies(c)

        W1 = np.where(pp_wre == 1, pre_AG, 0)
        W2 = np.where(pp_gre == 1, pre_RS, 0)
        W1d = np.where(pp_wre == 1, 0, pre_AG)
        W2d = np.where(pp_gre == 1, 0, pre_RS)
        stable_pre = stable + pre_fwd + pre_bwd + W1 + W2
        delta_pre = delta + W1d + W2d

        k = "ck" if last_ck else "nock"
        PS1 = np.where(pp_wre == 1, nAG[k], 0)
        PS2 = np.where(pp_gre == 1, nRS[k], 0)
        PD1 = np.where(pp_wre == 1, 0, nAG[k])
        PD2 = np.where(pp_gre == 1, 0, nRS[k])
        stable_post = stable + post_fwd + opb + PS1 + PS2
        delta_post = delta + PD1 + PD2
        stable_pp = stable + pre_fwd + pre_bwd + post_fwd + opb + W1 + W2 + PS1 + PS2
        delta_pp = delta + W1d + W2d + PD1 + PD2

        cur_if_eq = (num_layers - 1) * S_ck
        cur_if_not = c * S_ck + (num_layers - c - 1) * S_nock
        cur_if_not = np.where(num_layers >= c, cur_if_not, MEM_INF)
        cur_saved = cur_if_eq * c_eq_l + cur_if_not * (1 - c_eq_l)
        mod_saved = S_ck * c + S_nock * (num_layers - c)
        mod_saved = np.where(num_layers >= c, mod_saved, MEM_INF)

        if analysis is not None:
            extra_of_c.clear()
            for i in range(n):
                extra_of_c[i] = extra_info(
                    i, c, ((stable, delta), (stable_pre, delta_pre), (stable_post, delta_post),
                           (stable_pp, delta_pp)), mod_saved)

        for p in pre_saved_micro_batches_candidates:
            pipe_saved = p * mod_saved + cur_saved
            ge = c >= (num_layers - 1)
            ck_delta = (D_ck * ge) + (D_nock * (1 - ge))
            peak_f = (
                fwd_states + pipe_saved + ck_delta + fwd_peak_nock + out * p * 2 + gcb
            )
            peak_b = (
                bwd_states + pipe_saved + ck_delta + bwd_peak + out * p * 2 + out * 2 + gcb
            )
            if analysis is not None:
                # :2212-2216: float32 stable + float32 delta / python int stays float32
                lat32 = stable + delta / G
                record(0, p, c, stable, delta, lat32 + p2p, peak_f, peak_b)
            mask = np.maximum(peak_f, peak_b) * (mf_pp + 0.01) <= cap
            ind, s_, d_, sol_ = reduce_and_gather(stable, delta, mask)
            costs_stable[p, valid_l, c] = s_[valid_l]
            costs_delta[p, valid_l, c] = d_[valid_l]
            solutions[p, valid_l, c] = sol_[valid_l]
            idx_base[p, valid_l, c] = ind[valid_l]

            pf = p * pre_saved + peak_f + pre_states_and_saved
            pb = p * pre_saved + peak_b + pre_states_and_saved
            if analysis is not None:
                record(1, p, c, stable_pre, delta_pre, stable_pre + delta_pre / G + p2p, pf, pb)
            mask = np.maximum(pf, pb) * mf_pp <= cap
            ind, s_, d_, sol_ = reduce_and_gather(stable_pre, delta_pre, mask)
            costs_stable_pre[p, valid_l, c] = s_[valid_l]
            costs_delta_pre[p, valid_l, c] = d_[valid_l]
            solutions_pre[p, valid_l, c] = sol_[valid_l]
            idx_pre[p, valid_l, c] = ind[valid_l]

            if p == 0:
                f_in = fwd_states + post_states + mod_saved + post_fwd_peak + gcb
                b_in = (
                    bwd_states
                    + post_states
                    + mod_saved
                    + post_bwd_peak
                    + (raw_nock - S_nock) * c_eq_0
                    + gcb
                )
                pf = np.maximum(f_in, peak_f + post_states)
                pb = np.maximum(b_in, peak_b - out + post_states) + post_output
                if analysis is not None:
                    record(2, p, c, stable_post, delta_post, stable_post + delta_post / G + p2p, pf, pb)
                mask = np.maximum(pf, pb) * mf_pp <= cap
                ind, s_, d_, sol_ = reduce_and_gather(stable_post, delta_post, mask)
                # The reference rebinds the layer mask here (:3021-3023); the narrowed mask
                # then also governs the base / with_pre writes of every later p of this c.
                valid_l = np.logical_and(valid_l, c != num_layers.flatten() - 1)
                costs_stable_post[valid_l, c] = s_[valid_l]
                costs_delta_post[valid_l, c] = d_[valid_l]
                solutions_post[valid_l, c] = sol_[valid_l]
                idx_post[valid_l, c] = ind[valid_l]

                pf = pf + pre_states + pre_saved
                pb = pb + pre_states + pre_saved
                if analysis is not None:  # no p2p term here (:3071)
                    record(3, p, c, stable_pp, delta_pp, stable_pp + delta_pp / G, pf, pb)
                mask = np.maximum(pf, pb) * mf <= cap
                ind, s_, d_, sol_ = reduce_and_gather(stable_pp, delta_pp, mask)
                if c != Cmax - 1:  # :3103
                    costs_stable_nopp[c] = s_[-1]
                    costs_delta_nopp[c] = d_[-1]
                    solutions_nopp[c] = sol_[-1]
                    idx_nopp[c] = ind[-1]

    return (
        (costs_stable, costs_delta, solutions, idx_base),
        (costs_stable_pre, costs_delta_pre, solutions_pre, idx_pre),
        (costs_stable_post, costs_delta_post, solutions_post, idx_post),
        (costs_stable_nopp, costs_delta_nopp, solutions_nopp, idx_nopp),
    )


def batched_tune_best_latency_for_stage(
    tables,
    config,
    pre_saved_micro_batches_candidates,
    num_layers_candidates,
    num_ckpt_layers_candidates,
    num_nodes,
    num_gpus_per_node,
    gradient_accumulation_steps,
    tp_size=None,
    sample_size=None,
    debug=None,
    inner="numpy",
    threads=0,
):
    """:581-684: enumerate the rows, return all-``inf`` tables when there are none."""
    for cands, lo in (
        (pre_saved_micro_batches_candidates, 0),
        (num_layers_candidates, 1),
        (num_ckpt_layers_candidates, 0),
    ):
        assert set(cands) == set(range(lo, max(cands) + 1)), f"{cands} is not sequential"
    if sample_size is None:
        sample_size = config.tuning.sample_size
    rows = create_search_space(
        num_nodes,
        num_gpus_per_node,
        config.training.global_batch_size,
        gradient_accumulation_steps,
        config,
        constraint_fn=tables.constraint,
        tp_size=tp_size,
    )
    if debug is not None:
        debug["rows"] = rows
    if rows.size == 0:
        P = max(pre_saved_micro_batches_candidates)
        L = max(num_layers_candidates)
        C = max(num_ckpt_layers_candidates)
        S, F = sample_size, 10
        inf = lambda *shape: np.full(shape, np.inf)
        neg = lambda *shape: np.full(shape, -1, dtype=np.int64)
        return (
            (inf(P + 1, L, C + 1, S), inf(P + 1, L, C + 1, S), inf(P + 1, L, C + 1, S, F), neg(P + 1, L, C + 1, S)),
            (inf(P + 1, L, C + 1, S), inf(P + 1, L, C + 1, S), inf(P + 1, L, C + 1, S, F), neg(P + 1, L, C + 1, S)),
            (inf(L, C + 1, S), inf(L, C + 1, S), inf(L, C + 1, S, F), neg(L, C + 1, S)),
            (inf(C + 1, S), inf(C + 1, S), inf(C + 1, S, F), neg(C + 1, S)),
        )
    return batched_stage_analyze(
        tables,
        config,
        pre_saved_micro_batches_candidates,
        num_layers_candidates,
        num_ckpt_layers_candidates,
        num_nodes,
        num_gpus_per_node,
        gradient_accumulation_steps,
        rows,
        sample_size,
        debug=debug,
        inner=inner,
        threads=threads,
    )
