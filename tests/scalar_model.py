"""Independent scalar re-derivation of Mist's per-stage cost model for ONE candidate cell.

Written from the mathematical description of the model (phases, resource overlap, memory
budget), one python float at a time, with its own data flow: no arrays, no broadcasting, no code
shared with ``oracle/``.  The oracle's vectorised tables are checked against it cell by cell, so
a dropped term, a wrong sign, a transposed operand or a wrong index in either formulation shows
up as a mismatch.  Floating-point association is not reproduced here, so comparisons use a
tolerance of a few ulps (1e-12 relative), and feasibility is compared away from the boundary.
"""
import itertools

MB = float(1 << 20)

# Overlap factor layout of the 28 interference parameters: the 4-way case, then the 3-way cases
# and the 2-way cases, each listed in lexicographic order of the *excluded* / included resources
# as in the reference's mask tables; resources are (compute, gpu<->gpu, cpu->gpu, gpu->cpu).
_THREE = [(0, 1, 2), (0, 1, 3), (0, 2, 3), (1, 2, 3)]
_TWO = [(0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3)]


def factor_lookup(params):
    table = {(0, 1, 2, 3): list(params[0:4])}
    for i, key in enumerate(_THREE):
        table[key] = list(params[4 + 3 * i: 7 + 3 * i])
    for i, key in enumerate(_TWO):
        table[key] = list(params[16 + 2 * i: 18 + 2 * i])
    return table


def overlap_time(compute, g2g, c2g, g2c, params):
    """Time to drain four concurrent resources: while several are busy each progresses at
    1/factor of its solo speed; the phase ends when the first one finishes."""
    left = [compute, g2g, c2g, g2c]
    table = factor_lookup(params)
    elapsed = 0.0
    while True:
        busy = tuple(i for i in range(4) if abs(left[i]) > 1e-8)
        if len(busy) <= 1:
            return elapsed + sum(left)
        f = table[busy]
        dt = min(left[i] * f[j] for j, i in enumerate(busy))
        for j, i in enumerate(busy):
            left[i] = (left[i] * f[j] - dt) / f[j]
        elapsed += dt


def alpha_beta(gbytes, inter, intra, gg_params, factor):
    n = inter * intra
    if gbytes < 1e-5 or n == 1:
        return 0.0
    idx = {1: 0, 2: 1, 4: 2}
    oi = idx.get(inter, 3)
    ii = idx.get(intra, 3)
    k, b = gg_params[(oi * 4 + ii) * 2], gg_params[(oi * 4 + ii) * 2 + 1]
    return (gbytes / k * (n - 1) / n + b) * factor


def host_link(gbytes, kb):
    return 0.0 if gbytes == 0 else gbytes / kb[0] + kb[1]


def exec_latency(tables, kind, b, tp, inter, intra, G):
    f = bw = ef = eb = 0.0
    for fwd, bwd, xf, xb in tables.op_profiles(kind, b, tp, inter, intra):
        if bwd != 0 and bwd > 2.3 * fwd:
            bwd = 2 * fwd
        fwd, bwd = fwd + xf, bwd + xb
        if fwd < 5e-5 or bwd < 1e-4:
            continue
        f, bw, ef, eb = f + fwd, bw + bwd, ef + xf, eb + xb
    for ga in tables.grad_accum_profiles(kind, b, tp):
        bw += ga * (G - 1) / G
    return f, bw, ef, eb


def evaluate_cell(config, tables, n, m, G, row, l, c, p, L):
    """Returns ``{variant: (stable, delta, peak_fwd, peak_bwd, factor)}`` for the four stage
    variants of one strategy row ``(b, dp, tp, wre, gre, ore, wo, go, oo, ao)`` with ``l`` layers,
    ``c`` checkpointed layers and ``p`` pre-saved micro-batches; stable / delta are the float64
    values before the float32 rounding of the middle-stage pair."""
    hw = config.hardware
    b, dp, tp, wre, gre, ore, wo, go, oo, ao = row
    b, dp, tp = int(b), int(dp), int(tp)
    B = config.training.global_batch_size
    gg, c2g_kb, g2c_kb = hw.gpu_gpu_comm_params, hw.cpu_gpu_comm_params, hw.gpu_cpu_comm_params
    params = hw.interference_model_params
    adv = bool(config.enable_advanced_opt_in_first_block)
    I = lambda comp, g2g, g2c, c2g: overlap_time(comp, g2g, c2g, g2c, params)

    # ---- block layer tables ----
    W = float(tables.mem_full_states("block", "weights", tp))
    Gr = float(tables.mem_full_states("block", "grads", tp))
    O = float(tables.mem_full_states("block", "opts", tp))
    raw = {True: float(tables.mem_saved("block", True, b, tp)), False: float(tables.mem_saved("block", False, b, tp))}
    fwd_peak = float(tables.mem_peak("block", "fwd", b, tp, False))
    bwd_peak = float(tables.mem_peak("block", "bwd", b, tp))
    out = float(tables.mem_output("block", b, tp))
    ws, gs, os_ = (dp if wre else 1), (dp if gre else 1), (dp if ore else 1)
    inter_tp, intra_tp = (tp // m, m) if tp > m else (1, tp)
    e_fwd, e_bwd, x_fwd, x_bwd = exec_latency(tables, "block", b, tp, inter_tp, intra_tp, G)

    # ---- swaps and collectives of one layer ----
    gb = lambda mb: mb / 1024.0
    so = lambda mb: host_link(gb(mb), g2c_kb)
    si = lambda mb: host_link(gb(mb), c2g_kb)
    wW, wG, wO = W / ws * wo, Gr / gs * go, O / os_ * oo
    inter_dp, intra_dp = (n, dp // n) if dp > n else (dp, 1)
    AG = alpha_beta(gb(W), inter_dp, intra_dp, gg, 1.0)
    RS = alpha_beta(gb(Gr), inter_dp, intra_dp, gg, 1.1)
    AR = alpha_beta(gb(Gr), inter_dp, intra_dp, gg, 2.1)
    grad_sync_last = RS if ore else AR

    def phase_costs(first_mb, ck):
        """(middle layer, first-layer family, last-layer family) of one micro-batch kind."""
        act_out, act_in = so(raw[ck] * ao), si(raw[ck] * ao)
        if first_mb:  # first forward / last backward micro-batch
            f_g2g, f_g2c, f_c2g = AG * ore, so(wO) + so(wW), si(wO) + si(wG)
            b_g2g = AG * wre + grad_sync_last
            b_red = grad_sync_last
        else:
            f_g2g, f_g2c, f_c2g = AG * wre, 0.0, si(wW)
            b_g2g = AG * wre + RS * gre
            b_red = RS * gre
        b_g2c, b_c2g = so(wG), si(wW) + si(wG) + act_in
        comp_f = e_fwd - x_fwd
        comp_b, x_b = ((e_fwd + e_bwd) - (x_fwd + x_bwd), x_fwd + x_bwd) if ck else (e_bwd - x_bwd, x_bwd)
        f_layer = I(comp_f, f_g2g, f_g2c + act_out, f_c2g) + x_fwd
        b_layer = I(comp_b, b_g2g, b_g2c, b_c2g) + x_b
        pre_g2g = f_g2g if (first_mb or adv) else 0.0
        pre_c2g = f_c2g if adv else 0.0
        first = (
            I(0.0, pre_g2g, 0.0, pre_c2g)                       # prologue before the first layer
            + I(0.0, b_red, b_g2c if adv else 0.0, 0.0)          # epilogue after its backward
            + I(comp_f, f_g2g, 0.0, f_c2g) + x_fwd
            + I(comp_b, b_red, b_g2c if adv else 0.0, 0.0) + x_b
        )
        last = (
            I(0.0, 0.0, f_g2c + act_out, 0.0)
            + I(0.0, AG * wre, 0.0, b_c2g)
            + I(comp_f, 0.0, f_g2c + act_out, 0.0) + x_fwd
            + I(comp_b, AG * wre, 0.0, b_c2g) + x_b
        )
        return f_layer + b_layer, first, last

    def stage_latency(first_mb):
        mid = {ck: phase_costs(first_mb, ck) for ck in (False, True)}
        inner = max(l - 2, 0)
        n_ck = min(max(c - 1, 0), inner)
        total = n_ck * mid[True][0] + (inner - n_ck) * mid[False][0]
        total += mid[c == l][1]     # first layer is checkpointed only when every layer is
        total += mid[c != 0][2]     # last layer is checkpointed as soon as any layer is
        return total

    if G == 1:
        stable, delta = stage_latency(True), 0.0
    else:
        stable = stage_latency(False)
        delta = stage_latency(True) - stable

    # ---- pre / post layers ----
    strategy = config.tuning.pre_post_strategy
    if strategy == "dp":
        pdp, ptp, pwre, pgre, pore = n * m, 1, False, False, True
    else:
        pdp, ptp, pwre, pgre, pore = n, m, False, True, strategy.endswith("with-ore")
    pb = B // G // pdp
    pinter, pintra = (ptp // m, m) if ptp > m else (1, ptp)
    pre_f, pre_b, _, _ = exec_latency(tables, "pre", pb, ptp, pinter, pintra, G)
    post_f, post_b, _, _ = exec_latency(tables, "post", pb, ptp, pinter, pintra, G)
    fs = lambda kind, item: float(tables.mem_full_states(kind, item, ptp))
    pin, pia = (n, pdp // n) if pdp > n else (pdp, 1)
    coll = lambda mb, fac: 0.0 if pdp == 1 else alpha_beta(gb(mb), pin, pia, gg, fac)
    pre_AG, post_AG = coll(fs("pre", "weights"), 1.0), coll(fs("post", "weights"), 1.0)
    pre_RS, post_RS = coll(fs("pre", "grads"), 1.1), coll(fs("post", "grads"), 1.1)
    shard = lambda on: pdp if on else 1
    pre_states = (fs("pre", "weights") / shard(pwre) + fs("pre", "grads") / shard(pgre)
                  + fs("pre", "opts") / shard(pore))
    pre_saved = float(tables.mem_saved("pre", False, pb, ptp))
    post_states = fs("post", "weights") + fs("post", "grads") + fs("post", "opts") / shard(pore)
    post_fwd_peak = float(tables.mem_peak("post", "fwd", pb, ptp, None))
    post_bwd_peak = float(tables.mem_peak("post", "bwd", pb, ptp))
    post_out = float(tables.mem_output("post", pb, ptp))

    pre_stable = pre_f + pre_b + (pre_AG if pwre else 0.0) + (pre_RS if pgre else 0.0)
    pre_delta = (0.0 if pwre else pre_AG) + (0.0 if pgre else pre_RS)
    ck_last = c > 0
    hidden_w = max(e_fwd - so(raw[ck_last] * ao), 0.0)
    hidden_g = max((e_fwd + e_bwd if ck_last else e_bwd) - AG * wre - (si(wW) + si(wG)) - si(raw[ck_last] * ao), 0.0)
    nAG, nRS = max(post_AG - hidden_w, 0.0), max(post_RS - hidden_g, 0.0)
    # the post layer's backward hides behind the prologue of the last layer's backward
    prologue_b = I(0.0, AG * wre, 0.0, si(wW) + si(wG) + si(raw[True] * ao))
    post_stable = post_f + max(post_b - prologue_b, 0.0) + (nAG if pwre else 0.0) + (nRS if pgre else 0.0)
    post_delta = (0.0 if pwre else nAG) + (0.0 if pgre else nRS)

    # ---- memory ----
    frag = max(0, config.model.hidden_size / 2048 - 1) * 0.005 + max(0, config.training.max_sequence_length / 2048 - 1) * 0.045
    mf = (1.0 + frag + 0.025 * (wo > 0) + 0.025 * (go > 0) + 0.03 * (oo > 0) + 0.04 * (ao > 0)
          + 0.025 * bool(wre) + 0.025 * bool(gre) + 0.04 * (tp > 1) + 0.01 * (b >= 4))
    gcb = 0.0 if config.model.use_flash_attn else 2 * b * config.model.num_attention_heads / tp * config.training.max_sequence_length**2 / 1024**2
    pW, pG, pO = W / ws * (1 - wo), Gr / gs * (1 - go), O / os_ * (1 - oo)
    Wbuf = max(fs("pre", "weights"), fs("post", "weights"), W) if (ws > 1 or pwre or wo > 0) else 0.0
    Gbuf = max(fs("pre", "grads"), fs("post", "grads"), Gr) if (gs > 1 or pgre or go > 0) else 0.0
    fwd_states = 2 * (Wbuf + Gbuf) + (O // os_) + l * (pW + pG) + (l - 1) * pO
    bwd_states = 2 * (Wbuf + Gbuf) + l * (pW + pG + pO)
    kept = {ck: raw[ck] * (1 - ao) for ck in (True, False)}
    module_saved = c * kept[True] + (l - c) * kept[False]
    current_saved = (l - 1) * kept[True] if c == l else c * kept[True] + (l - c - 1) * kept[False]
    resident = p * module_saved + current_saved + raw[c >= l - 1] * ao
    peak_f = fwd_states + resident + fwd_peak + 2 * p * out + gcb
    peak_b = bwd_states + resident + bwd_peak + 2 * p * out + 2 * out + gcb
    res = {
        "base": (stable, delta, peak_f, peak_b, mf + 0.025 + 0.01),
        "with_pre": (stable + pre_stable, delta + pre_delta,
                     peak_f + (p + 1) * pre_saved + pre_states, peak_b + (p + 1) * pre_saved + pre_states,
                     mf + 0.025),
    }
    if p == 0:
        f_in = fwd_states + post_states + module_saved + post_fwd_peak + gcb
        b_in = bwd_states + post_states + module_saved + post_bwd_peak + (raw[False] * ao if c == 0 else 0.0) + gcb
        pf = max(f_in, peak_f + post_states)
        pb_ = max(b_in, peak_b - out + post_states) + post_out
        res["with_post"] = (stable + post_stable, delta + post_delta, pf, pb_, mf + 0.025)
        res["no_pp"] = (stable + pre_stable + post_stable, delta + pre_delta + post_delta,
                        pf + pre_states + pre_saved, pb_ + pre_states + pre_saved, mf)
    return res
