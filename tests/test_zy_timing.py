"""Timing comparisons on the GPU, kept apart from the parity tests and collected after them
(the file name sorts behind every other test file except the no-allocation entry point's):
the launch shape the model picks against its measured competitors, and a bucket-width fold
the MI355X cost model asks for against the unfolded widths.

Every comparison interleaves the candidates (A, B, C, A, B, C, ...) and compares medians, so
that a slow or noisy box scales all of them alike; the bounds are far above the 8 % spread seen
between boxes and only catch a choice that is plainly wrong."""
import numpy as np
import pytest

from liteform_ae_amd.format_matrix_market import MTX

pytestmark = pytest.mark.gpu

ROUNDS = 5


def interleaved_medians(plans, B, C, rounds=ROUNDS):
    """plans: {name: HybSpMM}.  One warm-up run each, then `rounds` rounds of one timed run per
    plan in turn; returns {name: median ms}."""
    for plan in plans.values():
        plan.time_ms(B, C, warmup=1, repeat=1)
    ms = {name: [] for name in plans}
    for _ in range(rounds):
        for name, plan in plans.items():
            ms[name].append(float(plan.time_ms(B, C, warmup=0, repeat=1)[0]))
    return {name: float(np.median(v)) for name, v in ms.items()}


@pytest.fixture(scope="module")
def big():
    import torch
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import make_workload
    return make_workload("cfg3"), fa, torch


@pytest.mark.parametrize("feat,shapes", [(128, [(1, 1), (1, 2), (2, 1), (2, 2)]),
                                         (256, [(1, 2), (1, 4), (2, 2), (2, 4)])])
def test_model_pick_against_measured_shapes(big, feat, shapes):
    """The launch shape the model picks for the 2.45M-row graph, timed against its nearest
    competitors (the shapes that were within a few percent of the fastest in the sweep the
    model was fitted to)."""
    wl, fa, torch = big
    g = wl.matrix
    pick = fa.predict_launch_shape(g, feat)
    assert pick in shapes, pick
    B = torch.rand((g.num_dst_nodes(), feat), device="cuda") - 0.5
    C = torch.empty((g.num_src_nodes(), feat), device="cuda")
    plans, fmts = {}, []
    for p in sorted({s[0] for s in shapes}):
        cfg = fa.search_bucket_config(g, p, fa.CostModelSettings(feat, p, cost_model="gfx950"))
        fmt = fa.build_hyb_format_device(g, cfg)
        fmts.append(fmt)
        for w in sorted({s[1] for s in shapes if s[0] == p}):
            plans[(p, w)] = fa.HybSpMM(fmt, feat, windows=w)
    ms = interleaved_medians(plans, B, C)
    for plan in plans.values():
        plan.close()
    print(f"\nN={feat}: pick {pick}, medians {ms}")
    assert ms[pick] <= 1.25 * min(ms.values()), (pick, ms)


def test_a_folded_choice_against_the_initial_widths():
    """33 entries per row: the MI355X fold model asks for 16-slot rows at N = 128 (measured 2.7 %
    faster than the initial 64-slot rows); it must at least not be plainly slower."""
    import torch
    from liteform_ae_amd import format_algos as fa
    from liteform_ae_amd.synthetic import csr_from_row_degrees
    rng = np.random.default_rng(33)
    n = 1_000_000
    indptr, indices = csr_from_row_degrees(np.full(n, 33), n, rng)
    g = MTX.from_csr(indptr, indices, (n, n), data=rng.random(len(indices), dtype=np.float32))
    feat = 128
    cfg = fa.search_bucket_config(g, 1, fa.CostModelSettings(feat, 1, cost_model="gfx950"))
    assert cfg == [[16]]
    B = torch.rand((n, feat), device="cuda") - 0.5
    C = torch.empty((n, feat), device="cuda")
    fmts = {"folded": fa.build_hyb_format_device(g, cfg),
            "initial": fa.build_hyb_format_device(g, [[32, 64]])}      # a few rows lost a duplicate: 32 entries
    plans = {name: fa.HybSpMM(fmt, feat) for name, fmt in fmts.items()}
    ms = interleaved_medians(plans, B, C, rounds=9)
    outs = {name: plan.run(B).clone() for name, plan in plans.items()}
    for plan in plans.values():
        plan.close()
    print(f"\nfold chain: {ms}")
    assert ms["folded"] <= 1.25 * ms["initial"], ms
    # same product either way (a row's terms are added in the same order, in pieces of 16 or 64)
    assert float((outs["folded"] - outs["initial"]).abs().max()) <= 1e-4
