"""Edge cases through the reference-shaped API on the GPU: empty and degenerate shapes,
many partitions, HIP-graph replay of the fused kernel."""
import numpy as np
import pytest

from liteform_ae_amd.format_matrix_market import MTX
from oracle import liteform_oracle as O

from helpers import assert_hyb_equal, mtx_from_rows, skewed_matrix

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa():
    from liteform_ae_amd import format_algos
    return format_algos


@pytest.fixture(scope="module")
def torch():
    import torch
    return torch


def product(fa, torch, g, cfg, feat=32, seed=0):
    rng = np.random.default_rng(seed)
    B = rng.uniform(-1, 1, size=(g.num_dst_nodes(), feat)).astype(np.float32)
    C = fa.spmm_hyb(fa.build_hyb_format_device(g, cfg), torch.from_numpy(B).cuda()).cpu().numpy()
    indptr, indices, data = g.adj_tensors("csr")
    ref = O.spmm_csr_f64(indptr, indices, data, g.coo_mtx.shape, B)
    bound = O.spmm_abs_bound(indptr, indices, data, g.coo_mtx.shape, B)
    assert C.shape == ref.shape
    assert (np.abs(C - ref) <= 1e-5 * bound).all()
    return C


def test_matrix_without_nonzeros(fa, torch):
    g = MTX.from_coo(np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64), (17, 9))
    cfg = fa.search_bucket_config(g, 2, fa.CostModelSettings(32, 2))
    assert cfg == [[], []] == O.search_bucket_config(g, 2, O.OracleCostModelSettings(32, 2))
    assert_hyb_equal(fa.build_hyb_format(g, cfg), O.build_hyb_format_sequential(g, cfg))
    C = product(fa, torch, g, cfg)
    assert (C == 0).all()


def test_single_entry_and_single_column(fa, torch):
    g = mtx_from_rows([[0, 0][:1], [0]], (2, 1))           # two rows, one column
    cfg = fa.search_bucket_config(g, 1, fa.CostModelSettings(32, 1))
    assert cfg == O.search_bucket_config(g, 1, O.OracleCostModelSettings(32, 1))
    assert_hyb_equal(fa.build_hyb_format(g, cfg), O.build_hyb_format_sequential(g, cfg))
    product(fa, torch, g, cfg)
    g = mtx_from_rows([[2]], (1, 5))                       # a single nonzero: the search refuses it
    with pytest.raises(ValueError):
        fa.search_bucket_config(g, 1, fa.CostModelSettings(32, 1))
    product(fa, torch, g, [[1]])                           # but a given config still works


def test_rectangular_both_ways(fa, torch):
    rng = np.random.default_rng(3)
    for shape in ((50, 4000), (4000, 50)):
        g = skewed_matrix(rng, shape[0], shape[1], mean_deg=4, heavy_rows=1, heavy_len=shape[1])
        for parts in (1, 3):
            try:
                want = O.search_bucket_config(g, parts, O.OracleCostModelSettings(64, parts))
            except ValueError:
                continue
            cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(64, parts))
            assert cfg == want
            assert_hyb_equal(fa.build_hyb_format(g, cfg), O.build_hyb_format_closed_form(g, cfg))
            product(fa, torch, g, cfg, feat=64)


def test_many_partitions(fa, torch):
    rng = np.random.default_rng(8)
    g = skewed_matrix(rng, 2000, 3000, mean_deg=30, heavy_rows=3, heavy_len=5000, values=True)
    for parts in (16, 37, 64):
        try:
            want = O.search_bucket_config(g, parts, O.OracleCostModelSettings(128, parts))
        except ValueError:
            with pytest.raises(ValueError):
                fa.search_bucket_config(g, parts, fa.CostModelSettings(128, parts))
            want = [[1, 4, 16, 64]] * parts
        else:
            assert fa.search_bucket_config(g, parts, fa.CostModelSettings(128, parts)) == want
        assert_hyb_equal(fa.build_hyb_format(g, want), O.build_hyb_format_closed_form(g, want))
        product(fa, torch, g, want, feat=128)


def test_more_partitions_than_columns(fa, torch):
    g = mtx_from_rows([[0, 1, 2], [1, 2], [0, 2], [0, 1]], (4, 3))
    widths = [[1, 2]] * 5                                  # partition size ceil(3/5) = 1; two empty partitions
    assert_hyb_equal(fa.build_hyb_format(g, widths), O.build_hyb_format_sequential(g, widths))
    product(fa, torch, g, widths)


def test_graph_replay_matches_eager(fa, torch):
    """The run entry point only launches kernels, so it can be captured in a HIP graph.
    Replays are interleaved with eager work and every replay is compared with the eager result."""
    rng = np.random.default_rng(12)
    g = skewed_matrix(rng, 6000, 20000, mean_deg=9, heavy_rows=3, heavy_len=60000)
    for parts in (1, 3):
        cfg = fa.search_bucket_config(g, parts, fa.CostModelSettings(128, parts, cost_model="gfx950"))
        fmt = fa.build_hyb_format_device(g, cfg)
        plan = fa.HybSpMM(fmt, 128)
        assert plan.info["heavy_rows"] >= 1, (cfg, plan.info, fmt.ell_rows)   # the partial-row kernel is in the graph
        B = torch.rand((20000, 128), device="cuda") - 0.5
        out = torch.empty((6000, 128), device="cuda")
        eager = plan.run(B).clone()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            plan.run(B, out)                            # warm-up on the capture stream
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                plan.run(B, out)
        torch.cuda.current_stream().wait_stream(side)
        for i in range(4):
            out.fill_(float("nan"))
            junk = (torch.rand((512, 512), device="cuda") @ torch.rand((512, 512), device="cuda")).sum()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {i} differs"
            assert torch.isfinite(junk)
        # new operand values through the same graph
        B.mul_(2.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, plan.run(B))
        plan.close()


def test_matrix_features_on_device(fa, torch):
    """Integer fields exact, float fields to 1e-9 relative against the host routine
    (numpy's two-pass standard deviation against sqrt(E[d^2] - E[d]^2) on exact sums)."""
    rng = np.random.default_rng(11)
    g = skewed_matrix(rng, 5000, 3000, mean_deg=7.0, heavy_rows=3, heavy_len=2500)
    # duplicated COO entries: "nnz" counts stored entries, row lengths come from the CSR
    row = np.concatenate([g.coo_mtx.row, g.coo_mtx.row[:100]])
    col = np.concatenate([g.coo_mtx.col, g.coo_mtx.col[:100]])
    for m in (g, MTX.from_coo(row, col, g.coo_mtx.shape), mtx_from_rows([[], [1], []], (3, 4))):
        want = m.matrix_features()
        got = fa.matrix_features_device(m)
        assert list(got) == list(want)
        for key in ("name", "num_rows", "num_cols", "nnz", "min_nnz_per_row", "max_nnz_per_row"):
            assert got[key] == want[key], key
        for key in want:
            if key.startswith(("avg", "std", "min_nnz_density", "max_nnz_density")):
                assert got[key] == pytest.approx(want[key], rel=1e-9, abs=1e-15), key
