"""CPU oracle for LiteForm's CELL/hyb SpMM hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain Python/numpy, what the reference computes on the
path  CSR in -> bucket-config search -> hyb composition -> SpMM.  It is the checker
the HIP implementation is compared against; nothing in the shipped package may
import it.  Only tests, the smoke entry and the benchmark's CPU-baseline leg use it.

Reference files are cited as
  FA = playground_pipline/format_algos.py
  FM = playground_pipline/format_matrix_market.py
  P5 = playground_pipline/proc05.spmm.end-to-end.py

Two independent formulations are kept on purpose:
  * ``*_sequential`` functions walk the data in the reference's order with Python
    dicts / lists / sets, so insertion order, aliasing and the strict-< tie rule
    are the same by construction (small inputs only);
  * ``*_closed_form`` functions compute the same result from per-(row, partition)
    counts with numpy (any size that fits in memory).
Tests pin the sequential forms with hand-evaluated examples and brute force, and
the closed forms against the sequential ones on random inputs.

Pinning status: every function of the format path (initial buckets, single-row
fix-up, cost function, fold search, hyb builder) is pinned twice: by hand-worked
known answers, invariants and brute force (tests/test_oracle_format.py,
tests/test_golden_examples.py), and bit for bit - float costs included - against
vectors produced by the reference's own functions on 21 seeded matrices
(tests/golden/search_vectors.*, tests/test_reference_vectors.py).  The reference's
GPU kernel comes from an external code generator and has no recorded outputs, so
the SpMM result is anchored on scipy CSR(f64) @ dense(f64), the reference's own
CPU product (FM:89-99).
"""
from __future__ import annotations

import bisect
import math
from typing import Dict, List, Sequence, Tuple

import numpy as np
import scipy.sparse as sp

WIDTH_LIMIT = 1024  # FA:821 default width_limit


# --------------------------------------------------------------------------- records
class OracleBucket:
    """Cost-model record of one (partition, width) bucket.  FM:12-37."""

    __slots__ = ("bucket_width", "num_rows", "nnz", "row_indices", "col_indices")

    def __init__(self, bucket_width, num_rows, nnz, row_indices, col_indices):
        self.bucket_width = bucket_width
        self.num_rows = num_rows          # cost-model rows (a >limit row counts pow2(deg)//limit)
        self.nnz = nnz
        self.row_indices = row_indices    # list of original rows (distinct)
        self.col_indices = col_indices    # set of distinct columns

    def key(self):
        return (self.bucket_width, self.num_rows, self.nnz,
                len(self.row_indices), len(self.col_indices))

    def __repr__(self):
        return "OracleBucket(w=%d, rows=%d, nnz=%d, |R|=%d, |C|=%d)" % self.key()


class OracleCostModelSettings:
    """FA:39-51: a (feat_size, num_parts) pair."""

    def __init__(self, feat_size: int, num_parts: int):
        self.feat_size = feat_size
        self.num_parts = num_parts

    def __str__(self):
        return f"(feat_size={self.feat_size}, num_parts={self.num_parts})"


def _coo_arrays(g):
    return np.asarray(g.coo_mtx.row), np.asarray(g.coo_mtx.col)


def partition_size(num_cols: int, num_parts: int) -> int:
    """ceil(num_cols / num_parts): FA:241 and FA:836."""
    return (num_cols + num_parts - 1) // num_parts


def initial_width(degree: int, width_limit: int = WIDTH_LIMIT) -> Tuple[int, int]:
    """(width, cost-model rows) of a row segment of `degree` nonzeros.  FA:875-882.

    The reference evaluates 2 ** ceil(log2(degree)) in floating point; that equals
    the next power of two for every degree below 2**40, which is what is used here.
    """
    assert degree > 0
    width = 1 << (int(degree) - 1).bit_length()
    rows = 1
    if width > width_limit:
        rows = width // width_limit
        width = width_limit
    return width, rows


# --------------------------------------------------------------------------- search
def get_init_buckets_sequential(g, num_parts: int, width_limit: int = WIDTH_LIMIT):
    """Initial power-of-two bucketing per column partition.  FA:819-900.

    Degrees and neighbour lists come from the raw COO triplets (FA:846-849), so
    duplicate COO entries count twice, exactly as in the reference.
    """
    num_rows = g.num_src_nodes()
    psize = partition_size(g.num_dst_nodes(), num_parts)
    rows, cols = _coo_arrays(g)
    # neighbours[p][r] -> list of columns in COO order
    neighbours: List[Dict[int, list]] = [dict() for _ in range(num_parts)]
    for r, c in zip(rows.tolist(), cols.tolist()):
        neighbours[c // psize].setdefault(r, []).append(c)

    out = []
    for p in range(num_parts):
        pool: Dict[int, OracleBucket] = {}
        for r in range(num_rows):                     # ascending row order: FA:868
            neigh = neighbours[p].get(r)
            if not neigh:
                continue
            deg = len(neigh)
            width, new_rows = initial_width(deg, width_limit)
            bk = pool.get(width)
            if bk is None:
                pool[width] = OracleBucket(width, new_rows, deg, [r], set(neigh))
            else:
                bk.nnz += deg
                bk.num_rows += new_rows
                bk.row_indices.append(r)
                bk.col_indices |= set(neigh)
        out.append(dict(sorted(pool.items())))        # FA:897 keys ascending
    return out


def move_largest_bucket(buckets: Dict[int, OracleBucket], pre_width: int, new_width: int):
    """Fold bucket `pre_width` into `new_width`.  FA:623-648.

    ratio is an integer division, so folding width 1 into a wider bucket moves
    zero cost-model rows (FA:638-639).  A new key is appended at the end of the
    dict order (FA:641); an existing one is merged in place (FA:643-646).
    """
    src = buckets[pre_width]
    moved_rows = src.num_rows * (pre_width // new_width)
    if new_width not in buckets:
        buckets[new_width] = OracleBucket(new_width, moved_rows, src.nnz,
                                          src.row_indices, src.col_indices)
    else:
        dst = buckets[new_width]
        dst.num_rows += moved_rows
        dst.nnz += src.nnz
        dst.row_indices += src.row_indices
        dst.col_indices |= src.col_indices
    del buckets[pre_width]


def move_width_one_bucket(buckets: Dict[int, OracleBucket], widths_snapshot: Sequence[int]):
    """FA:903-923.  `widths_snapshot` is the key list taken before any fold in this
    partition, so it may name a width that no longer exists."""
    new_width = 2
    max_width = max(widths_snapshot)
    while new_width <= max_width and new_width not in widths_snapshot:
        new_width *= 2
    if new_width > max_width:
        raise ValueError("The partition is too small, only having 1 non-zero element.")
    move_largest_bucket(buckets, 1, new_width)


def modify_single_row_buckets(buckets: List[Dict[int, OracleBucket]]):
    """FA:928-954: a bucket with exactly one cost-model row is folded away."""
    for pool in buckets:
        snapshot = sorted(pool.keys(), reverse=True)
        for width in snapshot:
            if pool[width].num_rows == 1:
                if width == 1:
                    move_width_one_bucket(pool, snapshot)
                else:
                    move_largest_bucket(pool, width, width // 2)


def get_memory_cost(bucket_dict: Dict[int, OracleBucket], cfg) -> Dict[str, float]:
    """FA:1035-1166.  Summation runs in dict order; cost3 is floating point."""
    feat_size = cfg.feat_size
    num_parts = cfg.num_parts
    max_w = max(bucket_dict.keys())
    cost = 0
    c1 = c2 = c3 = 0
    for width, bk in bucket_dict.items():
        block = max_w // width                                   # FA:1067
        padded_rows = (bk.num_rows + block - 1) // block * block  # FA:1068-1069
        b1 = 2 * padded_rows * width                             # FA:1071
        b2 = len(bk.col_indices) * feat_size                     # FA:1078
        atomic = num_parts > 1 or width == max_w                 # FA:1081
        out_rows = len(bk.row_indices)
        weight = padded_rows / out_rows if atomic else 1         # FA:1084 (true division)
        b3 = weight * out_rows * feat_size                       # FA:1087
        cost += b1 + b2 + b3                                     # FA:1093-1095
        c1 += b1
        c2 += b2
        c3 += b3
    # both load-imbalance penalties are identically zero in the reference (FA:1101-1119)
    return {"cost": cost, "cost1": c1, "cost2": c2, "cost3": c3, "load_imbalance_penalty": 0}


def modify_bucket_widths(bucket_dict: Dict[int, OracleBucket], cfg) -> List[int]:
    """FA:709-774: greedily fold the widest bucket into half its width, all the way
    down to width 1, and keep the key set of the cheapest state (strict <)."""
    best_cost = get_memory_cost(bucket_dict, cfg)["cost"]
    best = sorted(bucket_dict.keys())
    pre = max(bucket_dict.keys())
    new = pre // 2
    while new >= 1:
        move_largest_bucket(bucket_dict, pre, new)
        c = get_memory_cost(bucket_dict, cfg)["cost"]
        if c < best_cost:
            best = sorted(bucket_dict.keys())
            best_cost = c
        pre = new
        new //= 2
    return best


def get_bucket_config(init_buckets, cfg) -> List[List[int]]:
    """FA:777-816."""
    return [modify_bucket_widths(pool, cfg) if pool else [] for pool in init_buckets]


def search_bucket_config(g, num_parts: int, cfg) -> List[List[int]]:
    """FA:988-1032: init buckets -> single-row fix-up -> per-partition fold search."""
    pools = get_init_buckets_sequential(g, num_parts)
    modify_single_row_buckets(pools)
    return get_bucket_config(pools, cfg)


def search_cost_trace(g, num_parts: int, cfg):
    """Every (sorted key list, cost) state the fold search visits, per partition.
    Not a reference function: exposes the intermediate values of FA:727-772 so
    tests can compare costs bit for bit, not only the arg-min."""
    pools = get_init_buckets_sequential(g, num_parts)
    modify_single_row_buckets(pools)
    traces = []
    for pool in pools:
        tr = []
        if pool:
            tr.append((sorted(pool.keys()), get_memory_cost(pool, cfg)["cost"]))
            pre = max(pool.keys())
            new = pre // 2
            while new >= 1:
                move_largest_bucket(pool, pre, new)
                tr.append((sorted(pool.keys()), get_memory_cost(pool, cfg)["cost"]))
                pre, new = new, new // 2
        traces.append(tr)
    return traces


# --------------------------------------------------------------------------- builder
def build_hyb_format_sequential(g, bucket_widths: List[List[int]]):
    """Scatter every CSR nonzero into padded ELL slabs.  FA:226-385.

    Returns (rows, cols, mask): lists over partitions of lists over buckets of
    numpy arrays with shapes (R,), (R, W), (R, W).  Integer dtype is int64.
    """
    num_parts = len(bucket_widths)
    num_rows = g.num_src_nodes()
    psize = partition_size(g.num_dst_nodes(), num_parts)

    coo_r, coo_c = _coo_arrays(g)
    degree = [dict() for _ in range(num_parts)]                 # FA:249-252, COO counts
    for r, c in zip(coo_r.tolist(), coo_c.tolist()):
        d = degree[c // psize]
        d[r] = d.get(r, 0) + 1

    indptr, indices, _ = g.adj_tensors("csr")                  # FA:254
    indptr = np.asarray(indptr).tolist()
    indices = np.asarray(indices).tolist()

    ell_rows = [[[] for _ in ws] for ws in bucket_widths]
    ell_cols = [[[] for _ in ws] for ws in bucket_widths]
    ell_mask = [[[] for _ in ws] for ws in bucket_widths]

    for r in range(num_rows):
        for k in range(indptr[r], indptr[r + 1]):
            c = indices[k]
            p = c // psize
            ws = bucket_widths[p]
            b = bisect.bisect_left(ws, degree[p][r])              # FA:275
            if b == len(ws):
                b -= 1                                           # FA:276-278
            w = ws[b]
            cl, ml, rl = ell_cols[p][b], ell_mask[p][b], ell_rows[p][b]
            rem = len(cl) & (w - 1)                              # FA:286
            open_row = rem == 0
            if not open_row:
                assert rl, f"row_indices[{p}][{b}] is empty"      # FA:292
                if rl[-1] != r:
                    open_row = True
                    cl.extend([0] * (w - rem))                   # FA:297-299
                    ml.extend([0] * (w - rem))
            if open_row:
                assert len(cl) & (w - 1) == 0, "invalid padding"  # FA:303
                rl.append(r)
            cl.append(c)
            ml.append(1)

    rows_nd, cols_nd, mask_nd = [], [], []
    for p, ws in enumerate(bucket_widths):
        rp, cp, mp = [], [], []
        for b, w in enumerate(ws):
            cl, ml, rl = ell_cols[p][b], ell_mask[p][b], ell_rows[p][b]
            rem = len(cl) & (w - 1)
            if rem:                                              # FA:344-350
                cl.extend([0] * (w - rem))
                ml.extend([0] * (w - rem))
            n = len(rl)
            assert len(cl) == n * w and len(ml) == n * w        # FA:357-358
            rp.append(np.asarray(rl, dtype=np.int64).reshape(n))
            cp.append(np.asarray(cl, dtype=np.int64).reshape(n, w))
            mp.append(np.asarray(ml, dtype=np.int64).reshape(n, w))
        rows_nd.append(rp)
        cols_nd.append(cp)
        mask_nd.append(mp)
    return rows_nd, cols_nd, mask_nd


# --------------------------------------------------------------------------- closed forms
def _segments(g, num_parts: int):
    """Per (row, partition) segment table from canonical CSR and raw COO.

    Returns dict with, for every segment that holds at least one CSR entry, in
    row-major / partition-ascending order: row, part, start (offset into CSR
    arrays), fill (CSR count) and deg (COO count, FA:250-252)."""
    num_rows = g.num_src_nodes()
    psize = partition_size(g.num_dst_nodes(), num_parts)
    indptr, indices, data = g.adj_tensors("csr")
    indptr = np.asarray(indptr, dtype=np.int64)
    indices = np.asarray(indices, dtype=np.int64)
    row_of = np.repeat(np.arange(num_rows, dtype=np.int64), np.diff(indptr))
    key = row_of * num_parts + indices // psize
    # CSR is row-major with ascending columns, hence `key` is non-decreasing
    uniq, start, fill = np.unique(key, return_index=True, return_counts=True)
    coo_r, coo_c = _coo_arrays(g)
    coo_key = coo_r.astype(np.int64) * num_parts + coo_c.astype(np.int64) // psize
    ck, cc = np.unique(coo_key, return_counts=True)
    deg = cc[np.searchsorted(ck, uniq)]
    return {"row": uniq // num_parts, "part": uniq % num_parts, "start": start,
            "fill": fill, "deg": deg, "indices": indices, "data": np.asarray(data)}


def build_hyb_format_closed_form(g, bucket_widths: List[List[int]], with_values: bool = False):
    """Same result as build_hyb_format_sequential, computed without walking nonzeros
    one at a time.  Justification (from FA:268-311): CSR is traversed row-major with
    ascending columns, so the nonzeros of one (row, partition) segment are contiguous;
    each bucket therefore receives whole segments in ascending row order, a segment of
    `fill` entries occupies ceil(fill / W) consecutive ELL rows carrying the same row
    id, and padding (col 0, mask 0) only ever follows the last entry of a segment."""
    num_parts = len(bucket_widths)
    seg = _segments(g, num_parts)
    rows_nd, cols_nd, mask_nd, vals_nd = [], [], [], []
    for p, ws in enumerate(bucket_widths):
        sel = np.nonzero(seg["part"] == p)[0]
        if len(sel) and not ws:
            raise IndexError("list index out of range")  # FA:279 on an empty width list
        warr = np.asarray(ws, dtype=np.int64)
        b = np.searchsorted(warr, seg["deg"][sel], side="left") if len(ws) else np.zeros(0, int)
        b = np.minimum(b, len(ws) - 1)
        rp, cp, mp, vp = [], [], [], []
        for bi, w in enumerate(ws):
            s = sel[b == bi]
            fill = seg["fill"][s]
            n_ell = -(-fill // w)
            first = np.concatenate(([0], np.cumsum(n_ell)))[:-1]
            R = int(n_ell.sum())
            rows = np.repeat(seg["row"][s], n_ell).astype(np.int64)
            cols = np.zeros(R * w, dtype=np.int64)
            mask = np.zeros(R * w, dtype=np.int64)
            vals = np.zeros(R * w, dtype=np.float64)
            # slot of k-th entry of a segment: first*w + k
            tot = int(fill.sum())
            if tot:
                seg_id = np.repeat(np.arange(len(s)), fill)
                k = np.arange(tot) - np.repeat(np.concatenate(([0], np.cumsum(fill)))[:-1], fill)
                dst = first[seg_id] * w + k
                src = seg["start"][s][seg_id] + k
                cols[dst] = seg["indices"][src]
                mask[dst] = 1
                vals[dst] = seg["data"][src]
            rp.append(rows)
            cp.append(cols.reshape(R, w))
            mp.append(mask.reshape(R, w))
            vp.append(vals.reshape(R, w))
        rows_nd.append(rp)
        cols_nd.append(cp)
        mask_nd.append(mp)
        vals_nd.append(vp)
    if with_values:
        return rows_nd, cols_nd, mask_nd, vals_nd
    return rows_nd, cols_nd, mask_nd


def init_bucket_stats_closed_form(g, num_parts: int, width_limit: int = WIDTH_LIMIT):
    """The five numbers per initial bucket that the cost model reads (width, cost-model
    rows, nnz, distinct rows, distinct columns), computed with numpy.  Same content as
    get_init_buckets_sequential(...)[p][w].key()."""
    psize = partition_size(g.num_dst_nodes(), num_parts)
    coo_r, coo_c = _coo_arrays(g)
    coo_r = coo_r.astype(np.int64)
    coo_c = coo_c.astype(np.int64)
    part = coo_c // psize
    key = coo_r * num_parts + part
    uk, inv, deg = np.unique(key, return_inverse=True, return_counts=True)
    p_of = uk % num_parts
    pw = np.ones_like(deg)
    nz = deg > 1
    pw[nz] = 1 << np.ceil(np.log2(deg[nz])).astype(np.int64)
    # guard the float log2 against off-by-one at exact powers of two
    too_small = pw < deg
    pw[too_small] *= 2
    half_ok = (pw // 2 >= deg) & (pw > 1)
    pw[half_ok] //= 2
    mrows = np.maximum(1, pw // width_limit)
    width = np.minimum(pw, width_limit)
    out = []
    for p in range(num_parts):
        d = {}
        m = p_of == p
        for w in np.unique(width[m]).tolist():
            s = m & (width == w)
            in_bucket = s[inv]
            d[w] = (w, int(mrows[s].sum()), int(deg[s].sum()), int(s.sum()),
                    int(len(np.unique(coo_c[in_bucket]))))
        out.append(d)
    return out


# --------------------------------------------------------------------------- SpMM
def spmm_reference_f64(g, B: np.ndarray) -> np.ndarray:
    """The reference's golden product: scipy CSC . dense (FM:89-99), in float64."""
    return g.coo_mtx.tocsc().astype(np.float64).dot(np.asarray(B, dtype=np.float64))


def spmm_csr_f64(indptr, indices, data, shape, B) -> np.ndarray:
    """scipy CSR(f64) @ dense(f64): the numeric anchor for the HIP kernel."""
    A = sp.csr_matrix((np.asarray(data, dtype=np.float64), indices, indptr), shape=shape)
    return A @ np.asarray(B, dtype=np.float64)


def spmm_abs_bound(indptr, indices, data, shape, B) -> np.ndarray:
    """Per-element magnitude sum_k |a_ik| |b_kj| that scales the 1e-5 tolerance."""
    A = sp.csr_matrix((np.abs(np.asarray(data, dtype=np.float64)), indices, indptr), shape=shape)
    return A @ np.abs(np.asarray(B, dtype=np.float64))


def spmm_from_hyb(rows_nd, cols_nd, vals_nd, num_rows: int, B: np.ndarray) -> np.ndarray:
    """What the fused kernel computes, stated on the slabs (FA:99-102 applied per
    (partition, bucket) ELL block, accumulated into C by row id as FA:508-515 does):
    C[rows[e], :] += sum_j vals[e, j] * B[cols[e, j], :]  in float64."""
    B = np.asarray(B, dtype=np.float64)
    C = np.zeros((num_rows, B.shape[1]), dtype=np.float64)
    for rp, cp, vp in zip(rows_nd, cols_nd, vals_nd):
        for rows, cols, vals in zip(rp, cp, vp):
            if len(rows) == 0:
                continue
            contrib = np.einsum("ew,ewn->en", np.asarray(vals, dtype=np.float64), B[cols])
            np.add.at(C, rows, contrib)
    return C


def spmm_bsr_f64(bsr_mat, X: np.ndarray) -> np.ndarray:
    """Block-sparse product in float64: what bench_bsrmm's kernel computes
    (format_algos.py:1182-1216: C[i, bi, f] = sum_j sum_bj A[i, j, bi, bj] * B[j, bj, f]),
    through scipy's BSR @ dense with both operands widened first."""
    return bsr_mat.astype(np.float64) @ np.asarray(X, dtype=np.float64)


def spmm_bsr_abs_bound(bsr_mat, X: np.ndarray) -> np.ndarray:
    """sum |a| |x| per output element, the scale of the accumulation error."""
    return abs(bsr_mat.astype(np.float64)) @ np.abs(np.asarray(X, dtype=np.float64))
