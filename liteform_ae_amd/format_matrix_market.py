"""Matrix container for the CELL/hyb SpMM path.

Mirrors the interface of the reference's ``format_matrix_market`` module
(playground_pipline/format_matrix_market.py:12-205): ``Bucket`` is the cost-model
record, ``MTX`` wraps a ``scipy.sparse.coo_matrix`` and hands out CSR/CSC/COO views.
Anything that accepted a reference ``MTX`` accepts this one (same attribute and
method names, same return types).

Differences, all additive:
  * ``MTX.from_coo`` / ``MTX.from_csr`` build a matrix from arrays without a file and
    may keep real values (the reference forces every stored value to 1.0,
    format_matrix_market.py:54, 63-64);
  * the graph-dataset names of the reference need the ``dgl``/``ogb`` packages and a
    network connection; they raise ``RuntimeError`` here.
"""
from __future__ import annotations

from os.path import basename, splitext

import numpy as np
from scipy import sparse as sp

__all__ = ["MTX", "Bucket"]

_GRAPH_DATASETS = ("cora", "citeseer", "pubmed", "ppi", "arxiv", "proteins", "reddit")


class Bucket:
    """One (partition, width) bucket as the cost model sees it
    (format_matrix_market.py:12-37)."""

    def __init__(self, bucket_width: int, num_rows: int, nnz: int,
                 row_indices: list, col_indices: set):
        self.bucket_width = bucket_width
        self.num_rows = num_rows
        self.nnz = nnz
        self.row_indices = row_indices
        self.col_indices = col_indices

    def __str__(self):
        head = (f"Bucket(bucket_width={self.bucket_width}, num_rows={self.num_rows}, "
                f"nnz={self.nnz}, len(row_indices)={len(self.row_indices)}, ")
        if len(self.row_indices) < 11 and len(self.col_indices) < 11:
            return (head + f"row_indices={self.row_indices}, "
                    f"len(col_indices)={len(self.col_indices)}, col_indices={self.col_indices})")
        return head + f"len(col_indices)={len(self.col_indices)})"


class MTX:
    """Sparse matrix held as scipy COO (format_matrix_market.py:40-205).

    ``MTX(None)`` gives an empty shell whose ``coo_mtx`` the caller assigns;
    ``MTX(path)`` reads a MatrixMarket file and sets every stored value to 1.
    """

    def __init__(self, filename):
        self._coo = None
        self._csr = None
        self._csr_source = None       # the CSR matrix this container was made from (from_csr), as given
        self._unit_values = False     # from_csr without data: every stored value is 1
        if filename is None:
            self.name = None
        elif filename in _GRAPH_DATASETS:
            raise RuntimeError(
                f"dataset '{filename}' is downloaded through dgl/ogb in the reference; "
                "those loaders are not part of this library - build the matrix with "
                "MTX.from_coo / MTX.from_csr or pass a MatrixMarket path")
        else:
            from scipy.io import mmread
            self.name = splitext(basename(filename))[0]
            coo = sp.coo_matrix(mmread(filename))
            coo.data = np.ones(len(coo.data))          # format_matrix_market.py:63-64
            self.coo_mtx = coo

    # ``coo_mtx`` is the reference's one data attribute (format_matrix_market.py:44-46).  A
    # container made from CSR arrays keeps them and builds the COO view only when it is asked
    # for, so that a CSR input can go to the GPU as it is.
    @property
    def coo_mtx(self):
        if self._coo is None and self._csr_source is not None:
            self._coo = self._csr_source.tocoo()
        return self._coo

    @coo_mtx.setter
    def coo_mtx(self, value):
        self._coo = value
        self._csr = None                               # cached views follow the COO
        self._csr_source = None
        self._unit_values = False

    # ---- constructors without a file -------------------------------------------------
    @classmethod
    def from_coo(cls, row, col, shape, data=None, name=None):
        m = cls(None)
        m.name = name
        row = np.asarray(row)
        col = np.asarray(col)
        if data is None:
            data = np.ones(len(row))
        m.coo_mtx = sp.coo_matrix((np.asarray(data), (row, col)), shape=shape)
        return m

    @classmethod
    def from_csr(cls, indptr, indices, shape, data=None, name=None):
        """Container around CSR arrays, kept as they are (no copy for int32 / float32 input).
        ``data=None`` stores ones, like every matrix of the reference."""
        indptr = np.asarray(indptr)
        indices = np.asarray(indices)
        unit = data is None
        if unit:
            data = np.ones(len(indices), dtype=np.float32)
        m = cls(None)
        m.name = name
        m._csr_source = sp.csr_matrix((np.asarray(data), indices, indptr), shape=shape)
        m._unit_values = unit
        return m

    # ---- the reference's accessors ----------------------------------------------------
    def _csr_view(self):
        """Canonical CSR (sorted columns, duplicates summed): what coo.tocsr() gives
        (format_matrix_market.py:74-76)."""
        if self._csr is None:
            src = self._csr_source
            if src is not None and src.has_canonical_format:
                self._csr = src
            else:
                self._csr = self.coo_mtx.tocsr()
        return self._csr

    def _shape(self):
        return (self._csr_source if self._coo is None and self._csr_source is not None else self.coo_mtx).shape

    def adj_tensors(self, format: str):
        if format == "coo":
            return self.coo_mtx.row, self.coo_mtx.col
        elif format == "csc":
            csc = self.coo_mtx.tocsc()
            return csc.indptr, csc.indices, csc.data
        elif format == "csr":
            csr = self._csr_view()
            return csr.indptr, csr.indices, csr.data
        raise TypeError(f"Format {format} is not suppoted.")

    def num_src_nodes(self):
        return self._shape()[0]

    def num_dst_nodes(self):
        return self._shape()[1]

    def num_edges(self):
        # stored entries: the COO view of a CSR matrix holds exactly its stored entries
        if self._coo is None and self._csr_source is not None:
            return self._csr_source.nnz
        return self.coo_mtx.nnz

    def dot(self, B):
        """A @ B through scipy (format_matrix_market.py:89-99)."""
        return self.coo_mtx.tocsc().dot(B)

    def tobsr(self, blocksize=None, copy=False):
        """scipy BSR view (format_matrix_market.py:101-112)."""
        return self.coo_mtx.tobsr(blocksize=blocksize, copy=copy)

    def tobsr_with_padding(self, shape, blocksize=None):
        """BSR matrix of the given (padded) shape with fp16-valued entries, shape % blocksize == 0
        (format_matrix_market.py:115-136).  The reference stores the values as float16; scipy
        1.15 no longer accepts that dtype in sparse containers, so the values are rounded to
        fp16 and held as float32 (every value is exactly representable in fp16)."""
        data = np.array(self.coo_mtx.data, dtype=np.float16).astype(np.float32)
        ij = [self.coo_mtx.row, self.coo_mtx.col]
        return sp.bsr_matrix((data, ij), blocksize=blocksize, shape=shape)

    def tocsr(self, copy=False):
        return self.coo_mtx.tocsr(copy=copy)

    def matrix_features(self):
        """Row-length statistics used by the format selector
        (format_matrix_market.py:153-202)."""
        num_rows, num_cols = self._shape()
        indptr = self._csr_view().indptr
        per_row = np.diff(indptr)
        avg = np.mean(per_row)
        lo = per_row.min()
        hi = per_row.max()
        return {
            "name": self.name,
            "num_rows": num_rows,
            "num_cols": num_cols,
            "nnz": self.num_edges(),
            "avg_nnz_per_row": avg,
            "min_nnz_per_row": lo,
            "max_nnz_per_row": hi,
            "std_dev_nnz_per_row": np.std(per_row),
            "avg_nnz_density_per_row": avg / num_cols,
            "min_nnz_density_per_row": lo / num_cols,
            "max_nnz_density_per_row": hi / num_cols,
            "std_dev_nnz_density_per_row": np.std(per_row / num_cols),
        }

    def __str__(self):
        return str(self.coo_mtx)
