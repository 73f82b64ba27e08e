"""Sorting / segmentation helpers for the constant tables (API of ``equitorch/utils/_indices.py``).

Implemented on numpy arrays: a lexicographic column sort is ``numpy.lexsort`` (stable, so equal keys keep
their input order like Python's ``sorted``), run-length segmentation is a boundary mask + ``flatnonzero``,
and ranking against the sorted unique tuples is ``numpy.unique(axis=0, return_inverse=True)``.
"""
from typing import Any, List, Sequence, Tuple

import numpy as np


def _lex_order(key_cols: Sequence[Sequence[Any]]) -> np.ndarray:
    # numpy.lexsort sorts by the LAST key first, so feed the columns reversed
    return np.lexsort([np.asarray(c) for c in reversed(key_cols)])


def sort_by_column_key(to_sort: List[List[Any]], key: List[List[Any]] = None) -> List[List[Any]]:
    """Reorder the columns of ``to_sort`` by the lexicographic order of the columns of ``key``
    (reference ``_indices.py:89-138``)."""
    if key is None:
        key = to_sort
    if not to_sort or not key or len(to_sort[0]) != len(key[0]):
        raise ValueError("to_sort and key must be non-empty and of equal length")
    order = _lex_order(key)
    return [[row[i] for i in order] for row in to_sort]


def extract_batch_segments(keys: List[List[int]]):
    """Run-length segmentation of sorted key columns -> ``(batch, seg, values)`` (reference ``:12-87``)."""
    if not keys or not keys[0]:
        return [], [], []
    cols = np.stack([np.asarray(k) for k in keys])
    n = cols.shape[1]
    change = np.ones(n, dtype=bool)
    change[1:] = (cols[:, 1:] != cols[:, :-1]).any(axis=0)
    starts = np.flatnonzero(change)
    batch = np.cumsum(change) - 1
    seg = starts.tolist() + [n]
    vals = [[k[s] for s in starts] for k in keys]
    return batch.tolist(), seg, vals


def extract_scatter_indices(keys: List[List[int]]) -> Tuple[List[int], List[List[int]]]:
    """Index of every key tuple in the sorted list of distinct tuples (reference ``:140-204``)."""
    if not keys or not keys[0]:
        return [], []
    rows = np.stack([np.asarray(k, dtype=np.int64) for k in keys], axis=1)
    uniq, inverse = np.unique(rows, axis=0, return_inverse=True)
    return inverse.reshape(-1).tolist(), [uniq[:, c].tolist() for c in range(uniq.shape[1])]


def expand_left(source, target, dim: int):
    if dim < 0:
        dim = source.ndim + dim
    return target.view([1] * dim + [-1])
