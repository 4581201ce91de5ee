"""Routing (router logits -> top-k experts -> rows sorted by expert + cumulative group_list),
restated in numpy.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  The reference has no routing code of its own: its
ops take the cumulative int64 group_list (grouped_gemm/op_kernel/grouped_matmul_utils.h:304-320;
the tests build it by hand, grouped_gemm/test/python/test_group_gemm_fp4.py:176) and rows already
sorted by expert.  What is restated here is therefore the definition itself: a stable sort of the
(token, choice) pairs by expert id.  Pinned in tests/test_oracle.py by brute force on small inputs
and by the invariants a sort must satisfy.
"""
from __future__ import annotations

import numpy as np


def route_topk(logits: np.ndarray, topk: int):
    """ids int32 [T, topk]: the experts with the largest logits, in decreasing order, ties to the
    lower id; weight fp32 [T, topk]: softmax(logits) at those experts (not renormalised)."""
    logits = np.asarray(logits, dtype=np.float32)
    T, E = logits.shape
    # stable argsort of -logits: equal logits keep ascending id order
    order = np.argsort(-logits, axis=1, kind="stable")[:, :topk].astype(np.int32)
    mx = logits.max(axis=1, keepdims=True)
    p = np.exp((logits - mx).astype(np.float32)).astype(np.float32)
    p = p / p.sum(axis=1, keepdims=True, dtype=np.float32)
    return order, np.take_along_axis(p, order.astype(np.int64), axis=1).astype(np.float32)


def route_sort(ids: np.ndarray, E: int):
    """ids int32 [T, topk] -> (group_list int64 [E] cumulative, row_token int32 [n_valid],
    row_of_choice int32 [T*topk]).  Rows sorted by expert id, then by flat choice index; ids outside
    [0, E) are dropped (row_of_choice -1)."""
    ids = np.asarray(ids, dtype=np.int64)
    T, topk = ids.shape
    flat = ids.reshape(-1)
    valid = (flat >= 0) & (flat < E)
    idx = np.nonzero(valid)[0]
    order = idx[np.argsort(flat[idx], kind="stable")]
    group_list = np.cumsum(np.bincount(flat[idx], minlength=E)[:E]).astype(np.int64)
    row_token = (order // topk).astype(np.int32)
    row_of_choice = np.full(T * topk, -1, dtype=np.int32)
    row_of_choice[order] = np.arange(order.size, dtype=np.int32)
    return group_list, row_token, row_of_choice
