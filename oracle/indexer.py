"""TEST INFRASTRUCTURE ONLY: a CPU restatement (numpy, float64) of crit's sparse index selection, the checker of the
gfx950 kernels behind crit_amd.sparse_indexer. Nothing the product ships imports this file.

Follows the reference's definition of the operation (inference/attention-state/code/sparse_index.py:13-40):

    score[t, s] = sum_h weights[t, h] * scale * max(0, q[t, h] . keys[s])     for s < ends[t], -inf at or past it
    picked[t]   = the positions of the k largest score[t, s] below ends[t], ascending (all of them where ends[t] <= k),
                  then -1; ties to the lower position, a NaN below every number (-inf included), -0 = +0

Pinned (tests/test_oracle.py): sparse_scores by a loop over tokens, heads and keys in Python floats on small cases, by
the closed form of one-hot queries, by ReLU's sign and by linearity in the weights; sparse_index by a selection that
takes the best remaining score k times (no sort), by the reference's own known answers for NaN and -inf
(kernels/techniques/attention/sparse-indexer/tests/test_sparse_indexer.py:97-103) and by the rule's invariants (every
picked score at or above every unpicked one, ascending positions, everything picked where ends[t] <= k).
"""
import numpy as np


def sparse_scores(q, keys, weights, ends, scale):
    """q [T][H][D], keys [N][D], weights [T][H], ends [T] -> score [T][N] float64 (sparse_index.py:13-20)."""
    q, keys, weights = np.asarray(q, np.float64), np.asarray(keys, np.float64), np.asarray(weights, np.float64)
    products = np.maximum(np.einsum("thd,nd->thn", q, keys), 0.0)
    out = (products * (weights * float(scale))[:, :, None]).sum(1)
    at = np.arange(keys.shape[0])
    out[at[None, :] >= np.asarray(ends, np.int64)[:, None]] = -np.inf
    return out


def sparse_index(score, ends, k):
    """score [T][N] -> int64 [T][k] (sparse_index.py:23-40): the larger score first, then the lower position, every
    NaN after every number; the k first of that order, ascending, then -1."""
    score = np.asarray(score, np.float64)
    t, n = score.shape
    picked = np.full((t, k), -1, np.int64)
    for i in range(t):
        end = max(0, min(int(ends[i]), n))
        row = score[i, :end]
        if end <= k:
            chosen = np.arange(end)
        else:
            nan = np.isnan(row)
            value = np.where(nan, -np.inf, row) + 0.0      # (-0 + 0 = +0: the two zeros tie)
            order = np.lexsort((np.arange(end), -value, nan))      # NaN last; larger first; lower position first
            chosen = np.sort(order[:k])
        picked[i, :len(chosen)] = chosen
    return picked
