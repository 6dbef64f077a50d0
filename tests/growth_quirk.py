"""Where the reference's outputs differ from those of a lattice with one vertex per distinct key.

The reference computes the start cell of a hash lookup before it checks whether its index must
double (src/PermutohedralLatticeCPU.h:163-165, then :62), so the one lookup that triggers a
doubling probes the doubled index from a stale cell.  That lookup can miss a key that is present
and enter it again as a second vertex (during the splat), enter a new key where later lookups do
not find it, or report a neighbour as absent (during the blur).  Whatever it does, it does it to
the key it was looking up: everything the reference then computes differently lies within one blur
step along each of the pd+1 axes of that key.  The helpers here name those vertices and the
points that touch them.
"""
import itertools

import numpy as np


def blur_neighbourhood(keys, pd):
    """The set (of key bytes) of all lattice keys within one blur step along every axis of the
    given [k, pd] keys: key + sum_a s_a * step_a, s_a in {-1, 0, 1}, where a blur step along axis
    a < pd adds (1, .., 1) - (pd+1) e_a to the stored coordinates and along axis pd adds
    (1, .., 1) (src/PermutohedralLatticeCPU.h:381-388)."""
    steps = []
    for a in range(pd + 1):
        d = np.ones(pd, np.int64)
        if a < pd:
            d[a] -= pd + 1
        steps.append(d)
    combos = np.array(list(itertools.product((-1, 0, 1), repeat=pd + 1)), np.int64) @ np.array(steps)
    out = set()
    for k in np.asarray(keys, np.int64).reshape(-1, pd):
        for row in (k + combos).astype(np.int16):
            out.add(row.tobytes())
    return out


def points_touching(point_keys, key_set):
    """point_keys [N, pd+1, pd] int16 -> bool [N]: the point has a simplex vertex in key_set."""
    n, d1, pd = point_keys.shape
    flat = np.ascontiguousarray(point_keys.reshape(-1, pd))
    hit = np.fromiter((flat[i].tobytes() in key_set for i in range(flat.shape[0])), bool,
                      flat.shape[0])
    return hit.reshape(n, d1).any(axis=1)


def duplicated_keys(vertex_keys):
    """Keys that the reference's first-touch list holds more than once, and how many entries of
    the list are second (third, ...) copies."""
    uniq, counts = np.unique(np.asarray(vertex_keys), axis=0, return_counts=True)
    return uniq[counts > 1], int((counts - 1).sum())
