"""The dense-CRF mean-field workload (five iterations of softmax(logits + bilateral(Q) +
spatial(Q)), batch 2, reverse pass on the last iteration) on lattices built once per item,
against the same loop over the CPU oracle with a fresh lattice per message."""
import numpy as np
import pytest
import torch

from conftest import MAX_ABS_TOL, REL_L2_TOL, rel_l2
from permutohedral_lattice_amd import synth
from permutohedral_lattice_amd.crf import MeanField

import oracle

pytestmark = pytest.mark.gpu


def _inputs(batch, h, w, classes, seed):
    guide = np.stack([synth.blob_image(h, w, seed=seed + b) * 255.0 for b in range(batch)])
    logits = synth.normal_image((batch, h, w, classes), seed + 10)
    upstream = synth.normal_image((batch, h, w, classes), seed + 11)
    return guide.astype(np.float32), logits, upstream


@pytest.mark.parametrize("h,w", [(128, 128), (72, 100)])
def test_mean_field_loop_matches_the_oracle(h, w):
    batch, classes = 2, 21
    guide, logits, upstream = _inputs(batch, h, w, classes, 300 + h)
    mf = MeanField(torch.from_numpy(guide).cuda(), classes)
    q = mf.infer(torch.from_numpy(logits).cuda(), iterations=5)
    rev = mf.reverse(torch.from_numpy(upstream).cuda())
    torch.cuda.synchronize()
    q, rev = q.cpu().numpy(), rev.cpu().numpy()
    want_q, want_rev = oracle.mean_field(logits, guide, 5, upstream=upstream)
    # Q is a distribution over the classes: data in [0, 1]
    assert np.isfinite(q).all() and np.abs(q.sum(axis=-1) - 1.0).max() <= 1e-5
    assert np.abs(q - want_q).max() <= MAX_ABS_TOL and rel_l2(q, want_q) <= REL_L2_TOL
    # the reverse pass filters N(0,1) values: tolerance scaled by their range
    scale = float(np.abs(want_rev).max())
    assert np.abs(rev - want_rev).max() <= MAX_ABS_TOL * max(1.0, scale)
    assert rel_l2(rev, want_rev) <= REL_L2_TOL
    mf.close()


def test_mean_field_messages_equal_the_op_called_per_iteration():
    """Lattices built once and applied equal the op called afresh for every message."""
    import permutohedral_lattice_amd as pla
    batch, h, w, classes = 2, 64, 80, 5
    guide, logits, _ = _inputs(batch, h, w, classes, 400)
    d_guide = torch.from_numpy(guide).cuda()
    q = torch.softmax(torch.from_numpy(logits).cuda(), dim=-1)
    mf = MeanField(d_guide, classes)
    got = mf.messages(q).view(batch, h, w, classes)
    want = (pla.lattice_filter(q, d_guide, True, 80.0, 13.0, 3.0)
            + pla.lattice_filter(q, d_guide, False, 80.0, 13.0, 3.0))
    torch.cuda.synchronize()
    assert float((got - want).abs().max()) <= 1e-5
    mf.close()
