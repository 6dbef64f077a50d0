"""Dense-CRF mean-field message passing on the lattice filter, the use the reference names for
its op (README.md:16 of the reference tree; the reference itself holds no CRF code, so this loop
is this library's own harness around the op's two filters).

Per iteration ``Q <- softmax(logits + bilateral(Q; theta_alpha, theta_beta) + spatial(Q;
theta_gamma))``, where both filters are the ``LatticeFilter`` op's (features and normalisation
as in src/LatticeFilterKernel.cpp:126-142).  The features never change between iterations, so
each batch item builds its two lattices once (``pl_build_image``) and every message is one
``pl_apply``; the reference's op would rebuild them for each of its calls
(src/LatticeFilterKernel.cpp:152-179).  The gradient pass is the reference's rule
(lattice_filter_op_loader.py:32-54): the same two filters with ``reverse=True`` on the upstream
gradient.

torch carries the tensors and does the softmax; the filters are the HIP library's.
"""
import torch

from . import PermutohedralLattice


class MeanField:
    """Lattices of one batch of guide images ``[B, H, W, C_ref]`` for ``n_classes`` labels."""

    def __init__(self, guide, n_classes, theta_alpha=80.0, theta_beta=13.0, theta_gamma=3.0):
        if guide.dim() < 3:
            raise ValueError("guide must be [batch, spatial..., channels]")
        self.batch = int(guide.shape[0])
        self.sdims = [int(s) for s in guide.shape[1:-1]]
        self.n = 1
        for s in self.sdims:
            self.n *= s
        self.n_classes = int(n_classes)
        self.thetas = (float(theta_alpha), float(theta_beta), float(theta_gamma))
        rc, k = int(guide.shape[-1]), len(self.sdims)
        self.bilateral = [PermutohedralLattice(k + rc, self.n_classes + 1, self.n)
                          for _ in range(self.batch)]
        self.spatial = [PermutohedralLattice(k, self.n_classes + 1, self.n)
                        for _ in range(self.batch)]
        shape = (self.batch, self.n, self.n_classes)
        self._msg_bi = torch.empty(shape, dtype=torch.float32, device=guide.device)
        self._msg_sp = torch.empty(shape, dtype=torch.float32, device=guide.device)
        self.rebuild(guide)

    def rebuild(self, guide):
        """Build the lattices again for another batch of guide images of the same shape."""
        self.guide = guide.contiguous()
        rc = int(guide.shape[-1])
        theta_alpha, theta_beta, theta_gamma = self.thetas
        for b in range(self.batch):
            self.bilateral[b].build_image(self.guide[b].reshape(self.n, rc), self.sdims,
                                          theta_alpha, theta_beta)
            self.spatial[b].build_image(None, self.sdims, theta_gamma)

    def messages(self, q, reverse=False):
        """bilateral(q) + spatial(q) for ``q [B, ..., n_classes]`` (any spatial shape of N points)."""
        q = q.contiguous().view(self.batch, self.n, self.n_classes)
        for b in range(self.batch):
            self.bilateral[b].apply(self._msg_bi[b], q[b], reverse)
            self.spatial[b].apply(self._msg_sp[b], q[b], reverse)
        return self._msg_bi + self._msg_sp

    def infer(self, logits, iterations=5):
        """-> Q after ``iterations`` mean-field updates, shaped like ``logits``."""
        flat = logits.contiguous().view(self.batch, self.n, self.n_classes)
        q = torch.softmax(flat, dim=-1)
        for _ in range(iterations):
            q = torch.softmax(flat + self.messages(q), dim=-1)
        return q.view(logits.shape)

    def reverse(self, upstream):
        """The op's registered gradient of one message-passing step with respect to its input:
        both filters with ``reverse=True`` on ``upstream``, summed."""
        return self.messages(upstream, reverse=True).view(upstream.shape).clone()

    def close(self):
        for lat in self.bilateral + self.spatial:
            lat.close()
        self.bilateral, self.spatial = [], []
