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

The 2 x batch lattices of a step are independent of each other, and at image sizes like 512 x 512
one apply is a chain of short kernels that leaves most of the GPU idle, so every lattice works on a
HIP stream of its own (default priority): a message-passing step waits for its input on the
caller's stream, runs the applies of all lattices side by side, and the caller's stream waits for
all of them before it adds the messages up.

torch carries the tensors and does the softmax; the filters are the HIP library's.
"""
import torch

from . import PermutohedralLattice


class MeanField:
    """Lattices of one batch of guide images ``[B, H, W, C_ref]`` for ``n_classes`` labels."""

    def __init__(self, guide, n_classes, theta_alpha=80.0, theta_beta=13.0, theta_gamma=3.0,
                 concurrent=True):
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
        self.concurrent = bool(concurrent)
        self._streams = [torch.cuda.Stream(device=guide.device) if self.concurrent else None
                         for _ in range(2 * self.batch)]
        self.bilateral = [PermutohedralLattice(k + rc, self.n_classes + 1, self.n,
                                               stream=self._streams[2 * b])
                          for b in range(self.batch)]
        self.spatial = [PermutohedralLattice(k, self.n_classes + 1, self.n,
                                             stream=self._streams[2 * b + 1])
                        for b in range(self.batch)]
        shape = (self.batch, self.n, self.n_classes)
        self._msg_bi = torch.empty(shape, dtype=torch.float32, device=guide.device)
        self._msg_sp = torch.empty(shape, dtype=torch.float32, device=guide.device)
        self.rebuild(guide)

    def rebuild(self, guide):
        """Build the lattices again for another batch of guide images of the same shape."""
        self.guide = guide.contiguous()
        rc = int(guide.shape[-1])
        theta_alpha, theta_beta, theta_gamma = self.thetas
        self._side_streams_wait_for_caller()
        # all builds are enqueued, each on its lattice's stream, before the first is waited for: a
        # build is a chain of a dozen short kernels, and 2 x batch of them run side by side
        for b in range(self.batch):
            self.bilateral[b].build_image_begin(self.guide[b].reshape(self.n, rc), self.sdims,
                                                theta_alpha, theta_beta)
            self.spatial[b].build_image_begin(None, self.sdims, theta_gamma)
        for lat in self.bilateral + self.spatial:
            lat.build_end()
        # (a build has ended when its lattice is complete: nothing to wait for here)

    def _side_streams_wait_for_caller(self):
        """What the caller's stream has been given so far is complete before any lattice's stream
        goes on (the guide, the tensor a message is computed from)."""
        if not self.concurrent:
            return
        ready = torch.cuda.Event()
        ready.record(torch.cuda.current_stream())
        for s in self._streams:
            s.wait_event(ready)

    def _caller_waits_for_side_streams(self):
        if not self.concurrent:
            return
        caller = torch.cuda.current_stream()
        for s in self._streams:
            done = torch.cuda.Event()
            done.record(s)
            caller.wait_event(done)

    def messages(self, q, reverse=False):
        """bilateral(q) + spatial(q) for ``q [B, ..., n_classes]`` (any spatial shape of N points)."""
        q = q.contiguous().view(self.batch, self.n, self.n_classes)
        self._side_streams_wait_for_caller()
        for b in range(self.batch):
            self.bilateral[b].apply(self._msg_bi[b], q[b], reverse)
            self.spatial[b].apply(self._msg_sp[b], q[b], reverse)
        self._caller_waits_for_side_streams()
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
