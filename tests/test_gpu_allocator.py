"""Caller-supplied scratch memory (pl_alloc): the way the reference's DeviceMemoryAllocator takes
the lattice's buffers from TensorFlow temporaries (src/DeviceMemoryAllocator.h:52-71).  Here the
callbacks hand out torch tensors; every byte of scratch must come from them and go back to them,
and a callback that runs out of memory must surface as PL_ENOMEM, not as a crash."""
import ctypes as C

import numpy as np
import pytest
import torch

from conftest import MAX_ABS_TOL, REL_L2_TOL, rel_l2
from permutohedral_lattice_amd import synth

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu

ALLOC_FN = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_size_t)
FREE_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)


class PlAlloc(C.Structure):
    _fields_ = [("alloc", ALLOC_FN), ("free", FREE_FN), ("ctx", C.c_void_p)]


class TorchScratch:
    """Allocator callbacks over torch tensors, with a budget after which alloc returns NULL."""

    def __init__(self, fail_after=None):
        self.live, self.n_alloc, self.n_free, self.bytes = {}, 0, 0, 0
        self.fail_after = fail_after
        self._alloc = ALLOC_FN(self.alloc)
        self._free = FREE_FN(self.free)
        self.struct = PlAlloc(self._alloc, self._free, None)

    def alloc(self, _ctx, nbytes):
        if self.fail_after is not None and self.n_alloc >= self.fail_after:
            return None
        t = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device="cuda")
        self.live[t.data_ptr()] = t
        self.n_alloc += 1
        self.bytes += int(nbytes)
        return t.data_ptr()

    def free(self, _ctx, ptr):
        if ptr:
            assert ptr in self.live, "free of a pointer this allocator did not hand out"
            del self.live[ptr]
            self.n_free += 1


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _case():
    h, w = 72, 64
    img = synth.blob_image(h, w, seed=95)
    return h, w, img, synth.bilateral_positions(img, 8.0, 0.125)


def test_lattice_takes_all_its_scratch_from_the_callbacks_and_returns_it():
    h, w, img, pos = _case()
    n = h * w
    scratch = TorchScratch()
    handle = C.c_void_p()
    assert pla._lib.pl_create(5, 4, n, None, C.byref(scratch.struct), C.byref(handle)) == pla.PL_OK
    out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
    d_val, d_pos = dev(img.reshape(-1, 3)), dev(pos)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    for reverse in (0, 1):
        assert pla._lib.pl_filter(handle, out.data_ptr(), d_val.data_ptr(), d_pos.data_ptr(),
                                  reverse) == pla.PL_OK
        torch.cuda.synchronize()
        want = oracle.Lattice(5, 4, n).filter(img.reshape(-1, 3), pos, bool(reverse))
        got = out.cpu().numpy()
        assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    assert scratch.n_alloc > 5 and scratch.bytes > 8 * 6 * n      # replay rows alone are 48 B per point
    assert torch.cuda.memory_allocated() >= before                 # it lives in torch's tensors
    assert pla._lib.pl_destroy(handle) == pla.PL_OK
    assert scratch.n_free == scratch.n_alloc and not scratch.live


@pytest.mark.parametrize("fail_after", [0, 1, 3, 6, 9, 12])
def test_allocation_failure_is_reported_and_leaks_nothing(fail_after):
    h, w, img, pos = _case()
    n = h * w
    scratch = TorchScratch(fail_after=fail_after)
    handle = C.c_void_p()
    rc = pla._lib.pl_create(5, 4, n, None, C.byref(scratch.struct), C.byref(handle))
    if rc == pla.PL_OK:
        out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
        d_val, d_pos = dev(img.reshape(-1, 3)), dev(pos)
        rc = pla._lib.pl_filter(handle, out.data_ptr(), d_val.data_ptr(), d_pos.data_ptr(), 0)
        if rc != pla.PL_OK:
            assert rc == pla.PL_ENOMEM
            # with memory again the same handle works
            scratch.fail_after = None
            assert pla._lib.pl_filter(handle, out.data_ptr(), d_val.data_ptr(), d_pos.data_ptr(),
                                      0) == pla.PL_OK
            torch.cuda.synchronize()
            want = oracle.Lattice(5, 4, n).filter(img.reshape(-1, 3), pos, False)
            assert np.abs(out.cpu().numpy() - want).max() <= MAX_ABS_TOL
        assert pla._lib.pl_destroy(handle) == pla.PL_OK
    else:
        assert rc == pla.PL_ENOMEM and not handle.value
    assert not scratch.live and scratch.n_free == scratch.n_alloc


def test_op_with_caller_scratch_returns_everything_before_it_returns():
    b, h, w = 2, 48, 56
    guide = np.stack([synth.blob_image(h, w, seed=96 + i) for i in range(b)])
    inp = synth.uniform_image((b, h, w, 2), 98)
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, False)
    scratch = TorchScratch()
    d_in, d_ref = dev(inp), dev(guide)
    out = torch.empty_like(d_in)
    dims = (C.c_int * 2)(h, w)
    rc = pla._lib.pl_lattice_filter_op(d_in.data_ptr(), d_ref.data_ptr(), out.data_ptr(), b, 2, dims,
                                       2, 3, 1, 8.0, 0.125, 1.0, 0, None, C.byref(scratch.struct))
    assert rc == pla.PL_OK
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    assert scratch.n_alloc > 0 and not scratch.live and scratch.n_free == scratch.n_alloc


def test_double_op_with_caller_scratch_returns_everything_before_it_returns():
    b, h, w = 2, 40, 44
    guide = np.stack([synth.blob_image(h, w, seed=99 + i) for i in range(b)]).astype(np.float64)
    inp = synth.uniform_image((b, h, w, 2), 101).astype(np.float64)
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, False)
    scratch = TorchScratch()
    d_in, d_ref = dev(inp), dev(guide)
    out = torch.empty_like(d_in)
    dims = (C.c_int * 2)(h, w)
    rc = pla._lib.pl_lattice_filter_op_f64(d_in.data_ptr(), d_ref.data_ptr(), out.data_ptr(), b, 2,
                                           dims, 2, 3, 1, 8.0, 0.125, 1.0, 0, None,
                                           C.byref(scratch.struct))
    assert rc == pla.PL_OK
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - want).max() <= 1e-12
    assert scratch.n_alloc > 0 and not scratch.live and scratch.n_free == scratch.n_alloc
    # and a failing allocator is reported, with nothing kept
    for fail_after in (0, 2, 7, 11):
        short = TorchScratch(fail_after=fail_after)
        rc = pla._lib.pl_lattice_filter_op_f64(d_in.data_ptr(), d_ref.data_ptr(), out.data_ptr(), b,
                                               2, dims, 2, 3, 1, 8.0, 0.125, 1.0, 0, None,
                                               C.byref(short.struct))
        assert rc in (pla.PL_ENOMEM, pla.PL_OK)
        assert not short.live and short.n_free == short.n_alloc
    assert rc == pla.PL_ENOMEM      # eleven allocations are not enough for a lattice
