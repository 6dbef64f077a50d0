"""MI355X (gfx950) permutohedral-lattice filter: Python mirror of the reference's interfaces over
the C ABI of ``libpermutohedral_hip.so`` (declared in ``include/permutohedral_lattice.h``).

* :class:`PermutohedralLattice` -- the lattice object ``(pd, vd, N)`` with
  ``filter(output, input, positions, reverse)`` on device tensors
  (reference: src/PermutohedralLatticeCPU.h:419-446, src/PermutohedralLatticeGPU.cuh:434-479).
* :func:`compute_positions` -- the feature builder (reference: src/PermutohedralLatticeCPU.h:452-474).
* :func:`lattice_filter` -- the ``LatticeFilter`` op with its registered gradient
  (reference: src/LatticeFilterKernel.cpp:30-43, 98-181; lattice_filter_op_loader.py:32-54).

torch is used for device memory, streams and autograd plumbing only; all computation is in the
HIP library.  There is no CPU fallback: importing this package without the built library raises.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpermutohedral_hip.so")

PL_OK, PL_EINVAL, PL_EUNSUPPORTED, PL_ENOMEM, PL_EOVERFLOW, PL_EHIP, PL_ESTATE = 0, -1, -2, -3, -4, -5, -6
PL_ETOOLARGE = -7
PL_OPT_NORMALIZE, PL_OPT_PROFILE, PL_OPT_TABLE_CELLS, PL_OPT_XCD_AWARE, PL_OPT_PAIR_BLUR = 1, 2, 3, 4, 5
PL_OPT_GUESS_GRID = 6
PL_OPT_MERGE_TILES = 7
PL_OPT_STOP_AFTER = 8
PL_OPT_ORDER_POINTS = 9
PL_OPT_VERTEX_LISTS = 10
PL_OPT_NUMBER_SEGMENTS = 11
PL_INFO_BUILD_MERGED, PL_INFO_TABLE_CELLS, PL_INFO_SCRATCH_BYTES, PL_INFO_FOREIGN_ROWS = 1, 2, 3, 4
PL_LIB_LAYOUT_VERSION, PL_LIB_REPLAY_ROW_BYTES, PL_LIB_SOURCE_HASH = 1, 2, 3
# The device-side array layouts this module (and the tests and benchmarks on top of it) were
# written for: PL_LAYOUT_VERSION of include/permutohedral_lattice.h and the size of a replay row.
# A library that reports other values is not driven at all: its kernels would read each other's
# arrays in a layout this side knows nothing of.
LAYOUT_VERSION = 3
REPLAY_ROW_BYTES = 8

# every symbol include/permutohedral_lattice.h declares
EXPORTS = (
    "pl_supported", "pl_strerror", "pl_last_hip_error", "pl_library_info", "pl_create", "pl_destroy", "pl_filter",
    "pl_filter_static", "pl_build", "pl_apply", "pl_set_point_grid", "pl_get_point_grid", "pl_num_vertices", "pl_set_option", "pl_get_info", "pl_stage_ms", "pl_debug_simplex",
    "pl_debug_keys", "pl_debug_values", "pl_debug_replay", "pl_compute_positions", "pl_filter_image", "pl_build_image",
    "pl_filter_begin", "pl_filter_image_begin", "pl_filter_end",
    "pl_build_begin", "pl_build_image_begin", "pl_build_end", "pl_lattice_filter_op",
    "pl_set_op_concurrency",
    "pl_create_f64", "pl_filter_f64", "pl_build_f64", "pl_apply_f64", "pl_debug_simplex_f64",
    "pl_compute_positions_f64", "pl_lattice_filter_op_f64",
)


class PermutohedralError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = _lib.pl_strerror(status).decode()
        if status == PL_EHIP:
            msg += " (hipError %d)" % _lib.pl_last_hip_error()
        super().__init__("%s: %s" % (where, msg))


def _library_property(lib, what):
    v = C.c_longlong()
    status = lib.pl_library_info(int(what), C.byref(v))
    if status != PL_OK:
        raise ImportError("pl_library_info(%d) failed with status %d" % (what, status))
    return v.value


def _load(path=LIB_PATH):
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with `python permutohedral_lattice_amd/build.py` "
            "(there is no CPU fallback)" % path)
    lib = C.CDLL(path)
    stale = [name for name in EXPORTS if not hasattr(lib, name)]
    if stale:
        raise ImportError("%s lacks %s: rebuild it with `python permutohedral_lattice_amd/build.py`"
                          % (path, ", ".join(stale)))
    lib.pl_library_info.argtypes = [C.c_int, C.POINTER(C.c_longlong)]
    got = (_library_property(lib, PL_LIB_LAYOUT_VERSION), _library_property(lib, PL_LIB_REPLAY_ROW_BYTES))
    if got != (LAYOUT_VERSION, REPLAY_ROW_BYTES):
        raise ImportError(
            "%s has array layout version %d with replay rows of %d bytes; this module drives version "
            "%d with rows of %d bytes: rebuild it with `python permutohedral_lattice_amd/build.py`"
            % (path, got[0], got[1], LAYOUT_VERSION, REPLAY_ROW_BYTES))
    vp, ci, cf = C.c_void_p, C.c_int, C.c_float
    lib.pl_supported.argtypes = [ci, ci]
    lib.pl_strerror.argtypes = [ci]
    lib.pl_strerror.restype = C.c_char_p
    lib.pl_create.argtypes = [ci, ci, ci, vp, vp, C.POINTER(vp)]
    lib.pl_destroy.argtypes = [vp]
    lib.pl_filter.argtypes = [vp, vp, vp, vp, ci]
    lib.pl_filter_static.argtypes = [ci, ci, ci, vp, vp, vp, ci, vp]
    lib.pl_build.argtypes = [vp, vp]
    lib.pl_apply.argtypes = [vp, vp, vp, ci]
    lib.pl_set_point_grid.argtypes = [vp, ci, C.POINTER(ci)]
    lib.pl_get_point_grid.argtypes = [vp, C.POINTER(ci), C.POINTER(ci)]
    lib.pl_num_vertices.argtypes = [vp, C.POINTER(ci)]
    lib.pl_set_option.argtypes = [vp, ci, C.c_long]
    lib.pl_get_info.argtypes = [vp, ci, C.POINTER(C.c_long)]
    lib.pl_stage_ms.argtypes = [vp, C.POINTER(cf)]
    lib.pl_debug_simplex.argtypes = [vp, vp, vp, vp, vp, vp]
    lib.pl_debug_keys.argtypes = [vp, vp]
    lib.pl_debug_values.argtypes = [vp, vp]
    lib.pl_debug_replay.argtypes = [vp, vp, vp]
    lib.pl_compute_positions.argtypes = [vp, vp, ci, ci, ci, C.POINTER(ci), cf, cf, vp]
    lib.pl_filter_image.argtypes = [vp, vp, vp, vp, ci, ci, C.POINTER(ci), cf, cf, ci]
    lib.pl_build_image.argtypes = [vp, vp, ci, ci, C.POINTER(ci), cf, cf]
    lib.pl_filter_begin.argtypes = [vp, vp, vp, vp, ci]
    lib.pl_filter_image_begin.argtypes = [vp, vp, vp, vp, ci, ci, C.POINTER(ci), cf, cf, ci]
    lib.pl_filter_end.argtypes = [vp]
    lib.pl_build_begin.argtypes = [vp, vp]
    lib.pl_build_image_begin.argtypes = [vp, vp, ci, ci, C.POINTER(ci), cf, cf]
    lib.pl_build_end.argtypes = [vp]
    lib.pl_set_op_concurrency.argtypes = [ci]
    lib.pl_lattice_filter_op.argtypes = [vp, vp, vp, ci, ci, C.POINTER(ci), ci, ci, ci, cf, cf, cf,
                                         ci, vp, vp]
    # T = double
    lib.pl_create_f64.argtypes = lib.pl_create.argtypes
    lib.pl_filter_f64.argtypes = lib.pl_filter.argtypes
    lib.pl_build_f64.argtypes = lib.pl_build.argtypes
    lib.pl_apply_f64.argtypes = lib.pl_apply.argtypes
    lib.pl_debug_simplex_f64.argtypes = lib.pl_debug_simplex.argtypes
    lib.pl_compute_positions_f64.argtypes = [vp, vp, ci, ci, ci, C.POINTER(ci), C.c_double,
                                             C.c_double, vp]
    lib.pl_lattice_filter_op_f64.argtypes = lib.pl_lattice_filter_op.argtypes
    return lib


_lib = _load()


def _check(status, where):
    if status != PL_OK:
        raise PermutohedralError(status, where)


def _dev(t, name, numel=None, dtype=torch.float32):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous()):
        raise TypeError("%s must be a contiguous %s tensor on the GPU" % (name, dtype))
    if numel is not None and t.numel() != numel:
        raise ValueError("%s has %d elements, expected %d" % (name, t.numel(), numel))
    return C.c_void_p(t.data_ptr())


def _dev_f32(t, name, numel=None):
    return _dev(t, name, numel, torch.float32)


def _value_type(dtype):
    """The reference's template parameter T: float (default) or double."""
    if dtype in (None, torch.float32):
        return torch.float32
    if dtype == torch.float64:
        return torch.float64
    raise TypeError("the lattice is built for float32 and float64 values, not %s" % dtype)


def _stream_ptr(stream=None):
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def supported(pd, vd):
    return bool(_lib.pl_supported(pd, vd))


def library_source_hash():
    """The hash of its sources the loaded library was built with, as 12 hex digits (what
    ``build.source_hash()`` gives for the sources it was compiled from)."""
    return "%012x" % _library_property(_lib, PL_LIB_SOURCE_HASH)


class PermutohedralLattice:
    """Lattice for ``(pd, vd, N)``; ``vd`` counts the homogeneous channel.  All tensors are
    contiguous tensors of ``dtype`` (float32, or float64 for the reference's ``T = double``) on
    the GPU; work is enqueued on the stream current at construction."""

    def __init__(self, pd, vd, N, stream=None, dtype=torch.float32):
        self.pd, self.vd, self.N = int(pd), int(vd), int(N)
        self.dtype = _value_type(dtype)
        self._f64 = self.dtype == torch.float64
        self._h = C.c_void_p()
        self._stream = stream if stream is not None else torch.cuda.current_stream()
        create = _lib.pl_create_f64 if self._f64 else _lib.pl_create
        _check(create(self.pd, self.vd, self.N, _stream_ptr(self._stream), None, C.byref(self._h)),
               "pl_create")
        self._normalize = True

    def _t(self, t, name, numel):
        return _dev(t, name, numel, self.dtype)

    def _float_only(self, what):
        if self._f64:
            raise TypeError("%s is for lattices of float32 values" % what)

    def close(self):
        if getattr(self, "_h", None):
            _lib.pl_destroy(self._h)
            self._h = None

    def __del__(self):
        # (at interpreter exit the module's globals may be gone before the last lattice: the
        # process's memory goes with it)
        if _lib is not None:
            self.close()

    # -- the reference's interface -------------------------------------------------------------
    def filter(self, output, input, positions, reverse=False):
        ch = self.vd - 1 if self._normalize else self.vd
        call = _lib.pl_filter_f64 if self._f64 else _lib.pl_filter
        _check(call(self._h, self._t(output, "output", self.N * ch),
                    self._t(input, "input", self.N * ch),
                    self._t(positions, "positions", self.N * self.pd), int(bool(reverse))),
               "pl_filter")
        return output

    # -- the same in two halves: enqueue, and later wait and check ---------------------------------
    def filter_begin(self, output, input, positions, reverse=False):
        self._float_only("filter_begin")
        ch = self.vd - 1 if self._normalize else self.vd
        self._in_flight = (output, input, positions)   # keep the tensors alive until filter_end
        _check(_lib.pl_filter_begin(self._h, _dev_f32(output, "output", self.N * ch),
                                    _dev_f32(input, "input", self.N * ch),
                                    _dev_f32(positions, "positions", self.N * self.pd),
                                    int(bool(reverse))), "pl_filter_begin")

    def filter_end(self):
        _check(_lib.pl_filter_end(self._h), "pl_filter_end")
        self._in_flight = None

    # -- build once, apply many ----------------------------------------------------------------
    def build(self, positions):
        call = _lib.pl_build_f64 if self._f64 else _lib.pl_build
        _check(call(self._h, self._t(positions, "positions", self.N * self.pd)), "pl_build")

    def build_begin(self, positions):
        """``build`` in two halves: enqueue, and ``build_end`` waits and checks (so that several
        lattices, each on a stream of its own, are built side by side)."""
        self._float_only("build_begin")
        self._in_flight = (positions,)   # keep the tensor alive until build_end
        _check(_lib.pl_build_begin(self._h, _dev_f32(positions, "positions", self.N * self.pd)),
               "pl_build_begin")

    def build_end(self):
        _check(_lib.pl_build_end(self._h), "pl_build_end")
        self._in_flight = None

    def apply(self, output, input, reverse=False):
        ch = self.vd - 1 if self._normalize else self.vd
        call = _lib.pl_apply_f64 if self._f64 else _lib.pl_apply
        _check(call(self._h, self._t(output, "output", self.N * ch),
                    self._t(input, "input", self.N * ch), int(bool(reverse))), "pl_apply")
        return output

    # -- features built on the fly from the reference image and the grid coordinates ------------
    def _image_args(self, reference, spatial_dims):
        self._float_only("the fused feature builder")
        dims = [int(d) for d in spatial_dims]
        rc = self.pd - len(dims)
        if rc < 0:
            raise ValueError("more spatial dimensions than pd")
        ref = _dev_f32(reference, "reference", self.N * rc) if rc > 0 else None
        return ref, rc, len(dims), (C.c_int * max(1, len(dims)))(*dims)

    def filter_image(self, output, input, reference, spatial_dims, spatial_std, feature_std=1.0,
                     reverse=False):
        """``filter`` under the features ``compute_positions(reference, spatial_dims, spatial_std,
        feature_std)`` would give, without building that array."""
        ch = self.vd - 1 if self._normalize else self.vd
        ref, rc, k, dims = self._image_args(reference, spatial_dims)
        _check(_lib.pl_filter_image(self._h, _dev_f32(output, "output", self.N * ch),
                                    _dev_f32(input, "input", self.N * ch), ref, rc, k, dims,
                                    float(spatial_std), float(feature_std), int(bool(reverse))),
               "pl_filter_image")
        return output

    def build_image(self, reference, spatial_dims, spatial_std, feature_std=1.0):
        ref, rc, k, dims = self._image_args(reference, spatial_dims)
        _check(_lib.pl_build_image(self._h, ref, rc, k, dims, float(spatial_std), float(feature_std)),
               "pl_build_image")

    def build_image_begin(self, reference, spatial_dims, spatial_std, feature_std=1.0):
        """``build_image`` enqueued; ``build_end`` completes it."""
        ref, rc, k, dims = self._image_args(reference, spatial_dims)
        self._in_flight = (reference,)
        _check(_lib.pl_build_image_begin(self._h, ref, rc, k, dims, float(spatial_std),
                                         float(feature_std)), "pl_build_image_begin")

    def set_point_grid(self, dims):
        """Hint: the N points form a row-major grid of these extents (None removes the hint)."""
        dims = [int(d) for d in (dims or [])]
        arr = (C.c_int * max(1, len(dims)))(*dims)
        _check(_lib.pl_set_point_grid(self._h, len(dims), arr), "pl_set_point_grid")

    @property
    def point_grid(self):
        """Extents of the grid the work is ordered by (given, or found in the positions); () if none."""
        n, dims = C.c_int(), (C.c_int * 3)()
        _check(_lib.pl_get_point_grid(self._h, C.byref(n), dims), "pl_get_point_grid")
        return tuple(dims[i] for i in range(n.value))

    @property
    def num_vertices(self):
        m = C.c_int()
        _check(_lib.pl_num_vertices(self._h, C.byref(m)), "pl_num_vertices")
        return m.value

    def set_option(self, option, value):
        _check(_lib.pl_set_option(self._h, option, int(value)), "pl_set_option")
        if option == PL_OPT_NORMALIZE:
            self._normalize = bool(value)

    def info(self, what):
        v = C.c_long()
        _check(_lib.pl_get_info(self._h, int(what), C.byref(v)), "pl_get_info")
        return v.value

    def stage_ms(self):
        ms = (C.c_float * 8)()
        _check(_lib.pl_stage_ms(self._h, ms), "pl_stage_ms")
        return dict(zip(("clear", "build", "ids", "neighbours", "fill", "splat", "blur", "slice"),
                        list(ms)))

    # -- parity exports ------------------------------------------------------------------------
    def debug_simplex(self, positions):
        """-> dict of device tensors rem0 [N,pd+1] i16, rank [N,pd+1] i16, keys [N,pd+1,pd] i16,
        barycentric [N,pd+1] of the lattice's value type."""
        d1, dev = self.pd + 1, positions.device
        out = dict(rem0=torch.empty((self.N, d1), dtype=torch.int16, device=dev),
                   rank=torch.empty((self.N, d1), dtype=torch.int16, device=dev),
                   keys=torch.empty((self.N, d1, self.pd), dtype=torch.int16, device=dev),
                   barycentric=torch.empty((self.N, d1), dtype=self.dtype, device=dev))
        call = _lib.pl_debug_simplex_f64 if self._f64 else _lib.pl_debug_simplex
        _check(call(self._h, self._t(positions, "positions", self.N * self.pd),
                    C.c_void_p(out["rem0"].data_ptr()), C.c_void_p(out["rank"].data_ptr()),
                    C.c_void_p(out["keys"].data_ptr()), C.c_void_p(out["barycentric"].data_ptr())),
               "pl_debug_simplex")
        return out

    def debug_keys(self):
        keys = torch.empty((self.num_vertices, self.pd), dtype=torch.int16, device="cuda")
        _check(_lib.pl_debug_keys(self._h, C.c_void_p(keys.data_ptr())), "pl_debug_keys")
        return keys

    def debug_values(self):
        """-> vertex values [M, vd] as the last filter/apply left them (rows as in debug_keys)."""
        v = torch.empty((self.num_vertices, self.vd), dtype=self.dtype, device="cuda")
        _check(_lib.pl_debug_values(self._h, C.c_void_p(v.data_ptr())), "pl_debug_values")
        return v

    def debug_replay(self):
        """-> (vertex [pd+1, N] i32, weight [pd+1, N] f32) of the last apply/filter."""
        self._float_only("debug_replay")
        v = torch.empty((self.pd + 1, self.N), dtype=torch.int32, device="cuda")
        w = torch.empty((self.pd + 1, self.N), dtype=torch.float32, device="cuda")
        _check(_lib.pl_debug_replay(self._h, C.c_void_p(v.data_ptr()), C.c_void_p(w.data_ptr())),
               "pl_debug_replay")
        return v, w


def filter_static(output, input, positions, pd, vd, reverse=False, stream=None):
    """``filter`` without a lattice object and without any allocation: the lattice lives in a
    static device array inside the library for the length of the call (N*(pd+1) <= 131072,
    vd <= 8, float32; ``PL_ETOOLARGE`` beyond)."""
    n = int(positions.shape[0]) if positions.dim() == 2 else positions.numel() // int(pd)
    _check(_lib.pl_filter_static(int(pd), int(vd), n, _dev_f32(output, "output", n * (vd - 1)),
                                 _dev_f32(input, "input", n * (vd - 1)),
                                 _dev_f32(positions, "positions", n * pd), int(bool(reverse)),
                                 _stream_ptr(stream)), "pl_filter_static")
    return output


def set_op_concurrency(lanes):
    """Batch items :func:`lattice_filter` keeps in flight at once (1..8, default 4)."""
    _check(_lib.pl_set_op_concurrency(int(lanes)), "pl_set_op_concurrency")


def compute_positions(reference, spatial_dims, spatial_std, feature_std=1.0, out=None, dtype=None):
    """Feature rows of one batch item.  ``reference``: ``[*spatial_dims, rc]`` device tensor, or
    None for spatial-only features.  -> ``[N, k + rc]``, in ``dtype`` (default: the reference
    tensor's, float32 without one)."""
    if dtype is None:
        dtype = out.dtype if out is not None else (reference.dtype if reference is not None
                                                   else torch.float32)
    dtype = _value_type(dtype)
    sd = [int(s) for s in spatial_dims]
    n = 1
    for s in sd:
        n *= s
    rc = 0 if reference is None else int(reference.shape[-1])
    pd = len(sd) + rc
    if out is None:
        out = torch.empty((n, pd), dtype=dtype, device="cuda")
    ref_ptr = None if reference is None else _dev(reference, "reference", n * rc, dtype)
    dims = (C.c_int * len(sd))(*sd)
    call = _lib.pl_compute_positions_f64 if dtype == torch.float64 else _lib.pl_compute_positions
    _check(call(ref_ptr, _dev(out, "positions", n * pd, dtype), n, rc, len(sd), dims,
                float(spatial_std), float(feature_std), _stream_ptr()), "pl_compute_positions")
    return out


def _lattice_filter_raw(input_image, reference_image, bilateral, theta_alpha, theta_beta,
                        theta_gamma, reverse):
    if input_image.dim() < 3:
        raise ValueError("input_image must be [batch, spatial..., channels]")
    inp = input_image.contiguous()
    dtype = _value_type(inp.dtype)
    sd = [int(s) for s in inp.shape[1:-1]]
    out = torch.empty_like(inp)
    ref_ptr, rc = None, 0
    if reference_image is not None:
        ref = reference_image.contiguous()
        rc = int(ref.shape[-1])
        if bilateral:
            if list(ref.shape[:-1]) != list(inp.shape[:-1]):
                raise ValueError("reference_image and input_image differ in batch or spatial shape")
            ref_ptr = _dev(ref, "reference_image", None, dtype)
    dims = (C.c_int * len(sd))(*sd)
    call = _lib.pl_lattice_filter_op_f64 if dtype == torch.float64 else _lib.pl_lattice_filter_op
    _check(call(_dev(inp, "input_image", None, dtype), ref_ptr, C.c_void_p(out.data_ptr()),
                int(inp.shape[0]), len(sd), dims, int(inp.shape[-1]), rc, int(bool(bilateral)),
                float(theta_alpha), float(theta_beta), float(theta_gamma), int(bool(reverse)),
                _stream_ptr(), None), "pl_lattice_filter_op")
    return out


class _LatticePool:
    """Lattices kept between calls, so that the forward and the backward pass of one op call can
    share what the forward pass built: the positions are the same, only the blur order differs
    (the reference rebuilds the lattice in the backward pass, src/LatticeFilterKernel.cpp:79)."""

    def __init__(self, max_idle_per_shape=4, max_lent=16):
        self.idle, self.lent = {}, 0
        self.max_idle_per_shape, self.max_lent = max_idle_per_shape, max_lent

    @staticmethod
    def _key(pd, vd, n, stream):
        return (torch.cuda.current_device(), pd, vd, n, stream.cuda_stream)

    def acquire(self, pd, vd, n, count):
        """``count`` lattices for the current stream, or None when too many are lent out."""
        if self.lent + count > self.max_lent:
            return None
        stream = torch.cuda.current_stream()
        idle = self.idle.setdefault(self._key(pd, vd, n, stream), [])
        lattices = [idle.pop() if idle else PermutohedralLattice(pd, vd, n, stream=stream)
                    for _ in range(count)]
        self.lent += count
        return _LentLattices(self, lattices, self._key(pd, vd, n, stream))

    def give_back(self, lattices, key):
        self.lent -= len(lattices)
        idle = self.idle.setdefault(key, [])
        for lat in lattices:
            if len(idle) < self.max_idle_per_shape:
                idle.append(lat)
            else:
                lat.close()


class _LentLattices:
    """Returns its lattices to the pool when the autograd graph lets go of it."""

    def __init__(self, pool, lattices, key):
        self.pool, self.lattices, self.key = pool, lattices, key

    def __del__(self):
        if self.lattices is not None:
            self.pool.give_back(self.lattices, self.key)
            self.lattices = None


_pool = _LatticePool()


class _LatticeFilterFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_image, reference_image, bilateral, theta_alpha, theta_beta, theta_gamma,
                reverse):
        ctx.save_for_backward(reference_image)
        ctx.attrs = (bilateral, theta_alpha, theta_beta, theta_gamma)
        ctx.lent = None
        if (ctx.needs_input_grad[0] and input_image.dim() >= 3 and input_image.shape[0] > 0
                and input_image.dtype == torch.float32):
            out = _LatticeFilterFunction._forward_keeping_lattices(
                ctx, input_image, reference_image, bilateral, theta_alpha, theta_beta, theta_gamma,
                reverse)
            if out is not None:
                return out
        return _lattice_filter_raw(input_image, reference_image, bilateral, theta_alpha, theta_beta,
                                   theta_gamma, reverse)

    @staticmethod
    def _forward_keeping_lattices(ctx, input_image, reference_image, bilateral, theta_alpha,
                                  theta_beta, theta_gamma, reverse):
        """One lattice per batch item, built here and applied again (reversed) in backward."""
        inp = input_image.contiguous()
        sd = [int(s) for s in inp.shape[1:-1]]
        n = 1
        for s in sd:
            n *= s
        rc = int(reference_image.shape[-1]) if (bilateral and reference_image is not None) else 0
        pd, vd = len(sd) + rc, int(inp.shape[-1]) + 1
        if bilateral and (reference_image is None or rc < 1 or
                          list(reference_image.shape[:-1]) != list(inp.shape[:-1])):
            return None         # let the op report it
        if not supported(pd, vd) or n == 0:
            return None
        lent = _pool.acquire(pd, vd, n, int(inp.shape[0]))
        if lent is None:
            return None
        ref = reference_image.contiguous() if rc else None
        out = torch.empty_like(inp)
        spatial_std = theta_alpha if bilateral else theta_gamma
        for b, lat in enumerate(lent.lattices):
            lat.filter_image(out[b].view(n, vd - 1), inp[b].view(n, vd - 1),
                             ref[b].view(n, rc) if rc else None, sd, spatial_std,
                             theta_beta if bilateral else 1.0, reverse)
        ctx.lent = lent
        return out

    @staticmethod
    def backward(ctx, grad):
        # the reference's registered gradient: the same op on the upstream gradient with
        # reverse=True, and zeros for the reference image (lattice_filter_op_loader.py:46-54)
        (reference_image,) = ctx.saved_tensors
        bilateral, theta_alpha, theta_beta, theta_gamma = ctx.attrs
        lent = ctx.lent
        if lent is not None and lent.lattices is not None and \
                lent.key[-1] == torch.cuda.current_stream().cuda_stream:
            g = grad.contiguous()
            grad_vals = torch.empty_like(g)
            for b, lat in enumerate(lent.lattices):
                lat.apply(grad_vals[b].view(lat.N, lat.vd - 1), g[b].view(lat.N, lat.vd - 1), True)
        else:
            grad_vals = _lattice_filter_raw(grad, reference_image, bilateral, theta_alpha,
                                            theta_beta, theta_gamma, True)
        grad_ref = torch.zeros_like(reference_image) if ctx.needs_input_grad[1] else None
        return grad_vals, grad_ref, None, None, None, None, None


def lattice_filter(input_image, reference_image, bilateral=True, theta_alpha=1.0, theta_beta=1.0,
                   theta_gamma=1.0, reverse=False):
    """The ``LatticeFilter`` op: channels-last ``[B, s_1..s_k, C]`` device tensors, output shaped
    like ``input_image``.  Differentiable in ``input_image`` by the reference's rule."""
    return _LatticeFilterFunction.apply(input_image, reference_image, bool(bilateral),
                                        float(theta_alpha), float(theta_beta), float(theta_gamma),
                                        bool(reverse))
