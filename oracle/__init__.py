"""ctypes bindings of the CPU oracle (``liboracle.so``) and, when it has been built, of the
library around the reference's own CPU header (``_ref/libplref.so``).

TEST INFRASTRUCTURE ONLY: used by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` as the checker.  The HIP library never imports this.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libplref.so")

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i16p = np.ctypeslib.ndpointer(np.int16, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build(with_reference=True):
    """Compile liboracle.so (and _ref/libplref.so when the reference tree is present)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "all"], stdout=subprocess.DEVNULL)
    if with_reference and os.path.exists("/root/reference/src/PermutohedralLatticeCPU.h"):
        subprocess.check_call(["make", "-C", _HERE, "-B", "ref"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build(with_reference=False)
    lib = C.CDLL(_LIB_PATH)
    lib.plo_scale_factor.argtypes = [C.c_int, _f32p]
    lib.plo_dump_simplex.argtypes = [C.c_int, C.c_int, _f32p] + [C.c_void_p] * 5
    lib.plo_compute_positions.argtypes = [C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int, _i32p,
                                          C.c_float, C.c_float]
    lib.plo_create.restype = C.c_void_p
    lib.plo_create.argtypes = [C.c_int, C.c_int, C.c_int]
    lib.plo_destroy.argtypes = [C.c_void_p]
    lib.plo_splat.argtypes = [C.c_void_p, _f32p, _f32p]
    lib.plo_blur.argtypes = [C.c_void_p, C.c_int]
    lib.plo_slice.argtypes = [C.c_void_p, _f32p, C.c_int]
    lib.plo_filter.argtypes = [C.c_void_p, _f32p, _f32p, _f32p, C.c_int]
    lib.plo_filter_raw.argtypes = [C.c_void_p, _f32p, _f32p, _f32p, C.c_int]
    lib.plo_set_reference_growth_quirk.argtypes = [C.c_void_p, C.c_int]
    lib.plo_num_growths.argtypes = [C.c_void_p]
    lib.plo_num_growths.restype = C.c_int
    lib.plo_num_vertices.argtypes = [C.c_void_p]
    lib.plo_num_vertices.restype = C.c_int
    for name, typ in (("plo_keys", C.c_int16), ("plo_values", C.c_float),
                      ("plo_replay_vertex", C.c_int32), ("plo_replay_weight", C.c_float)):
        getattr(lib, name).argtypes = [C.c_void_p]
        getattr(lib, name).restype = C.POINTER(typ)
    lib.plo_stage_seconds.argtypes = [C.c_void_p] + [C.POINTER(C.c_double)] * 3
    lib.plo_lattice_filter_op.restype = C.c_int
    lib.plo_lattice_filter_op.argtypes = [_f32p, C.c_void_p, _f32p, C.c_int, C.c_int, _i32p,
                                          C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                                          C.c_float, C.c_int]
    return lib


_lib = _load()


def _opt(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def scale_factor(pd):
    out = np.empty(pd, np.float32)
    _lib.plo_scale_factor(pd, out)
    return out


def dump_simplex(positions, want_elevated=False):
    """positions [N, pd] -> dict(rem0 [N,pd+1] i16, rank [N,pd+1] i16, keys [N,pd+1,pd] i16,
    barycentric [N,pd+1] f32[, elevated [N,pd+1] f32])."""
    positions = np.ascontiguousarray(positions, np.float32)
    n, pd = positions.shape
    d1 = pd + 1
    out = dict(rem0=np.empty((n, d1), np.int16), rank=np.empty((n, d1), np.int16),
               keys=np.empty((n, d1, pd), np.int16), barycentric=np.empty((n, d1), np.float32))
    el = np.empty((n, d1), np.float32) if want_elevated else None
    _lib.plo_dump_simplex(pd, n, positions, _opt(out["rem0"]), _opt(out["rank"]),
                          _opt(out["keys"]), _opt(out["barycentric"]), _opt(el))
    if want_elevated:
        out["elevated"] = el
    return out


def compute_positions(reference, spatial_dims, spatial_std, feature_std, n_reference_channels):
    """One batch item.  reference: [N, rc] (ignored when rc == 0) -> positions [N, k+rc]."""
    sd = np.ascontiguousarray(spatial_dims, np.int32)
    n = int(np.prod(sd))
    pd = len(sd) + n_reference_channels
    pos = np.empty((n, pd), np.float32)
    ref = None
    if n_reference_channels:
        ref = np.ascontiguousarray(reference, np.float32).reshape(n, n_reference_channels)
    _lib.plo_compute_positions(_opt(ref), pos, n, n_reference_channels, len(sd), sd,
                               float(spatial_std), float(feature_std))
    return pos


class Lattice:
    """Lattice object for (pd, vd, N); vd includes the homogeneous channel."""

    def __init__(self, pd, vd, n, reference_growth_quirk=False):
        """reference_growth_quirk=True reproduces the reference's duplicate vertex at index
        doublings (bit-exact with the reference); False is one vertex per distinct key."""
        self.pd, self.vd, self.n = pd, vd, n
        self._h = _lib.plo_create(pd, vd, n)
        if not self._h:
            raise ValueError("bad lattice dimensions")
        _lib.plo_set_reference_growth_quirk(self._h, int(reference_growth_quirk))

    @property
    def num_growths(self):
        return _lib.plo_num_growths(self._h)

    def __del__(self):
        if getattr(self, "_h", None):
            _lib.plo_destroy(self._h)
            self._h = None

    def filter(self, inp, positions, reverse=False):
        inp = np.ascontiguousarray(inp, np.float32).reshape(self.n, self.vd - 1)
        positions = np.ascontiguousarray(positions, np.float32).reshape(self.n, self.pd)
        out = np.empty_like(inp)
        _lib.plo_filter(self._h, out, inp, positions, int(reverse))
        return out

    def filter_raw(self, inp_vd, positions, reverse=False):
        """The unnormalised linear operator on values that carry all vd channels."""
        inp_vd = np.ascontiguousarray(inp_vd, np.float32).reshape(self.n, self.vd)
        positions = np.ascontiguousarray(positions, np.float32).reshape(self.n, self.pd)
        out = np.empty_like(inp_vd)
        _lib.plo_filter_raw(self._h, out, inp_vd, positions, int(reverse))
        return out

    def splat(self, inp, positions):
        inp = np.ascontiguousarray(inp, np.float32).reshape(self.n, self.vd - 1)
        positions = np.ascontiguousarray(positions, np.float32).reshape(self.n, self.pd)
        _lib.plo_splat(self._h, positions, inp)

    def blur(self, reverse=False):
        _lib.plo_blur(self._h, int(reverse))

    def slice(self, normalize=True):
        out = np.empty((self.n, self.vd - 1 if normalize else self.vd), np.float32)
        _lib.plo_slice(self._h, out, int(normalize))
        return out

    @property
    def num_vertices(self):
        return _lib.plo_num_vertices(self._h)

    def keys(self):
        m = self.num_vertices
        return np.ctypeslib.as_array(_lib.plo_keys(self._h), (m, self.pd)).copy()

    def values(self):
        m = self.num_vertices
        return np.ctypeslib.as_array(_lib.plo_values(self._h), (m, self.vd)).copy()

    def replay(self):
        shape = (self.n, self.pd + 1)
        return (np.ctypeslib.as_array(_lib.plo_replay_vertex(self._h), shape).copy(),
                np.ctypeslib.as_array(_lib.plo_replay_weight(self._h), shape).copy())

    def stage_seconds(self):
        s = [C.c_double() for _ in range(3)]
        _lib.plo_stage_seconds(self._h, *[C.byref(x) for x in s])
        return dict(splat=s[0].value, blur=s[1].value, slice=s[2].value)


def lattice_filter(input_image, reference_image, bilateral=True, theta_alpha=1.0, theta_beta=1.0,
                   theta_gamma=1.0, reverse=False):
    """The LatticeFilter op on channels-last arrays [B, s_1..s_k, C]."""
    inp = np.ascontiguousarray(input_image, np.float32)
    sd = np.ascontiguousarray(inp.shape[1:-1], np.int32)
    ref = None
    rc = 0
    if reference_image is not None:
        ref = np.ascontiguousarray(reference_image, np.float32)
        rc = ref.shape[-1]
    out = np.empty_like(inp)
    rcode = _lib.plo_lattice_filter_op(inp, _opt(ref), out, inp.shape[0], len(sd), sd,
                                       inp.shape[-1], rc, int(bilateral), theta_alpha,
                                       theta_beta, theta_gamma, int(reverse))
    if rcode != 0:
        raise ValueError("plo_lattice_filter_op: bad arguments")
    return out


# ---------------------------------------------------------------------------------------------
# The reference's own CPU header behind C entry points (present only after `make -C oracle ref`)
# ---------------------------------------------------------------------------------------------

def have_reference():
    return os.path.exists(_REF_PATH)


class _Ref:
    def __init__(self):
        lib = C.CDLL(_REF_PATH)
        lib.plref_scale_factor.argtypes = [C.c_int, _f32p]
        lib.plref_dump_simplex.argtypes = [C.c_int, C.c_int, _f32p] + [C.c_void_p] * 5
        lib.plref_compute_positions.argtypes = [C.c_void_p, _f32p, C.c_int, C.c_int, C.c_int,
                                                _i32p, C.c_float, C.c_float]
        lib.plref_filter.argtypes = [C.c_int, C.c_int, C.c_int, _f32p, _f32p, _f32p, C.c_int,
                                     C.POINTER(C.c_int), C.c_void_p, C.POINTER(C.c_double)]
        lib.plref_filter_stages.argtypes = [C.c_int, C.c_int, C.c_int, _f32p, _f32p, _f32p,
                                            C.c_int, C.POINTER(C.c_int), C.c_void_p, C.c_void_p,
                                            C.c_void_p]
        lib.plref_lattice_filter_op.argtypes = [_f32p, C.c_void_p, _f32p, C.c_int, C.c_int, _i32p,
                                                C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                                                C.c_float, C.c_int]
        self.lib = lib

    def scale_factor(self, pd):
        out = np.empty(pd, np.float32)
        self.lib.plref_scale_factor(pd, out)
        return out

    def dump_simplex(self, positions):
        positions = np.ascontiguousarray(positions, np.float32)
        n, pd = positions.shape
        d1 = pd + 1
        out = dict(rem0=np.empty((n, d1), np.int16), rank=np.empty((n, d1), np.int16),
                   keys=np.empty((n, d1, pd), np.int16),
                   barycentric=np.empty((n, d1), np.float32),
                   elevated=np.empty((n, d1), np.float32))
        self.lib.plref_dump_simplex(pd, n, positions, _opt(out["rem0"]), _opt(out["rank"]),
                                    _opt(out["keys"]), _opt(out["barycentric"]),
                                    _opt(out["elevated"]))
        return out

    def compute_positions(self, reference, spatial_dims, spatial_std, feature_std,
                          n_reference_channels):
        sd = np.ascontiguousarray(spatial_dims, np.int32)
        n = int(np.prod(sd))
        pos = np.empty((n, len(sd) + n_reference_channels), np.float32)
        ref = None
        if n_reference_channels:
            ref = np.ascontiguousarray(reference, np.float32).reshape(n, n_reference_channels)
        self.lib.plref_compute_positions(_opt(ref), pos, n, n_reference_channels, len(sd), sd,
                                         float(spatial_std), float(feature_std))
        return pos

    def filter(self, pd, vd, inp, positions, reverse=False):
        """-> (output, M, keys [M, pd], seconds)"""
        inp = np.ascontiguousarray(inp, np.float32)
        n = inp.size // (vd - 1)
        inp = inp.reshape(n, vd - 1)
        positions = np.ascontiguousarray(positions, np.float32).reshape(n, pd)
        out = np.empty_like(inp)
        m = C.c_int()
        sec = C.c_double()
        keys = np.empty((n * (pd + 1), pd), np.int16)
        self.lib.plref_filter(pd, vd, n, out, inp, positions, int(reverse), C.byref(m),
                              _opt(keys), C.byref(sec))
        return out, m.value, keys[:m.value].copy(), sec.value

    def filter_stages(self, pd, vd, inp, positions, reverse=False, want_values=True):
        """-> dict(output, M, after_splat [M,vd], after_blur [M,vd], seconds{splat,blur,slice})"""
        inp = np.ascontiguousarray(inp, np.float32)
        n = inp.size // (vd - 1)
        inp = inp.reshape(n, vd - 1)
        positions = np.ascontiguousarray(positions, np.float32).reshape(n, pd)
        out = np.empty_like(inp)
        m = C.c_int()
        a = np.empty((n * (pd + 1), vd), np.float32) if want_values else None
        b = np.empty((n * (pd + 1), vd), np.float32) if want_values else None
        sec = np.zeros(3, np.float64)
        self.lib.plref_filter_stages(pd, vd, n, out, inp, positions, int(reverse), C.byref(m),
                                     _opt(a), _opt(b), _opt(sec))
        res = dict(output=out, M=m.value,
                   seconds=dict(splat=sec[0], blur=sec[1], slice=sec[2]))
        if want_values:
            res["after_splat"] = a[:m.value].copy()
            res["after_blur"] = b[:m.value].copy()
        return res

    def lattice_filter(self, input_image, reference_image, bilateral=True, theta_alpha=1.0,
                       theta_beta=1.0, theta_gamma=1.0, reverse=False):
        inp = np.ascontiguousarray(input_image, np.float32)
        sd = np.ascontiguousarray(inp.shape[1:-1], np.int32)
        ref = np.ascontiguousarray(reference_image, np.float32)
        out = np.empty_like(inp)
        self.lib.plref_lattice_filter_op(inp, _opt(ref), out, inp.shape[0], len(sd), sd,
                                         inp.shape[-1], ref.shape[-1], int(bilateral),
                                         theta_alpha, theta_beta, theta_gamma, int(reverse))
        return out


_ref_singleton = None


def reference():
    """Bindings of oracle/_ref/libplref.so, or None when it has not been built."""
    global _ref_singleton
    if _ref_singleton is None and have_reference():
        _ref_singleton = _Ref()
    return _ref_singleton
