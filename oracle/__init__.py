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


def _variants():
    """(suffix of the C names, numpy type, ctypes type) for T = float and T = double"""
    return (("", np.float32, C.c_float), ("_f64", np.float64, C.c_double))


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return ""
    if dtype == np.float64:
        return "_f64"
    raise TypeError("the lattice is built for float32 and float64, not %s" % dtype)


def _load():
    if not os.path.exists(_LIB_PATH):
        build(with_reference=False)
    lib = C.CDLL(_LIB_PATH)
    for sfx, npt, ct in _variants():
        fp = np.ctypeslib.ndpointer(npt, flags="C_CONTIGUOUS")

        def fn(name):
            return getattr(lib, "plo_" + name + sfx)
        fn("scale_factor").argtypes = [C.c_int, fp]
        fn("dump_simplex").argtypes = [C.c_int, C.c_int, fp] + [C.c_void_p] * 5
        fn("compute_positions").argtypes = [C.c_void_p, fp, C.c_int, C.c_int, C.c_int, _i32p,
                                            ct, ct]
        fn("create").restype = C.c_void_p
        fn("create").argtypes = [C.c_int, C.c_int, C.c_int]
        fn("destroy").argtypes = [C.c_void_p]
        fn("splat").argtypes = [C.c_void_p, fp, fp]
        fn("blur").argtypes = [C.c_void_p, C.c_int]
        fn("slice").argtypes = [C.c_void_p, fp, C.c_int]
        fn("filter").argtypes = [C.c_void_p, fp, fp, fp, C.c_int]
        fn("filter_raw").argtypes = [C.c_void_p, fp, fp, fp, C.c_int]
        fn("set_reference_growth_quirk").argtypes = [C.c_void_p, C.c_int]
        fn("num_growths").argtypes = [C.c_void_p]
        fn("num_growths").restype = C.c_int
        fn("growth_keys").argtypes = [C.c_void_p, np.ctypeslib.ndpointer(np.int16, flags="C_CONTIGUOUS")]
        fn("growth_keys").restype = C.c_int
        fn("num_vertices").argtypes = [C.c_void_p]
        fn("num_vertices").restype = C.c_int
        for name, typ in (("keys", C.c_int16), ("values", ct), ("replay_vertex", C.c_int32),
                          ("replay_weight", ct)):
            fn(name).argtypes = [C.c_void_p]
            fn(name).restype = C.POINTER(typ)
        fn("stage_seconds").argtypes = [C.c_void_p] + [C.POINTER(C.c_double)] * 3
        fn("lattice_filter_op").restype = C.c_int
        fn("lattice_filter_op").argtypes = [fp, C.c_void_p, fp, C.c_int, C.c_int, _i32p, C.c_int,
                                            C.c_int, C.c_int, C.c_float, C.c_float, C.c_float,
                                            C.c_int]
    return lib


_lib = _load()


def _fn(name, dtype):
    return getattr(_lib, "plo_" + name + _suffix(dtype))


def _opt(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def scale_factor(pd, dtype=np.float32):
    out = np.empty(pd, dtype)
    _fn("scale_factor", dtype)(pd, out)
    return out


def dump_simplex(positions, want_elevated=False, dtype=np.float32):
    """positions [N, pd] -> dict(rem0 [N,pd+1] i16, rank [N,pd+1] i16, keys [N,pd+1,pd] i16,
    barycentric [N,pd+1][, elevated [N,pd+1]]), floats in `dtype`."""
    positions = np.ascontiguousarray(positions, dtype)
    n, pd = positions.shape
    d1 = pd + 1
    out = dict(rem0=np.empty((n, d1), np.int16), rank=np.empty((n, d1), np.int16),
               keys=np.empty((n, d1, pd), np.int16), barycentric=np.empty((n, d1), dtype))
    el = np.empty((n, d1), dtype) if want_elevated else None
    _fn("dump_simplex", dtype)(pd, n, positions, _opt(out["rem0"]), _opt(out["rank"]),
                          _opt(out["keys"]), _opt(out["barycentric"]), _opt(el))
    if want_elevated:
        out["elevated"] = el
    return out


def compute_positions(reference, spatial_dims, spatial_std, feature_std, n_reference_channels,
                      dtype=np.float32):
    """One batch item.  reference: [N, rc] (ignored when rc == 0) -> positions [N, k+rc]."""
    sd = np.ascontiguousarray(spatial_dims, np.int32)
    n = int(np.prod(sd))
    pd = len(sd) + n_reference_channels
    pos = np.empty((n, pd), dtype)
    ref = None
    if n_reference_channels:
        ref = np.ascontiguousarray(reference, dtype).reshape(n, n_reference_channels)
    _fn("compute_positions", dtype)(_opt(ref), pos, n, n_reference_channels, len(sd), sd,
                                     float(spatial_std), float(feature_std))
    return pos


class Lattice:
    """Lattice object for (pd, vd, N); vd includes the homogeneous channel."""

    def __init__(self, pd, vd, n, reference_growth_quirk=False, dtype=np.float32):
        """reference_growth_quirk=True reproduces the reference's duplicate vertex at index
        doublings (bit-exact with the reference); False is one vertex per distinct key.
        dtype: the reference's template parameter T, float32 or float64."""
        self.pd, self.vd, self.n = pd, vd, n
        self.dtype = np.dtype(dtype)
        self._sfx = _suffix(dtype)
        self._h = self._fn("create")(pd, vd, n)
        if not self._h:
            raise ValueError("bad lattice dimensions")
        self._fn("set_reference_growth_quirk")(self._h, int(reference_growth_quirk))

    def _fn(self, name):
        return getattr(_lib, "plo_" + name + self._sfx)

    @property
    def num_growths(self):
        return self._fn("num_growths")(self._h)

    @property
    def growth_keys(self):
        """[doublings, pd] int16: the key that was being looked up when the index doubled, per
        doubling: with the quirk on, the lookups that probed from a stale cell."""
        out = np.zeros((24, self.pd), np.int16)
        n = self._fn("growth_keys")(self._h, out)
        return out[:n].copy()

    def __del__(self):
        if getattr(self, "_h", None):
            self._fn("destroy")(self._h)
            self._h = None

    def filter(self, inp, positions, reverse=False):
        inp = np.ascontiguousarray(inp, self.dtype).reshape(self.n, self.vd - 1)
        positions = np.ascontiguousarray(positions, self.dtype).reshape(self.n, self.pd)
        out = np.empty_like(inp)
        self._fn("filter")(self._h, out, inp, positions, int(reverse))
        return out

    def filter_raw(self, inp_vd, positions, reverse=False):
        """The unnormalised linear operator on values that carry all vd channels."""
        inp_vd = np.ascontiguousarray(inp_vd, self.dtype).reshape(self.n, self.vd)
        positions = np.ascontiguousarray(positions, self.dtype).reshape(self.n, self.pd)
        out = np.empty_like(inp_vd)
        self._fn("filter_raw")(self._h, out, inp_vd, positions, int(reverse))
        return out

    def splat(self, inp, positions):
        inp = np.ascontiguousarray(inp, self.dtype).reshape(self.n, self.vd - 1)
        positions = np.ascontiguousarray(positions, self.dtype).reshape(self.n, self.pd)
        self._fn("splat")(self._h, positions, inp)

    def blur(self, reverse=False):
        self._fn("blur")(self._h, int(reverse))

    def slice(self, normalize=True):
        out = np.empty((self.n, self.vd - 1 if normalize else self.vd), self.dtype)
        self._fn("slice")(self._h, out, int(normalize))
        return out

    @property
    def num_vertices(self):
        return self._fn("num_vertices")(self._h)

    def keys(self):
        m = self.num_vertices
        return np.ctypeslib.as_array(self._fn("keys")(self._h), (m, self.pd)).copy()

    def values(self):
        m = self.num_vertices
        return np.ctypeslib.as_array(self._fn("values")(self._h), (m, self.vd)).copy()

    def replay(self):
        shape = (self.n, self.pd + 1)
        return (np.ctypeslib.as_array(self._fn("replay_vertex")(self._h), shape).copy(),
                np.ctypeslib.as_array(self._fn("replay_weight")(self._h), shape).copy())

    def stage_seconds(self):
        s = [C.c_double() for _ in range(3)]
        self._fn("stage_seconds")(self._h, *[C.byref(x) for x in s])
        return dict(splat=s[0].value, blur=s[1].value, slice=s[2].value)


def lattice_filter(input_image, reference_image, bilateral=True, theta_alpha=1.0, theta_beta=1.0,
                   theta_gamma=1.0, reverse=False):
    """The LatticeFilter op on channels-last arrays [B, s_1..s_k, C]; float64 input selects
    T = double, anything else T = float."""
    dtype = np.float64 if np.asarray(input_image).dtype == np.float64 else np.float32
    inp = np.ascontiguousarray(input_image, dtype)
    sd = np.ascontiguousarray(inp.shape[1:-1], np.int32)
    ref = None
    rc = 0
    if reference_image is not None:
        ref = np.ascontiguousarray(reference_image, dtype)
        rc = ref.shape[-1]
    out = np.empty_like(inp)
    rcode = _fn("lattice_filter_op", dtype)(inp, _opt(ref), out, inp.shape[0], len(sd), sd,
                                       inp.shape[-1], rc, int(bilateral), theta_alpha,
                                       theta_beta, theta_gamma, int(reverse))
    if rcode != 0:
        raise ValueError("plo_lattice_filter_op: bad arguments")
    return out


def _softmax(z):
    z = np.asarray(z, np.float64)
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)


def mean_field(logits, guide, iterations=5, theta_alpha=80.0, theta_beta=13.0, theta_gamma=3.0,
               upstream=None, op=None):
    """CPU twin of permutohedral_lattice_amd.crf.MeanField, for checking it: Q <- softmax(logits +
    bilateral(Q) + spatial(Q)) `iterations` times on channels-last arrays [B, s_1..s_k, C], every
    message a fresh lattice_filter call as the reference's op would make it; with `upstream` also
    the reverse pass, bilateral_reverse(upstream) + spatial_reverse(upstream).  `op`: the
    lattice_filter to use (default this module's; pass reference().lattice_filter for the
    reference's own header).  -> (Q, reverse or None)"""
    op = op or lattice_filter
    logits = np.ascontiguousarray(logits, np.float32)
    guide = np.ascontiguousarray(guide, np.float32)

    def messages(q, reverse):
        return (op(q, guide, True, theta_alpha, theta_beta, theta_gamma, reverse)
                + op(q, guide, False, theta_alpha, theta_beta, theta_gamma, reverse))

    q = _softmax(logits)
    for _ in range(iterations):
        q = _softmax(logits.astype(np.float64) + messages(q, False))
    rev = None if upstream is None else messages(np.ascontiguousarray(upstream, np.float32), True)
    return q, rev


# ---------------------------------------------------------------------------------------------
# The reference's own CPU header behind C entry points (present only after `make -C oracle ref`)
# ---------------------------------------------------------------------------------------------

def have_reference():
    return os.path.exists(_REF_PATH)


class _Ref:
    def __init__(self):
        lib = C.CDLL(_REF_PATH)
        for sfx, npt, ct in _variants():
            fp = np.ctypeslib.ndpointer(npt, flags="C_CONTIGUOUS")

            def fn(name):
                return getattr(lib, "plref_" + name + sfx)
            fn("scale_factor").argtypes = [C.c_int, fp]
            fn("dump_simplex").argtypes = [C.c_int, C.c_int, fp] + [C.c_void_p] * 5
            fn("compute_positions").argtypes = [C.c_void_p, fp, C.c_int, C.c_int, C.c_int, _i32p,
                                                ct, ct]
            fn("filter").argtypes = [C.c_int, C.c_int, C.c_int, fp, fp, fp, C.c_int,
                                     C.POINTER(C.c_int), C.c_void_p, C.POINTER(C.c_double)]
            fn("filter_stages").argtypes = [C.c_int, C.c_int, C.c_int, fp, fp, fp, C.c_int,
                                            C.POINTER(C.c_int), C.c_void_p, C.c_void_p, C.c_void_p]
            fn("filter_replay").argtypes = [C.c_int, C.c_int, C.c_int, fp, fp, fp, C.c_int,
                                            C.POINTER(C.c_int), C.c_void_p, C.c_void_p, C.c_void_p]
            fn("lattice_filter_op").argtypes = [fp, C.c_void_p, fp, C.c_int, C.c_int, _i32p,
                                                C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                                                C.c_float, C.c_int]
        self.lib = lib

    def _fn(self, name, dtype):
        return getattr(self.lib, "plref_" + name + _suffix(dtype))

    def scale_factor(self, pd, dtype=np.float32):
        out = np.empty(pd, dtype)
        self._fn("scale_factor", dtype)(pd, out)
        return out

    def dump_simplex(self, positions, dtype=np.float32):
        positions = np.ascontiguousarray(positions, dtype)
        n, pd = positions.shape
        d1 = pd + 1
        out = dict(rem0=np.empty((n, d1), np.int16), rank=np.empty((n, d1), np.int16),
                   keys=np.empty((n, d1, pd), np.int16),
                   barycentric=np.empty((n, d1), dtype),
                   elevated=np.empty((n, d1), dtype))
        self._fn("dump_simplex", dtype)(pd, n, positions, _opt(out["rem0"]), _opt(out["rank"]),
                                        _opt(out["keys"]), _opt(out["barycentric"]),
                                        _opt(out["elevated"]))
        return out

    def compute_positions(self, reference, spatial_dims, spatial_std, feature_std,
                          n_reference_channels, dtype=np.float32):
        sd = np.ascontiguousarray(spatial_dims, np.int32)
        n = int(np.prod(sd))
        pos = np.empty((n, len(sd) + n_reference_channels), dtype)
        ref = None
        if n_reference_channels:
            ref = np.ascontiguousarray(reference, dtype).reshape(n, n_reference_channels)
        self._fn("compute_positions", dtype)(_opt(ref), pos, n, n_reference_channels, len(sd), sd,
                                             float(spatial_std), float(feature_std))
        return pos

    def filter(self, pd, vd, inp, positions, reverse=False, dtype=np.float32):
        """-> (output, M, keys [M, pd], seconds)"""
        inp = np.ascontiguousarray(inp, dtype)
        n = inp.size // (vd - 1)
        inp = inp.reshape(n, vd - 1)
        positions = np.ascontiguousarray(positions, dtype).reshape(n, pd)
        out = np.empty_like(inp)
        m = C.c_int()
        sec = C.c_double()
        keys = np.empty((n * (pd + 1), pd), np.int16)
        self._fn("filter", dtype)(pd, vd, n, out, inp, positions, int(reverse), C.byref(m),
                                  _opt(keys), C.byref(sec))
        return out, m.value, keys[:m.value].copy(), sec.value

    def filter_stages(self, pd, vd, inp, positions, reverse=False, want_values=True,
                      dtype=np.float32):
        """-> dict(output, M, after_splat [M,vd], after_blur [M,vd], seconds{splat,blur,slice})"""
        inp = np.ascontiguousarray(inp, dtype)
        n = inp.size // (vd - 1)
        inp = inp.reshape(n, vd - 1)
        positions = np.ascontiguousarray(positions, dtype).reshape(n, pd)
        out = np.empty_like(inp)
        m = C.c_int()
        a = np.empty((n * (pd + 1), vd), dtype) if want_values else None
        b = np.empty((n * (pd + 1), vd), dtype) if want_values else None
        sec = np.zeros(3, np.float64)
        self._fn("filter_stages", dtype)(pd, vd, n, out, inp, positions, int(reverse),
                                         C.byref(m), _opt(a), _opt(b), _opt(sec))
        res = dict(output=out, M=m.value,
                   seconds=dict(splat=sec[0], blur=sec[1], slice=sec[2]))
        if want_values:
            res["after_splat"] = a[:m.value].copy()
            res["after_blur"] = b[:m.value].copy()
        return res

    def filter_replay(self, pd, vd, inp, positions, reverse=False, dtype=np.float32):
        """-> dict(output, M, keys [M, pd] in first-touch order, replay_vertex [N, pd+1],
        replay_weight [N, pd+1]): one filter call and the rows its slice replayed."""
        inp = np.ascontiguousarray(inp, dtype)
        n = inp.size // (vd - 1)
        inp = inp.reshape(n, vd - 1)
        positions = np.ascontiguousarray(positions, dtype).reshape(n, pd)
        out = np.empty_like(inp)
        m = C.c_int()
        keys = np.empty((n * (pd + 1), pd), np.int16)
        vertex = np.empty((n, pd + 1), np.int32)
        weight = np.empty((n, pd + 1), dtype)
        self._fn("filter_replay", dtype)(pd, vd, n, out, inp, positions, int(reverse), C.byref(m),
                                         _opt(keys), _opt(vertex), _opt(weight))
        return dict(output=out, M=m.value, keys=keys[:m.value].copy(), replay_vertex=vertex,
                    replay_weight=weight)

    def lattice_filter(self, input_image, reference_image, bilateral=True, theta_alpha=1.0,
                       theta_beta=1.0, theta_gamma=1.0, reverse=False):
        dtype = np.float64 if np.asarray(input_image).dtype == np.float64 else np.float32
        inp = np.ascontiguousarray(input_image, dtype)
        sd = np.ascontiguousarray(inp.shape[1:-1], np.int32)
        ref = np.ascontiguousarray(reference_image, dtype)
        out = np.empty_like(inp)
        self._fn("lattice_filter_op", dtype)(inp, _opt(ref), out, inp.shape[0], len(sd), sd,
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
