"""ctypes loader for the CPU checker (test infrastructure; never imported by the
shipped package).  Builds oracle/liboracle.so with g++ when it is missing."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


class OrcParams(ctypes.Structure):
    _fields_ = [
        ("objective", ctypes.c_int),
        ("depth", ctypes.c_int),
        ("min_child_weight", ctypes.c_float),
        ("min_leaf_size", ctypes.c_uint),
        ("gamma_absolute", ctypes.c_float),
        ("gamma_relative", ctypes.c_float),
        ("lambda_", ctypes.c_float),
        ("alpha", ctypes.c_float),
        ("initial_y", ctypes.c_float),
        ("eta", ctypes.c_float),
        ("max_leaf_weight", ctypes.c_float),
        ("hist_size", ctypes.c_int),
        ("double_precision", ctypes.c_int),
        ("accum", ctypes.c_int),
        ("use_trick", ctypes.c_int),
        ("labels_count", ctypes.c_int),
        ("threads", ctypes.c_int),
        ("colsample_bytree", ctypes.c_float),
        ("colsample_bylevel", ctypes.c_float),
        ("seed", ctypes.c_uint),
        ("method", ctypes.c_int),
    ]


def build(force=False):
    src = os.path.join(_HERE, "arboretum_oracle.cpp")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.orc_expf.restype = ctypes.c_float
        L.orc_expf.argtypes = [ctypes.c_float]
        L.orc_sigmoid.restype = ctypes.c_float
        L.orc_sigmoid.argtypes = [ctypes.c_float]
        L.orc_quantize_column.restype = ctypes.c_int
        L.orc_quantize_column.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
                                          ctypes.c_void_p]
        L.orc_gain.restype = ctypes.c_float
        L.orc_gain.argtypes = [ctypes.c_int, ctypes.c_double, ctypes.c_double, ctypes.c_uint64,
                               ctypes.c_double, ctypes.c_double, ctypes.c_uint64, ctypes.c_uint,
                               ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                               ctypes.c_float, ctypes.c_float]
        L.orc_weight.restype = ctypes.c_float
        L.orc_weight.argtypes = [ctypes.c_int, ctypes.c_double, ctypes.c_double, ctypes.c_uint,
                                 ctypes.c_uint, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                 ctypes.c_float]
        L.orc_fix_shift.restype = ctypes.c_int
        L.orc_fix_shift.argtypes = [ctypes.c_float]
        L.orc_to_fixed.restype = ctypes.c_int64
        L.orc_to_fixed.argtypes = [ctypes.c_float, ctypes.c_int]
        L.orc_hist_fixed_u8.restype = None
        L.orc_hist_fixed_u8.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p]
        L.orc_create.restype = ctypes.c_void_p
        L.orc_create.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
                                 ctypes.c_void_p, ctypes.POINTER(OrcParams)]
        L.orc_create_binned.restype = ctypes.c_void_p
        L.orc_create_binned.argtypes = L.orc_create.argtypes
        L.orc_free.argtypes = [ctypes.c_void_p]
        L.orc_grow_round.restype = ctypes.c_char_p
        L.orc_grow_round.argtypes = [ctypes.c_void_p]
        L.orc_get_active.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        L.orc_hist_size.argtypes = [ctypes.c_void_p]
        L.orc_num_trees.argtypes = [ctypes.c_void_p]
        L.orc_updates.restype = ctypes.c_uint64
        L.orc_updates.argtypes = [ctypes.c_void_p]
        L.orc_get_tree.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5
        L.orc_get_leaf.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.orc_get_yhat.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.orc_get_grad.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        L.orc_force_wide_ranks.argtypes = [ctypes.c_int]
        L.orc_get_bins.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        L.orc_get_thresholds.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                         ctypes.POINTER(ctypes.c_int)]
        L.orc_get_shifts.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int),
                                     ctypes.POINTER(ctypes.c_int)]
        L.orc_get_level_hist.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        L.orc_predict.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                                  ctypes.c_void_p]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def params_from_config(config, accum=0, threads=0):
    """Maps the reference's JSON configuration (src/core/json_conversion.h:55-167,
    defaults src/core/param.h:21-57) to OrcParams."""
    t = config.get("tree", {})
    it = config.get("internals", {})
    return OrcParams(
        objective=int(config.get("objective", 0)),
        depth=int(t.get("max_depth", 7)) + 1,
        min_child_weight=float(t.get("min_child_weight", 1.0)),
        min_leaf_size=int(t.get("min_leaf_size", 1)),
        gamma_absolute=float(t.get("gamma_absolute", 0.0)),
        gamma_relative=float(t.get("gamma_relative", 0.0)),
        lambda_=float(t.get("lambda", 1.0)),
        alpha=float(t.get("alpha", 0.0)),
        initial_y=float(t.get("initial_y", 0.5)),
        eta=float(t.get("eta", 0.3)),
        max_leaf_weight=float(t.get("max_leaf_weight", 0.0)),
        hist_size=int(it.get("hist_size", 255)),
        double_precision=int(bool(it.get("double_precision", False))),
        accum=accum,
        use_trick=int(bool(it.get("use_hist_subtraction_trick", True))),
        labels_count=int(t.get("labels_count", 1)),
        threads=threads,
        colsample_bytree=float(t.get("colsample_bytree", 1.0)),
        colsample_bylevel=float(t.get("colsample_bylevel", 1.0)),
        seed=int(it.get("seed", 0)),
        method=int(config.get("method", 1)),
    )


def force_wide_ranks(on):
    """Test switch: exact-mode boosters created from now on keep 32-bit ranks (the branch of more
    than 65535 distinct values per feature)."""
    lib().orc_force_wide_ranks(1 if on else 0)


def quantize_column(x, hist_size):
    x = np.ascontiguousarray(x, dtype=np.float32)
    thr = np.empty(hist_size, dtype=np.float32)
    bins = np.empty(x.size, dtype=np.uint16)
    size = lib().orc_quantize_column(_p(x), x.size, hist_size, _p(thr), _p(bins))
    return thr, bins, size


def hist_fixed_u8(bins, g, h, shift_g, shift_h, sel=None, n_features=None):
    bins = np.ascontiguousarray(bins, dtype=np.uint8)
    n, stride = bins.shape
    F = n_features or stride
    g = np.ascontiguousarray(g, dtype=np.float32)
    h = None if h is None else np.ascontiguousarray(h, dtype=np.float32)
    sel = None if sel is None else np.ascontiguousarray(sel, dtype=np.uint8)
    out = np.zeros((F, 256, 3), dtype=np.int64)
    lib().orc_hist_fixed_u8(_p(bins), n, F, stride, _p(g), _p(h), shift_g, shift_h, _p(sel), _p(out))
    return out


class Booster:
    def __init__(self, X, y=None, labels=None, config=None, accum=0, threads=0, binned=False):
        self.params = params_from_config(config, accum, threads)
        self.n, self.F = X.shape
        y = None if y is None else np.ascontiguousarray(y, dtype=np.float32)
        labels = None if labels is None else np.ascontiguousarray(labels, dtype=np.uint8)
        if binned:
            X = np.ascontiguousarray(X, dtype=np.uint8)
            self.h = lib().orc_create_binned(_p(X), self.n, self.F, _p(y), _p(labels),
                                             ctypes.byref(self.params))
        else:
            X = np.ascontiguousarray(X, dtype=np.float32)
            self.h = lib().orc_create(_p(X), self.n, self.F, _p(y), _p(labels),
                                      ctypes.byref(self.params))
        if not self.h:
            raise ValueError("the checker could not take the matrix")
        self.K = self.params.labels_count
        self.params.hist_size = lib().orc_hist_size(self.h)   # exact method: the largest number of distinct values

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_free(self.h)
            self.h = None

    def grow(self, rounds=1):
        for _ in range(rounds):
            err = lib().orc_grow_round(self.h)
            if err is not None:      # the literal the reference throws (garden.cu:127-140)
                raise ValueError(err.decode())

    def active_features(self, t, level):
        """Feature ids tree `t` may split on at `level` (garden.cu:162-165, 252-253)."""
        n = lib().orc_get_active(self.h, t, level, None)
        if n < 0:
            raise IndexError((t, level))
        out = np.empty(n, np.uint32)
        lib().orc_get_active(self.h, t, level, _p(out))
        return out

    @property
    def num_trees(self):
        return lib().orc_num_trees(self.h)

    @property
    def updates(self):
        return lib().orc_updates(self.h)

    def tree(self, t):
        D = self.params.depth
        ni, nl = (1 << (D - 1)) - 1, 1 << (D - 1)
        fid = np.empty(ni, np.int32)
        q = np.empty(ni, np.int32)
        thr = np.empty(ni, np.float32)
        gain = np.empty(ni, np.float32)
        w = np.empty(nl, np.float32)
        lib().orc_get_tree(self.h, t, _p(fid), _p(q), _p(thr), _p(gain), _p(w))
        return {"fid": fid, "quantized": q, "threshold": thr, "gain": gain, "weights": w}

    def leaf(self):
        out = np.empty(self.n, np.uint32)
        lib().orc_get_leaf(self.h, _p(out))
        return out

    def yhat(self):
        out = np.empty(self.n * self.K, np.float32)
        lib().orc_get_yhat(self.h, _p(out))
        return out

    def grad(self):
        g = np.empty(self.n * self.K, np.float32)
        h = np.empty(self.n * self.K, np.float32)
        lib().orc_get_grad(self.h, _p(g), _p(h))
        return g, h

    def bins(self):
        if self.params.hist_size > 65535:
            raise ValueError("ranks beyond 16 bits (exact mode, more than 65535 distinct values) are not handed out")
        out = np.empty((self.n, self.F), np.uint16)
        lib().orc_get_bins(self.h, _p(out))
        return out

    def thresholds(self, f):
        thr = np.empty(self.params.hist_size, np.float32)
        size = ctypes.c_int()
        lib().orc_get_thresholds(self.h, f, _p(thr), ctypes.byref(size))
        return thr, size.value

    def shifts(self):
        a, b = ctypes.c_int(), ctypes.c_int()
        lib().orc_get_shifts(self.h, ctypes.byref(a), ctypes.byref(b))
        return a.value, b.value

    def level_hist(self, level, mode=0):
        L = 1 << level
        slots = self.params.hist_size + 1
        out = np.empty((L, self.F, slots, 3), np.int64 if mode == 0 else np.float64)
        r = lib().orc_get_level_hist(self.h, level, mode, _p(out))
        assert r == L * self.F * slots
        return out

    def predict(self, X, n_rounds=-1):
        X = np.ascontiguousarray(X, dtype=np.float32)
        out = np.empty(X.shape[0] * self.K, np.float32)
        lib().orc_predict(self.h, _p(X), X.shape[0], n_rounds, _p(out))
        return out if self.K == 1 else out.reshape(X.shape[0], self.K)

    def model_dict(self):
        """Model in the reference's JSON layout (src/core/json_conversion.h:13-40)."""
        D = self.params.depth
        ni = (1 << (D - 1)) - 1
        trees = []
        for t in range(self.num_trees):
            tr = self.tree(t)
            nodes = []
            for i in range((1 << D) - 1):
                if i < ni:
                    thr = float(tr["threshold"][i])
                    nodes.append({"id": i, "leaf": False, "left": 2 * i + 1, "right": 2 * i + 2,
                                  "threshold": None if np.isinf(thr) else thr, "fid": int(tr["fid"][i])})
                else:
                    nodes.append({"id": i, "leaf": True, "idx": i - ni})
            trees.append({"nodes": nodes, "weights": [float(w) for w in tr["weights"]], "depth": D})
        return {"model": trees}
