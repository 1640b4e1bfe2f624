"""Python face of libarboretum.so: the `DMatrix` / `Garden` / `train` / `load`
API and the scikit-learn style estimators of the reference's package
(python-package/arboretum/core.py:51-339, 342-732), over the same ctypes
boundary (core.py:21-48).  Everything here is marshalling; the work happens in
the shared library (host C++ and HIP kernels)."""
import ctypes
import json
import os

import numpy as np


class ArboretumError(Exception):
    pass


def _load_lib():
    here = os.path.dirname(os.path.abspath(os.path.expanduser(__file__)))
    path = os.path.join(here, "libarboretum.so")
    if not os.path.exists(path):
        raise ArboretumError(
            "libarboretum.so is not built: run `python arboretum_amd/build.py` (needs hipcc)")
    lib = ctypes.cdll.LoadLibrary(path)
    c_char_p, c_void_p, c_int, c_float = ctypes.c_char_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    P = ctypes.POINTER
    sigs = {
        # reference boundary (python-wrapper/arboretum_wrapper.h:6-39)
        "ACreateFromDenseMatrix": [P(c_float), P(ctypes.c_uint), c_int, c_int, c_int, c_float, P(c_void_p)],
        "ASetY": [c_void_p, P(c_float)],
        "ASetLabel": [c_void_p, P(ctypes.c_ubyte)],
        "ASetWeights": [c_void_p, P(c_float)],
        "AInitGarden": [c_char_p, P(c_void_p)],
        "AGrowTree": [c_void_p, c_void_p, c_void_p],
        "AAppendLastTree": [c_void_p, c_void_p],
        "AGetY": [c_void_p, c_void_p, P(P(c_float))],
        "APredict": [c_void_p, c_void_p, P(P(c_float)), c_int],
        "ADumpModel": [P(c_char_p), c_void_p],
        "ALoadModel": [c_char_p, c_void_p],
        "AFreeDMatrix": [c_void_p],
        "AFreeGarden": [c_void_p],
        "ADeleteArray": [P(c_float)],
        # extensions (include/arboretum_ext.h)
        "ADeviceCount": [P(c_int)],
        "ADeviceCopyProbe": [ctypes.c_ulonglong],
        "ACreateFromQuantized": [c_void_p, ctypes.c_longlong, c_int, P(c_void_p)],
        "ACreateFromQuantizedBlocks": [c_void_p, c_int, ctypes.c_longlong, ctypes.c_longlong, c_int, P(c_void_p)],
        "AQuantize": [c_void_p, c_int],
        "AGetBins": [c_void_p, c_void_p],
        "AGetBins16": [c_void_p, c_void_p],
        "AGetBinLayout": [c_void_p, P(c_int), P(c_int)],
        "AGetThresholds": [c_void_p, c_int, c_void_p, P(c_int)],
        "AGardenSetInspect": [c_void_p, c_int],
        "AGardenPredictOnDevice": [c_void_p, c_int],
        "AGardenNumTrees": [c_void_p, P(c_int)],
        "AGardenGetTree": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
        "AGardenGetTreeDepth": [c_void_p, c_int, P(c_int)],
        "AGardenGetLeaves": [c_void_p, c_void_p],
        "AGardenGetTrainYHat": [c_void_p, c_void_p],
        "AGardenGetGrad": [c_void_p, c_void_p, c_void_p],
        "AGardenGetLevelHist": [c_void_p, c_int, c_void_p, P(c_int)],
        "AGardenGetShifts": [c_void_p, P(c_int), P(c_int)],
        "AGardenEnableTiming": [c_void_p, c_int],
        "AGardenGetTimings": [c_void_p, c_void_p],
        "AGardenRowsScanned": [c_void_p, P(ctypes.c_ulonglong)],
        "AGardenRowsScannedByLevel": [c_void_p, c_void_p],
        "AGardenStreamResidency": [c_void_p, P(ctypes.c_ulonglong), P(ctypes.c_ulonglong)],
        "AGardenSynchronize": [c_void_p],
        "AHistSum": [c_void_p] * 10 + [ctypes.c_ulonglong, ctypes.c_longlong, c_int, c_int, c_int, c_int, c_int,
                                       c_void_p],
        "AHistSumPlan": [ctypes.c_longlong, c_int, P(ctypes.c_uint), P(ctypes.c_uint)],
        "AHistSumNoAlloc": [c_void_p] * 10 + [ctypes.c_ulonglong, ctypes.c_longlong, c_int, c_int, c_int, c_int,
                                              c_int, c_void_p, c_void_p],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.restype = c_char_p
        fn.argtypes = args
    return lib


_LIB = _load_lib()


def _check(ret):
    if ret is not None:
        raise ArboretumError(ValueError(ret.decode("utf-8", "replace")))


def device_count():
    n = ctypes.c_int(0)
    _check(_LIB.ADeviceCount(ctypes.byref(n)))
    return n.value


def copy_probe(nbytes):
    """One device-to-device copy kernel of known size (profile calibration)."""
    _check(_LIB.ADeviceCopyProbe(int(nbytes)))


def hist_sum(sum_g, sum_h, bin_count, grad, hess, node_size, bins, stride, nrow, ncol, nodes, shift_g,
             shift_h=0, use_trick=False, parent_g=None, parent_h=None, parent_c=None, stream=None):
    """Histogram sums of node segments for data that lives on the GPU (AHistSum; the
    reference's HistTreeGrower::HistSum over every feature at once).  Every array argument
    is a DEVICE address (an int, e.g. `tensor.data_ptr()`), or None."""
    _check(_LIB.AHistSum(sum_g, sum_h, bin_count, parent_g, parent_h, parent_c, grad, hess, node_size, bins,
                         int(stride), int(nrow), int(ncol), int(nodes), int(bool(use_trick)), int(shift_g),
                         int(shift_h), stream))


def hist_sum_plan(nrow, nodes):
    """(rows per work item, work items) of the plan hist_sum makes (AHistSumPlan; no GPU needed)."""
    a, b = ctypes.c_uint(), ctypes.c_uint()
    _check(_LIB.AHistSumPlan(int(nrow), int(nodes), ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def hist_sum_no_alloc(sum_g, sum_h, bin_count, grad, hess, node_size, bins, stride, nrow, ncol, nodes, shift_g,
                      shift_h=0, use_trick=False, parent_g=None, parent_h=None, parent_c=None, stream=None,
                      status=None):
    """hist_sum without any device allocation (AHistSumNoAlloc): static work memory, limited
    sizes, enqueues on `stream` and returns without waiting; `status` is an optional device word."""
    _check(_LIB.AHistSumNoAlloc(sum_g, sum_h, bin_count, parent_g, parent_h, parent_c, grad, hess, node_size,
                                bins, int(stride), int(nrow), int(ncol), int(nodes), int(bool(use_trick)),
                                int(shift_g), int(shift_h), stream, status))


def _fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


class DMatrix(object):
    """Data matrix (core.py:51-120 of the reference).  `quantized=True` takes
    `data` as uint8 bin ids instead of floats (extension)."""

    def __init__(self, data, data_category=None, y=None, labels=None, weights=None, missing=0.0,
                 quantized=False):
        self.handle = None
        self.labels_count = 1
        if len(data.shape) != 2:
            raise ValueError('Input numpy.ndarray must be 2 dimensional')
        self.rows = data.shape[0]
        self.columns = data.shape[1]
        handle = ctypes.c_void_p()
        if quantized:
            bins = np.ascontiguousarray(data, dtype=np.uint8)
            _check(_LIB.ACreateFromQuantized(bins.ctypes.data_as(ctypes.c_void_p), self.rows, self.columns,
                                             ctypes.byref(handle)))
        else:
            if data_category is not None and not np.issubdtype(data_category.dtype, np.integer):
                raise ValueError("Category's type must be int like")
            flat = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
            cat, ccol = None, 0
            if data_category is not None:
                ccol = data_category.shape[1]
                cat = np.ascontiguousarray(data_category, dtype=np.uint32).reshape(-1)
            _check(_LIB.ACreateFromDenseMatrix(
                _fptr(flat), None if cat is None else cat.ctypes.data_as(ctypes.POINTER(ctypes.c_uint)),
                self.rows, self.columns, ccol, float(missing), ctypes.byref(handle)))
        self.handle = handle
        if y is not None and labels is not None:
            raise ValueError(
                'y and labels both are not None. Specify labels only for multi label classification')
        if y is not None:
            assert self.rows == len(y)
            yy = np.ascontiguousarray(np.asarray(y).reshape(self.rows), dtype=np.float32)
            _check(_LIB.ASetY(self.handle, _fptr(yy)))
        elif labels is not None:
            assert self.rows == len(labels)
            self.labels_count = int(np.max(labels)) + 1
            ll = np.ascontiguousarray(np.asarray(labels).reshape(self.rows), dtype=np.uint8)
            _check(_LIB.ASetLabel(self.handle, ll.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte))))
        if weights is not None:
            assert weights.shape[0] == self.rows and weights.size == self.rows
            ww = np.ascontiguousarray(weights.reshape(self.rows), dtype=np.float32)
            _check(_LIB.ASetWeights(self.handle, _fptr(ww)))

    def __del__(self):
        if getattr(self, "handle", None):
            _LIB.AFreeDMatrix(self.handle)
            self.handle = None

    # ---- extensions
    @classmethod
    def from_blocks(cls, block_addresses, block_rows, rows, columns, y=None, labels=None):
        """Matrix over bin ids that stay in caller-owned host blocks (ACreateFromQuantizedBlocks): for
        matrices beyond HBM and beyond 2^31 rows.  block_addresses: host addresses (ints) of the
        blocks, each 32-bit words [ceil(columns / 4)][block_rows]; the caller keeps them alive.
        Train with internals.upload_features = False."""
        self = cls.__new__(cls)
        self.handle = None
        self.labels_count = 1
        self.rows, self.columns = int(rows), int(columns)
        ptrs = (ctypes.c_void_p * len(block_addresses))(*[int(a) for a in block_addresses])
        handle = ctypes.c_void_p()
        _check(_LIB.ACreateFromQuantizedBlocks(ptrs, len(block_addresses), int(block_rows), self.rows, self.columns,
                                               ctypes.byref(handle)))
        self.handle = handle
        if y is not None:
            assert self.rows == len(y)
            yy = np.ascontiguousarray(np.asarray(y).reshape(self.rows), dtype=np.float32)
            _check(_LIB.ASetY(self.handle, _fptr(yy)))
        elif labels is not None:
            assert self.rows == len(labels)
            self.labels_count = int(np.max(labels)) + 1
            ll = np.ascontiguousarray(np.asarray(labels).reshape(self.rows), dtype=np.uint8)
            _check(_LIB.ASetLabel(self.handle, ll.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte))))
        return self

    def quantize(self, hist_size):
        _check(_LIB.AQuantize(self.handle, int(hist_size)))

    def bin_layout(self):
        """(bits per bin id, histogram slots per feature) of the quantised matrix."""
        bits, slots = ctypes.c_int(), ctypes.c_int()
        _check(_LIB.AGetBinLayout(self.handle, ctypes.byref(bits), ctypes.byref(slots)))
        return bits.value, slots.value

    def bins(self):
        bits, slots = self.bin_layout()
        if bits == 16 or slots > 256:      # ids above 255: 16-bit ids, or bytes with a ninth bit
            out = np.empty((self.rows, self.columns), dtype=np.uint16)
            _check(_LIB.AGetBins16(self.handle, out.ctypes.data_as(ctypes.c_void_p)))
            return out
        out = np.empty((self.rows, self.columns), dtype=np.uint8)
        _check(_LIB.AGetBins(self.handle, out.ctypes.data_as(ctypes.c_void_p)))
        return out

    def thresholds(self, fid, hist_size):
        thr = np.empty(hist_size, dtype=np.float32)
        size = ctypes.c_int()
        _check(_LIB.AGetThresholds(self.handle, fid, thr.ctypes.data_as(ctypes.c_void_p), ctypes.byref(size)))
        return thr, size.value


class Garden(object):
    """Low level booster object (core.py:123-294 of the reference)."""

    def __init__(self, config, data=None):
        self.handle = None
        self.config = config
        self.data = data
        self._init = False
        self.labels_count = config.get('tree', {}).get('labels_count', 1)
        self.config_str = json.dumps(config)

    def __del__(self):
        if getattr(self, "handle", None):
            _LIB.AFreeGarden(self.handle)
            self.handle = None
        if hasattr(self, 'data'):
            del self.data

    def _ensure(self):
        if not self._init:
            handle = ctypes.c_void_p()
            _check(_LIB.AInitGarden(self.config_str.encode('UTF-8'), ctypes.byref(handle)))
            self.handle = handle
            self._init = True

    def load(self, json_model_str):
        self._init = False
        if self.handle:
            _LIB.AFreeGarden(self.handle)
            self.handle = None
        self._ensure()
        _check(_LIB.ALoadModel(json_model_str.encode('UTF-8'), self.handle))

    def grow_tree(self, grad=None):
        self._ensure()
        if grad is not None:
            assert len(grad) == self.data.rows
            g = np.ascontiguousarray(np.asarray(grad).reshape(self.data.rows), dtype=np.float32)
            _check(_LIB.AGrowTree(self.handle, self.data.handle, g.ctypes.data_as(ctypes.c_void_p)))
        else:
            _check(_LIB.AGrowTree(self.handle, self.data.handle, None))

    def append_last_tree(self, data):
        self._ensure()
        _check(_LIB.AAppendLastTree(self.handle, data.handle))

    def _take(self, preds, length):
        shape = (length,) if self.labels_count == 1 else (length, self.labels_count)
        res = np.copy(np.ctypeslib.as_array(preds, shape=shape))
        _check(_LIB.ADeleteArray(preds))
        return res

    def get_y(self, data):
        self._ensure()
        preds = ctypes.POINTER(ctypes.c_float)()
        _check(_LIB.AGetY(self.handle, data.handle, ctypes.byref(preds)))
        return self._take(preds, int(data.rows))

    def predict(self, data, n_rounds=-1):
        self._ensure()
        preds = ctypes.POINTER(ctypes.c_float)()
        _check(_LIB.APredict(self.handle, data.handle, ctypes.byref(preds), int(n_rounds)))
        return self._take(preds, int(data.rows))

    def dump(self):
        self._ensure()
        json_p = ctypes.c_char_p()
        _check(_LIB.ADumpModel(ctypes.byref(json_p), self.handle))
        return json_p.value.decode('utf-8')

    # ---- extensions (include/arboretum_ext.h)
    def predict_on_device(self, on=True):
        """Tree walks of predict() on the GPU (default) or on the host; the results are bit-identical."""
        self._ensure()
        _check(_LIB.AGardenPredictOnDevice(self.handle, int(on)))

    def set_inspect(self, on=True):
        self._ensure()
        _check(_LIB.AGardenSetInspect(self.handle, int(on)))

    def enable_timing(self, level=1):
        """0: off; 1: every phase; 2: only the deeper-level histogram kernels; 3: those on every fourth tree."""
        self._ensure()
        _check(_LIB.AGardenEnableTiming(self.handle, int(level)))

    def timings(self):
        out = np.zeros(16, dtype=np.float64)
        _check(_LIB.AGardenGetTimings(self.handle, out.ctypes.data_as(ctypes.c_void_p)))
        keys = ["grad_ms", "hist_root_ms", "hist_deep_ms", "reduce_ms", "split_ms", "partition_ms", "leaf_ms",
                "plan_ms", "hist_root_launches", "hist_root_rows", "hist_deep_launches", "fused_last_ms",
                "fused_last_launches"]
        return dict(zip(keys, out.tolist()))

    def rows_scanned(self):
        v = ctypes.c_ulonglong()
        _check(_LIB.AGardenRowsScanned(self.handle, ctypes.byref(v)))
        return v.value

    def stream_residency(self):
        """(row blocks kept in device memory, row blocks) of a streamed matrix; (0, 0) otherwise."""
        a, b = ctypes.c_ulonglong(), ctypes.c_ulonglong()
        _check(_LIB.AGardenStreamResidency(self.handle, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def rows_scanned_by_level(self):
        """Rows accumulated into histograms so far, per tree level (root = 0)."""
        out = np.zeros(32, dtype=np.uint64)
        _check(_LIB.AGardenRowsScannedByLevel(self.handle, out.ctypes.data_as(ctypes.c_void_p)))
        return out

    def synchronize(self):
        _check(_LIB.AGardenSynchronize(self.handle))

    def num_trees(self):
        n = ctypes.c_int()
        _check(_LIB.AGardenNumTrees(self.handle, ctypes.byref(n)))
        return n.value

    def tree(self, t):
        # a loaded model's trees carry their own depth, which need not be the configuration's
        d = ctypes.c_int(0)
        _check(_LIB.AGardenGetTreeDepth(self.handle, t, ctypes.byref(d)))
        depth = d.value
        ni, nl = (1 << (depth - 1)) - 1, 1 << (depth - 1)
        fid, q = np.empty(ni, np.int32), np.empty(ni, np.int32)
        thr, gain, w = np.empty(ni, np.float32), np.empty(ni, np.float32), np.empty(nl, np.float32)
        vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
        _check(_LIB.AGardenGetTree(self.handle, t, vp(fid), vp(q), vp(thr), vp(gain), vp(w)))
        return {"fid": fid, "quantized": q, "threshold": thr, "gain": gain, "weights": w}

    def leaves(self):
        out = np.empty(self.data.rows, dtype=np.uint32)
        _check(_LIB.AGardenGetLeaves(self.handle, out.ctypes.data_as(ctypes.c_void_p)))
        return out

    def train_yhat(self):
        out = np.empty(self.data.rows * self.labels_count, dtype=np.float32)
        _check(_LIB.AGardenGetTrainYHat(self.handle, out.ctypes.data_as(ctypes.c_void_p)))
        return out

    def grad(self):
        g = np.empty(self.data.rows * self.labels_count, dtype=np.float32)
        h = np.empty_like(g)
        _check(_LIB.AGardenGetGrad(self.handle, g.ctypes.data_as(ctypes.c_void_p), h.ctypes.data_as(ctypes.c_void_p)))
        return g, h

    def level_hist(self, level):
        nodes = 1 << level
        slots = self.data.bin_layout()[1]
        out = np.empty((nodes, self.data.columns, slots, 3), dtype=np.int64)
        cells = ctypes.c_int()
        _check(_LIB.AGardenGetLevelHist(self.handle, level, out.ctypes.data_as(ctypes.c_void_p), ctypes.byref(cells)))
        assert cells.value == nodes * self.data.columns * slots
        return out

    def shifts(self):
        a, b = ctypes.c_int(), ctypes.c_int()
        _check(_LIB.AGardenGetShifts(self.handle, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value


def train(config, data, num_round):
    """core.py:297-319 of the reference."""
    model = Garden(config)
    model.data = data
    model.labels_count = data.labels_count
    for _ in range(num_round):
        model.grow_tree(None)
    return model


def load(json_model_str):
    """core.py:322-339 of the reference."""
    config = json.loads(json_model_str)['configuration']
    model = Garden(config)
    model.load(json_model_str)
    return model


class _Estimator(object):
    _objective = 0

    def __init__(self, max_depth=6, learning_rate=0.1, n_estimators=100, verbosity=1, gamma_absolute=0.0,
                 gamma_relative=0.0, min_child_weight=1.0, min_leaf_size=0, max_leaf_weight=0.0,
                 colsample_bytree=0.8, colsample_bylevel=1.0, l1=1.0, l2=1.0, scale_pos_weight=1.0,
                 initial_y=0.5, seed=0, double_precision=False, method='hist', hist_size=255, **kwargs):
        # config layout: core.py:398-429 / 595-626 of the reference
        self._config = {
            'objective': self._objective,
            'method': 1 if method == 'hist' else 0,
            'internals': {'double_precision': double_precision, 'compute_overlap': 2,
                          'use_hist_subtraction_trick': True, 'dynamic_parallelism': True,
                          'upload_features': True, 'hist_size': hist_size, 'seed': seed},
            'verbose': {'gpu': verbosity > 0, 'booster': verbosity > 0, 'data': verbosity > 0},
            'tree': {'eta': learning_rate, 'max_depth': max_depth, 'gamma_absolute': gamma_absolute,
                     'gamma_relative': gamma_relative, 'min_child_weight': min_child_weight,
                     'min_leaf_size': min_leaf_size, 'colsample_bytree': colsample_bytree,
                     'colsample_bylevel': colsample_bylevel, 'max_leaf_weight': max_leaf_weight,
                     'lambda': l2, 'alpha': l1}}
        if self._objective == 1:
            self._config['tree']['scale_pos_weight'] = scale_pos_weight
            self._config['tree']['initial_y'] = initial_y
        self.n_estimators = n_estimators
        self._garden = Garden(self._config)
        self.verbosity = verbosity
        self.best_round = -1
        self.best_score = np.inf

    def _default_metric(self, y, p):
        raise NotImplementedError

    def fit(self, X, y=None, eval_set=None, eval_labels=None, early_stopping_rounds=5, eval_metric=None):
        if isinstance(X, DMatrix):
            data = X
        elif isinstance(X, np.ndarray) and isinstance(y, np.ndarray):
            data = DMatrix(X, y=y)
        else:
            raise ValueError("Only DMatrix and numpy array are supported")
        self._garden.data = data
        eval_data = None
        if eval_set is not None:
            if isinstance(eval_set, DMatrix):
                eval_data = eval_set
            elif isinstance(eval_set, np.ndarray):
                eval_data = DMatrix(eval_set)
            else:
                raise ValueError("Only DMatrix and numpy array are supported")
        metric = eval_metric or self._default_metric
        self.best_round, self.best_score = -1, np.inf
        for i in range(self.n_estimators):
            self._garden.grow_tree()
            if eval_data is not None:
                self._garden.append_last_tree(eval_data)
                score = metric(eval_labels, self._garden.get_y(eval_data))
                if score < self.best_score:
                    if self.verbosity > 0:
                        print("improved score {0} {1}->{2}".format(i, self.best_score, score))
                    self.best_score, self.best_round = score, i
                if early_stopping_rounds + self.best_round < i:
                    if self.verbosity > 0:
                        print("early stopping at {0} score {1}, use 'best_round' and 'best_score' to get it".format(
                            self.best_round, self.best_score))
                    break
        return self

    def predict(self, X, n_rounds=-1):
        if isinstance(X, DMatrix):
            data = X
        elif isinstance(X, np.ndarray):
            data = DMatrix(X)
        else:
            raise ValueError("Only DMatrix and numpy array are supported")
        return self._garden.predict(data, n_rounds)


class ArboretumRegression(_Estimator):
    """Scikit-learn style regressor (core.py:342-536 of the reference)."""
    _objective = 0

    def _default_metric(self, y, p):
        return float(np.mean((np.asarray(y) - p) ** 2))


class ArboretumClassifier(_Estimator):
    """Scikit-learn style binary classifier (core.py:539-732 of the reference)."""
    _objective = 1

    def _default_metric(self, y, p):
        from sklearn.metrics import roc_auc_score
        return -roc_auc_score(y, p)
