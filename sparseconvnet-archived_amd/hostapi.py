"""ctypes view of ``libscn_host.so``: the C++ host classes (SparseConvNet,
SparseConvTriangLeNet, SpatiallySparseDataset, BatchProducer) through the C
facade in ``host/scn_host_c.h``.  Harness plumbing only."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libscn_host.so")

TRAINBATCH, TESTBATCH, UNLABELEDBATCH, RESCALEBATCH = range(4)
LAYER_KINDS = ["conv", "conv_tri", "nin", "nin_prelu", "maxpool", "maxpool_tri", "terminal", "fmp"]
POFMP, PDFMP, ROFMP, RDFMP = range(4)  # pseudorandom / random, overlapping / disjoint fractional max-pooling


def build(force=True):
    args = ["make", "-C", os.path.join(_HERE, "host"), "-s", "-j8"]
    if force:
        args.append("-B")
    subprocess.check_call(args)


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libscn_host.so is not built; run __graft_entry__.build()")
    L = C.CDLL(LIB_PATH)
    vp, i32, i64, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_float
    P = C.POINTER
    sig = {
        "scnh_net_create": (vp, [i32] * 6),
        "scnh_net_destroy": (None, [vp]),
        "scnh_add_lenet_layer_mp": (None, [vp] + [i32] * 6 + [f32, i32]),
        "scnh_add_terminal_pooling_layer": (None, [vp, i32]),
        "scnh_add_softmax_layer": (None, [vp]),
        "scnh_finish_headless": (i32, [vp, i32]),
        "scnh_set_precision": (None, [vp, i32]),
        "scnh_set_fused_convolutions": (None, [vp, i32]),
        "scnh_set_producer_streams": (None, [vp, i32]),
        "scnh_producer_streams_in_use": (i32, [vp]),
        "scnh_set_chained_rule_books": (None, [vp, i32]),
        "scnh_input_spatial_size": (i32, [vp]),
        "scnh_n_layers": (i32, [vp]),
        "scnh_layer_info": (i32, [vp, i32, P(i32), P(i32), P(i32)]),
        "scnh_set_weights": (i32, [vp, i32, vp, vp, vp]),
        "scnh_save_weights": (None, [vp, C.c_char_p, i32, i32]),
        "scnh_load_weights": (None, [vp, C.c_char_p, i32, i32]),
        "scnh_dataset_create": (vp, [C.c_char_p, i32, i32, i32]),
        "scnh_dataset_destroy": (None, [vp]),
        "scnh_dataset_add_points": (None, [vp, i32, i32, i64, vp, vp, i32]),
        "scnh_dataset_size": (i64, [vp]),
        "scnh_dataset_label": (i32, [vp, i64]),
        "scnh_dataset_add_off_file": (i32, [vp, C.c_char_p, i32, i32]),
        "scnh_dataset_add_mesh": (None, [vp, i64, vp, i64, vp, i32, i32]),
        "scnh_dataset_add_strokes": (i32, [vp, i32, vp, vp, i32, i32, i32, i32]),
        "scnh_dataset_add_pendigits_file": (i64, [vp, C.c_char_p, i32, i32]),
        "scnh_constant_speed": (i64, [vp, i32, f32, i32, vp, i64]),
        "scnh_dataset_add_image": (i32, [vp, i32, i32, i32, vp, i32, i32, i32]),
        "scnh_dataset_add_mnist_files": (i64, [vp, C.c_char_p, C.c_char_p]),
        "scnh_dataset_add_cifar10_file": (i64, [vp, C.c_char_p]),
        "scnh_dataset_add_cifar100_file": (i64, [vp, C.c_char_p]),
        "scnh_codify_picture": (i64, [vp, i64, i32, i64, i64, vp, vp, vp, vp]),
        "scnh_process_dataset": (f32, [vp, vp, i32]),
        "scnh_add_lenet_layer_fmp": (i32, [vp, i32, i32, i32, i32, i32, f32, i32, f32, i32]),
        "scnh_iface_features_present": (i32, [vp, i32, vp]),
        "scnh_iface_region_ticks_size": (i64, [vp, i32]),
        "scnh_iface_region_ticks": (None, [vp, i32, vp]),
        "scnh_process_dataset_train": (f32, [vp, vp, i32, f32, f32]),
        "scnh_set_training": (None, [vp, f32, f32, i32]),
        "scnh_get_weights": (i32, [vp, i32, i32, vp, vp, vp]),
        "scnh_iface_dfeatures_size": (i64, [vp, i32]),
        "scnh_iface_dfeatures": (None, [vp, i32, vp]),
        "scnh_process_dataset_repeat_test": (None, [vp, vp, i32, i32]),
        "scnh_process_dataset_dump_top_level_features": (None, [vp, vp, i32, i32]),
        "scnh_calculate_input_regularizing_constants": (None, [vp, vp]),
        "scnh_input_normalizing_constants": (i32, [vp, vp, i32]),
        "scnh_begin": (None, [vp, vp, i32]),
        "scnh_next_batch": (i32, [vp]),
        "scnh_end": (None, [vp]),
        "scnh_batch_size": (i32, [vp]),
        "scnh_batch_mistakes": (i32, [vp]),
        "scnh_batch_nll": (f32, [vp]),
        "scnh_batch_probabilities": (None, [vp, vp]),
        "scnh_batch_predictions": (None, [vp, vp]),
        "scnh_batch_sample_numbers": (None, [vp, vp]),
        "scnh_iface_info": (None, [vp, i32, P(i32), P(i32), P(i32), P(i64), P(i64), P(i64), P(i64)]),
        "scnh_iface_rules": (None, [vp, i32, vp]),
        "scnh_iface_features": (None, [vp, i32, vp]),
        "scnh_iface_choices": (None, [vp, i32, vp]),
        "scnh_iface_grids": (None, [vp, i32, vp, vp, vp, vp]),
        "scnh_forward_resident": (i32, [vp, i32, vp, vp, vp, vp, i64, i32, vp, vp]),
        "scnh_forward_resident_stream": (i32, [vp, i32, i32, vp, vp, vp, vp, i64, i32, vp, vp]),
        "scnh_forward_stream_timed": (i32, [vp, i32, i32, i32, vp, vp, vp, vp, i64, i32, vp, i32, vp, P(C.c_double)]),
        "scnh_forward_stream_timed_many": (i32, [vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp, P(C.c_double)]),
        "scnh_set_stream_tail": (None, [vp, i32]),
        "scnh_stream_ready_at_start": (i32, [vp]),
        "scnh_collect_probabilities": (None, [vp, vp, i64]),
        "scnh_chain_counts": (None, [vp, P(i64), P(i64)]),
        "scnh_context": (vp, [vp]),
        "scnh_take_multiply_add_count": (C.c_double, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class Dataset:
    def __init__(self, name, nFeatures, nClasses, batch_type=TESTBATCH):
        self.nFeatures, self.nClasses = nFeatures, nClasses
        self.h = lib().scnh_dataset_create(name.encode(), nFeatures, nClasses, batch_type)

    def add_points(self, dimension, latticeSize, coords, features, label=-1):
        coords = np.ascontiguousarray(coords, np.int32).reshape(-1, dimension)
        features = np.ascontiguousarray(features, np.float32).reshape(coords.shape[0], self.nFeatures)
        lib().scnh_dataset_add_points(self.h, dimension, latticeSize, coords.shape[0], _p(coords), _p(features), label)

    def add_off_file(self, path, renderSize, label=-1):
        """OffSurfaceModelPicture from an OFF file."""
        if lib().scnh_dataset_add_off_file(self.h, str(path).encode(), renderSize, label) != 0:
            raise IOError("%s is not a readable OFF mesh" % path)

    def add_mesh(self, points, triangles, renderSize, label=-1):
        """OffSurfaceModelPicture from arrays (points n x 3, triangles m x 3)."""
        points = np.ascontiguousarray(points, np.float64).reshape(-1, 3)
        triangles = np.ascontiguousarray(triangles, np.int32).reshape(-1, 3)
        lib().scnh_dataset_add_mesh(self.h, len(points), _p(points), len(triangles), _p(triangles), renderSize, label)

    def add_strokes(self, strokes, renderSize, encoding, label=-1, normalize=True):
        """OnlineHandwritingPicture from a list of strokes (each n x 2)."""
        strokes = [np.ascontiguousarray(s, np.float64).reshape(-1, 2) for s in strokes]
        lengths = np.array([len(s) for s in strokes], np.int32)
        xy = np.ascontiguousarray(np.concatenate(strokes) if strokes else np.zeros((0, 2)))
        if lib().scnh_dataset_add_strokes(self.h, len(strokes), _p(lengths), _p(xy), renderSize, encoding, label,
                                          1 if normalize else 0) != 0:
            raise ValueError("strokes: encoding %d is not available, does not match nFeatures %d, or the "
                             "character is empty" % (encoding, self.nFeatures))

    def add_image(self, pixels, backgroundColor, label=-1, trainingJiggle=0):
        """OpenCVPicture from an array [rows x cols x channels] of values 0..255."""
        pixels = np.ascontiguousarray(pixels, np.float32)
        if pixels.ndim == 2:
            pixels = pixels[:, :, None]
        r, c, ch = pixels.shape
        if lib().scnh_dataset_add_image(self.h, r, c, ch, _p(pixels), backgroundColor, label, trainingJiggle) != 0:
            raise ValueError("image: %d channels into a dataset of %d features" % (ch, self.nFeatures))

    def add_mnist_files(self, images, labels):
        n = lib().scnh_dataset_add_mnist_files(self.h, str(images).encode(), str(labels).encode())
        if n < 0:
            raise IOError("%s / %s: not a readable MNIST idx pair (or nFeatures != 1)" % (images, labels))
        return int(n)

    def add_cifar10_file(self, path):
        n = lib().scnh_dataset_add_cifar10_file(self.h, str(path).encode())
        if n < 0:
            raise IOError("%s: not a readable CIFAR-10 batch (or nFeatures != 3)" % path)
        return int(n)

    def add_cifar100_file(self, path):
        n = lib().scnh_dataset_add_cifar100_file(self.h, str(path).encode())
        if n < 0:
            raise IOError("%s: not a readable CIFAR-100 file (or nFeatures != 3)" % path)
        return int(n)

    def add_pendigits_file(self, path, renderSize, encoding):
        """every character of a UCI pen-digits file; returns how many."""
        n = lib().scnh_dataset_add_pendigits_file(self.h, str(path).encode(), renderSize, encoding)
        if n < 0:
            raise IOError("%s: not readable, or encoding %d not available for nFeatures %d"
                          % (path, encoding, self.nFeatures))
        return int(n)

    def codify(self, index, spatialSize, seed=-1):
        """distort (seed >= 0) + codifyInputData of one picture on the CPU:
        (keys, rows in insertion order, background row, features [rows x nFeatures])."""
        cap = 1 << 12
        while True:
            keys, rows = np.empty(cap, np.int64), np.empty(cap, np.int32)
            bg = C.c_int32()
            feats = np.empty((cap, self.nFeatures), np.float32)
            n = lib().scnh_codify_picture(self.h, index, spatialSize, seed, cap, _p(keys), _p(rows), C.byref(bg), _p(feats))
            if n <= cap:
                return keys[:n - 1].copy(), rows[:n - 1].copy(), bg.value, feats[:n].copy()
            cap = int(n)

    def __len__(self):
        return lib().scnh_dataset_size(self.h)

    def label(self, index):
        return lib().scnh_dataset_label(self.h, index)

    def close(self):
        if getattr(self, "h", None):
            lib().scnh_dataset_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Net:
    """SparseConvNet (or SparseConvTriangLeNet with triangular=True)."""

    def __init__(self, dimension, nInputFeatures, nClasses, nTop=1, threads=2, triangular=False):
        self.dimension, self.nInputFeatures, self.nClasses, self.nTop = dimension, nInputFeatures, nClasses, nTop
        self.h = lib().scnh_net_create(dimension, nInputFeatures, nClasses, nTop, threads, int(triangular))

    def close(self):
        if getattr(self, "h", None):
            lib().scnh_net_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # builders, named as in the reference
    def addLeNetLayerMP(self, nFeatures, filterSize, filterStride, poolSize, poolStride, activationFn=1, dropout=0.0,
                        minActiveInputs=1):
        lib().scnh_add_lenet_layer_mp(self.h, nFeatures, filterSize, filterStride, poolSize, poolStride, activationFn,
                                      dropout, minActiveInputs)

    def addLeNetLayerFMP(self, kind, nFeatures, filterSize, filterStride, poolSize, fmpShrink, activationFn=1,
                         dropout=0.0, minActiveInputs=1):
        """addLeNetLayerPOFMP / PDFMP / ROFMP / RDFMP of the reference (kind = POFMP ...)"""
        rc = lib().scnh_add_lenet_layer_fmp(self.h, kind, nFeatures, filterSize, filterStride, poolSize, fmpShrink,
                                            activationFn, dropout, minActiveInputs)
        assert rc == 0, "fractional max-pooling builders exist on the square-lattice net only"

    def addTerminalPoolingLayer(self, poolSize):
        lib().scnh_add_terminal_pooling_layer(self.h, poolSize)

    def addSoftmaxLayer(self):
        lib().scnh_add_softmax_layer(self.h)

    def finishHeadless(self, topSpatialSize):
        return lib().scnh_finish_headless(self.h, topSpatialSize)

    def setFusedConvolutions(self, on=True):
        lib().scnh_set_fused_convolutions(self.h, int(on))

    def setProducerStreams(self, n):
        lib().scnh_set_producer_streams(self.h, int(n))

    def producerStreamsInUse(self):
        return lib().scnh_producer_streams_in_use(self.h)

    def setChainedRuleBooks(self, on=True):
        lib().scnh_set_chained_rule_books(self.h, int(on))

    def setPrecision(self, precision):
        lib().scnh_set_precision(self.h, precision)

    @property
    def inputSpatialSize(self):
        return lib().scnh_input_spatial_size(self.h)

    def layers(self):
        out = []
        for i in range(lib().scnh_n_layers(self.h)):
            a, b, c = C.c_int(), C.c_int(), C.c_int()
            kind = lib().scnh_layer_info(self.h, i, C.byref(a), C.byref(b), C.byref(c))
            out.append(dict(kind=LAYER_KINDS[kind], nIn=a.value, nOut=b.value, act=c.value))
        return out

    def set_weights(self, layer, W, B, prelu=None):
        W = np.ascontiguousarray(W, np.float32)
        B = np.ascontiguousarray(B, np.float32)
        pr = np.ascontiguousarray(prelu, np.float32) if prelu is not None else None
        rc = lib().scnh_set_weights(self.h, layer, _p(W), _p(B), _p(pr) if pr is not None else None)
        assert rc == 0, "layer %d has no weights" % layer

    def get_weights(self, layer, momentum=False):
        """(W [K x N], B [N], PReLU slopes [N] or None) of a NiN layer, or their momentum vectors"""
        l = self.layers()[layer]
        W = np.empty((l["nIn"], l["nOut"]), np.float32)
        B = np.empty(l["nOut"], np.float32)
        pr = np.empty(l["nOut"], np.float32) if l["kind"] == "nin_prelu" else None
        rc = lib().scnh_get_weights(self.h, layer, int(momentum), _p(W), _p(B), _p(pr) if pr is not None else None)
        assert rc == 0, "layer %d has no weights" % layer
        return W, B, pr

    def set_training(self, learningRate, momentum, shuffle=True):
        """learning rate and momentum of TRAINBATCH batches run by next_batch(); shuffled order or not"""
        lib().scnh_set_training(self.h, learningRate, momentum, int(shuffle))

    def processDatasetTrain(self, ds, batchSize=100, learningRate=0.0, momentum=0.99):
        return lib().scnh_process_dataset_train(self.h, ds.h, batchSize, learningRate, momentum)

    def features_present(self, i):
        """featuresPresent of interface i: which features the columns of its feature matrix are"""
        n = lib().scnh_iface_features_present(self.h, i, None)
        out = np.empty(n, np.int32)
        lib().scnh_iface_features_present(self.h, i, _p(out))
        return out

    def region_ticks(self, i):
        """(inputL, inputR), each [batch, dimension, spatialSize of interface i]: the regions a fractional
        max-pooling layer drew for the current batch; None for any other interface"""
        n = lib().scnh_iface_region_ticks_size(self.h, i)
        if n == 0:
            return None
        t = np.empty(n, np.int32)
        lib().scnh_iface_region_ticks(self.h, i, _p(t))
        b = lib().scnh_batch_size(self.h)
        t = t.reshape(2, b, self.dimension, -1)
        return t[0].copy(), t[1].copy()

    def dfeatures(self, i):
        """gradient left in interface i by the last TRAINBATCH, flat; empty if the backward pass stopped above it"""
        n = lib().scnh_iface_dfeatures_size(self.h, i)
        out = np.empty(n, np.float32)
        if n:
            lib().scnh_iface_dfeatures(self.h, i, _p(out))
        return out

    def saveWeights(self, base, epoch, momentum=False):
        lib().scnh_save_weights(self.h, base.encode(), epoch, int(momentum))

    def loadWeights(self, base, epoch, momentum=False):
        lib().scnh_load_weights(self.h, base.encode(), epoch, int(momentum))

    def processDataset(self, ds, batchSize=100):
        return lib().scnh_process_dataset(self.h, ds.h, batchSize)

    def processDatasetRepeatTest(self, ds, batchSize=100, nReps=2):
        lib().scnh_process_dataset_repeat_test(self.h, ds.h, batchSize, nReps)

    # batch-by-batch with inspection
    def processDatasetDumpTopLevelFeatures(self, ds, batchSize=100, reps=1):
        """writes "<dataset name>.features" into the working directory."""
        lib().scnh_process_dataset_dump_top_level_features(self.h, ds.h, batchSize, reps)

    def calculateInputRegularizingConstants(self, ds):
        lib().scnh_calculate_input_regularizing_constants(self.h, ds.h)
        return self.inputNormalizingConstants()

    def inputNormalizingConstants(self):
        out = np.zeros(4096, np.float32)
        n = lib().scnh_input_normalizing_constants(self.h, _p(out), len(out))
        return out[:n].copy()

    def begin(self, ds, batchSize):
        lib().scnh_begin(self.h, ds.h, batchSize)

    def next_batch(self):
        return bool(lib().scnh_next_batch(self.h))

    def end(self):
        lib().scnh_end(self.h)

    def batch_outputs(self):
        L = lib()
        b = L.scnh_batch_size(self.h)
        probs = np.empty((b, self.nClasses), np.float32)
        pred = np.empty((b, self.nTop), np.int32)
        nums = np.empty(b, np.int32)
        L.scnh_batch_probabilities(self.h, _p(probs))
        L.scnh_batch_predictions(self.h, _p(pred))
        L.scnh_batch_sample_numbers(self.h, _p(nums))
        return dict(probabilities=probs, predictions=pred, sampleNumbers=nums, mistakes=L.scnh_batch_mistakes(self.h),
                    nll=L.scnh_batch_nll(self.h), batchSize=b)

    def interface(self, i, want_features=True):
        L = lib()
        nf, ns, ss = C.c_int(), C.c_int(), C.c_int()
        nr, ne, nc, ng = C.c_int64(), C.c_int64(), C.c_int64(), C.c_int64()
        L.scnh_iface_info(self.h, i, C.byref(nf), C.byref(ns), C.byref(ss), C.byref(nr), C.byref(ne), C.byref(nc),
                          C.byref(ng))
        out = dict(nFeatures=nf.value, nSpatialSites=ns.value, spatialSize=ss.value)
        rules = np.empty(nr.value, np.int32)
        if nr.value:
            L.scnh_iface_rules(self.h, i, _p(rules))
        out["rules"] = rules
        if want_features:
            # None: a convolution's output whose gather was fused into the next NiN layer
            feats = np.empty((ns.value, nf.value), np.float32) if (ne.value or ns.value == 0) else None
            if ne.value:
                L.scnh_iface_features(self.h, i, _p(feats))
            out["features"] = feats
        ch = np.empty(nc.value, np.int32)
        if nc.value:
            L.scnh_iface_choices(self.h, i, _p(ch))
        out["choices"] = ch
        b = L.scnh_batch_size(self.h)
        s, k, r, bg = np.empty(ng.value, np.int32), np.empty(ng.value, np.int64), np.empty(ng.value, np.int32), np.empty(b, np.int32)
        L.scnh_iface_grids(self.h, i, _p(s), _p(k), _p(r), _p(bg))
        out["grids"] = (s, k, r, bg)
        return out

    # resident input (device pointers as integers)
    def forward_resident(self, batch, d_sample, d_key, d_row, d_bg, nActive, nSpatialSites, d_features, h_probs=None):
        return lib().scnh_forward_resident(self.h, batch, d_sample, d_key, d_row, d_bg, nActive, nSpatialSites,
                                           d_features, _p(h_probs) if h_probs is not None else None)

    def forward_resident_stream(self, nBatches, batch, d_sample, d_key, d_row, d_bg, nActive, nSpatialSites, d_features,
                                h_probs=None):
        return lib().scnh_forward_resident_stream(self.h, nBatches, batch, d_sample, d_key, d_row, d_bg, nActive,
                                                  nSpatialSites, d_features, _p(h_probs) if h_probs is not None else None)

    def forward_stream_timed(self, nWarmup, nTimed, batch, sample, key, row, bg, nActive, nSpatialSites, features,
                             inputs_on_host=False, h_probs=None):
        """nWarmup + nTimed batches in one pass; returns the wall time of the timed ones in seconds.  The five
        arrays are device pointers, or pinned host pointers with inputs_on_host (uploaded for every batch)."""
        sec = C.c_double()
        done = lib().scnh_forward_stream_timed(self.h, nWarmup, nTimed, batch, sample, key, row, bg, nActive,
                                               nSpatialSites, features, int(inputs_on_host),
                                               _p(h_probs) if h_probs is not None else None, C.byref(sec))
        assert done == nWarmup + nTimed
        return sec.value

    def forward_stream_timed_many(self, nWarmup, nTimed, batches, inputs_on_host=False, h_probs=None):
        """The same over several different batches taken in turn; batches: list of (batch, sample, key, row, bg,
        nActive, nSpatialSites, features) with pointers as integers."""
        n = len(batches)
        vpa = C.c_void_p * n
        col = lambda i: vpa(*[b[i] for b in batches])
        sizes = (C.c_int * n)(*[b[0] for b in batches])
        act = (C.c_int64 * n)(*[b[5] for b in batches])
        sites = (C.c_int * n)(*[b[6] for b in batches])
        sec = C.c_double()
        done = lib().scnh_forward_stream_timed_many(self.h, nWarmup, nTimed, n, sizes, col(1), col(2), col(3), col(4),
                                                    act, sites, col(7), int(inputs_on_host),
                                                    _p(h_probs) if h_probs is not None else None, C.byref(sec))
        assert done == nWarmup + nTimed
        return sec.value

    def setStreamTail(self, nTail):
        """batches that follow the timed ones of every later forward_stream_timed(_many) pass, untimed"""
        lib().scnh_set_stream_tail(self.h, int(nTail))

    def streamReadyAtStart(self):
        return lib().scnh_stream_ready_at_start(self.h)

    def collect_probabilities(self, out):
        """out: float32 array that later stream passes fill with every batch's probabilities in batch order
        (None: switched off).  The caller keeps it alive."""
        self._collect = out
        lib().scnh_collect_probabilities(self.h, _p(out) if out is not None else None, 0 if out is None else out.size)

    def chain_counts(self):
        """(runs of recorded plans, plans in them) so far, over every stream that builds rule books"""
        a, b = C.c_int64(), C.c_int64()
        lib().scnh_chain_counts(self.h, C.byref(a), C.byref(b))
        return a.value, b.value

    def context_handle(self):
        return lib().scnh_context(self.h)


# OnlineHandwritingEncoding (types.h:29-39 of the reference)
SIMPLE, OCTOGRAM, UNDIRECTED_OCTOGRAM, SPACETIME3D, VECTOR_SPACETIME3D = 0, 1, 2, 7, 8
ENCODING_FEATURES = {0: 1, 1: 8, 2: 4, 7: 1, 8: 3}


def constant_speed(stroke, density, multiplier=1):
    """constantSpeed of one stroke (n x 2) -> resampled points."""
    xy = np.ascontiguousarray(stroke, np.float64).reshape(-1, 2)
    cap = 1 << 12
    while True:
        out = np.empty((cap, 2), np.float64)
        n = lib().scnh_constant_speed(_p(xy), len(xy), density, multiplier, _p(out), cap)
        if n <= cap:
            return out[:n].copy()
        cap = int(n)


def take_multiply_add_count():
    return lib().scnh_take_multiply_add_count()
