"""ctypes view of ``libscn_hip.so`` (the C ABI in ``include/scn_hip.h``).

This module is plumbing for tests, the smoke check and the benchmark: it loads
the in-tree HIP library, raises if it is missing (there is no CPU fallback) and
wraps device buffers.  The product's host side is the C++ library in ``host/``.
"""
import ctypes as C
import os
import re
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
LIB_PATH = os.path.join(_HERE, "libscn_hip.so")
HEADER = os.path.join(ROOT, "include", "scn_hip.h")

# ActivationFunction (reference types.h:11-20)
NOSIGMOID, RELU, VLEAKYRELU, LEAKYRELU, TANH, SOFTMAX, PRELU, SIGMOID = range(8)
FP32, BF16, BF16X3 = 0, 1, 2
OK, ERR_ARG, ERR_HIP, ERR_CAPACITY, ERR_STATE = range(5)
K_GRID_BUILD, K_RULES, K_GATHER, K_NIN, K_MAXPOOL, K_TERMINAL, K_SOFTMAX, K_CONV_NIN, K_PROBE, K_BACKWARD = range(10)
KERNEL_FAMILIES = ["grid_build", "rules", "gather", "nin", "maxpool", "terminal", "softmax", "conv_nin", "probe",
                   "backward"]


class ScnError(RuntimeError):
    pass


NAG_MAX = 4


class NagItem(C.Structure):
    """scn_nag_item of the C header."""
    _fields_ = [("d_delta", C.c_void_p), ("d_momentum", C.c_void_p), ("d_weights", C.c_void_p),
                ("n", C.c_int64), ("keepPositive", C.c_int)]


def build(force=True):
    """Compile the HIP library for gfx950 (works without a GPU)."""
    args = ["make", "-C", os.path.join(_HERE, "csrc"), "-s", "-j8"]
    if force:
        args.append("-B")
    subprocess.check_call(args)


def declared_symbols():
    """Names of every function the C header declares."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(scn_[A-Za-z0-9_]+)\s*\(", text)))


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ScnError(
            "libscn_hip.so is not built (run `python -c 'import __graft_entry__ as g; g.build()'`); "
            "there is no CPU fallback for the sparse forward path")
    L = C.CDLL(LIB_PATH)
    vp, i32, i64, f32, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t
    P = C.POINTER
    sig = {
        "scn_last_error": (C.c_char_p, []),
        "scn_version": (C.c_char_p, []),
        "scn_ctx_create": (C.c_int, [C.c_int, P(vp)]),
        "scn_ctx_destroy": (C.c_int, [vp]),
        "scn_ctx_stream": (vp, [vp]),
        "scn_sync": (C.c_int, [vp]),
        "scn_malloc": (C.c_int, [vp, sz, P(vp)]),
        "scn_free": (C.c_int, [vp, vp]),
        "scn_h2d": (C.c_int, [vp, vp, vp, sz]),
        "scn_d2h": (C.c_int, [vp, vp, vp, sz]),
        "scn_host_alloc": (C.c_int, [vp, sz, C.POINTER(vp)]),
        "scn_host_free": (C.c_int, [vp, vp]),
        "scn_h2d_async": (C.c_int, [vp, vp, vp, C.c_size_t]),
        "scn_copy": (C.c_int, [vp, vp, vp, C.c_size_t]),
        "scn_d2h_async": (C.c_int, [vp, vp, vp, sz]),
        "scn_event_create": (C.c_int, [vp, C.POINTER(vp)]),
        "scn_event_destroy": (C.c_int, [vp]),
        "scn_event_record": (C.c_int, [vp, vp]),
        "scn_event_wait": (C.c_int, [vp]),
        "scn_d2d": (C.c_int, [vp, vp, vp, sz]),
        "scn_fill32": (C.c_int, [vp, vp, C.c_uint32, sz]),
        "scn_grids_create": (C.c_int, [vp, P(vp)]),
        "scn_grids_clear_many": (C.c_int, [vp, C.POINTER(vp), C.c_int]),
        "scn_ctx_defer_counts": (C.c_int, [vp, C.c_int]),
        "scn_ctx_chain_rules": (C.c_int, [vp, C.c_int]),
        "scn_ctx_chain_count": (C.c_int, [vp, P(i64), P(i64)]),
        "scn_rules_settle": (C.c_int, [vp]),
        "scn_grids_destroy": (C.c_int, [vp, vp]),
        "scn_grids_build": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, vp, vp, vp, i64, vp, i32]),
        "scn_grids_info": (C.c_int, [vp, P(C.c_int), P(C.c_int), P(C.c_int), P(i64), P(i32)]),
        "scn_grids_download": (C.c_int, [vp, vp, vp, vp, vp, vp]),
        "scn_grids_find": (C.c_int, [vp, vp, vp, vp, i64, vp]),
        "scn_rules_square_plan": (C.c_int, [vp, vp, vp] + [C.c_int] * 5 + [P(i64)]),
        "scn_rules_triangular_plan": (C.c_int, [vp, vp, vp] + [C.c_int] * 5 + [P(i64)]),
        "scn_rules_terminal_plan": (C.c_int, [vp, vp, vp, P(i64)]),
        "scn_rules_fmp_plan": (C.c_int, [vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, vp, P(i64)]),
        "scn_rules_width": (C.c_int, [vp, P(i64)]),
        "scn_rules_fill": (C.c_int, [vp, vp, vp, vp, i64]),
        "scn_gather_rows": (C.c_int, [vp, vp, vp, vp, i64, C.c_int]),
        "scn_nin_forward": (C.c_int, [vp] * 6 + [i64, C.c_int, C.c_int, f32, C.c_int, C.c_int]),
        "scn_conv_nin_supported": (C.c_int, [C.c_int, C.c_int, C.c_int]),
        "scn_conv_nin_forward": (C.c_int, [vp, vp, vp, C.c_int, C.c_int, vp, vp, vp, vp, i64, C.c_int, f32, C.c_int]),
        "scn_conv_nin_supported_p": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int]),
        "scn_conv_nin_forward_p": (C.c_int, [vp, vp, vp, C.c_int, C.c_int, vp, vp, vp, vp, i64, C.c_int, f32, C.c_int,
                                             C.c_int]),
        "scn_conv_nin_forward_a16": (C.c_int, [vp, vp, i64, vp, vp, C.c_int, C.c_int, vp, vp, vp, vp, i64, C.c_int, f32,
                                               C.c_int]),
        "scn_maxpool": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int, vp]),
        "scn_maxpool_checked": (C.c_int, [vp, vp, i64, vp, vp, i64, C.c_int, C.c_int, vp]),
        "scn_terminal_pool": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int]),
        "scn_softmax_rows": (C.c_int, [vp, vp, vp, i64, C.c_int]),
        "scn_softmax_grad": (C.c_int, [vp, vp, vp, vp, i64, C.c_int]),
        "scn_activation_backward": (C.c_int, [vp, vp, vp, i64, C.c_int, C.c_int, vp, vp, vp]),
        "scn_sgemm_AtB": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int]),
        "scn_sgemm_ABt_workspace": (i64, [C.c_int, C.c_int]),
        "scn_sgemm_ABt": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int, vp]),
        "scn_sgemm_ABt_static_limit": (i64, []),
        "scn_sgemm_ABt_static": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int]),
        "scn_nag_update": (C.c_int, [vp, vp, vp, vp, i64, f32, f32, C.c_int]),
        "scn_nag_update_many": (C.c_int, [vp, P(NagItem), C.c_int, f32, f32, C.c_int]),
        "scn_activation_backward_acc": (C.c_int, [vp, vp, vp, i64, C.c_int, C.c_int, vp, vp, vp]),
        "scn_sgemm_AtB_acc": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int]),
        "scn_shrink_matrix": (C.c_int, [vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int]),
        "scn_nag_update_shrunk": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, f32, f32]),
        "scn_sum_abs": (C.c_int, [vp, vp, i64, P(C.c_double)]),
        "scn_scale": (C.c_int, [vp, vp, i64, f32]),
        "scn_gather_rows_backward": (C.c_int, [vp, vp, vp, vp, i64, C.c_int]),
        "scn_maxpool_backward": (C.c_int, [vp, vp, vp, i64, C.c_int, vp]),
        "scn_terminal_pool_backward": (C.c_int, [vp, vp, vp, vp, i64, C.c_int, C.c_int]),
        "scn_prof_enable": (C.c_int, [vp, C.c_int]),
        "scn_prof_reset": (C.c_int, [vp]),
        "scn_prof_probe": (C.c_int, [vp, C.c_int]),
        "scn_prof_tag": (C.c_int, [vp, C.c_int]),
        "scn_prof_spans": (C.c_int, [vp, C.c_int, vp, vp, vp, P(i32)]),
        "scn_prof_read": (C.c_int, [vp, C.c_int, P(C.c_double), P(i64)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    L._signatures = sig
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise ScnError("scn error %d: %s" % (rc, lib().scn_last_error().decode()))


class PinnedBuf:
    def __init__(self, ctx, nbytes):
        self.ctx, self.nbytes = ctx, int(nbytes)
        p = C.c_void_p()
        _check(lib().scn_host_alloc(ctx.h, max(self.nbytes, 16), C.byref(p)))
        self.ptr = p.value

    def buffer(self):
        return (C.c_char * self.nbytes).from_address(self.ptr)

    def free(self):
        if self.ptr:
            lib().scn_host_free(self.ctx.h, C.c_void_p(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class DevArray:
    """A typed device buffer allocated through the C ABI."""

    def __init__(self, ctx, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        p = C.c_void_p()
        _check(lib().scn_malloc(ctx.h, max(self.nbytes, 16), C.byref(p)))
        self.ptr = p.value

    def free(self):
        if getattr(self, "ptr", None):
            lib().scn_free(self.ctx.h, self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.size == self.size, (a.shape, self.shape)
        _check(lib().scn_h2d(self.ctx.h, self.ptr, a.ctypes.data_as(C.c_void_p), self.nbytes))
        return self

    def download(self):
        out = np.empty(self.shape, self.dtype)
        _check(lib().scn_d2h(self.ctx.h, out.ctypes.data_as(C.c_void_p), self.ptr, self.nbytes))
        return out


class Context:
    def __init__(self, device=0, handle=None):
        """A new context, or a view of one owned elsewhere (handle)."""
        self.owned = handle is None
        if handle is None:
            h = C.c_void_p()
            _check(lib().scn_ctx_create(device, C.byref(h)))
            handle = h.value
        self.h = handle

    def close(self):
        if getattr(self, "h", None) and self.owned:
            lib().scn_ctx_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def sync(self):
        _check(lib().scn_sync(self.h))

    def stream(self):
        return lib().scn_ctx_stream(self.h)

    def array(self, a, dtype=None):
        a = np.ascontiguousarray(a, dtype=dtype)
        return DevArray(self, a.shape, a.dtype).upload(a)

    def empty(self, shape, dtype):
        return DevArray(self, shape, dtype)

    def host_alloc(self, nbytes):
        """Pinned host memory (scn_host_alloc), freed with the object."""
        return PinnedBuf(self, nbytes)

    # ---- profiling
    def prof_enable(self, on=True):
        _check(lib().scn_prof_enable(self.h, int(on)))

    def prof_probe(self, with_kernel=True):
        _check(lib().scn_prof_probe(self.h, int(with_kernel)))

    def prof_reset(self):
        _check(lib().scn_prof_reset(self.h))

    def prof_read(self):
        out = {}
        for i, name in enumerate(KERNEL_FAMILIES):
            ms, calls = C.c_double(), C.c_int64()
            _check(lib().scn_prof_read(self.h, i, C.byref(ms), C.byref(calls)))
            out[name] = (ms.value, calls.value)
        return out

    def prof_spans(self, capacity=1 << 16):
        """[(family name, tag, ms)] of every span since the last read."""
        fam = np.empty(capacity, np.int32)
        tag = np.empty(capacity, np.int32)
        ms = np.empty(capacity, np.float64)
        n = C.c_int32()
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        _check(lib().scn_prof_spans(self.h, capacity, vp(fam), vp(tag), vp(ms), C.byref(n)))
        return [(KERNEL_FAMILIES[fam[i]], int(tag[i]), float(ms[i])) for i in range(n.value)]

    # ---- feature kernels
    def gather_rows(self, d_in, d_out, d_rules, count, nIn):
        _check(lib().scn_gather_rows(self.h, d_in.ptr, d_out.ptr, d_rules.ptr, count, nIn))

    def nin_forward(self, d_A, d_W, d_B, d_prelu, d_out, M, K, N, p=1.0, act=RELU, precision=FP32):
        _check(lib().scn_nin_forward(self.h, d_A.ptr, d_W.ptr, d_B.ptr,
                                     d_prelu.ptr if d_prelu is not None else None,
                                     d_out.ptr, M, K, N, p, act, precision))

    def conv_nin_forward(self, d_in, d_rules, fs, nIn, d_W, d_B, d_prelu, d_out, M, N, p=1.0, act=RELU, precision=FP32):
        _check(lib().scn_conv_nin_forward_p(self.h, d_in.ptr, d_rules.ptr, fs, nIn, d_W.ptr, d_B.ptr,
                                            d_prelu.ptr if d_prelu is not None else None, d_out.ptr, M, N, p, act,
                                            precision))

    def conv_nin_forward_a16(self, d_in, nInRows, d_in16, d_rules, fs, nIn, d_W, d_B, d_prelu, d_out, M, N, p=1.0, act=RELU):
        _check(lib().scn_conv_nin_forward_a16(self.h, d_in.ptr, nInRows, d_in16.ptr, d_rules.ptr, fs, nIn, d_W.ptr,
                                              d_B.ptr, d_prelu.ptr if d_prelu is not None else None, d_out.ptr, M, N,
                                              p, act))

    def maxpool(self, d_in, d_out, d_rules, nOutSites, ps, Cn, d_choice):
        _check(lib().scn_maxpool(self.h, d_in.ptr, d_out.ptr, d_rules.ptr, nOutSites, ps, Cn, d_choice.ptr))

    def terminal_pool(self, d_in, d_out, d_rules, count, S, Cn):
        _check(lib().scn_terminal_pool(self.h, d_in.ptr, d_out.ptr, d_rules.ptr, count, S, Cn))

    def softmax_rows(self, d_in, d_out, M, N):
        _check(lib().scn_softmax_rows(self.h, d_in.ptr, d_out.ptr, M, N))

    # ---- backward pass
    def softmax_grad(self, d_probs, d_labels, d_delta, batch, N):
        _check(lib().scn_softmax_grad(self.h, d_probs.ptr, d_labels.ptr, d_delta.ptr, batch, N))

    def activation_backward(self, d_out, d_delta, M, N, act, d_prelu, d_db, d_dprelu, accumulate=False):
        f = lib().scn_activation_backward_acc if accumulate else lib().scn_activation_backward
        _check(f(self.h, d_out.ptr, d_delta.ptr, M, N, act,
                 d_prelu.ptr if d_prelu is not None else None, d_db.ptr,
                 d_dprelu.ptr if d_dprelu is not None else None))

    def sgemm_AtB(self, d_A, d_D, d_dW, M, K, N, accumulate=False):
        f = lib().scn_sgemm_AtB_acc if accumulate else lib().scn_sgemm_AtB
        _check(f(self.h, d_A.ptr, d_D.ptr, d_dW.ptr, M, K, N))

    def nag_update_many(self, items, learningRate, momentum, clearGradients=False):
        """items: (d_delta, d_momentum, d_weights, n, keepPositive) tuples, at most NAG_MAX of them."""
        arr = (NagItem * max(1, len(items)))()
        for k, (d, m, w, n, kp) in enumerate(items):
            arr[k] = NagItem(d.ptr, m.ptr, w.ptr, n, int(kp))
        _check(lib().scn_nag_update_many(self.h, arr, len(items), learningRate, momentum, int(clearGradients)))

    def sgemm_ABt(self, d_D, d_W, d_dA, M, N, K, d_workspace):
        assert d_workspace.size >= lib().scn_sgemm_ABt_workspace(N, K)
        _check(lib().scn_sgemm_ABt(self.h, d_D.ptr, d_W.ptr, d_dA.ptr, M, N, K, d_workspace.ptr))

    def sgemm_ABt_static(self, d_D, d_W, d_dA, M, N, K):
        _check(lib().scn_sgemm_ABt_static(self.h, d_D.ptr, d_W.ptr, d_dA.ptr, M, N, K))

    def nag_update(self, d_delta, d_momentum, d_weights, n, learningRate, momentum, keepPositive=False):
        _check(lib().scn_nag_update(self.h, d_delta.ptr, d_momentum.ptr, d_weights.ptr, n, learningRate, momentum,
                                    int(keepPositive)))

    def shrink_matrix(self, d_W, d_w, d_inPresent, d_outPresent, nOut, nInP, nOutP):
        _check(lib().scn_shrink_matrix(self.h, d_W.ptr, d_w.ptr, d_inPresent.ptr, d_outPresent.ptr, nOut, nInP, nOutP))

    def nag_update_shrunk(self, d_delta, d_mom, d_wts, d_inPresent, d_outPresent, nOut, nInP, nOutP, lr, momentum):
        _check(lib().scn_nag_update_shrunk(self.h, d_delta.ptr, d_mom.ptr, d_wts.ptr, d_inPresent.ptr,
                                           d_outPresent.ptr, nOut, nInP, nOutP, lr, momentum))

    def sum_abs(self, d_x, n):
        out = C.c_double()
        _check(lib().scn_sum_abs(self.h, d_x.ptr, n, C.byref(out)))
        return out.value

    def scale(self, d_x, n, multiplier):
        _check(lib().scn_scale(self.h, d_x.ptr, n, multiplier))

    def gather_rows_backward(self, d_din, d_dconv, d_rules, count, nIn):
        _check(lib().scn_gather_rows_backward(self.h, d_din.ptr, d_dconv.ptr, d_rules.ptr, count, nIn))

    def maxpool_backward(self, d_din, d_dout, count, Cn, d_choice):
        _check(lib().scn_maxpool_backward(self.h, d_din.ptr, d_dout.ptr, count, Cn, d_choice.ptr))

    def terminal_pool_backward(self, d_din, d_dout, d_rules, count, Cn, S):
        _check(lib().scn_terminal_pool_backward(self.h, d_din.ptr, d_dout.ptr, d_rules.ptr, count, Cn, S))


class Grids:
    """Device-resident SparseGrids of one depth of a batch."""

    def __init__(self, ctx):
        self.ctx = ctx
        h = C.c_void_p()
        _check(lib().scn_grids_create(ctx.h, C.byref(h)))
        self.h = h.value

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            lib().scn_grids_destroy(self.ctx.h, self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def build(self, batch, dimension, spatialSize, sample, key, row, background, nSpatialSites):
        """Host arrays in, as Picture::codifyInputData leaves them."""
        c = self.ctx
        self._keep = (c.array(sample, np.int32), c.array(key, np.int64), c.array(row, np.int32),
                      c.array(np.asarray(background, np.int32) if batch else np.zeros(1, np.int32), np.int32))
        self.build_device(batch, dimension, spatialSize, *self._keep, len(np.asarray(key)), nSpatialSites)

    def build_device(self, batch, dimension, spatialSize, d_sample, d_key, d_row, d_bg, n, nSpatialSites):
        _check(lib().scn_grids_build(self.ctx.h, self.h, batch, dimension, spatialSize,
                                     d_sample.ptr, d_key.ptr, d_row.ptr, n, d_bg.ptr, nSpatialSites))

    def info(self):
        b, d, n = C.c_int(), C.c_int(), C.c_int()
        na, ns = C.c_int64(), C.c_int32()
        _check(lib().scn_grids_info(self.h, C.byref(b), C.byref(d), C.byref(n), C.byref(na), C.byref(ns)))
        return dict(batch=b.value, dimension=d.value, spatialSize=n.value, nActive=na.value, nSpatialSites=ns.value)

    def download(self):
        info = self.info()
        n, b = info["nActive"], info["batch"]
        s = np.empty(n, np.int32)
        k = np.empty(n, np.int64)
        r = np.empty(n, np.int32)
        bg = np.empty(b, np.int32)
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        _check(lib().scn_grids_download(self.ctx.h, self.h, vp(s), vp(k), vp(r), vp(bg)))
        return s, k, r, bg

    def find(self, sample, key):
        c = self.ctx
        ds, dk = c.array(sample, np.int32), c.array(key, np.int64)
        out = c.empty(len(sample), np.int32)
        _check(lib().scn_grids_find(c.h, self.h, ds.ptr, dk.ptr, len(sample), out.ptr))
        return out.download()

    # ---- rule books: plan on `self` as the input, returns (out grids, nOutSites)
    def plan_square(self, out, nIn, nOut, size, stride, minActive=1):
        n = C.c_int64()
        _check(lib().scn_rules_square_plan(self.ctx.h, self.h, out.h, nIn, nOut, size, stride, minActive, C.byref(n)))
        return n.value

    def plan_triangular(self, out, nIn, nOut, size, stride, minActive=1):
        n = C.c_int64()
        _check(lib().scn_rules_triangular_plan(self.ctx.h, self.h, out.h, nIn, nOut, size, stride, minActive, C.byref(n)))
        return n.value

    def plan_fmp(self, out, nIn, nOut, poolSize, inputL, inputR):
        """inputL / inputR: [batch, dimension, nOut] int32 host arrays (fractional max-pooling regions)"""
        inputL = np.ascontiguousarray(inputL, np.int32)
        inputR = np.ascontiguousarray(inputR, np.int32)
        info = self.info()
        assert inputL.shape == (info["batch"], info["dimension"], nOut) == inputR.shape
        n = C.c_int64()
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        _check(lib().scn_rules_fmp_plan(self.ctx.h, self.h, out.h, nIn, nOut, poolSize, vp(inputL), vp(inputR),
                                        C.byref(n)))
        return n.value

    def plan_terminal(self, out):
        S = C.c_int64()
        _check(lib().scn_rules_terminal_plan(self.ctx.h, self.h, out.h, C.byref(S)))
        return S.value

    def rules_width(self):
        w = C.c_int64()
        _check(lib().scn_rules_width(self.h, C.byref(w)))
        return w.value

    def fill(self, out, d_rules, capacity=None):
        cap = d_rules.size if capacity is None else capacity
        _check(lib().scn_rules_fill(self.ctx.h, self.h, out.h, d_rules.ptr, cap))


def defer_counts(ctx, on):
    _check(lib().scn_ctx_defer_counts(ctx.h, int(on)))


def chain_rules(ctx, on):
    """Record plan / fill calls that continue from one another and run them together (needs deferred counts)."""
    _check(lib().scn_ctx_chain_rules(ctx.h, int(on)))


def chain_count(ctx):
    """(chains run, plans they held) so far on this context"""
    a, b = C.c_int64(), C.c_int64()
    _check(lib().scn_ctx_chain_count(ctx.h, C.byref(a), C.byref(b)))
    return a.value, b.value


def settle(ctx):
    """Collect deferred counts; returns False when a bound was outgrown (plan again with deferral off)."""
    rc = lib().scn_rules_settle(ctx.h)
    if rc == ERR_CAPACITY:
        return False
    _check(rc)
    return True


def clear_many(ctx, grids):
    """Empty the tables and masks of several Grids in one launch (start of a batch)."""
    arr = (C.c_void_p * len(grids))(*[g.h for g in grids])
    _check(lib().scn_grids_clear_many(ctx.h, arr, len(grids)))


def rules_square(ctx, grids, nIn, nOut, size, stride, minActive=1, triangular=False, out=None):
    """plan + fill; returns (out grids, device rules, nOutSites, width)."""
    out = out if out is not None else Grids(ctx)
    plan = grids.plan_triangular if triangular else grids.plan_square
    n = plan(out, nIn, nOut, size, stride, minActive)
    w = out.rules_width()
    rules = ctx.empty(max(n * w, 1), np.int32)
    grids.fill(out, rules, n * w)
    return out, rules, n, w


def rules_fmp(ctx, grids, nIn, nOut, poolSize, inputL, inputR, out=None):
    """plan + fill over fractional max-pooling regions; returns (out grids, device rules, nOutSites, width)."""
    out = out if out is not None else Grids(ctx)
    n = grids.plan_fmp(out, nIn, nOut, poolSize, inputL, inputR)
    w = out.rules_width()
    rules = ctx.empty(max(n * w, 1), np.int32)
    grids.fill(out, rules, n * w)
    return out, rules, n, w


def rules_terminal(ctx, grids):
    out = Grids(ctx)
    S = grids.plan_terminal(out)
    batch = grids.info()["batch"]
    rules = ctx.empty(max(batch * S, 1), np.int32)
    grids.fill(out, rules, batch * S)
    return out, rules, S
