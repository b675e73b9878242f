"""ctypes access to oracle/liboracle.so for the tests (the checker side only)."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "liboracle.so")

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            subprocess.run(["make", "-C", ORACLE_DIR], check=True, capture_output=True)
        _lib = ctypes.CDLL(LIB_PATH)
    return Oracle(_lib)


_CT = {np.dtype(np.float32): ctypes.c_float, np.dtype(np.float64): ctypes.c_double}
_SUF = {np.dtype(np.float32): "_f32", np.dtype(np.float64): "_f64"}


def _arg(x, dtype):
    """numpy array -> pointer, python int -> c_int, python float -> REAL."""
    if isinstance(x, np.ndarray):
        assert x.dtype == dtype and x.flags["C_CONTIGUOUS"], (x.dtype, dtype)
        return x.ctypes.data_as(ctypes.c_void_p)
    if isinstance(x, (int, np.integer)):
        return ctypes.c_int(int(x))
    if isinstance(x, float):
        return _CT[dtype](x)
    if x is None:
        return ctypes.c_void_p(0)
    raise TypeError(type(x))


class Oracle:
    def __init__(self, lib):
        self.lib = lib

    def call(self, name, dtype, *args):
        """Calls oracle_<name>_f32/_f64 with numpy arrays / ints / floats."""
        dtype = np.dtype(dtype)
        fn = getattr(self.lib, "oracle_" + name + _SUF[dtype])
        fn.restype = None
        fn(*[_arg(a, dtype) for a in args])

    def chain_one(self, inputs, dtype):
        """inputs = (sx, sy, theta, o, px, py) -> (w, grads[6], q)."""
        dtype = np.dtype(dtype)
        x = np.asarray(inputs, dtype=dtype)
        w = np.zeros(1, dtype)
        g = np.zeros(6, dtype)
        q = np.zeros(1, dtype)
        self.call("chain_one", dtype, x, w, g, q)
        return w[0], g, q[0]

    def chain_soa(self, inputs, dtype):
        """Six arrays -> array of shape (7, n): w and the six gradients."""
        dtype = np.dtype(dtype)
        arrays = [np.ascontiguousarray(a, dtype=dtype) for a in inputs]
        n = arrays[0].size
        outs = [np.empty(n, dtype) for _ in range(7)]
        fn = getattr(self.lib, "oracle_chain_soa" + _SUF[dtype])
        fn.restype = None
        fn(ctypes.c_long(n), *[a.ctypes.data_as(ctypes.c_void_p) for a in arrays],
           *[a.ctypes.data_as(ctypes.c_void_p) for a in outs])
        return np.stack(outs)

    def set_threads(self, n):
        self.lib.oracle_set_threads(ctypes.c_int(n))

    def max_threads(self):
        return self.lib.oracle_max_threads()

    def accumulate_chain(self, inputs, slot, num_slots, chain_in_double=True):
        """fp64 per-slot sums of the six chain gradients and of their magnitudes: two (num_slots, 6) arrays."""
        arrays = [np.ascontiguousarray(a, dtype=np.float32) for a in inputs]
        slot = np.ascontiguousarray(slot, dtype=np.int32)
        n = slot.size
        sums = np.zeros((num_slots, 6), np.float64)
        mass = np.zeros((num_slots, 6), np.float64)
        fn = self.lib.oracle_accumulate_chain
        fn.restype = None
        fn(ctypes.c_long(n), *[a.ctypes.data_as(ctypes.c_void_p) for a in arrays], slot.ctypes.data_as(ctypes.c_void_p),
           ctypes.c_int(num_slots), ctypes.c_int(1 if chain_in_double else 0),
           sums.ctypes.data_as(ctypes.c_void_p), mass.ctypes.data_as(ctypes.c_void_p))
        return sums, mass

    # ---- splatting -----------------------------------------------------------

    def splat_step(self, width, height, params, depth, target, dtype=np.float32, want_grads=True, rects_in=None,
                   want_bounds=False):
        """Tile-binned step on the CPU.  params (9, G).  Returns dict with image (H, W, 3),
        grads (9, G) or None, loss, pairs, longest_list, seconds (5 stages), rects (G, 4: first/last tile
        column and row of every Gaussian).  rects_in: bin with these rectangles instead of deriving them
        (an fp64 run then bins exactly like the fp32 run they came from).  want_bounds adds grad_mass and
        grad_bound (9, G, float64): the sum of the magnitudes of the per-pixel terms behind every gradient,
        and a first-order bound on the distance of an fp32 evaluation of the step from this one, and
        image_bound (H, W, 3), the same kind of bound for the image."""
        dtype = np.dtype(dtype)
        params = np.ascontiguousarray(params, dtype=dtype)
        depth = np.ascontiguousarray(depth, dtype=dtype)
        target = np.ascontiguousarray(target, dtype=dtype)
        G = params.shape[1]
        image = np.zeros((height, width, 3), dtype)
        grads = np.zeros((9, G), dtype) if want_grads else None
        rects = np.zeros((G, 4), np.int32)
        if rects_in is not None:
            rects_in = np.ascontiguousarray(rects_in, dtype=np.int32)
            assert rects_in.shape == (G, 4)
        mass = np.zeros((9, G), np.float64) if want_bounds else None
        bound = np.zeros((9, G), np.float64) if want_bounds else None
        image_bound = np.zeros((height, width, 3), np.float64) if want_bounds else None
        assert want_grads or not want_bounds
        stats = (ctypes.c_long * 2)()
        seconds = (ctypes.c_double * 5)()
        fn = getattr(self.lib, "oracle_splat_step_ex" + _SUF[dtype])
        fn.restype = ctypes.c_double
        P = ctypes.c_void_p
        ptr = lambda a: a.ctypes.data_as(P) if a is not None else P(0)
        loss = fn(ctypes.c_int(width), ctypes.c_int(height), ctypes.c_int(G), ptr(params), ptr(depth), ptr(target), ptr(image),
                  ptr(grads), stats, seconds, ptr(rects_in), ptr(rects), ptr(mass), ptr(bound), ptr(image_bound))
        return {"image": image, "grads": grads, "loss": loss, "pairs": stats[0], "longest_list": stats[1], "seconds": list(seconds),
                "rects": rects, "grad_mass": mass, "grad_bound": bound, "image_bound": image_bound}

    def splat_bruteforce(self, width, height, params, depth, target, dtype=np.float64):
        """Every pixel against every Gaussian.  Returns (image, loss)."""
        dtype = np.dtype(dtype)
        params = np.ascontiguousarray(params, dtype=dtype)
        depth = np.ascontiguousarray(depth, dtype=dtype)
        target = np.ascontiguousarray(target, dtype=dtype)
        image = np.zeros((height, width, 3), dtype)
        fn = getattr(self.lib, "oracle_splat_bruteforce" + _SUF[dtype])
        fn.restype = ctypes.c_double
        P = ctypes.c_void_p
        loss = fn(ctypes.c_int(width), ctypes.c_int(height), ctypes.c_int(params.shape[1]), params.ctypes.data_as(P),
                  depth.ctypes.data_as(P), target.ctypes.data_as(P), image.ctypes.data_as(P))
        return image, loss

    def adam_step(self, p, g, m, v, lr, beta1, beta2, eps, iteration):
        """In place on float32 numpy arrays (any shape, one learning rate)."""
        for a in (p, g, m, v):
            assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
        fn = self.lib.oracle_adam_step_f32
        fn.restype = None
        P = ctypes.c_void_p
        fn(ctypes.c_long(p.size), p.ctypes.data_as(P), g.ctypes.data_as(P), m.ctypes.data_as(P), v.ctypes.data_as(P),
           ctypes.c_float(lr), ctypes.c_float(beta1), ctypes.c_float(beta2), ctypes.c_float(eps), ctypes.c_int(iteration))

    def linreg_gradient(self, x1, x2, y, params, rows=None):
        """-> array of 5: gradient sums for (a, b, c, d) and the loss sum."""
        x1, x2, y, params = (np.ascontiguousarray(a, dtype=np.float64) for a in (x1, x2, y, params))
        if rows is not None:
            rows = np.ascontiguousarray(rows, dtype=np.int32)
        n = rows.size if rows is not None else x1.size
        out = np.zeros(5, np.float64)
        fn = self.lib.oracle_linreg_gradient_f64
        fn.restype = None
        P = ctypes.c_void_p
        fn(ctypes.c_long(n), x1.ctypes.data_as(P), x2.ctypes.data_as(P), y.ctypes.data_as(P),
           rows.ctypes.data_as(P) if rows is not None else P(0), params.ctypes.data_as(P), out.ctypes.data_as(P))
        return out

    def linreg_sgd(self, x1, x2, y, rows, params, batch, epochs, lr_first, lr_last):
        """rows: int32 (epochs * batch).  -> (final params, loss history)."""
        x1, x2, y = (np.ascontiguousarray(a, dtype=np.float64) for a in (x1, x2, y))
        rows = np.ascontiguousarray(rows, dtype=np.int32)
        assert rows.size == batch * epochs
        p = np.array(params, dtype=np.float64)
        history = np.zeros(epochs, np.float64)
        fn = self.lib.oracle_linreg_sgd_f64
        fn.restype = None
        P = ctypes.c_void_p
        fn(x1.ctypes.data_as(P), x2.ctypes.data_as(P), y.ctypes.data_as(P), rows.ctypes.data_as(P), p.ctypes.data_as(P),
           ctypes.c_int(batch), ctypes.c_int(epochs), ctypes.c_double(lr_first), ctypes.c_double(lr_last),
           history.ctypes.data_as(P))
        return p, history
