"""Tile-binned 2D Gaussian splatting step and Adam (GPU), host-side access.

Plays the part of the reference example's host code around its kernel launch
(examples/mini-gaussian-splatting/gaussian_splatting_training.cu:127-175 in
xyz-autodiff-cuda): zero/compute gradients, read the loss, Adam step.
"""
import ctypes
import math
import warnings

from . import _lib, rng

PARAM_ROWS = ("cx", "cy", "log_sx", "log_sy", "theta", "r", "g", "b", "opacity")
STAGES = ("sort", "project", "binning", "render_forward", "render_backward", "parameter_backward")
DEPTH_MODES = {"checked": 0, "static": 1, "every_step": 2}


def _check_tensor(t, shape, name, dtype=None):
    import torch

    dtype = dtype or torch.float32
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous() and tuple(t.shape) == tuple(shape)):
        raise ValueError("%s must be a contiguous %s CUDA tensor of shape %s" % (name, dtype, tuple(shape)))


class SplatContext:
    """Owns the device workspace of the step for one image size and Gaussian count."""

    def __init__(self, width, height, num_gaussians, pair_capacity_hint=0, device=None, depth_mode="checked"):
        """depth_mode: "checked" (every call looks whether a depth changed since the Gaussians were last ordered:
        one wait per call), "static" (a promise that depth does not change: calls that do not ask for the loss
        only queue work) or "every_step" (the order is recomputed by every call, on the device)."""
        import torch

        self.width, self.height, self.num_gaussians = int(width), int(height), int(num_gaussians)
        self.device = torch.device(device if device is not None else "cuda:0")
        self._lib = _lib.load()
        handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            st = self._lib.xad_splat_create(self.width, self.height, self.num_gaussians, int(pair_capacity_hint), ctypes.byref(handle))
        _lib.check(st, "xad_splat_create")
        self._handle = handle
        if depth_mode != "checked":
            self.set_depth_mode(depth_mode)

    def close(self):
        if getattr(self, "_handle", None):
            self._lib.xad_splat_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _stream(self, stream):
        import torch

        return (stream if stream is not None else torch.cuda.current_stream(self.device)).cuda_stream

    def set_depth_mode(self, mode):
        _lib.check(self._lib.xad_splat_set_depth_mode(self._handle, DEPTH_MODES[mode] if isinstance(mode, str) else int(mode)),
                   "xad_splat_set_depth_mode")

    def lists(self):
        """The tile lists of the last call: (range_begin, range_end, gaussians) as numpy uint32 arrays; tile t
        (row-major) holds gaussians[range_begin[t]:range_end[t]] in compositing order.  Waits for the device."""
        import numpy as np

        tiles = ((self.width + 15) // 16) * ((self.height + 15) // 16)
        begin, end = np.zeros(tiles, np.uint32), np.zeros(tiles, np.uint32)
        pairs = self.stats()["pairs"]
        ids = np.zeros(max(pairs, 1), np.uint32)
        st = self._lib.xad_splat_get_lists(self._handle, begin.ctypes.data, end.ctypes.data, ids.ctypes.data, ids.size)
        _lib.check(st, "xad_splat_get_lists")
        return begin, end, ids[:pairs]

    def overflow_word(self):
        """Device address of the word that is not zero while a step's lists have overflowed unseen by the host."""
        word = ctypes.c_void_p()
        _lib.check(self._lib.xad_splat_overflow_word(self._handle, ctypes.byref(word)), "xad_splat_overflow_word")
        return word.value

    def set_profiling(self, enabled):
        _lib.check(self._lib.xad_splat_set_profiling(self._handle, 1 if enabled else 0), "xad_splat_set_profiling")

    def forward(self, params, depth, image=None, stream=None):
        import torch

        G = self.num_gaussians
        _check_tensor(params, (9, G), "params")
        _check_tensor(depth, (G,), "depth")
        if image is None:
            image = torch.empty(self.height, self.width, 3, dtype=torch.float32, device=self.device)
        _check_tensor(image, (self.height, self.width, 3), "image")
        with torch.cuda.device(self.device):
            st = self._lib.xad_splat_forward(self._handle, params.data_ptr(), depth.data_ptr(), image.data_ptr(), self._stream(stream))
        _lib.check(st, "xad_splat_forward")
        return image

    def step(self, params, depth, target, image=None, grads=None, want_loss=True, stream=None):
        """Render, loss, gradients.  Returns (image, grads, loss or None)."""
        import torch

        G = self.num_gaussians
        _check_tensor(params, (9, G), "params")
        _check_tensor(depth, (G,), "depth")
        _check_tensor(target, (self.height, self.width, 3), "target")
        if image is None:
            image = torch.empty(self.height, self.width, 3, dtype=torch.float32, device=self.device)
        if grads is None:
            grads = torch.empty(9, G, dtype=torch.float32, device=self.device)
        _check_tensor(image, (self.height, self.width, 3), "image")
        _check_tensor(grads, (9, G), "grads")
        loss = ctypes.c_double(0.0)
        with torch.cuda.device(self.device):
            st = self._lib.xad_splat_step(self._handle, params.data_ptr(), depth.data_ptr(), target.data_ptr(), image.data_ptr(),
                                          grads.data_ptr(), ctypes.byref(loss) if want_loss else None, self._stream(stream))
        if st == _lib.XAD_ERR_INCOMPLETE:
            # this step's outputs are complete; an earlier step that did not wait lacked pairs (lists since enlarged)
            warnings.warn(self._lib.xad_last_error().decode("utf-8", "replace"), RuntimeWarning)
        else:
            _lib.check(st, "xad_splat_step")
        return image, grads, (loss.value if want_loss else None)

    def stats(self, longest_list=False):
        pairs = ctypes.c_uint64(0)
        longest = ctypes.c_uint32(0)
        ms = (ctypes.c_float * len(STAGES))()
        st = self._lib.xad_splat_get_stats(self._handle, ctypes.byref(pairs), ctypes.byref(longest) if longest_list else None, ms)
        _lib.check(st, "xad_splat_get_stats")
        out = {"pairs": pairs.value, "stage_ms": dict(zip(STAGES, [float(x) for x in ms]))}
        if longest_list:
            out["longest_list"] = longest.value
        return out


def depth_order(depth, stream=None):
    """(order, rank) of a float32 CUDA tensor of depths: order[i] = the i-th element by (depth, index), rank its
    inverse; int32 tensors holding the unsigned values (xad_depth_order_f32)."""
    import torch

    _check_tensor(depth, (depth.numel(),), "depth")
    order = torch.empty(depth.numel(), dtype=torch.int32, device=depth.device)
    rank = torch.empty_like(order)
    s = (stream if stream is not None else torch.cuda.current_stream(depth.device)).cuda_stream
    with torch.cuda.device(depth.device):
        st = _lib.load().xad_depth_order_f32(depth.numel(), depth.data_ptr(), order.data_ptr(), rank.data_ptr(), s)
    _lib.check(st, "xad_depth_order_f32")
    return order, rank


def host_step(params, depth, target, width, height, want_grads=True, num_threads=0):
    """The step on the host cores (xad_host_splat_step_f32), numpy in and out: the CPU figure
    the GPU step is reported beside.  params (9, G), depth (G,), target (height, width, 3), all
    float32.  Returns a dict with image, grads (None unless wanted), loss and pairs."""
    import numpy as np

    params = np.ascontiguousarray(params, dtype=np.float32)
    depth = np.ascontiguousarray(depth, dtype=np.float32)
    target = np.ascontiguousarray(target, dtype=np.float32)
    if params.ndim != 2 or params.shape[0] != len(PARAM_ROWS):
        raise ValueError("params must have shape (9, G)")
    G = params.shape[1]
    if depth.shape != (G,) or target.shape != (height, width, 3):
        raise ValueError("depth must have shape (G,) and target (height, width, 3)")
    image = np.empty((height, width, 3), dtype=np.float32)
    grads = np.empty_like(params) if want_grads else None
    loss = ctypes.c_double(0.0)
    pairs = ctypes.c_uint64(0)
    st = _lib.load().xad_host_splat_step_f32(width, height, G, params.ctypes.data, depth.ctypes.data, target.ctypes.data,
                                             image.ctypes.data, grads.ctypes.data if want_grads else None, ctypes.byref(loss),
                                             ctypes.byref(pairs), int(num_threads))
    _lib.check(st, "xad_host_splat_step_f32")
    return {"image": image, "grads": grads, "loss": loss.value, "pairs": pairs.value}


def adam_step(params, grads, m, v, learning_rates, iteration, beta1=0.9, beta2=0.999, eps=1e-8, stream=None,
              hold_if_nonzero=None, held_count=None):
    """In-place Adam over (rows, n) tensors; learning_rates: one float per row (or one float for all).
    hold_if_nonzero (a device address, e.g. SplatContext.overflow_word(), or a one-element int32 CUDA tensor): the
    update is decided on the device and withheld when that word is not zero; held_count (one-element int32 CUDA
    tensor) then counts it."""
    import torch

    rows, n = params.shape
    for t, name in ((params, "params"), (grads, "grads"), (m, "m"), (v, "v")):
        _check_tensor(t, (rows, n), name)
    if isinstance(learning_rates, (int, float)):
        learning_rates = [float(learning_rates)] * rows
    if len(learning_rates) != rows:
        raise ValueError("need one learning rate per row")
    lrs = (ctypes.c_float * rows)(*[float(x) for x in learning_rates])
    s = (stream if stream is not None else torch.cuda.current_stream(params.device)).cuda_stream
    with torch.cuda.device(params.device):
        if hold_if_nonzero is None:
            st = _lib.load().xad_adam_step_f32(n, rows, params.data_ptr(), grads.data_ptr(), m.data_ptr(), v.data_ptr(), lrs,
                                               beta1, beta2, eps, int(iteration), s)
        else:
            gate = hold_if_nonzero.data_ptr() if hasattr(hold_if_nonzero, "data_ptr") else int(hold_if_nonzero)
            st = _lib.load().xad_adam_step_gated_f32(n, rows, params.data_ptr(), grads.data_ptr(), m.data_ptr(), v.data_ptr(), lrs,
                                                     beta1, beta2, eps, int(iteration), gate,
                                                     held_count.data_ptr() if held_count is not None else None, s)
    _lib.check(st, "xad_adam_step_f32")


def synthetic_scene(num_gaussians, width, height, seed, scale_px=(1.0, 20.0), device="cuda:0"):
    """Random Gaussians with the benchmark's distributions: centre ~ U(image),
    log-scale ~ U(log lo, log hi) px, theta ~ U(-pi, pi), RGB ~ U(0, 1),
    opacity logit ~ N(0, 1), depth ~ U(0, 1).  Returns (params (9, G), depth (G,))."""
    import torch

    G = int(num_gaussians)
    params = torch.empty(9, G, dtype=torch.float32, device=device)
    depth = torch.empty(G, dtype=torch.float32, device=device)
    lo, hi = math.log(scale_px[0]), math.log(scale_px[1])
    rng.uniform_(params[0], seed, 0, 0.0, float(width))
    rng.uniform_(params[1], seed, 1, 0.0, float(height))
    rng.uniform_(params[2], seed, 2, lo, hi)
    rng.uniform_(params[3], seed, 3, lo, hi)
    rng.uniform_(params[4], seed, 4, -math.pi, math.pi)
    for row, stream_id in ((5, 5), (6, 6), (7, 7)):
        rng.uniform_(params[row], seed, stream_id, 0.0, 1.0)
    rng.normal_(params[8], seed, 8, 0.0, 1.0)
    rng.uniform_(depth, seed, 9, 0.0, 1.0)
    return params, depth


def synthetic_target(num_gaussians, width, height, seed, scale_px=(1.0, 20.0), noise=0.02, device="cuda:0"):
    """Target image: a render of a separate random scene plus N(0, noise) per value."""
    import torch

    params, depth = synthetic_scene(num_gaussians, width, height, seed, scale_px, device)
    ctx = SplatContext(width, height, num_gaussians, device=device)
    image = ctx.forward(params, depth)
    torch.cuda.synchronize()
    ctx.close()
    if noise:
        eps = torch.empty_like(image)
        rng.normal_(eps.view(-1), seed, 20, 0.0, float(noise))
        image += eps
    return image
