"""Splatting trainer front-end: configuration, image files, training run, checkpoints.

Thin ctypes layer over the trainer entry points of libxad_hip.so, the host-side
counterpart of examples/mini-gaussian-splatting/{gaussian_splatting_training.cu,
training_config.cpp, image_utils.cpp} in xyz-autodiff-cuda.  The command-line
program built next to the library, xad_splat_train, uses the same entry points.
"""
import ctypes
import os

import numpy as np

from . import _lib

PROGRAM_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "xad_splat_train")
HELP_REQUESTED = 4


class TrainingConfig(ctypes.Structure):
    """xad_training_config (include/xad_capi.h)."""

    _fields_ = [
        ("lr_center", ctypes.c_float), ("lr_scale", ctypes.c_float), ("lr_rotation", ctypes.c_float),
        ("lr_color", ctypes.c_float), ("lr_opacity", ctypes.c_float),
        ("max_iterations", ctypes.c_int), ("save_interval", ctypes.c_int), ("num_gaussians", ctypes.c_int),
        ("save_images", ctypes.c_int),
        ("beta1", ctypes.c_float), ("beta2", ctypes.c_float), ("epsilon", ctypes.c_float),
        ("target_image_path", ctypes.c_char * 1024),
        ("seed", ctypes.c_uint64),
        ("checkpoint_interval", ctypes.c_int),
        ("output_dir", ctypes.c_char * 1024),
        ("checkpoint_path", ctypes.c_char * 1024),
        ("resume_path", ctypes.c_char * 1024),
        ("image_format", ctypes.c_char * 8),
    ]

    @classmethod
    def defaults(cls, **overrides):
        config = cls()
        _lib.load().xad_training_config_defaults(ctypes.byref(config))
        for key, value in overrides.items():
            if isinstance(value, str):
                value = value.encode()
            setattr(config, key, value)
        return config

    def validate(self):
        _lib.check(_lib.load().xad_training_config_validate(ctypes.byref(self)), "xad_training_config_validate")


def parse_args(argv):
    """argv as given to main (program name first).  Returns a TrainingConfig, or None for --help;
    raises XadError with the reference's messages otherwise."""
    lib = _lib.load()
    config = TrainingConfig()
    args = (ctypes.c_char_p * len(argv))(*[a.encode() for a in argv])
    status = lib.xad_training_config_parse(len(argv), args, ctypes.byref(config))
    if status == HELP_REQUESTED:
        return None
    _lib.check(status, "xad_training_config_parse")
    return config


def usage():
    return _lib.load().xad_training_usage().decode()


def load_image(path):
    """-> float32 array (height, width, 3) in [0, 1]."""
    lib = _lib.load()
    width, height = ctypes.c_int(0), ctypes.c_int(0)
    data = ctypes.POINTER(ctypes.c_float)()
    _lib.check(lib.xad_image_load(os.fsencode(path), ctypes.byref(width), ctypes.byref(height), ctypes.byref(data)), "xad_image_load")
    try:
        return np.ctypeslib.as_array(data, shape=(height.value, width.value, 3)).copy()
    finally:
        lib.xad_image_free(data)


def save_image(path, rgb, quality=None):
    """By the extension of `path` (.jpg / .jpeg / .png / .ppm); with a quality (1..100), a JPEG whatever the extension."""
    rgb = np.ascontiguousarray(rgb, dtype=np.float32)
    if rgb.ndim != 3 or rgb.shape[2] != 3:
        raise ValueError("expected an array of shape (height, width, 3)")
    lib, data = _lib.load(), rgb.ctypes.data_as(ctypes.c_void_p)
    if quality is None:
        _lib.check(lib.xad_image_save(os.fsencode(path), rgb.shape[1], rgb.shape[0], data), "xad_image_save")
    else:
        _lib.check(lib.xad_image_save_jpeg(os.fsencode(path), rgb.shape[1], rgb.shape[0], data, int(quality)), "xad_image_save_jpeg")


def test_pattern(width, height):
    out = np.empty((height, width, 3), np.float32)
    _lib.check(_lib.load().xad_image_test_pattern(width, height, out.ctypes.data_as(ctypes.c_void_p)), "xad_image_test_pattern")
    return out


class Trainer:
    """One training run on the current GPU (see xad_trainer_create)."""

    def __init__(self, config, target):
        self._lib = _lib.load()
        target = np.ascontiguousarray(target, dtype=np.float32)
        if target.ndim != 3 or target.shape[2] != 3:
            raise ValueError("target must have shape (height, width, 3)")
        self.height, self.width = target.shape[:2]
        self.num_gaussians = config.num_gaussians
        handle = ctypes.c_void_p()
        st = self._lib.xad_trainer_create(ctypes.byref(config), self.width, self.height, target.ctypes.data_as(ctypes.c_void_p), ctypes.byref(handle))
        _lib.check(st, "xad_trainer_create")
        self._handle = handle

    def close(self):
        if getattr(self, "_handle", None):
            self._lib.xad_trainer_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def run(self, iterations, want_loss=True):
        loss = ctypes.c_double(0.0)
        status = self._lib.xad_trainer_run(self._handle, int(iterations), ctypes.byref(loss) if want_loss else None)
        _lib.check(status, "xad_trainer_run")
        return loss.value if want_loss else None

    @property
    def repeated_iterations(self):
        """Iterations run a second time because their tile lists had outgrown the buffers (their first run changed nothing)."""
        return self._lib.xad_trainer_repeated_iterations(self._handle)

    @property
    def iteration(self):
        return self._lib.xad_trainer_iteration(self._handle)

    def image(self):
        out = np.empty((self.height, self.width, 3), np.float32)
        _lib.check(self._lib.xad_trainer_download_image(self._handle, out.ctypes.data_as(ctypes.c_void_p)), "xad_trainer_download_image")
        return out

    def state(self):
        """-> dict of host copies: params, m, v (9, G) and depth (G,)."""
        G = self.num_gaussians
        out = {k: np.empty((9, G), np.float32) for k in ("params", "m", "v")}
        out["depth"] = np.empty(G, np.float32)
        P = ctypes.c_void_p
        st = self._lib.xad_trainer_get_state(self._handle, *[out[k].ctypes.data_as(P) for k in ("params", "m", "v", "depth")])
        _lib.check(st, "xad_trainer_get_state")
        return out

    def set_params(self, params=None, depth=None):
        G = self.num_gaussians
        P = ctypes.c_void_p
        if params is not None:
            params = np.ascontiguousarray(params, dtype=np.float32)
            assert params.shape == (9, G)
        if depth is not None:
            depth = np.ascontiguousarray(depth, dtype=np.float32)
            assert depth.shape == (G,)
        st = self._lib.xad_trainer_set_params(self._handle, params.ctypes.data_as(P) if params is not None else None,
                                              depth.ctypes.data_as(P) if depth is not None else None)
        _lib.check(st, "xad_trainer_set_params")

    def save_checkpoint(self, path):
        _lib.check(self._lib.xad_trainer_save_checkpoint(self._handle, os.fsencode(path)), "xad_trainer_save_checkpoint")

    def load_checkpoint(self, path):
        _lib.check(self._lib.xad_trainer_load_checkpoint(self._handle, os.fsencode(path)), "xad_trainer_load_checkpoint")
