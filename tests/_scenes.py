"""Small synthetic splatting scenes for the tests (numpy, CPU)."""
import numpy as np


def random_scene(G, width, height, seed, scale_px=(1.0, 20.0)):
    """Benchmark distributions: centre ~ U(image), log-scale ~ U(log lo, log hi),
    theta ~ U(-pi, pi), RGB ~ U(0, 1), opacity logit ~ N(0, 1), depth ~ U(0, 1)."""
    r = np.random.default_rng(seed)
    params = np.stack([
        r.uniform(0, width, G), r.uniform(0, height, G),
        r.uniform(np.log(scale_px[0]), np.log(scale_px[1]), G), r.uniform(np.log(scale_px[0]), np.log(scale_px[1]), G),
        r.uniform(-np.pi, np.pi, G),
        r.uniform(0, 1, G), r.uniform(0, 1, G), r.uniform(0, 1, G),
        r.normal(0, 1, G),
    ]).astype(np.float32)
    depth = r.uniform(0, 1, G).astype(np.float32)
    return params, depth


def one_gaussian(cx, cy, log_sx, log_sy, theta, rgb, opacity):
    return np.array([[cx], [cy], [log_sx], [log_sy], [theta], [rgb[0]], [rgb[1]], [rgb[2]], [opacity]], np.float32)
