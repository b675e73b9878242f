"""The host side under AddressSanitizer + UndefinedBehaviorSanitizer (tests/native/sanitized_host.cpp):
the templates' host build (API cases, benchmark graph, gradient testers), the trainer's command-line
parser, and the image / checkpoint readers on valid files and on random mutations of them."""
import io
import os
import struct
import subprocess
import zlib

import numpy as np

from tests.test_trainer_host import _make_png

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NATIVE = os.path.join(ROOT, "tests", "native")
TRAINER = os.path.join(ROOT, "xyz_autodiff_cuda_amd", "csrc", "trainer")
MUTATIONS = 4000


def _png(width, height, colour_type, depth, rows, palette=None, split=1):
    def chunk(tag, data):
        return struct.pack(">I", len(data)) + tag + data + struct.pack(">I", zlib.crc32(tag + data) & 0xFFFFFFFF)

    raw = b"".join(bytes([r % 5 if False else 0]) + row for r, row in enumerate(rows))
    data = zlib.compress(raw, 6)
    parts = [data[i * len(data) // split:(i + 1) * len(data) // split] for i in range(split)]
    out = b"\x89PNG\r\n\x1a\n" + chunk(b"IHDR", struct.pack(">IIBBBBB", width, height, depth, colour_type, 0, 0, 0))
    if palette is not None:
        out += chunk(b"PLTE", palette)
    for part in parts:
        out += chunk(b"IDAT", part)
    return out + chunk(b"IEND", b"")


def _corpus(directory):
    r = np.random.default_rng(3)
    w, h = 19, 7
    rgb = r.integers(0, 256, (h, w, 3), dtype=np.uint8)
    files = {
        "rgb8.png": _png(w, h, 2, 8, [row.tobytes() for row in rgb], split=3),
        "grey8.png": _png(w, h, 0, 8, [row[:, 0].tobytes() for row in rgb]),
        "rgba16.png": _png(w, h, 6, 16, [r.integers(0, 256, w * 8, dtype=np.uint8).tobytes() for _ in range(h)]),
        "palette4.png": _png(w, h, 3, 4, [r.integers(0, 256, (w + 1) // 2, dtype=np.uint8).tobytes() for _ in range(h)],
                             palette=r.integers(0, 256, 48, dtype=np.uint8).tobytes()),
        "grey1.png": _png(w, h, 0, 1, [r.integers(0, 256, (w + 7) // 8, dtype=np.uint8).tobytes() for _ in range(h)]),
        "p6.ppm": b"P6\n# comment\n%d %d\n255\n" % (w, h) + rgb.tobytes(),
        "p6_16.ppm": b"P6 %d %d 65535\n" % (w, h) + r.integers(0, 256, w * h * 6, dtype=np.uint8).tobytes(),
        "p5.pgm": b"P5\n%d %d\n255\n" % (w, h) + rgb[:, :, 0].tobytes(),
        "interlaced.png": _make_png(rgb.astype(np.int64), 8, 2, interlace=True),
        "interlaced_grey2.png": _make_png(r.integers(0, 4, (h, w, 1)), 2, 0, interlace=True),
    }
    from PIL import Image

    smooth = np.clip(np.add.outer(np.arange(24) * 9, np.arange(40) * 5)[:, :, None] + rgb[0, 0] * 0.3, 0, 255).astype(np.uint8)
    kinds = {"baseline420.jpg": dict(subsampling=2), "progressive444.jpg": dict(subsampling=0, progressive=True),
             "restarts422.jpg": dict(subsampling=1, restart_marker_blocks=2), "optimised411.jpg": dict(subsampling="4:1:1", optimize=True),
             "progressive420_restarts.jpg": dict(subsampling=2, progressive=True, restart_marker_rows=1)}
    for name, options in kinds.items():
        buffer = io.BytesIO()
        Image.fromarray(smooth).save(buffer, "JPEG", quality=85, **options)
        files[name] = buffer.getvalue()
    buffer = io.BytesIO()
    Image.fromarray(smooth[:, :, 0]).save(buffer, "JPEG", quality=60, progressive=True)
    files["grey_progressive.jpg"] = buffer.getvalue()
    for name, image in {"rgb.bmp": Image.fromarray(rgb), "palette.bmp": Image.fromarray(rgb).quantize(colors=16),
                        "bilevel.bmp": Image.fromarray(rgb[:, :, 0]).convert("1"), "rgba.bmp": Image.fromarray(np.dstack([rgb, rgb[:, :, :1]]))}.items():
        buffer = io.BytesIO()
        image.save(buffer, "BMP")
        files[name] = buffer.getvalue()
    for name, data in files.items():
        with open(os.path.join(directory, name), "wb") as f:
            f.write(data)
    return len(files)


def test_host_tier_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    exe = str(tmp_path / "sanitized_host")
    hip_include = os.path.join(os.path.dirname(os.path.dirname(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"))), "include")
    cmd = [os.environ.get("CXX", "g++"), "-std=c++20", "-O0", "-g1", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-fno-omit-frame-pointer", "-march=x86-64-v3", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "include", "mini-gaussian-splatting"), "-I" + hip_include,
           "-I" + NATIVE,
           os.path.join(NATIVE, "sanitized_host.cpp"), os.path.join(TRAINER, "image_io.cpp"), os.path.join(TRAINER, "jpeg_codec.cpp"),
           os.path.join(TRAINER, "checkpoint.cpp"),
           os.path.join(TRAINER, "training_config.cpp"), "-o", exe, "-lz", "-lpthread"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    corpus, scratch = tmp_path / "corpus", tmp_path / "scratch"
    corpus.mkdir()
    scratch.mkdir()
    files = _corpus(str(corpus))
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1:abort_on_error=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    run = subprocess.run([exe, str(corpus), str(scratch), str(MUTATIONS)], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout[-2000:], run.stderr[-6000:])
    assert "sanitized host tier ok" in run.stdout, run.stdout
    assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr, run.stderr[-6000:]
    # all of the generated files were readable, the checkpoint and the four written images joined them, and
    # the mutation loop both accepted and rejected files (so it reached the decoders, not only the magic check)
    summary = run.stdout.strip().splitlines()[-1]
    assert "corpus %d files" % (files + 5) in summary, summary
    accepted, rejected = (int(summary.split(key)[0].split()[-1]) for key in (" mutations accepted", " rejected"))
    assert accepted > 50 and rejected > 50 and accepted + rejected == MUTATIONS, summary
