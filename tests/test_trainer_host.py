"""Trainer front-end, host side (no GPU): command line and image files.

The command line is checked against the behaviour of TrainingConfigParser
(examples/mini-gaussian-splatting/training_config.cpp:29-146 in xyz-autodiff-cuda):
defaults, every option, and the failure messages.  The image reader is checked
against PNG/PPM files produced here with Python's zlib (all colour types, bit
depths and row filters), the writer by decoding its files with an independent
decoder written in this test.
"""
import struct
import zlib

import numpy as np
import pytest

from xyz_autodiff_cuda_amd import trainer

LR = ["0.01", "0.005", "0.02", "0.03", "0.04"]


# ---- command line ---------------------------------------------------------------------

def test_defaults_match_the_reference(xad):
    c = trainer.TrainingConfig.defaults()
    # training_config.h:9-27
    assert [c.lr_center, c.lr_scale, c.lr_rotation, c.lr_color, c.lr_opacity] == [np.float32(0.01)] * 5
    assert (c.max_iterations, c.save_interval, c.num_gaussians, c.save_images) == (500, 25, 1000, 1)
    assert (c.beta1, c.beta2, c.epsilon) == (np.float32(0.9), np.float32(0.999), np.float32(1e-8))
    assert c.target_image_path == b"" and c.output_dir == b"output" and c.seed == 0


def test_parse_reference_example(xad):
    # the example line of print_usage (training_config.cpp:111)
    c = trainer.parse_args(["prog"] + "0.01 0.005 0.02 0.01 0.01 --target data/target.png --max-iterations 1000 --save-interval 50".split())
    assert c.lr_scale == np.float32(0.005) and c.lr_rotation == np.float32(0.02)
    assert c.target_image_path == b"data/target.png" and c.max_iterations == 1000 and c.save_interval == 50
    assert c.num_gaussians == 1000 and c.save_images == 1


def test_parse_every_option(xad):
    c = trainer.parse_args(["prog"] + LR + ["--num-gaussians", "77", "--no-save-images", "--beta1", "0.8", "--beta2", "0.95",
                                             "--epsilon", "1e-6", "--target", "t.ppm", "--seed", "12345678901234", "--output-dir", "o",
                                             "--checkpoint", "c.bin", "--checkpoint-interval", "5", "--resume", "r.bin"])
    assert [c.lr_center, c.lr_scale, c.lr_rotation, c.lr_color, c.lr_opacity] == [np.float32(float(x)) for x in LR]
    assert c.num_gaussians == 77 and c.save_images == 0
    assert (c.beta1, c.beta2, c.epsilon) == (np.float32(0.8), np.float32(0.95), np.float32(1e-6))
    assert c.seed == 12345678901234 and c.output_dir == b"o" and c.checkpoint_path == b"c.bin"
    assert c.checkpoint_interval == 5 and c.resume_path == b"r.bin"


@pytest.mark.parametrize("args,message", [
    (LR[:4], "Insufficient arguments"),                       # argc < 6 (training_config.cpp:32-35)
    (LR + ["--target", "t.png", "--bogus"], "Invalid argument"),           # :71-75
    (LR + ["--target"], "Invalid argument"),                                # option without its value falls through to the same branch
    (LR + ["--max-iterations", "10"], "Target image path must be specified with --target"),
    (["0", "1", "1", "1", "1", "--target", "t"], "All learning rates must be positive"),
    (["abc", "1", "1", "1", "1", "--target", "t"], "All learning rates must be positive"),  # atof("abc") = 0
    (LR + ["--target", "t", "--max-iterations", "0"], "Max iterations must be positive"),
    (LR + ["--target", "t", "--save-interval", "-1"], "Save interval must be positive"),
    (LR + ["--target", "t", "--num-gaussians", "0"], "Number of Gaussians must be positive"),
    (LR + ["--target", "t", "--beta1", "1.0"], "Beta1 must be in range (0, 1)"),
    (LR + ["--target", "t", "--beta2", "0"], "Beta2 must be in range (0, 1)"),
    (LR + ["--target", "t", "--epsilon", "0"], "Epsilon must be positive"),
    (LR + ["--target", "t", "--checkpoint-interval", "3"], "needs a checkpoint path"),
    (LR + ["--target", "x" * 2000], "too long"),
])
def test_parse_failures(xad, args, message):
    with pytest.raises(xad.XadError, match=message.replace("(", r"\(").replace(")", r"\)")):
        trainer.parse_args(["prog"] + args)


def test_help(xad):
    assert trainer.parse_args(["prog", "--help"]) is None
    assert trainer.parse_args(["prog"] + LR + ["--target", "t", "--help"]) is None
    text = trainer.usage()
    for option in ("--target", "--max-iterations", "--save-interval", "--num-gaussians", "--no-save-images", "--beta1", "--beta2",
                   "--epsilon", "--help", "--resume", "--checkpoint"):
        assert option in text


# ---- images ---------------------------------------------------------------------------

def _chunk(kind, data):
    return struct.pack(">I", len(data)) + kind + data + struct.pack(">I", zlib.crc32(kind + data))


def _paeth(a, b, c):
    p = a + b - c
    pa, pb, pc = abs(p - a), abs(p - b), abs(p - c)
    return a if pa <= pb and pa <= pc else (b if pb <= pc else c)


def _filter_rows(rows, bpp, filters):
    """rows: list of bytes; applies PNG filter type filters[y] to each row."""
    out = bytearray()
    prev = bytes(len(rows[0]))
    for y, row in enumerate(rows):
        f = filters[y % len(filters)]
        out.append(f)
        for i, x in enumerate(row):
            a = row[i - bpp] if i >= bpp else 0
            b = prev[i]
            c = prev[i - bpp] if i >= bpp else 0
            pred = (0, a, b, (a + b) >> 1, _paeth(a, b, c))[f]
            out.append((x - pred) & 255)
        prev = row
    return bytes(out)


def _make_png(samples, depth, colour, palette=None, filters=(0, 1, 2, 3, 4), idat_split=1, extra=b""):
    """samples: uint array (H, W, channels) of `depth`-bit values."""
    h, w, ch = samples.shape
    rows = []
    for y in range(h):
        flat = samples[y].reshape(-1)
        if depth == 16:
            rows.append(flat.astype(">u2").tobytes())
        elif depth == 8:
            rows.append(flat.astype(np.uint8).tobytes())
        else:
            bits = "".join(format(int(v), "0%db" % depth) for v in flat)
            bits += "0" * (-len(bits) % 8)
            rows.append(bytes(int(bits[i:i + 8], 2) for i in range(0, len(bits), 8)))
    bpp = max(1, ch * depth // 8)
    packed = zlib.compress(_filter_rows(rows, bpp, filters), 9)
    step = -(-len(packed) // idat_split)
    idat = b"".join(_chunk(b"IDAT", packed[i:i + step]) for i in range(0, len(packed), step))
    out = b"\x89PNG\r\n\x1a\n" + _chunk(b"IHDR", struct.pack(">IIBBBBB", w, h, depth, colour, 0, 0, 0))
    if palette is not None:
        out += _chunk(b"PLTE", bytes(palette))
    return out + extra + idat + _chunk(b"IEND", b"")


def _decode_png_rgb8(data):
    """Independent decoder for what save_image writes: 8-bit RGB, one or more IDAT chunks."""
    assert data[:8] == b"\x89PNG\r\n\x1a\n"
    pos, idat, header = 8, b"", None
    while pos < len(data):
        (length,), kind = struct.unpack(">I", data[pos:pos + 4]), data[pos + 4:pos + 8]
        body = data[pos + 8:pos + 8 + length]
        assert struct.unpack(">I", data[pos + 8 + length:pos + 12 + length])[0] == zlib.crc32(kind + body)
        if kind == b"IHDR":
            header = struct.unpack(">IIBBBBB", body)
        elif kind == b"IDAT":
            idat += body
        pos += 12 + length
    w, h, depth, colour, comp, filt, lace = header
    assert (depth, colour, comp, filt, lace) == (8, 2, 0, 0, 0)
    raw = zlib.decompress(idat)
    assert len(raw) == h * (1 + 3 * w)
    out = np.zeros((h, w * 3), np.uint8)
    for y in range(h):
        row = raw[y * (1 + 3 * w):(y + 1) * (1 + 3 * w)]
        assert row[0] == 0
        out[y] = np.frombuffer(row[1:], np.uint8)
    return out.reshape(h, w, 3)


@pytest.mark.parametrize("colour,channels,depths", [(0, 1, (1, 2, 4, 8, 16)), (2, 3, (8, 16)), (4, 2, (8, 16)), (6, 4, (8, 16))])
def test_png_reader_colour_types_depths_and_filters(xad, tmp_path, colour, channels, depths):
    rng = np.random.default_rng(colour)
    for depth in depths:
        h, w = 13, 11  # odd sizes: rows of sub-byte samples end inside a byte
        samples = rng.integers(0, 1 << depth, (h, w, channels))
        path = tmp_path / ("c%dd%d.png" % (colour, depth))
        path.write_bytes(_make_png(samples, depth, colour, idat_split=3, extra=_chunk(b"tEXt", b"Comment\0hello")))
        got = trainer.load_image(path)
        scale = np.float32((1 << depth) - 1)
        colour_samples = samples[:, :, :3] if channels >= 3 else np.repeat(samples[:, :, :1], 3, axis=2)
        np.testing.assert_array_equal(got, colour_samples.astype(np.float32) / scale)


def test_png_reader_palette(xad, tmp_path):
    rng = np.random.default_rng(3)
    palette = rng.integers(0, 256, (16, 3))
    for depth in (1, 2, 4, 8):
        index = rng.integers(0, min(16, 1 << depth), (9, 10, 1))
        path = tmp_path / ("p%d.png" % depth)
        path.write_bytes(_make_png(index, depth, 3, palette=palette.reshape(-1).tolist()))
        np.testing.assert_array_equal(trainer.load_image(path), palette[index[:, :, 0]].astype(np.float32) / np.float32(255))


def test_png_reader_rejects_damage(xad, tmp_path):
    samples = np.random.default_rng(0).integers(0, 256, (8, 8, 3))
    good = _make_png(samples, 8, 2)
    cases = {
        "truncated": good[:-20],
        "checksum": good[:40] + bytes([good[40] ^ 1]) + good[41:],
        "interlaced": good[:8] + _chunk(b"IHDR", struct.pack(">IIBBBBB", 8, 8, 8, 2, 0, 0, 1)) + good[33:],
        "critical": good[:33] + _chunk(b"ABCD", b"") + good[33:],
        "size": _make_png(samples[:7], 8, 2)[:8] + good[8:33] + _make_png(samples[:7], 8, 2)[33:],
        "jpeg": b"\xff\xd8\xff\xe0" + bytes(100),
        "text": b"hello world, not an image",
    }
    for name, data in cases.items():
        path = tmp_path / (name + ".png")
        path.write_bytes(data)
        with pytest.raises(xad.XadError):
            trainer.load_image(path)
    with pytest.raises(xad.XadError, match="cannot open"):
        trainer.load_image(tmp_path / "missing.png")


def test_ppm_and_pgm_reader(xad, tmp_path):
    rng = np.random.default_rng(1)
    rgb = rng.integers(0, 256, (5, 7, 3)).astype(np.uint8)
    (tmp_path / "a.ppm").write_bytes(b"P6\n# a comment\n7 5\n# another\n255\n" + rgb.tobytes())
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "a.ppm"), rgb.astype(np.float32) / np.float32(255))
    grey = rng.integers(0, 1000, (4, 3)).astype(">u2")
    (tmp_path / "b.pgm").write_bytes(b"P5 3 4 999\n" + grey.tobytes())
    want = np.repeat((grey.astype(np.float32) / np.float32(999))[:, :, None], 3, axis=2)
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "b.pgm"), want)
    (tmp_path / "short.ppm").write_bytes(b"P6 7 5 255\n" + rgb.tobytes()[:-1])
    with pytest.raises(xad.XadError, match="shorter"):
        trainer.load_image(tmp_path / "short.ppm")


def test_writer_quantisation_and_round_trip(xad, tmp_path):
    rng = np.random.default_rng(2)
    image = rng.uniform(-0.2, 1.2, (17, 23, 3)).astype(np.float32)
    image[0, 0] = [np.nan, np.inf, -np.inf]
    image[0, 1] = [0.5, 0.49803922, 1.0 / 510.0]  # around rounding boundaries
    # image_utils.cpp:42-46: clamp to [0, 1], then (unsigned char)(v * 255 + 0.5) in fp32
    clamped = np.where(image > 0, np.minimum(image, np.float32(1)), np.float32(0)).astype(np.float32)
    want = (clamped * np.float32(255) + np.float32(0.5)).astype(np.uint8)
    for name in ("out.png", "out.PPM"):
        trainer.save_image(tmp_path / name, image)
    np.testing.assert_array_equal(_decode_png_rgb8((tmp_path / "out.png").read_bytes()), want)
    raw = (tmp_path / "out.PPM").read_bytes()
    assert raw.startswith(b"P6\n23 17\n255\n")
    np.testing.assert_array_equal(np.frombuffer(raw[len(b"P6\n23 17\n255\n"):], np.uint8).reshape(17, 23, 3), want)
    # and our reader reads our writer
    for name in ("out.png", "out.PPM"):
        np.testing.assert_array_equal(trainer.load_image(tmp_path / name), want.astype(np.float32) / np.float32(255))
    with pytest.raises(xad.XadError, match="png or .ppm"):
        trainer.save_image(tmp_path / "out.jpg", image)
    with pytest.raises(xad.XadError, match="cannot create"):
        trainer.save_image(tmp_path / "no_such_dir" / "out.png", image)


def test_test_pattern(xad):
    # create_test_image (image_utils.cpp:58-77): r = x / width, g = y / height, b = (r + g) / 2, in fp32
    got = trainer.test_pattern(40, 24)
    x = np.arange(40, dtype=np.float32)[None, :] / np.float32(40)
    y = np.arange(24, dtype=np.float32)[:, None] / np.float32(24)
    np.testing.assert_array_equal(got[:, :, 0], np.broadcast_to(x, (24, 40)))
    np.testing.assert_array_equal(got[:, :, 1], np.broadcast_to(y, (24, 40)))
    np.testing.assert_array_equal(got[:, :, 2], np.float32(0.5) * (x + y))
