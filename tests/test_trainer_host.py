"""Trainer front-end, host side (no GPU): command line and image files.

The command line is checked against the behaviour of TrainingConfigParser
(examples/mini-gaussian-splatting/training_config.cpp:29-146 in xyz-autodiff-cuda):
defaults, every option, and the failure messages.  The image reader is checked
against PNG/PPM files produced here with Python's zlib (all colour types, bit
depths and row filters, plain and interlaced), the writer by decoding its files
with an independent decoder written in this test.  The JPEG reader and writer
are checked against Pillow (libjpeg): the reader on Pillow's files of every
kind it writes, the writer by having Pillow read its files and by comparing
them with Pillow's own files of the same image.  Decoders of this format may
differ by a level or two per sample (transform and interpolation rounding); the
tolerances say so.
"""
import io
import itertools
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
    assert c.image_format == b"jpg"  # gaussian_splatting_training.cu:106, :124 write .jpg


def test_parse_reference_example(xad):
    # the example line of print_usage (training_config.cpp:111)
    c = trainer.parse_args(["prog"] + "0.01 0.005 0.02 0.01 0.01 --target data/target.png --max-iterations 1000 --save-interval 50".split())
    assert c.lr_scale == np.float32(0.005) and c.lr_rotation == np.float32(0.02)
    assert c.target_image_path == b"data/target.png" and c.max_iterations == 1000 and c.save_interval == 50
    assert c.num_gaussians == 1000 and c.save_images == 1


def test_parse_every_option(xad):
    c = trainer.parse_args(["prog"] + LR + ["--num-gaussians", "77", "--no-save-images", "--beta1", "0.8", "--beta2", "0.95",
                                             "--epsilon", "1e-6", "--target", "t.ppm", "--seed", "12345678901234", "--output-dir", "o",
                                             "--checkpoint", "c.bin", "--checkpoint-interval", "5", "--resume", "r.bin",
                                             "--image-format", "png"])
    assert [c.lr_center, c.lr_scale, c.lr_rotation, c.lr_color, c.lr_opacity] == [np.float32(float(x)) for x in LR]
    assert c.num_gaussians == 77 and c.save_images == 0
    assert (c.beta1, c.beta2, c.epsilon) == (np.float32(0.8), np.float32(0.95), np.float32(1e-6))
    assert c.seed == 12345678901234 and c.output_dir == b"o" and c.checkpoint_path == b"c.bin"
    assert c.checkpoint_interval == 5 and c.resume_path == b"r.bin" and c.image_format == b"png"


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
    (LR + ["--target", "t", "--image-format", "gif"], "Image format must be jpg, png or ppm"),
    (LR + ["--target", "t", "--image-format", "portable-network-graphics"], "Image format must be jpg, png or ppm"),
])
def test_parse_failures(xad, args, message):
    with pytest.raises(xad.XadError, match=message.replace("(", r"\(").replace(")", r"\)")):
        trainer.parse_args(["prog"] + args)


def test_help(xad):
    assert trainer.parse_args(["prog", "--help"]) is None
    assert trainer.parse_args(["prog"] + LR + ["--target", "t", "--help"]) is None
    text = trainer.usage()
    for option in ("--target", "--max-iterations", "--save-interval", "--num-gaussians", "--no-save-images", "--beta1", "--beta2",
                   "--epsilon", "--help", "--resume", "--checkpoint", "--image-format"):
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


def _packed_rows(samples, depth):
    rows = []
    for y in range(samples.shape[0]):
        flat = samples[y].reshape(-1)
        if depth == 16:
            rows.append(flat.astype(">u2").tobytes())
        elif depth == 8:
            rows.append(flat.astype(np.uint8).tobytes())
        else:
            bits = "".join(format(int(v), "0%db" % depth) for v in flat)
            bits += "0" * (-len(bits) % 8)
            rows.append(bytes(int(bits[i:i + 8], 2) for i in range(0, len(bits), 8)))
    return rows


# Adam7 (PNG specification, section 8.2): pass k holds the pixels (x0 + i dx, y0 + j dy)
ADAM7 = ((0, 0, 8, 8), (4, 0, 8, 8), (0, 4, 4, 8), (2, 0, 4, 4), (0, 2, 2, 4), (1, 0, 2, 2), (0, 1, 1, 2))


def _make_png(samples, depth, colour, palette=None, filters=(0, 1, 2, 3, 4), idat_split=1, extra=b"", interlace=False):
    """samples: uint array (H, W, channels) of `depth`-bit values."""
    h, w, ch = samples.shape
    bpp = max(1, ch * depth // 8)
    if interlace:
        filtered = b""
        for x0, y0, dx, dy in ADAM7:
            part = samples[y0::dy, x0::dx]
            if part.shape[0] and part.shape[1]:
                filtered += _filter_rows(_packed_rows(part, depth), bpp, filters)
    else:
        filtered = _filter_rows(_packed_rows(samples, depth), bpp, filters)
    packed = zlib.compress(filtered, 9)
    step = -(-len(packed) // idat_split)
    idat = b"".join(_chunk(b"IDAT", packed[i:i + step]) for i in range(0, len(packed), step))
    out = b"\x89PNG\r\n\x1a\n" + _chunk(b"IHDR", struct.pack(">IIBBBBB", w, h, depth, colour, 0, 0, int(interlace)))
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


@pytest.mark.parametrize("size", [(1, 1), (2, 3), (3, 2), (5, 9), (8, 8), (13, 11), (33, 17)])
def test_png_reader_interlaced(xad, tmp_path, size):
    # sizes below 5 x 5 leave some of the seven passes empty; every pass is filtered on its own
    h, w = size
    rng = np.random.default_rng(h * 100 + w)
    for colour, channels, depth in ((2, 3, 8), (0, 1, 1), (0, 1, 4), (6, 4, 16), (4, 2, 8)):
        samples = rng.integers(0, 1 << depth, (h, w, channels))
        path = tmp_path / ("i%d_%d.png" % (colour, depth))
        path.write_bytes(_make_png(samples, depth, colour, interlace=True, idat_split=2))
        colour_samples = samples[:, :, :3] if channels >= 3 else np.repeat(samples[:, :, :1], 3, axis=2)
        np.testing.assert_array_equal(trainer.load_image(path), colour_samples.astype(np.float32) / np.float32((1 << depth) - 1))
        plain = tmp_path / "plain.png"
        plain.write_bytes(_make_png(samples, depth, colour))
        np.testing.assert_array_equal(trainer.load_image(path), trainer.load_image(plain))
    palette = rng.integers(0, 256, (4, 3))
    index = rng.integers(0, 4, (h, w, 1))
    path = tmp_path / "ip.png"
    path.write_bytes(_make_png(index, 2, 3, palette=palette.reshape(-1).tolist(), interlace=True))
    np.testing.assert_array_equal(trainer.load_image(path), palette[index[:, :, 0]].astype(np.float32) / np.float32(255))


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
        "interlace_flag_on_plain_data": good[:8] + _chunk(b"IHDR", struct.pack(">IIBBBBB", 8, 8, 8, 2, 0, 0, 1)) + good[33:],
        "interlace_method": good[:8] + _chunk(b"IHDR", struct.pack(">IIBBBBB", 8, 8, 8, 2, 0, 0, 2)) + good[33:],
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
    with pytest.raises(xad.XadError, match="must end in"):
        trainer.save_image(tmp_path / "out.gif", image)
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


# ---- BMP ------------------------------------------------------------------------------

def _bmp(width, height, bits, rows, palette=b"", compression=0, masks=b"", top_down=False, core=False):
    """rows: top-to-bottom list of unpadded row bytes."""
    padded = [r + bytes(-len(r) % 4) for r in (rows if top_down else rows[::-1])]
    if core:
        info = struct.pack("<IHHHH", 12, width, height, 1, bits)
    else:
        info = struct.pack("<IiiHHIIiiII", 40, width, -height if top_down else height, 1, bits, compression, 0, 2835, 2835,
                           len(palette) // 4, 0)
    offset = 14 + len(info) + len(masks) + len(palette)
    body = b"".join(padded)
    return b"BM" + struct.pack("<IHHI", offset + len(body), 0, 0, offset) + info + masks + palette + body


def test_bmp_reader_against_pillow(xad, tmp_path):
    from PIL import Image

    rng = np.random.default_rng(11)
    rgb = rng.integers(0, 256, (9, 13, 3), dtype=np.uint8)  # 13 x 3 bytes per row: padding is exercised
    images = {"rgb": Image.fromarray(rgb), "grey": Image.fromarray(rgb[:, :, 0]),
              "palette": Image.fromarray(rgb).quantize(colors=37), "bilevel": Image.fromarray(rgb[:, :, 1]).convert("1"),
              "rgba": Image.fromarray(np.dstack([rgb, rgb[:, :, :1]]))}
    for name, image in images.items():
        path = tmp_path / (name + ".bmp")
        image.save(path, "BMP")
        want = np.asarray(Image.open(path).convert("RGB")).astype(np.float32) / np.float32(255)
        np.testing.assert_array_equal(trainer.load_image(path), want, err_msg=name)


def test_bmp_reader_layouts(xad, tmp_path):
    rng = np.random.default_rng(12)
    h, w = 5, 7
    rgb = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    want = rgb.astype(np.float32) / np.float32(255)
    bgr_rows = [rgb[y, :, ::-1].tobytes() for y in range(h)]
    for name, data in {"bottom_up": _bmp(w, h, 24, bgr_rows), "top_down": _bmp(w, h, 24, bgr_rows, top_down=True),
                       "core": _bmp(w, h, 24, bgr_rows, core=True)}.items():
        (tmp_path / (name + ".bmp")).write_bytes(data)
        np.testing.assert_array_equal(trainer.load_image(tmp_path / (name + ".bmp")), want, err_msg=name)
    # 4 bits per pixel with a colour table of 11 entries (blue, green, red, unused)
    table = rng.integers(0, 256, (11, 4), dtype=np.uint8)
    index = rng.integers(0, 11, (h, w))
    rows = [bytes((int(a) << 4) | int(b) for a, b in zip(list(r[0::2]), list(r[1::2]) + [0])) for r in index]
    (tmp_path / "p4.bmp").write_bytes(_bmp(w, h, 4, rows, palette=table.tobytes()))
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "p4.bmp"), table[index][:, :, 2::-1].astype(np.float32) / np.float32(255))
    # 16 bits: five bits a channel by default, 5-6-5 by masks; 32 bits with masks in another order
    r5, g6, b5 = rng.integers(0, 32, (h, w)), rng.integers(0, 64, (h, w)), rng.integers(0, 32, (h, w))
    rows = [((r5[y] << 10) | ((g6[y] >> 1) << 5) | b5[y]).astype("<u2").tobytes() for y in range(h)]
    (tmp_path / "x555.bmp").write_bytes(_bmp(w, h, 16, rows))
    want555 = np.stack([r5 / 31, (g6 >> 1) / 31, b5 / 31], axis=2).astype(np.float32)
    np.testing.assert_allclose(trainer.load_image(tmp_path / "x555.bmp"), want555, rtol=0, atol=1e-7)
    rows = [((r5[y] << 11) | (g6[y] << 5) | b5[y]).astype("<u2").tobytes() for y in range(h)]
    (tmp_path / "r565.bmp").write_bytes(_bmp(w, h, 16, rows, compression=3, masks=struct.pack("<III", 0xF800, 0x07E0, 0x001F)))
    want565 = np.stack([r5 / 31, g6 / 63, b5 / 31], axis=2).astype(np.float32)
    np.testing.assert_allclose(trainer.load_image(tmp_path / "r565.bmp"), want565, rtol=0, atol=1e-7)
    packed = (rgb[:, :, 0].astype(np.uint32) << 8) | (rgb[:, :, 1].astype(np.uint32) << 24) | (rgb[:, :, 2].astype(np.uint32) << 16)
    (tmp_path / "masks32.bmp").write_bytes(_bmp(w, h, 32, [packed[y].astype("<u4").tobytes() for y in range(h)], compression=3,
                                                masks=struct.pack("<III", 0x0000FF00, 0xFF000000, 0x00FF0000)))
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "masks32.bmp"), want)


def test_bmp_reader_rejects_damage(xad, tmp_path):
    rgb = np.random.default_rng(13).integers(0, 256, (4, 4, 3), dtype=np.uint8)
    rows = [rgb[y].tobytes() for y in range(4)]
    good = _bmp(4, 4, 24, rows)
    table = bytes(range(16))  # four entries
    cases = {
        "run_length": (_bmp(4, 4, 8, [bytes(4)] * 4, palette=table, compression=1), "compressed"),
        "short": (good[:-5], "shorter"),
        "depth": (_bmp(4, 4, 7, rows), "bit depth"),
        "empty": (_bmp(0, 4, 24, rows), "size"),
        "huge": (_bmp(70000, 70000, 24, rows), "size"),
        "index": (_bmp(4, 4, 8, [bytes([0, 1, 2, 9])] * 4, palette=table), "colour index"),
        "table": (_bmp(4, 4, 8, [bytes(4)] * 4, palette=table)[:60], "colour table"),
        "header": (b"BM" + bytes(12) + struct.pack("<I", 13) + bytes(40), "header"),
    }
    for name, (data, message) in cases.items():
        (tmp_path / (name + ".bmp")).write_bytes(data)
        with pytest.raises(xad.XadError, match=message):
            trainer.load_image(tmp_path / (name + ".bmp"))


# ---- JPEG -----------------------------------------------------------------------------

def _scene(width, height, seed):
    """Smooth blobs, noise, a sharp white bar and a thin coloured line: what a transform codec finds easy and hard."""
    rng = np.random.default_rng(seed)
    y, x = np.mgrid[0:height, 0:width].astype(np.float64)
    image = np.zeros((height, width, 3))
    for _ in range(12):
        cx, cy, s = rng.uniform(0, width), rng.uniform(0, height), rng.uniform(3, 3 + width / 3)
        image += np.exp(-((x - cx) ** 2 + (y - cy) ** 2) / (2 * s * s))[..., None] * rng.uniform(0, 1, 3)
    image = image / image.max() + rng.normal(0, 0.02, image.shape)
    image[height // 3:height // 3 + 5] = 1.0
    image[:, width // 2:width // 2 + 2, 0] = 0.0
    return (np.clip(image, 0, 1) * 255).astype(np.uint8)


def _pillow_jpeg(pixels, **options):
    from PIL import Image

    buffer = io.BytesIO()
    Image.fromarray(pixels).save(buffer, "JPEG", **options)
    return buffer.getvalue()


def _pillow_decode(data):
    from PIL import Image

    return np.asarray(Image.open(io.BytesIO(data)).convert("RGB")).astype(np.int32)


def _load_levels(path):
    return np.rint(trainer.load_image(path) * np.float32(255)).astype(np.int32)


def _psnr(a, b):
    return 10 * np.log10(255.0 ** 2 / max(np.mean((a.astype(np.float64) - b) ** 2), 1e-12))


JPEG_KINDS = [{}, {"progressive": True}, {"optimize": True}, {"restart_marker_blocks": 3}, {"progressive": True, "restart_marker_rows": 1}]


@pytest.mark.parametrize("size", [(64, 48), (33, 17), (1, 1), (7, 100), (257, 131)])
def test_jpeg_reader_against_pillow(xad, tmp_path, size):
    """Every kind of file Pillow writes: sequential and progressive, default and optimised Huffman tables, restart
    intervals, chroma at full, half-horizontal, half-both and quarter-horizontal rate, grey; image sizes that are
    not multiples of the coding unit.  Both decoders are conforming; they may differ by rounding."""
    width, height = size
    source = _scene(width, height, width * 1000 + height)
    path = tmp_path / "file.jpg"
    for grey in (False, True):
        pixels = source[:, :, 0] if grey else source
        for quality, kind in itertools.product((30, 75, 90, 100), JPEG_KINDS):
            for subsampling in ((None,) if grey else (0, 1, 2, "4:1:1")):
                options = dict(quality=quality, **kind)
                if subsampling is not None:
                    options["subsampling"] = subsampling
                data = _pillow_jpeg(pixels, **options)
                path.write_bytes(data)
                got, want = _load_levels(path), _pillow_decode(data)
                assert got.shape == want.shape == (height, width, 3), options
                difference = np.abs(got - want)
                assert difference.max() <= 4 and difference.mean() <= 0.3, (options, difference.max(), difference.mean())
                # and near the source where the file is: a wrong table, sign or scan would be tens of levels off
                if quality == 100 and subsampling in (None, 0):
                    assert np.abs(got - (np.repeat(pixels[:, :, None], 3, 2) if grey else pixels)).mean() < 2.0


def test_jpeg_reader_progressive_is_exactly_sequential(xad, tmp_path):
    # the same coefficients reach the decoder in one scan or in ten: the samples must be the same to the bit
    source = _scene(120, 90, 4)
    for subsampling, quality in itertools.product((0, 2), (40, 95)):
        (tmp_path / "s.jpg").write_bytes(_pillow_jpeg(source, quality=quality, subsampling=subsampling))
        (tmp_path / "p.jpg").write_bytes(_pillow_jpeg(source, quality=quality, subsampling=subsampling, progressive=True))
        np.testing.assert_array_equal(trainer.load_image(tmp_path / "s.jpg"), trainer.load_image(tmp_path / "p.jpg"))


def test_jpeg_reader_colour_spaces(xad, tmp_path):
    source = _scene(40, 30, 2)
    data = _pillow_jpeg(source, quality=95, subsampling=0)
    assert data[2:4] == b"\xff\xe0" and data[6:11] == b"JFIF\0"
    length = int.from_bytes(data[4:6], "big")
    # the same coefficients declared as RGB by an Adobe segment (transform 0) in place of the JFIF one
    adobe = b"\xff\xee" + (14).to_bytes(2, "big") + b"Adobe" + bytes([0, 100, 0, 0, 0, 0, 0])
    crafted = data[:2] + adobe + data[4 + length:]
    (tmp_path / "rgb.jpg").write_bytes(crafted)
    assert np.abs(_load_levels(tmp_path / "rgb.jpg") - _pillow_decode(crafted)).max() <= 2
    # ... and as YCbCr by transform 1
    crafted = data[:2] + adobe[:-1] + b"\x01" + data[4 + length:]
    (tmp_path / "ycc.jpg").write_bytes(crafted)
    assert np.abs(_load_levels(tmp_path / "ycc.jpg") - _pillow_decode(data)).max() <= 3
    # a comment and an unknown application segment are stepped over
    extra = data[:2] + b"\xff\xfe\x00\x07hello" + b"\xff\xe5\x00\x04ab" + data[2:]
    (tmp_path / "extra.jpg").write_bytes(extra)
    (tmp_path / "plain.jpg").write_bytes(data)
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "extra.jpg"), trainer.load_image(tmp_path / "plain.jpg"))


def test_jpeg_reader_rejects_what_it_does_not_read(xad, tmp_path):
    from PIL import Image

    source = _scene(48, 32, 1)
    good = _pillow_jpeg(source, quality=80)
    frame = good.index(b"\xff\xc0")
    buffer = io.BytesIO()
    Image.new("CMYK", (16, 16)).save(buffer, "JPEG")
    cases = {
        "cmyk": (buffer.getvalue(), "four-component"),
        "arithmetic": (good[:frame] + b"\xff\xc9" + good[frame + 2:], "arithmetic"),
        "lossless": (good[:frame] + b"\xff\xc3" + good[frame + 2:], "lossless"),
        "twelve_bit": (good[:frame + 4] + b"\x0c" + good[frame + 5:], "8-bit"),
        "no_tables": (good[:2] + good[frame:], "not defined"),
        "cut_in_header": (good[:frame + 6], None),
        "cut_in_data": (good[:len(good) * 2 // 3], "ends inside the compressed data"),
        "only_start": (b"\xff\xd8\xff\xd9", "no frame header"),
    }
    for name, (data, message) in cases.items():
        path = tmp_path / (name + ".jpg")
        path.write_bytes(data)
        with pytest.raises(xad.XadError, match=message):
            trainer.load_image(path)
    # a file that lacks only its end marker is complete
    (tmp_path / "no_end.jpg").write_bytes(good[:-2])
    (tmp_path / "good.jpg").write_bytes(good)
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "no_end.jpg"), trainer.load_image(tmp_path / "good.jpg"))


def _jpeg_segments(data):
    """marker -> list of payloads, up to the first scan."""
    out, pos = {}, 2
    while data[pos + 1] != 0xDA:
        assert data[pos] == 0xFF
        length = int.from_bytes(data[pos + 2:pos + 4], "big")
        out.setdefault(data[pos + 1], []).append(data[pos + 4:pos + 2 + length])
        pos += 2 + length
    return out


@pytest.mark.parametrize("size", [(64, 48), (33, 17), (1, 1), (257, 131)])
def test_jpeg_writer_against_pillow(xad, tmp_path, size):
    """Pillow reads the writer's files; they are as close to the source and as large as Pillow's own files of the
    same image, quality and chroma rate; quantisation and Huffman tables are the ones libjpeg writes (annex K)."""
    from PIL import Image

    width, height = size
    source = _scene(width, height, 5)
    image = source.astype(np.float32) / np.float32(255)
    for quality in (10, 50, 90, 95, 100):
        path = tmp_path / ("q%d.jpg" % quality)
        trainer.save_image(path, image, quality=quality)
        data = path.read_bytes()
        opened = Image.open(io.BytesIO(data))
        assert opened.size == (width, height) and opened.mode == "RGB"
        half_rate = quality <= 90  # chroma at half the rate each way up to 90, full rate above (the reference's writer)
        own_layers = [(1, 2 if half_rate else 1), (2, 1), (3, 1)]
        assert [(c[0], c[1]) for c in opened.layer] == own_layers and all(c[1] == c[2] for c in opened.layer)
        theirs = _pillow_jpeg(source, quality=quality, subsampling=2 if half_rate else 0)
        assert opened.quantization == Image.open(io.BytesIO(theirs)).quantization
        tables = [sorted(t for seg in _jpeg_segments(d)[0xC4] for t in _split_tables(seg)) for d in (data, theirs)]
        assert len(tables[0]) == 4 and tables[0] == tables[1]
        decoded, reference = _pillow_decode(data), _pillow_decode(theirs)
        if width > 1:
            assert _psnr(decoded, source) > _psnr(reference, source) - 0.3, quality
            assert len(data) < 1.1 * len(theirs) + 64, quality
        # and the reader reads the writer
        assert np.abs(_load_levels(path) - decoded).max() <= 4


def _split_tables(segment):
    """The tables of one define-Huffman-tables segment, each as a segment of its own (libjpeg may write several in one)."""
    out, pos = [], 0
    while pos < len(segment):
        count = sum(segment[pos + 1:pos + 17])
        out.append(segment[pos:pos + 17 + count])
        pos += 17 + count
    return out


def test_jpeg_writer_by_extension_and_quantisation(xad, tmp_path):
    # .jpg and .jpeg: quality 90 (image_utils.h:21); input is clamped and rounded like the other formats (image_utils.cpp:42-46)
    rng = np.random.default_rng(8)
    image = (_scene(50, 40, 3).astype(np.float32) / np.float32(255) * np.float32(1.4) - np.float32(0.2)).astype(np.float32)
    image[0, 0] = [np.nan, np.inf, -np.inf]
    trainer.save_image(tmp_path / "a.jpg", image)
    trainer.save_image(tmp_path / "b.JPEG", image)
    trainer.save_image(tmp_path / "c.jpg", image, quality=90)
    assert (tmp_path / "a.jpg").read_bytes() == (tmp_path / "b.JPEG").read_bytes() == (tmp_path / "c.jpg").read_bytes()
    clamped = np.where(image > 0, np.minimum(image, np.float32(1)), np.float32(0)).astype(np.float32)
    bytes_in = (clamped * np.float32(255) + np.float32(0.5)).astype(np.uint8)
    own = _psnr(_pillow_decode((tmp_path / "a.jpg").read_bytes()), bytes_in)
    assert own > _psnr(_pillow_decode(_pillow_jpeg(bytes_in, quality=90, subsampling=2)), bytes_in) - 0.3 and own > 20
    trainer.save_image(tmp_path / "d.png", image, quality=100)  # save_image_jpeg: a JPEG whatever the name
    assert (tmp_path / "d.png").read_bytes()[:2] == b"\xff\xd8"
    for bad in (0, 101):
        with pytest.raises(xad.XadError, match="quality"):
            trainer.save_image(tmp_path / "e.jpg", image, quality=bad)
    del rng
