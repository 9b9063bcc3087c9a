"""ImageStack / ImageDataset: the behaviour the reference's tests/test_image_dataset.py
checks, on files written here without the optional image libraries (the package's own
TIFF writer, Pillow for PNG/JPEG when it is installed, numpy for .npy)."""
import logging

import numpy as np
import pytest
import torch

import msd_pytorch_amd.image_dataset as img_ds
from msd_pytorch_amd.errors import InputError

try:
    from PIL import Image
except ImportError:            # pragma: no cover - Pillow ships with this image
    Image = None


def test_convert_to_integral():
    # reference tests/test_image_dataset.py:11-20
    img = np.ones(10)
    assert np.mean(img_ds._convert_to_integral(img.astype(np.int8))) == 1
    assert np.mean(img_ds._convert_to_integral(img.astype(bool))) == 1
    assert img_ds._convert_to_integral(img.astype(bool)).dtype == np.uint8
    assert img_ds._convert_to_integral((-img).astype(np.int8)).dtype == np.uint64
    u = img.astype(np.uint16)
    assert img_ds._convert_to_integral(u) is u
    for t in (np.float16, np.float32, np.float64):
        with pytest.raises(InputError):
            img_ds._convert_to_integral(img.astype(t))


def test_relabel_image():
    # reference tests/test_image_dataset.py:23-41
    img0 = np.ones(10, dtype=np.uint8)
    assert img_ds._relabel_image(img0, 2).mean() == 1
    with pytest.raises(InputError):
        img_ds._relabel_image(img0 - 2, 2)        # wraps to 255
    img = img0 + 2
    with pytest.raises(InputError):
        img_ds._relabel_image(img, 2)
    with pytest.raises(InputError):
        img_ds._relabel_image(img, [2])
    assert img_ds._relabel_image(img, [3]).mean() == 0
    assert img_ds._relabel_image(img, 4).mean() == 3
    # a label set renumbers in its own order and leaves the argument alone
    mixed = np.array([5, 1, 2, 5], dtype=np.uint8)
    assert img_ds._relabel_image(mixed, [1, 2, 5]).tolist() == [2, 0, 1, 2]
    assert img_ds._relabel_image(mixed, [5, 2, 1]).tolist() == [0, 2, 1, 0]
    assert mixed.tolist() == [5, 1, 2, 5]
    assert img_ds._relabel_image(mixed, range(6)).tolist() == [5, 1, 2, 5]


def test_natural_sort():
    names = ["scan10.tif", "scan2.tif", "scan1.tif", "a_3_b_20", "a_3_b_3"]
    assert img_ds._natural_sort(names) == ["a_3_b_3", "a_3_b_20", "scan1.tif", "scan2.tif", "scan10.tif"]


def test_empty_stack(tmp_path, caplog):
    # reference tests/test_image_dataset.py:44-57
    with caplog.at_level(logging.WARNING):
        assert len(img_ds.ImageStack(tmp_path / "non_existing.tif")) == 0
        assert len(img_ds.ImageStack(tmp_path / "non_existing*.tif")) == 0
    assert len(caplog.record_tuples) == 2
    assert all(level == logging.WARNING and "empty" in msg for (_, level, msg) in caplog.record_tuples)


def test_stack_no_glob(tmp_path):
    # a directory is all its files; a file is itself (reference :60-63)
    img_ds.write_tiff(tmp_path / "image.tif", np.ones((10, 10)))
    assert len(img_ds.ImageStack(tmp_path)) == 1
    single = img_ds.ImageStack(tmp_path / "image.tif")
    assert len(single) == 1 and single[0].shape == (1, 10, 10) and single[0].dtype == torch.float32


@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.int16, np.uint32, np.float32, np.float64])
@pytest.mark.parametrize("byteorder", ["<", ">"])
def test_tiff_reader_round_trip(tmp_path, dtype, byteorder):
    rng = np.random.default_rng(1)
    a = (rng.random((3, 6, 9)) * 200).astype(dtype)
    img_ds.write_tiff(tmp_path / "s.tif", a)
    data = bytearray((tmp_path / "s.tif").read_bytes())
    assert bytes(data[:2]) == b"II"
    if byteorder == ">":
        # the same stack as one big-endian page with three planar samples, built by hand
        import struct
        be = a.astype(a.dtype.newbyteorder(">")).tobytes()
        fmt = {"u": 1, "i": 2, "f": 3}[a.dtype.kind]
        tags = [(256, 4, 9), (257, 4, 6), (258, 3, 8 * a.dtype.itemsize), (259, 3, 1), (273, 4, 8),
                (277, 3, 3), (279, 4, len(be)), (284, 3, 2), (339, 3, fmt)]
        out = b"MM" + struct.pack(">HI", 42, 8 + len(be)) + be + struct.pack(">H", len(tags))
        for tag, typ, value in tags:
            out += struct.pack(">HHI", tag, typ, 1) + (struct.pack(">I", value) if typ == 4 else struct.pack(">HH", value, 0))
        out += struct.pack(">I", 0)
        (tmp_path / "s.tif").write_bytes(out)
    b = img_ds._read_tiff_uncompressed(tmp_path / "s.tif")
    assert b.dtype == a.dtype and b.shape == a.shape and np.array_equal(a, b)
    img_ds.write_tiff(tmp_path / "p.tif", a[0])
    assert np.array_equal(img_ds._read_tiff_uncompressed(tmp_path / "p.tif"), a[0])


def test_tiff_reader_refuses_what_it_cannot_read(tmp_path):
    (tmp_path / "x.tif").write_bytes(b"not a tiff at all")
    with pytest.raises(ValueError):
        img_ds._read_tiff_uncompressed(tmp_path / "x.tif")
    with pytest.raises(InputError):
        img_ds.ImageStack(tmp_path / "x.tif")[0]
    with pytest.raises(ValueError):
        img_ds.write_tiff(tmp_path / "y.tif", np.zeros((2, 2), dtype=np.complex64))


@pytest.mark.skipif(Image is None, reason="needs Pillow")
def test_tiff_agrees_with_pillow(tmp_path):
    rng = np.random.default_rng(2)
    f = rng.random((5, 7)).astype(np.float32)
    img_ds.write_tiff(tmp_path / "ours.tif", f)
    assert np.array_equal(np.array(Image.open(tmp_path / "ours.tif")), f)
    Image.fromarray(f).save(tmp_path / "theirs.tif")
    assert np.array_equal(img_ds._read_tiff_uncompressed(tmp_path / "theirs.tif"), f)
    rgb = (rng.random((5, 7, 3)) * 255).astype(np.uint8)
    Image.fromarray(rgb).save(tmp_path / "rgb.tif")
    assert np.array_equal(img_ds._read_tiff_uncompressed(tmp_path / "rgb.tif"), rgb)
    u16 = (rng.random((5, 7)) * 60000).astype(np.uint16)
    Image.fromarray(u16).save(tmp_path / "u16.tif")
    assert np.array_equal(img_ds._read_tiff_uncompressed(tmp_path / "u16.tif"), u16)
    Image.fromarray(rgb).save(tmp_path / "lzw.tif", compression="tiff_lzw")
    with pytest.raises(ValueError, match="compressed"):
        img_ds._read_tiff_uncompressed(tmp_path / "lzw.tif")


def _write_colour_files(tmp_path, prefix, n, num_channels):
    """n colour images per format, as the reference's test writes them (:66-75)."""
    rng = np.random.default_rng(3)
    for i in range(n):
        img = rng.standard_normal((num_channels, 10, 10))
        u8 = np.clip(img * 60 + 128, 0, 255).astype(np.uint8)
        if Image is not None:
            Image.fromarray(u8.swapaxes(0, 2)).save(tmp_path / f"{prefix}imio_{i}.png")
            Image.fromarray(u8.swapaxes(0, 2)).save(tmp_path / f"{prefix}imio_{i}.jpeg")
        np.save(tmp_path / f"{prefix}npy_{i}.npy", img)
        img_ds.write_tiff(tmp_path / f"{prefix}tiff_{i}.tif", img)
        img_ds.write_tiff(tmp_path / f"{prefix}tiff2d_{i}.tif", img[0])
        img_ds.write_tiff(tmp_path / f"{prefix}tiff0_{i:05}.tif", img)


def test_image_stack(tmp_path):
    # reference tests/test_image_dataset.py:66-106
    num_channels, n = 3, 10
    _write_colour_files(tmp_path, "", n, num_channels)
    utiffs = img_ds.ImageStack(tmp_path / "tiff_*.tif")
    utiffs_c = img_ds.ImageStack(tmp_path / "tiff_*.tif", collapse_channels=True)
    utiffs_2d = img_ds.ImageStack(tmp_path / "tiff2d_*.tif")
    otiffs = img_ds.ImageStack(tmp_path / "tiff0_*.tif")
    npys = img_ds.ImageStack(tmp_path / "npy_*.npy")
    with pytest.raises(RuntimeError):
        utiffs.num_labels
    assert len(utiffs) == len(utiffs_2d) == len(otiffs) == len(npys) == n
    # natural order: ..._2 before ..._10 also without zero padding
    assert [p.rsplit("_", 1)[1] for p in utiffs.paths] == [f"{i}.tif" for i in range(n)]
    for i in range(n):
        assert utiffs[i].shape == (num_channels, 10, 10) and utiffs[i].dtype == torch.float32
        assert utiffs_2d[i].shape == (1, 10, 10)
        assert utiffs_c[i].shape == (1, 10, 10)
        assert torch.allclose(utiffs_c[i], utiffs[i].mean(0, keepdim=True))
        assert torch.equal(otiffs[i], utiffs[i])
        assert torch.equal(npys[i], utiffs[i])
        assert torch.equal(utiffs_2d[i][0], utiffs[i][0])
    if Image is not None:
        pngs = img_ds.ImageStack(tmp_path / "imio_*.png")
        pngs_c = img_ds.ImageStack(tmp_path / "imio_*.png", collapse_channels=True)
        jpegs = img_ds.ImageStack(tmp_path / "imio_*.jpeg")
        jpegs_c = img_ds.ImageStack(tmp_path / "imio_*.jpeg", collapse_channels=True)
        assert len(pngs) == len(pngs_c) == len(jpegs) == len(jpegs_c) == n
        for i in range(n):
            assert pngs[i].dim() == 3 and pngs[i].shape[0] == num_channels
            assert jpegs[i].dim() == 3 and jpegs[i].shape[0] == num_channels
            assert pngs_c[i].shape[0] == 1 and jpegs_c[i].shape[0] == 1
        # PNG is lossless: channel c of the stack item is channel c of what was written
        rng = np.random.default_rng(3)
        first = np.clip(rng.standard_normal((num_channels, 10, 10)) * 60 + 128, 0, 255).astype(np.uint8)
        assert torch.equal(pngs[0], torch.from_numpy(first.astype(np.float32)))


def test_image_stack_labels(tmp_path):
    # reference tests/test_image_dataset.py:109-141
    num_labels, n = 10, 10
    rng = np.random.default_rng(4)
    for i in range(n):
        img = rng.integers(num_labels, size=(1, 10, 10), dtype=np.uint8)
        img[0, 0, 0] = num_labels - 1              # every image holds the largest label
        img_ds.write_tiff(tmp_path / f"tiff_{i}.tif", img)
        img_ds.write_tiff(tmp_path / f"tiff2d_{i}.tif", img[0])
        img_ds.write_tiff(tmp_path / f"tiff0_{i:05}.tif", img)
    with pytest.raises(InputError):
        list(img_ds.ImageStack(tmp_path / "tiff0_*.tif", labels=range(9)))
    with pytest.raises(InputError):
        list(img_ds.ImageStack(tmp_path / "tiff0_*.tif", labels=9))
    utiffs = img_ds.ImageStack(tmp_path / "tiff_*.tif", labels=num_labels)
    utiffs_2d = img_ds.ImageStack(tmp_path / "tiff2d_*.tif", labels=num_labels)
    otiffs = img_ds.ImageStack(tmp_path / "tiff0_*.tif", labels=range(num_labels))
    for s in (utiffs, utiffs_2d, otiffs):
        assert len(s) == n and s.num_labels == num_labels
        for i in range(n):
            assert s[i].shape == (1, 10, 10) and not s[i].dtype.is_floating_point
            assert torch.equal(otiffs[i], s[i])
    with pytest.raises(AssertionError):
        img_ds.ImageStack(tmp_path / "tiff_*.tif", labels=num_labels, collapse_channels=True)[0]


def test_image_dataset(tmp_path):
    # reference tests/test_image_dataset.py:144-193
    num_channels, n = 3, 6
    _write_colour_files(tmp_path, "train_", n, num_channels)
    _write_colour_files(tmp_path, "val_", n, num_channels)
    utiffs = img_ds.ImageDataset(tmp_path / "train_tiff_*.tif", tmp_path / "val_tiff_*.tif")
    utiffs_c = img_ds.ImageDataset(tmp_path / "train_tiff_*.tif", tmp_path / "val_tiff_*.tif",
                                   collapse_channels=True)
    utiffs_2d = img_ds.ImageDataset(tmp_path / "train_tiff2d_*.tif", tmp_path / "val_tiff2d_*.tif")
    otiffs = img_ds.ImageDataset(tmp_path / "train_tiff0_*.tif", tmp_path / "val_tiff0_*.tif")
    with pytest.raises(RuntimeError):
        utiffs.num_labels
    assert len(utiffs) == len(utiffs_c) == len(utiffs_2d) == len(otiffs) == n
    for i in range(n):
        for j in (0, 1):
            assert utiffs[i][j].shape == (num_channels, 10, 10)
            assert utiffs_c[i][j].shape == (1, 10, 10)
            assert utiffs_2d[i][j].dim() == 3
            assert torch.equal(otiffs[i][j], utiffs[i][j])
    with pytest.raises(InputError):
        img_ds.ImageDataset(tmp_path / "train_tiff_*.tif", tmp_path / "val_tiff_1*.tif")
    # through a DataLoader: batches of B x C x H x W, labels on the target only
    rng = np.random.default_rng(5)
    for i in range(n):
        img_ds.write_tiff(tmp_path / f"lab_{i}.tif", rng.integers(3, size=(10, 10)).astype(np.uint8) * 2)
    seg = img_ds.ImageDataset(tmp_path / "train_tiff2d_*.tif", tmp_path / "lab_*.tif", labels=[0, 2, 4],
                              collapse_channels=True)
    assert seg.num_labels == 3
    x, y = next(iter(torch.utils.data.DataLoader(seg, batch_size=4)))
    assert x.shape == (4, 1, 10, 10) and x.dtype == torch.float32
    assert y.shape == (4, 1, 10, 10) and y.dtype == torch.uint8 and int(y.max()) <= 2
