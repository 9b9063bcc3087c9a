"""Image stacks on disk as a torch Dataset of (input, target) pairs
(reference image_dataset.py:13-382).

Same interface and conventions as the reference: a path specifier is a file, a
directory or a glob pattern; files are ordered naturally ("scan2" before
"scan10"); every item is a C x H x W tensor, float32 unless ``labels`` asks for
integral class indices.

The readers are chosen when an image is read, not when the module is imported,
so the package imports on a machine without the optional image libraries:

* ``.tif`` / ``.tiff``: ``tifffile`` when it is installed, otherwise the reader
  in this file, which understands uncompressed strip-based TIFF (any integer or
  float sample type, several samples per pixel, several pages) - what tomography
  pipelines usually write;
* ``.npy``: ``numpy.load`` (an addition; nothing is unpickled);
* anything else: ``imageio`` when it is installed, otherwise Pillow.
"""
import logging
import re
import struct
from collections.abc import Iterable
from pathlib import Path

import numpy as np
import torch
from torch.utils.data import Dataset

from .errors import InputError

_TIFF_SUFFIXES = (".tif", ".tiff")


def _natural_sort(names):
    """Sort strings so that embedded numbers compare by value."""
    def key(name):
        return [int(part) if part.isdigit() else part for part in re.split(r"(\d+)", name)]

    return sorted(names, key=key)


def _convert_to_integral(img):
    """Unsigned and boolean arrays pass (booleans as uint8), signed integers are
    reinterpreted as uint64 with a warning, anything else is an InputError
    (reference image_dataset.py:22-43)."""
    kind = img.dtype.kind
    if kind == "u":
        return img
    if kind == "b":
        return img.astype(np.uint8)
    if kind == "i":
        logging.warning("Converting signed integer image to unsigned integer.")
        return img.astype(np.uint64)
    raise InputError(f"Image could not be converted to an integral value. Its type is {img.dtype}.")


def _relabel_image(img, labels):
    """``labels`` a collection: value ``labels[i]`` becomes ``i`` and any other value is
    an InputError.  ``labels`` an int k: values must already lie in 0..k-1
    (reference image_dataset.py:46-67)."""
    img = _convert_to_integral(img)
    if isinstance(labels, Iterable):
        labels = list(labels)
        unexpected = set(np.unique(img).tolist()) - set(labels)
        if unexpected:
            raise InputError(f"Encountered unexpected values {unexpected} that are not in the label set.")
        out = img.copy()
        for index, value in enumerate(labels):
            out[img == value] = index
        return out
    low, high = img.min(), img.max()
    if low < 0 or labels <= high:
        raise InputError(f"Image pixel value range {[low, high]} exceeded range {[0, labels - 1]}.")
    return img


# ---- built-in reader for uncompressed TIFF -------------------------------------------------

_TIFF_TYPE_CODES = {1: "B", 2: "c", 3: "H", 4: "I", 5: "II", 6: "b", 8: "h", 9: "i", 10: "ii",
                    11: "f", 12: "d", 16: "Q", 17: "q", 18: "Q"}


def _read_tiff_uncompressed(path):
    """All pages of a classic or Big TIFF file whose pixel data is stored uncompressed in
    strips, as one array: (H, W) or (H, W, S) for a single page, pages stacked in front
    otherwise.  Tiled or compressed files raise ValueError naming what is needed."""
    data = Path(path).read_bytes()
    if data[:2] == b"II":
        bo = "<"
    elif data[:2] == b"MM":
        bo = ">"
    else:
        raise ValueError("not a TIFF file")
    magic = struct.unpack_from(bo + "H", data, 2)[0]
    if magic == 42:
        big, offset = False, struct.unpack_from(bo + "I", data, 4)[0]
    elif magic == 43:
        big, offset = True, struct.unpack_from(bo + "Q", data, 8)[0]
    else:
        raise ValueError("not a TIFF file")
    count_fmt, entry_size, inline, off_fmt = ("Q", 20, 8, "Q") if big else ("H", 12, 4, "I")

    def directory(at):
        n = struct.unpack_from(bo + count_fmt, data, at)[0]
        at += struct.calcsize(count_fmt)
        tags = {}
        for i in range(n):
            entry = at + i * entry_size
            tag, typ = struct.unpack_from(bo + "HH", data, entry)
            cnt = struct.unpack_from(bo + off_fmt, data, entry + 4)[0]
            code = _TIFF_TYPE_CODES.get(typ)
            if code is None:
                continue
            fmt = bo + code * cnt if len(code) == 1 else bo + code[0] * (2 * cnt)
            value_at = entry + 4 + struct.calcsize(off_fmt)
            if struct.calcsize(fmt) > inline:
                value_at = struct.unpack_from(bo + off_fmt, data, value_at)[0]
            tags[tag] = struct.unpack_from(fmt, data, value_at)
        return tags, struct.unpack_from(bo + off_fmt, data, at + n * entry_size)[0]

    pages = []
    seen = set()
    while offset and offset not in seen:
        seen.add(offset)
        tags, offset = directory(offset)
        if 256 not in tags or 257 not in tags:
            continue
        if tags.get(259, (1,))[0] != 1:
            raise ValueError("compressed TIFF: install tifffile to read it")
        if 273 not in tags:
            raise ValueError("tiled TIFF: install tifffile to read it")
        width, height = tags[256][0], tags[257][0]
        samples = tags.get(277, (1,))[0]
        bits = tags.get(258, (1,))[0]
        kind = {1: "u", 2: "i", 3: "f"}.get(tags.get(339, (1,))[0], "u")
        if bits % 8 or (kind == "f" and bits not in (16, 32, 64)) or bits not in (8, 16, 32, 64):
            raise ValueError(f"{bits}-bit samples: install tifffile to read them")
        dtype = np.dtype(f"{bo}{kind}{bits // 8}")
        planar = tags.get(284, (1,))[0] == 2 and samples > 1
        need = width * height * samples * dtype.itemsize
        counts = tags.get(279, (need,) if len(tags[273]) == 1 else None)
        if counts is None:
            raise ValueError("TIFF strips without byte counts")
        raw = b"".join(data[o:o + c] for o, c in zip(tags[273], counts))
        if len(raw) < need:
            raise ValueError("truncated TIFF pixel data")
        arr = np.frombuffer(raw[:need], dtype=dtype)
        if samples == 1:
            arr = arr.reshape(height, width)
        elif planar:
            arr = arr.reshape(samples, height, width)
        else:
            arr = arr.reshape(height, width, samples)
        pages.append(arr.astype(dtype.newbyteorder("=")))
    if not pages:
        raise ValueError("no image in TIFF file")
    return pages[0] if len(pages) == 1 else np.stack(pages)


def write_tiff(path, array):
    """Write a 2-D array as a one-page, or a 3-D array as a multi-page (page, H, W),
    uncompressed little-endian TIFF that any TIFF reader opens.  For saving predictions
    and making test data without an image library; use ``tifffile`` for anything more."""
    array = np.asarray(array)
    if array.ndim == 2:
        array = array[None]
    if array.ndim != 3:
        raise ValueError("write_tiff expects a 2-D image or a 3-D stack of pages")
    if array.dtype == np.bool_:
        array = array.astype(np.uint8)
    fmt = {"u": 1, "i": 2, "f": 3}.get(array.dtype.kind)
    if fmt is None or (fmt == 3 and array.dtype.itemsize < 4):
        raise ValueError(f"write_tiff cannot store {array.dtype}")
    array = np.ascontiguousarray(array.astype(array.dtype.newbyteorder("<")))
    pages, height, width = array.shape
    nbytes = height * width * array.dtype.itemsize
    entries = 9
    ifd_size = 2 + 12 * entries + 4
    if 8 + pages * (ifd_size + nbytes) >= 2 ** 32:
        raise ValueError("too large for a classic TIFF file")
    out = bytearray(b"II" + struct.pack("<HI", 42, 8))
    for page in range(pages):
        here = len(out)
        pixels = here + ifd_size
        last = page == pages - 1
        out += struct.pack("<H", entries)
        for tag, typ, value in ((256, 4, width), (257, 4, height), (258, 3, 8 * array.dtype.itemsize),
                                (259, 3, 1), (262, 3, 1), (273, 4, pixels), (278, 4, height),
                                (279, 4, nbytes), (339, 3, fmt)):
            out += struct.pack("<HHI", tag, typ, 1) + struct.pack("<I" if typ == 4 else "<HH", *((value,) if typ == 4 else (value, 0)))
        out += struct.pack("<I", 0 if last else pixels + nbytes)
        out += array[page].tobytes()
    Path(path).write_bytes(bytes(out))


def _load_tiff(path):
    try:
        import tifffile
    except ImportError:
        return _read_tiff_uncompressed(path)
    return np.array(tifffile.imread(path))


def _load_natural_image(path):
    """PNG, JPEG, ...: H x W or H x W x C from the reader; colour images get their first
    and last axes swapped, as the reference does (image_dataset.py:70-78), so the
    channels lead (C x W x H)."""
    try:
        import imageio
        img = np.array(imageio.imread(path))
    except ImportError:
        try:
            from PIL import Image
        except ImportError:
            raise ImportError("reading this file type needs imageio or Pillow") from None
        with Image.open(path) as im:
            img = np.array(im)
    if img.ndim == 3 and img.shape[2] in (1, 3, 4):
        return img.swapaxes(0, 2)
    return img


def _load_image(path):
    suffix = Path(path).suffix.lower()
    if suffix in _TIFF_SUFFIXES:
        return _load_tiff(path)
    if suffix == ".npy":
        return np.load(path, allow_pickle=False)
    return _load_natural_image(path)


class ImageStack(object):
    """The images that match one path specifier, indexable; ``stack[i]`` is a
    C x H x W tensor (reference image_dataset.py:81-262).

    ``path_specifier``: a directory (all files in it), a single file, or a pattern
    with ``*`` in its last component; ``~`` is expanded.
    ``collapse_channels``: average the channels into one.
    ``labels``: ``None`` for float32 images; an int k for class images with values
    0..k-1; a collection of values to be renumbered 0, 1, ... in its order."""

    def __init__(self, path_specifier, *, collapse_channels=False, labels=None):
        super().__init__()
        self.path_specifier = Path(path_specifier).expanduser().resolve()
        self.collapse_channels = collapse_channels
        self.labels = labels
        self.paths = ImageStack.find_images(self.path_specifier)

    @staticmethod
    def find_images(path_specifier):
        spec = Path(path_specifier)
        if spec.name and "*" in spec.name:
            found = spec.parent.glob(spec.name)
        elif spec.is_file():
            found = [spec]
            logging.warning(f"Image stack consists of single file {spec}")
        elif spec.is_dir():
            found = spec.glob("*")
        else:
            found = []
        paths = _natural_sort([str(p) for p in found])
        if not paths:
            logging.warning(f"Image stack is empty for path specification {spec}")
        return paths

    @property
    def num_labels(self):
        """Number of classes; RuntimeError for a stack without labels."""
        if self.labels is None:
            raise RuntimeError("This image stack has no labels")
        if isinstance(self.labels, Iterable):
            return len(list(self.labels))
        return int(self.labels)

    def __len__(self):
        return len(self.paths)

    def __getitem__(self, i):
        path = self.paths[i]
        try:
            img = _load_image(path)
        except Exception as e:
            raise InputError(f"Could not read image from {path}. Got error {e}")
        if self.labels is None:
            img = img.astype(np.float32)
        else:
            try:
                img = _relabel_image(img, self.labels)
            except InputError as e:
                raise InputError(f"Expected labeled image from path {path}. Got error {e}")
        if img.ndim > 3:
            raise InputError(f"Image in {path} has more than 3 dimensions.")
        if img.ndim < 2:
            raise InputError(f"Image in {path} has less than 2 dimensions.")
        if img.ndim == 2:
            img = img[None]
        assert not (self.labels is not None and self.collapse_channels), \
            "Cannot collapse channels of segmentation image stack."
        if self.collapse_channels:
            img = img.mean(axis=0, keepdims=True)
        return torch.from_numpy(np.ascontiguousarray(img))


class ImageDataset(Dataset):
    """Pairs ``(input_stack[i], target_stack[i])`` (reference image_dataset.py:265-382).

    ``labels`` applies to the targets only (segmentation); ``collapse_channels``
    applies to the inputs, and to the targets when they are not labels.  Stacks of
    different length raise InputError."""

    def __init__(self, input_path_specifier, target_path_specifier, *, collapse_channels=False, labels=None):
        super().__init__()
        self.input_path_specifier = input_path_specifier
        self.target_path_specifier = target_path_specifier
        self.collapse_channels = collapse_channels
        self.labels = labels
        self.input_stack = ImageStack(input_path_specifier, collapse_channels=collapse_channels)
        self.target_stack = ImageStack(target_path_specifier,
                                       collapse_channels=collapse_channels and labels is None, labels=labels)
        if len(self.input_stack) != len(self.target_stack):
            raise InputError("Number of input and target images does not match. "
                             f"Got {len(self.input_stack)} input images and "
                             f"{len(self.target_stack)} target images.")

    def __len__(self):
        return len(self.input_stack)

    def __getitem__(self, i):
        return self.input_stack[i], self.target_stack[i]

    @property
    def num_labels(self):
        """Number of classes of the targets; RuntimeError when they are not labels."""
        return self.target_stack.num_labels
