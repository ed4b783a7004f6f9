"""The MNIST reader of the host side (dlmi::MNIST; the reference's is
data/dataset/mnist.cpp:56-227, which needs fmt and the Boost-based File helpers and
cannot be compiled here).  What pins it: the IDX format is a published one
(big-endian int32 header: magic 2051 / 2049, count[, rows, cols], then unsigned
bytes), and the reference's mapping is closed-form: pixel / 255 as float, one-hot
labels over ten classes, train pair for ENV::TRAIN and the t10k pair otherwise.
The files here are synthetic ones of that shape (there is no network to fetch the
real set).  Host code only: no GPU involved."""
import ctypes
import struct

import numpy as np
import pytest

from conftest import load_package


@pytest.fixture(scope="module")
def lib():
    pkg = load_package()
    return ctypes.CDLL(pkg.LIB_PATH)


def write_idx(dirname, prefix, images, labels, image_magic=2051, label_magic=2049, announce=None):
    n, r, c = images.shape
    with open(dirname / f"{prefix}-images-idx3-ubyte", "wb") as f:
        f.write(struct.pack(">iiii", image_magic, n if announce is None else announce, r, c))
        f.write(images.astype(np.uint8).tobytes())
    with open(dirname / f"{prefix}-labels-idx1-ubyte", "wb") as f:
        f.write(struct.pack(">ii", label_magic, labels.size))
        f.write(labels.astype(np.uint8).tobytes())


def test_reads_idx_pair(lib, tmp_path):
    from deep_learning_amd.model import load_mnist
    rng = np.random.default_rng(0)
    tr_img, tr_lab = rng.integers(0, 256, (37, 28, 28)), rng.integers(0, 10, 37)
    te_img, te_lab = rng.integers(0, 256, (5, 28, 28)), rng.integers(0, 10, 5)
    tr_img[0, 0, :3] = (0, 255, 128)
    write_idx(tmp_path, "train", tr_img, tr_lab)
    write_idx(tmp_path, "t10k", te_img, te_lab)
    for train, img, lab in ((True, tr_img, tr_lab), (False, te_img, te_lab)):
        X, Y = load_mnist(lib, tmp_path, train=train)
        assert X.shape == (img.shape[0], 784) and Y.shape == (img.shape[0], 10)
        # float(byte) / 255.0f, row-major pixels (mnist.cpp:176-181)
        assert np.array_equal(X, (img.reshape(-1, 784).astype(np.float32) / np.float32(255)))
        assert np.array_equal(Y, np.eye(10, dtype=np.float32)[lab])
    X, _ = load_mnist(lib, tmp_path, train=True)
    assert X[0, 0] == 0.0 and X[0, 1] == 1.0 and X[0, 2] == np.float32(128) / np.float32(255)


def test_other_geometry(lib, tmp_path):
    """Rows and columns come from the header, not from a constant."""
    from deep_learning_amd.model import load_mnist
    img = np.arange(3 * 4 * 6).reshape(3, 4, 6) % 256
    write_idx(tmp_path, "train", img, np.array([9, 0, 4]))
    X, Y = load_mnist(lib, tmp_path)
    assert X.shape == (3, 24) and np.array_equal(np.argmax(Y, 1), [9, 0, 4])
    assert np.array_equal(np.rint(X * 255).astype(int), img.reshape(3, 24))


@pytest.mark.parametrize("case", ["missing", "bad_image_magic", "bad_label_magic", "count_mismatch", "truncated", "empty",
                                  "bad_label"])
def test_refusals(lib, tmp_path, case):
    from deep_learning_amd.model import load_mnist
    img, lab = np.zeros((4, 2, 2), int), np.array([1, 2, 3, 4])
    if case == "bad_image_magic":
        write_idx(tmp_path, "train", img, lab, image_magic=2049)
    elif case == "bad_label_magic":
        write_idx(tmp_path, "train", img, lab, label_magic=2051)
    elif case == "count_mismatch":
        write_idx(tmp_path, "train", img, lab[:3])
    elif case == "truncated":
        write_idx(tmp_path, "train", img, lab, announce=5)
    elif case == "empty":
        write_idx(tmp_path, "train", img[:0], lab[:0])
    elif case == "bad_label":
        write_idx(tmp_path, "train", img, np.array([1, 2, 10, 4]))
    with pytest.raises(RuntimeError, match="MNIST::load failed"):
        load_mnist(lib, tmp_path)
