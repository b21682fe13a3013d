"""Dataset readers and the accuracy check (data.cpp / utility.h:198-233 of the reference): the numpy
mirror against what the file formats and the arithmetic fix, and the C++ twin against the mirror bit
for bit on the same files.  CPU only; the files are synthetic (the datasets are not distributed)."""
import os
import struct
import subprocess

import numpy as np
import pytest

from tcbnn_amd import data

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F = np.float32


@pytest.fixture(scope="module")
def cli(tmp_path_factory):
    """bin/read_dataset when built, else compiled here from the same sources with g++."""
    built = os.path.join(ROOT, "tcbnn_amd", "bin", "read_dataset")
    src = os.path.join(ROOT, "tcbnn_amd", "drivers", "read_dataset.cpp")
    hdr = os.path.join(ROOT, "tcbnn_amd", "host", "tcbnn_data.hpp")
    if os.path.exists(built) and os.path.getmtime(built) >= max(os.path.getmtime(src), os.path.getmtime(hdr)):
        return built
    exe = str(tmp_path_factory.mktemp("cli") / "read_dataset")
    subprocess.check_call(["g++", "-O2", "-std=c++17", src, "-o", exe])
    return exe


def _mnist_files(tmp_path, n, seed):
    rng = np.random.default_rng(seed)
    px = rng.integers(0, 256, size=(n, 28, 28), dtype=np.uint8)
    lab = rng.integers(0, 10, size=n, dtype=np.uint8)
    fi, fl = str(tmp_path / "img-idx3"), str(tmp_path / "lab-idx1")
    with open(fi, "wb") as f:
        f.write(struct.pack(">4i", 2051, n, 28, 28) + px.tobytes())
    with open(fl, "wb") as f:
        f.write(struct.pack(">2i", 2049, n) + lab.tobytes())
    return fi, fl, px, lab


def _cifar_file(tmp_path, n, seed):
    rng = np.random.default_rng(seed)
    chw = rng.integers(0, 256, size=(n, 3, 32, 32), dtype=np.uint8)
    lab = rng.integers(0, 10, size=n, dtype=np.uint8)
    path = str(tmp_path / "test_batch.bin")
    with open(path, "wb") as f:
        for i in range(n):
            f.write(bytes([lab[i]]) + chw[i].tobytes())
    return path, chw, lab


def _write_ppm(path, hwc, comment=False):
    h, w = hwc.shape[:2]
    with open(path, "wb") as f:
        f.write(b"P6\n" + (b"# made by a test\n" if comment else b"") + b"%d %d\n255\n" % (w, h) + hwc.tobytes())


def test_mnist_readers(tmp_path):
    fi, fl, px, lab = _mnist_files(tmp_path, 37, 1)
    raw, l0 = data.read_MNIST_raw(fi, fl, 20)
    assert np.array_equal(raw, px[:20]) and np.array_equal(l0, lab[:20])
    img, l1 = data.read_MNIST_normalized(fi, fl, 37)
    assert img.shape == (37, 1, 28, 28) and img.dtype == F and np.array_equal(l1, lab)
    # the 256 possible values, each through the reference's expression in float32, one scalar at a time
    table = np.array([(F(v) / F(255.0) - F(0.1307)) / F(0.3081) for v in range(256)], dtype=F)
    assert np.array_equal(img.reshape(37, 28, 28), table[px])
    # the published normalisation: mean 0.1307, std 0.3081 of v/255
    assert np.allclose(img.reshape(37, 28, 28) * 0.3081 + 0.1307, px / 255.0, atol=1e-6)
    with pytest.raises(IOError):
        data.read_MNIST_normalized(fi, fl, 38)


def test_cifar10_readers(tmp_path):
    path, chw, lab = _cifar_file(tmp_path, 9, 2)
    words, l0 = data.read_CIFAR10_raw(path, 9)
    assert words.shape == (9, 32, 32) and np.array_equal(l0, lab)
    for c in range(3):
        assert np.array_equal((words >> (8 * c)) & 0xFF, chw[:, c])
    assert np.all(words >> 24 == 0)
    img, l1 = data.read_CIFAR10_normalized(path, 5)
    assert img.shape == (5, 3, 32, 32) and img.dtype == F and np.array_equal(l1, lab[:5])
    mean, std = [0.4914, 0.4822, 0.4465], [0.2470, 0.2435, 0.2616]
    for c in range(3):
        table = np.array([(F(v) / F(255.0) - F(mean[c])) / F(std[c]) for v in range(256)], dtype=F)
        assert np.array_equal(img[:, c], table[chw[:5, c]])


def test_imagenet_preprocess_closed_forms():
    mul, sub = [4.3668, 4.4643, 4.4444], [2.1179, 2.0357, 1.8044]
    # a constant image stays constant through any interpolation
    const = np.empty((300, 411, 3), dtype=np.uint8)
    const[...] = [10, 128, 250]
    out = data.imagenet_preprocess(const)
    assert out.shape == (3, 224, 224)
    for c, v in enumerate([10, 128, 250]):
        assert np.all(out[c] == F(F(v) / F(255.0)) * F(mul[c]) - F(sub[c]))
    # a ramp along the width, portrait: width 200 -> 256, height 300 -> 384; bilinear on a linear ramp is the
    # ramp, truncation gives floor; crop offsets (384-224)/2 = 80 rows and 16 columns
    ramp = np.broadcast_to(np.arange(200, dtype=np.uint8)[None, :, None], (300, 200, 3))
    out = data.imagenet_preprocess(ramp)
    want = np.floor((np.arange(224) + 16) / 256.0 * 199.0)
    for c in range(3):
        got = np.rint((out[c].astype(np.float64) + sub[c]) / mul[c] * 255.0)
        assert np.array_equal(got, np.broadcast_to(want[None, :], (224, 224)))
    # a ramp along the height, landscape: height 200 -> 256, width 300 -> 384
    ramp = np.broadcast_to(np.arange(200, dtype=np.uint8)[:, None, None], (200, 300, 3))
    out = data.imagenet_preprocess(ramp)
    for c in range(3):
        got = np.rint((out[c].astype(np.float64) + sub[c]) / mul[c] * 255.0)
        assert np.array_equal(got, np.broadcast_to(want[:, None], (224, 224)))
    # channels are kept apart and in order
    rgb = np.zeros((256, 256, 3), dtype=np.uint8)
    rgb[..., 1] = 255
    out = data.imagenet_preprocess(rgb)
    assert np.all(out[0] == F(0) * F(mul[0]) - F(sub[0])) and np.all(out[1] == F(1) * F(mul[1]) - F(sub[1]))


def test_score_prediction():
    rng = np.random.default_rng(5)
    logits = rng.normal(size=(64, 50)).astype(F)
    labels = rng.integers(0, 50, size=64).astype(np.uint32)
    labels[:20] = np.argmax(logits[:20], axis=1)
    top1, top5, pos = data.score_prediction(logits, labels)
    assert pos == list(np.argmax(logits, axis=1))                     # strict ">" keeps the first maximum
    assert top1 == int(np.sum(np.argmax(logits, axis=1) == labels)) >= 20
    assert top5 >= top1
    # by hand: scores 1 5 4 3 2 9.  5 then 9 take the best slot (5 is dropped, not moved down); 4, 3, 2 cannot
    # beat slot 1 once it holds 4 ... slot1 <- 4, slot2 <- 3, slot3 <- 2; slot 4 keeps category 0
    one = np.array([[1, 5, 4, 3, 2, 9]], dtype=F)
    for lab, hit in [(5, True), (2, True), (3, True), (4, True), (0, True), (1, False)]:
        t1, t5, p = data.score_prediction(one, np.array([lab], dtype=np.uint32))
        assert p == [5] and t1 == int(lab == 5) and t5 == int(hit), lab
    # ties: an equal value never replaces
    assert data.score_prediction(np.zeros((1, 7), dtype=F), np.array([0], dtype=np.uint32))[:2] == (1, 1)
    assert data.score_prediction(np.zeros((1, 7), dtype=F), np.array([3], dtype=np.uint32))[:2] == (0, 0)


def test_cpp_readers_agree_with_the_mirror(tmp_path, cli):
    def run(*args):
        return subprocess.run([cli] + [str(a) for a in args], check=True, capture_output=True, text=True).stdout

    out_f, out_l = tmp_path / "x.f32", tmp_path / "l.u32"
    fi, fl, _, _ = _mnist_files(tmp_path, 33, 7)
    run("mnist", fi, fl, 33, out_f, out_l)
    img, lab = data.read_MNIST_normalized(fi, fl, 33)
    assert np.array_equal(np.fromfile(out_f, dtype=F), img.ravel())
    assert np.array_equal(np.fromfile(out_l, dtype=np.uint32), lab)

    path, _, _ = _cifar_file(tmp_path, 6, 8)
    run("cifar10", path, 6, out_f, out_l)
    img, lab = data.read_CIFAR10_normalized(path, 6)
    assert np.array_equal(np.fromfile(out_f, dtype=F), img.ravel())
    assert np.array_equal(np.fromfile(out_l, dtype=np.uint32), lab)

    rng = np.random.default_rng(9)
    shapes = [(256, 256), (231, 500), (375, 260), (480, 640)]
    with open(tmp_path / "list.csv", "w") as f:
        for i, (h, w) in enumerate(shapes):
            # smooth + noise, so that interpolation weights and truncation both matter
            yy, xx = np.mgrid[0:h, 0:w]
            base = (127 + 100 * np.sin(yy / 17.0 + i)[..., None] * np.cos(xx / 23.0)[..., None] * [1, 0.5, -1])
            img = np.clip(base + rng.integers(-25, 26, size=(h, w, 3)), 0, 255).astype(np.uint8)
            name = str(tmp_path / ("img%d.ppm" % i))
            _write_ppm(name, img, comment=(i == 1))
            f.write("%s,%d\n" % (name, 100 + i))
    run("imagenet", tmp_path / "list.csv", len(shapes), out_f, out_l)
    img, lab = data.read_ImageNet_normalized(str(tmp_path / "list.csv"), len(shapes))
    assert list(lab) == [100, 101, 102, 103]
    assert np.array_equal(np.fromfile(out_l, dtype=np.uint32), lab)
    assert np.array_equal(np.fromfile(out_f, dtype=F), img.ravel())

    logits = rng.normal(size=(40, 17)).astype(F)
    labels = rng.integers(0, 17, size=40).astype(np.uint32)
    labels[::3] = np.argmax(logits[::3], axis=1)
    logits.tofile(out_f)
    labels.tofile(out_l)
    text = run("validate", out_f, out_l, 17, 40)
    top1, top5, pos = data.score_prediction(logits, labels)
    lines = text.splitlines()
    assert lines[0] == "======Label======" and lines[1].split() == [str(int(v)) for v in labels]
    assert lines[3].split() == [str(v) for v in pos]
    assert lines[4] == "=====Batch Accuracy:40======="
    pct = lambda n: float(F(n) / F(40) * F(100))  # the reference prints float32
    assert lines[5] == "Top-1:%f%%" % pct(top1) and lines[6] == "Top-5:%f%%" % pct(top5)

    bad = subprocess.run([cli, "mnist", fi, fl, "34", str(out_f), str(out_l)], capture_output=True, text=True)
    assert bad.returncode == 1 and "ended early" in bad.stderr
    bad = subprocess.run([cli, "cifar10", str(tmp_path / "nope.bin"), "1", str(out_f), str(out_l)],
                         capture_output=True, text=True)
    assert bad.returncode == 1 and "Error in reading" in bad.stderr
