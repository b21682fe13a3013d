"""Dataset readers and the accuracy check of the reference's host side, in numpy.

Same names, argument meaning, layouts and float32 arithmetic as data.h:36-119 / data.cpp and
utility.h:198-233 of the reference; the C++ twin is host/tcbnn_data.hpp and the two agree bit
for bit on the same files.  ImageNet images are decoded with PIL when it is importable (any
format it reads), binary PPM otherwise.
"""
import struct

import numpy as np

_F = np.float32


def _read_exact(f, n, path):
    b = f.read(n)
    if len(b) != n:
        raise IOError("File '%s' ended early." % path)
    return b


def _mnist_bytes(filename, labelname, batch):
    with open(filename, "rb") as f:
        struct.unpack(">4i", _read_exact(f, 16, filename))  # magic, count, rows, cols: not checked (data.cpp:57-64)
        px = np.frombuffer(_read_exact(f, batch * 784, filename), dtype=np.uint8).reshape(batch, 28, 28)
    with open(labelname, "rb") as f:
        struct.unpack(">2i", _read_exact(f, 8, labelname))
        lab = np.frombuffer(_read_exact(f, batch, labelname), dtype=np.uint8).astype(np.uint32)
    return px, lab


def read_MNIST_raw(filename, labelname, batch):
    """[batch][28][28] uint8 and uint32 labels (data.cpp:28-110)."""
    return _mnist_bytes(filename, labelname, batch)


def read_MNIST_normalized(filename, labelname, batch):
    """[batch][1][28][28] float32, (v/255 - 0.1307) / 0.3081 (data.cpp:112-194)."""
    px, lab = _mnist_bytes(filename, labelname, batch)
    img = ((px.astype(_F) / _F(255.0)) - _F(0.1307)) / _F(0.3081)
    return img.reshape(batch, 1, 28, 28), lab


def _cifar_records(filename, batch):
    with open(filename, "rb") as f:
        rec = np.frombuffer(_read_exact(f, batch * 3073, filename), dtype=np.uint8).reshape(batch, 3073)
    return rec[:, 1:].reshape(batch, 3, 32, 32), rec[:, 0].astype(np.uint32)


def read_CIFAR10_raw(filename, batch):
    """[batch][32][32] uint32 words, byte c = channel c, fourth byte 0 (data.cpp:198-245)."""
    chw, lab = _cifar_records(filename, batch)
    words = np.zeros((batch, 32, 32, 4), dtype=np.uint8)
    words[..., :3] = chw.transpose(0, 2, 3, 1)
    return words.view("<u4").reshape(batch, 32, 32), lab


def read_CIFAR10_normalized(filename, batch):
    """[batch][3][32][32] float32, (v/255 - mean_c) / std_c (data.cpp:248-316)."""
    chw, lab = _cifar_records(filename, batch)
    mean = np.array([0.4914, 0.4822, 0.4465], dtype=_F).reshape(1, 3, 1, 1)
    std = np.array([0.2470, 0.2435, 0.2616], dtype=_F).reshape(1, 3, 1, 1)
    return (chw.astype(_F) / _F(255.0) - mean) / std, lab


def imagenet_preprocess(hwc, out_h=224, out_w=224):
    """Decoded [H][W][3] uint8 image -> [3][out_h][out_w] float32: short side to 256 with the reference's
    byte-truncating bilinear resize (scale_transform, data.cpp:407-431), centre crop, normalise
    (data.cpp:478-552).  Only the pixels of the scaled image are computed; the reference's loop also
    writes one element past each row and one row past the end, which the crop never reads."""
    hwc = np.ascontiguousarray(hwc, dtype=np.uint8)
    org_h, org_w = hwc.shape[:2]
    scale = _F(256.0) / _F(min(org_w, org_h))
    if org_w < org_h:
        sw, sh = 256, int(scale * _F(org_h))
    else:
        sh, sw = 256, int(scale * _F(org_w))
    if sh < out_h or sw < out_w:
        raise ValueError("image %dx%d is too small for a %dx%d crop" % (org_h, org_w, out_h, out_w))
    chw = hwc.transpose(2, 0, 1).astype(_F)
    gx = np.arange(sw, dtype=_F) / _F(sw) * _F(org_w - 1)
    gy = np.arange(sh, dtype=_F) / _F(sh) * _F(org_h - 1)
    gxi, gyi = gx.astype(np.int64), gy.astype(np.int64)
    tx = (gx - gxi.astype(_F))[None, None, :]
    ty = (gy - gyi.astype(_F))[None, :, None]
    c00 = chw[:, gyi][:, :, gxi]
    c10 = chw[:, gyi][:, :, gxi + 1]
    c01 = chw[:, gyi + 1][:, :, gxi]
    c11 = chw[:, gyi + 1][:, :, gxi + 1]
    top = c00 + (c10 - c00) * tx
    bot = c01 + (c11 - c01) * tx
    scaled = (top + (bot - top) * ty).astype(np.uint8)  # values are in [0, 255]: the cast truncates like C
    y0, x0 = (sh - out_h) // 2, (sw - out_w) // 2
    crop = scaled[:, y0:y0 + out_h, x0:x0 + out_w].astype(_F)
    mul = np.array([4.3668, 4.4643, 4.4444], dtype=_F).reshape(3, 1, 1)
    sub = np.array([2.1179, 2.0357, 1.8044], dtype=_F).reshape(3, 1, 1)
    return (crop / _F(255.0)) * mul - sub


def _read_ppm(path):
    with open(path, "rb") as f:
        data = f.read()
    pos, vals = 0, []
    if data[:2] != b"P6":
        raise IOError("'%s' is not a binary PPM (P6) file." % path)
    pos = 2
    while len(vals) < 3:
        while pos < len(data) and data[pos:pos + 1].isspace():
            pos += 1
        if data[pos:pos + 1] == b"#":
            while pos < len(data) and data[pos:pos + 1] != b"\n":
                pos += 1
            continue
        end = pos
        while end < len(data) and not data[end:end + 1].isspace():
            end += 1
        vals.append(int(data[pos:end]))
        pos = end
    w, h, maxval = vals
    if maxval != 255 or w <= 0 or h <= 0 or len(data) < pos + 1 + 3 * w * h:
        raise IOError("'%s': unsupported PPM header or short file." % path)
    return np.frombuffer(data, dtype=np.uint8, count=3 * w * h, offset=pos + 1).reshape(h, w, 3)


def _decode(path):
    with open(path, "rb") as f:
        is_ppm = f.read(2) == b"P6"
    if is_ppm:
        return _read_ppm(path)
    from PIL import Image  # JPEG and the rest: needs PIL

    return np.asarray(Image.open(path).convert("RGB"))


def read_ImageNet_normalized(descfilename, batch):
    """[batch][3][224][224] float32 and uint32 labels from a list of "<image file>,<label>" lines
    (data.cpp:554-593)."""
    images = np.zeros((batch, 3, 224, 224), dtype=_F)
    labels = np.zeros(batch, dtype=np.uint32)
    with open(descfilename, "r") as f:
        entries = [ln.strip() for ln in f if ln.strip()]
    if len(entries) < batch:
        raise IOError("Imagenet Description File '%s' ended after %d of %d entries." % (descfilename, len(entries), batch))
    for i in range(batch):
        name, tag = entries[i].rsplit(",", 1)
        labels[i] = int(tag)
        images[i] = imagenet_preprocess(_decode(name.strip()))
    return images, labels


def score_prediction(prediction, labels):
    """(top1 correct, top5 correct, top-1 positions) of a [batch][categories] logit array, ranked the way
    validate_prediction does (utility.h:198-233): one pass keeps a best value and four runner-up slots,
    all starting at category 0's score; a value that beats the best replaces it without moving the old
    best down, otherwise the first slot it beats takes it.  "top-5" is therefore the reference's count,
    not the textbook one."""
    prediction = np.asarray(prediction, dtype=_F)
    top1 = top5 = 0
    positions = []
    for p, lab in zip(prediction, labels):
        best = [p[0]] * 5
        pos = [0] * 5
        for j, v in enumerate(p):
            for k in range(5):
                if v > best[k]:
                    best[k], pos[k] = v, j
                    break
        positions.append(pos[0])
        top1 += int(pos[0] == int(lab))
        top5 += int(int(lab) in pos)
    return top1, top5, positions


def validate_prediction(prediction, labels, categories=None, batch=None):
    """Prints the reference's report (utility.h:198-233) and returns (top-1 %, top-5 %)."""
    prediction = np.asarray(prediction, dtype=_F)
    if categories is not None and batch is not None:
        prediction = prediction.reshape(batch, categories)
    n = prediction.shape[0]
    top1, top5, positions = score_prediction(prediction, labels)
    print("======Label======")
    print(" ".join(str(int(v)) for v in labels[:n]) + " ")
    print("=====Predict=======")
    print(" ".join(str(v) for v in positions) + " ")
    print("=====Batch Accuracy:%d=======" % n)
    a1 = float(_F(top1) / _F(n) * _F(100))
    a5 = float(_F(top5) / _F(n) * _F(100))
    print("Top-1:%f%%" % a1)
    print("Top-5:%f%%" % a5)
    return a1, a5
