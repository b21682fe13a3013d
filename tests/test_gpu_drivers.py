"""The C++ host layer (tcbnn_layers.hpp classes + drivers) against the CPU oracle: the driver
binaries read a weight file in the reference's text format and a raw input file, and their
logits must match the oracle's on the same data."""
import os
import subprocess

import numpy as np
import pytest

from oracle import nets as orc_nets

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tcbnn_amd", "bin")


def _write_weight_file(path, arrays):
    with open(path, "w") as f:
        for a in arrays:
            a = np.asarray(a, np.float32).ravel()
            if np.all(np.abs(a) == 1.0):
                f.write(" ".join("1" if v > 0 else "-1" for v in a))
            else:
                f.write(" ".join(repr(float(v)) for v in a))  # repr(float(float32)) round-trips
            f.write("\n")


def _run_driver(tmp_path, name, spec, extra, seed, variant, exact=True):
    import tcbnn_amd
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "%s is not built (run __graft_entry__.build())" % exe
    weights = tcbnn_amd.synthetic_weights(spec, seed)
    x = tcbnn_amd.synthetic_input(spec, seed)
    wf, xf, of = (str(tmp_path / n) for n in ("w.csv", "x.f32", "logits.f32"))
    _write_weight_file(wf, weights)
    x.astype(np.float32).tofile(xf)
    batch = spec[0]["batch"]
    cmd = [exe, "--batch", str(batch), "--weights", wf, "--input", xf, "--out", of, "--reps", "2", "--warmup", "1",
           "--variant", variant] + extra
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=280)
    assert proc.returncode == 0, proc.stdout
    classes = spec[-1]["out"]
    got = np.fromfile(of, np.float32).reshape(batch, classes)
    want = orc_nets.run(spec, weights, x)[spec[-1]["name"]]["out"]
    if exact:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)
        np.testing.assert_array_equal(got, want)
    else:  # fp32 head: 1e-5 of the logits' scale
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * float(np.abs(want).max()))
    return proc.stdout


@pytest.mark.parametrize("variant", ["popc", "mfma_f4"])
def test_mnist_mlp_driver(gpu, tmp_path, variant):
    from tcbnn_amd import nets
    out = _run_driver(tmp_path, "mnist_mlp", nets.mnist_mlp_spec(batch=200), [], 5, variant)
    assert '"net": "mnist_mlp"' in out


def test_cifar10_vgg_driver(gpu, tmp_path):
    from tcbnn_amd import nets
    _run_driver(tmp_path, "cifar10_vgg", nets.cifar10_vgg_spec(batch=8, image=16), ["--image", "16"], 6, "popc")


def test_imagenet_resnet_driver(gpu, tmp_path):
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_spec(batch=8, image=64, output_size=100)
    _run_driver(tmp_path, "imagenet_resnet", spec, ["--image", "64", "--classes", "100"], 7, "mfma_f4")


def test_imagenet_resnet_driver_packed_input(gpu, tmp_path):
    """The C++ classes with the packed first-layer input (the upload packs, the first layer reads without staging)."""
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_spec(batch=70, image=64, output_size=100)
    _run_driver(tmp_path, "imagenet_resnet", spec, ["--image", "64", "--classes", "100", "--packed-input"], 9, "mfma_f4")


def test_alexnet_driver(gpu, tmp_path):
    from tcbnn_amd import nets
    spec = nets.alexnet_spec(batch=8, image=96, output_size=100)
    _run_driver(tmp_path, "alexnet", spec, ["--image", "96", "--classes", "100"], 8, "mfma_f4")


def test_cifar10_resnet_driver(gpu, tmp_path):
    from tcbnn_amd import nets
    _run_driver(tmp_path, "cifar10_resnet", nets.cifar10_resnet_spec(batch=8), [], 9, "mfma_f4")


def test_imagenet_vgg_driver(gpu, tmp_path):
    from tcbnn_amd import nets
    spec = nets.imagenet_vgg_spec(batch=8, image=32, output_size=100)
    _run_driver(tmp_path, "imagenet_vgg", spec, ["--image", "32", "--classes", "100"], 10, "popc")


def test_imagenet_resnet_textbook_driver(gpu, tmp_path):
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_textbook_spec(batch=8, image=64, output_size=100)
    _run_driver(tmp_path, "imagenet_resnet_textbook", spec, ["--image", "64", "--classes", "100"], 15, "mfma_f4",
                exact=False)
    exe = os.path.join(BIN, "imagenet_resnet_textbook")  # synthetic mode
    proc = subprocess.run([exe, "--batch", "8", "--image", "64", "--classes", "10", "--reps", "2"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and '"images_per_s"' in proc.stdout, proc.stdout


def test_driver_synthetic_mode_runs(gpu):
    exe = os.path.join(BIN, "imagenet_resnet")
    proc = subprocess.run([exe, "--batch", "8", "--image", "64", "--classes", "10", "--reps", "2"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and '"images_per_s"' in proc.stdout, proc.stdout


def test_driver_error_convention_is_print_and_exit(gpu):
    """Reference convention (utility.h:57-92): message on stderr and exit(-1), no exception."""
    exe = os.path.join(BIN, "mnist_mlp")
    proc = subprocess.run([exe, "--weights", "/nonexistent.csv"], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=60)
    assert proc.returncode != 0 and "NULL pointer" in proc.stderr


def test_mnist_mlp_driver_on_a_dataset_file(gpu, tmp_path):
    """idx files -> read_dataset -> mnist_mlp --input/--labels: the evaluation flow of the reference's main
    (read_MNIST_normalized ... validate_prediction, mnist_mlp.cu:80-156), on synthetic idx files."""
    import struct
    import tcbnn_amd
    from tcbnn_amd import data, nets
    batch = 96
    rng = np.random.default_rng(11)
    px = rng.integers(0, 256, size=(batch, 28, 28), dtype=np.uint8)
    lab = rng.integers(0, 10, size=batch, dtype=np.uint8)
    fi, fl = str(tmp_path / "img-idx3"), str(tmp_path / "lab-idx1")
    with open(fi, "wb") as f:
        f.write(struct.pack(">4i", 2051, batch, 28, 28) + px.tobytes())
    with open(fl, "wb") as f:
        f.write(struct.pack(">2i", 2049, batch) + lab.tobytes())
    xf, lf, wf, of = (str(tmp_path / n) for n in ("x.f32", "y.u32", "w.csv", "logits.f32"))
    subprocess.check_call([os.path.join(BIN, "read_dataset"), "mnist", fi, fl, str(batch), xf, lf])
    x, labels = data.read_MNIST_normalized(fi, fl, batch)
    assert np.array_equal(np.fromfile(xf, np.float32), x.ravel())

    spec = nets.mnist_mlp_spec(batch=batch)
    weights = tcbnn_amd.synthetic_weights(spec, 12)
    _write_weight_file(wf, weights)
    proc = subprocess.run([os.path.join(BIN, "mnist_mlp"), "--batch", str(batch), "--weights", wf, "--input", xf,
                           "--labels", lf, "--out", of, "--reps", "1", "--warmup", "0"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout
    got = np.fromfile(of, np.float32).reshape(batch, 10)
    want = orc_nets.run(spec, weights, x.reshape(batch, 784))[spec[-1]["name"]]["out"]
    np.testing.assert_array_equal(got, want)
    top1, top5, pos = data.score_prediction(want, labels)
    lines = proc.stdout.splitlines()
    i = lines.index("=====Predict=======")
    assert lines[i + 1].split() == [str(v) for v in pos]
    pct = lambda n: float(np.float32(n) / np.float32(batch) * np.float32(100))  # the reference prints float32
    assert lines[i + 3] == "Top-1:%f%%" % pct(top1) and lines[i + 4] == "Top-5:%f%%" % pct(top5)


@pytest.mark.parametrize("variant", ["popc", "mfma_f4"])
def test_reference_layout_accessors_of_the_cpp_classes(gpu, tmp_path, variant):
    """drivers/reference_fmt_interop.cpp: the same small residual network with engine-layout and with
    reference-layout buffers between the C++ layer objects; the binary compares the two itself."""
    exe = os.path.join(BIN, "reference_fmt_interop")
    assert os.path.exists(exe), "%s is not built (run __graft_entry__.build())" % exe
    proc = subprocess.run([exe, "--batch", "12", "--seed", "3", "--variant", variant], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout
    assert '"ok": true' in proc.stdout and '"c2_residual_nonzero": 0,' not in proc.stdout


def test_first_layer_set_input_refuses_a_batch_beyond_its_residual_bound(gpu):
    """The C++ first layer picks the residual storage format from the first batch's window sums of |x|; a later
    batch whose sums no longer fit that format must end in the reference's error convention (message +
    exit(-1)), not in wrapped residuals.  (The same binary, without the flag, checks that admissible later batches,
    a smaller one and a larger one that the format still holds, give what a fresh layer gives: the test above.)"""
    exe = os.path.join(BIN, "reference_fmt_interop")
    proc = subprocess.run([exe, "--batch", "12", "--seed", "3", "--oversize-input"], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 255 and "exceed what the residual formats" in proc.stderr, (proc.returncode, proc.stderr)
