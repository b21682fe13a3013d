"""Network drivers: the layer wiring of the reference's mnist_mlp.cu, cifar10_vgg.cu,
imagenet_resnet.cu, alexnet.cu, cifar10_resnet.cu and imagenet_vgg.cu mains, as host loops over
layer.forward(stream).

A network is described by a list of layer specs (plain dicts, constructor arguments in
the reference's order) so the same description can drive other implementations of the
layer semantics.  `synthetic_weights` produces seeded weights in the order the
reference's weight file is consumed (utility.h:188-196).
"""
import numpy as np

from . import _lib
from .layers import (ArrayWeights, AvgPoolFcLayerParam, Conv128LayerParam, Fc128LayerParam, In128LayerParam,
                     InConv128LayerParam, Out128LayerParam, PAD128, Pool128LayerParam)


def _conv_out(h, r, s, padding=True, pool=1):
    buf = (h + s - 1) // s if padding else (h - r) // s + 1
    return (buf + pool - 1) // pool


def mnist_mlp_spec(batch=8192, n_hidden=1024, image_size=784, output_size=10):
    """mnist_mlp.cu:111-124: In -> Fc x3 -> Out."""
    return [
        dict(kind="in", name="Fin", batch=batch, features=image_size),
        dict(kind="fc", name="Fc1", batch=batch, inp=image_size, out=n_hidden, src="Fin"),
        dict(kind="fc", name="Fc2", batch=batch, inp=n_hidden, out=n_hidden, src="Fc1"),
        dict(kind="fc", name="Fc3", batch=batch, inp=n_hidden, out=n_hidden, src="Fc2"),
        dict(kind="out", name="Fout", batch=batch, inp=n_hidden, out=output_size, src="Fc3"),
    ]


def _conv(name, h, cin, cout, batch, src, stride=1, pool=1, ahead_fc=False, save_residual=False,
          inject_residual=False, residual_channels=0, residual_pool=False, res_src=None, r=3):
    return dict(kind="conv", name=name, h=h, w=h, r=r, s=r, cin=cin, cout=cout, batch=batch,
                stride=stride, padding=True, pool=pool, ahead_fc=ahead_fc, save_residual=save_residual,
                inject_residual=inject_residual, residual_channels=residual_channels,
                residual_pool=residual_pool, src=src, res_src=res_src)


def cifar10_vgg_spec(batch=256, image=32, n_hidden=1024, output_size=10):
    """cifar10_vgg.cu:162-199."""
    spec = [dict(kind="inconv", name="Conv1", h=image, w=image, r=3, s=3, cin=3, cout=128, batch=batch,
                 stride=1, padding=True, pool=1, save_residual=False)]
    h = image
    spec.append(_conv("Conv2", h, 128, 128, batch, "Conv1", pool=2)); h //= 2
    spec.append(_conv("Conv3", h, 128, 256, batch, "Conv2"))
    spec.append(_conv("Conv4", h, 256, 256, batch, "Conv3", pool=2)); h //= 2
    spec.append(_conv("Conv5", h, 256, 512, batch, "Conv4"))
    spec.append(_conv("Conv6", h, 512, 512, batch, "Conv5", pool=2, ahead_fc=True)); h //= 2
    spec.append(dict(kind="fc", name="Fc1", batch=batch, inp=h * h * 512, out=n_hidden, src="Conv6"))
    spec.append(dict(kind="fc", name="Fc2", batch=batch, inp=n_hidden, out=n_hidden, src="Fc1"))
    spec.append(dict(kind="out", name="Fout", batch=batch, inp=n_hidden, out=output_size, src="Fc2"))
    return spec


def imagenet_resnet_spec(batch=256, image=224, output_size=1000):
    """imagenet_resnet.cu:223-325 (ResNet-18 as the reference wires it: 7x7 stride-4 stem with
    saved residual, int32 residual carried between blocks, 2x2-max-pooled at stage entry)."""
    spec = [dict(kind="inconv", name="Conv1", h=image, w=image, r=7, s=7, cin=3, cout=64, batch=batch,
                 stride=4, padding=True, pool=1, save_residual=True)]
    h = _conv_out(image, 7, 4)
    B = batch
    spec.append(_conv("L1B1C1", h, 64, 64, B, "Conv1"))
    spec.append(_conv("L1B1C2", h, 64, 64, B, "L1B1C1", save_residual=True, inject_residual=True,
                      residual_channels=64, res_src="Conv1"))
    spec.append(_conv("L1B2C1", h, 64, 64, B, "L1B1C2"))
    spec.append(_conv("L1B2C2", h, 64, 64, B, "L1B2C1", save_residual=True, inject_residual=True,
                      residual_channels=128, res_src="L1B1C2"))
    prev, prev_res, cin = "L1B2C2", "L1B2C2", 64
    for stage, cout in ((2, 128), (3, 256), (4, 512)):
        n = "L%dB1C1" % stage
        spec.append(_conv(n, h, cin, cout, B, prev, stride=2))
        h = _conv_out(h, 3, 2)
        # stage-entry shortcut: previous stage's residual, 2x2 max-pooled, first residual_channels
        # output channels only (imagenet_resnet.cu:256-259, 279-282, 302-305)
        res_ch = {2: 128, 3: 128, 4: 256}[stage]
        n2 = "L%dB1C2" % stage
        spec.append(_conv(n2, h, cout, cout, B, n, save_residual=True, inject_residual=True,
                          residual_channels=res_ch, residual_pool=True, res_src=prev_res))
        n3 = "L%dB2C1" % stage
        spec.append(_conv(n3, h, cout, cout, B, n2))
        n4 = "L%dB2C2" % stage
        last = stage == 4
        spec.append(_conv(n4, h, cout, cout, B, n3, ahead_fc=last, save_residual=not last,
                          inject_residual=True, residual_channels=cout if stage != 2 else 128,
                          res_src=n2))
        prev, prev_res, cin = n4, n4, cout
    spec.append(dict(kind="fc", name="Fc1", batch=B, inp=h * h * 512, out=512, src=prev))
    spec.append(dict(kind="out", name="Fout", batch=B, inp=512, out=output_size, src="Fc1"))
    return spec


def alexnet_spec(batch=256, image=224, n_hidden=4096, output_size=1000):
    """alexnet.cu:143-177: 11x11 stride-4 first layer with 2x2 pooling, a 5x5 layer, channel counts
    that are not multiples of 128 (192, 384)."""
    spec = [dict(kind="inconv", name="Conv1", h=image, w=image, r=11, s=11, cin=3, cout=64, batch=batch,
                 stride=4, padding=True, pool=2, save_residual=False)]
    h = _conv_out(image, 11, 4, pool=2)
    spec.append(_conv("Conv2", h, 64, 192, batch, "Conv1", pool=2, r=5)); h = _conv_out(h, 5, 1, pool=2)
    spec.append(_conv("Conv3", h, 192, 384, batch, "Conv2"))
    spec.append(_conv("Conv4", h, 384, 256, batch, "Conv3"))
    spec.append(_conv("Conv5", h, 256, 256, batch, "Conv4", pool=2, ahead_fc=True)); h = _conv_out(h, 3, 1, pool=2)
    spec.append(dict(kind="fc", name="Fc1", batch=batch, inp=h * h * 256, out=n_hidden, src="Conv5"))
    spec.append(dict(kind="fc", name="Fc2", batch=batch, inp=n_hidden, out=n_hidden, src="Fc1"))
    spec.append(dict(kind="out", name="Fout", batch=batch, inp=n_hidden, out=output_size, src="Fc2"))
    return spec


def cifar10_resnet_spec(batch=256, image=32, output_size=10):
    """cifar10_resnet.cu:189-259: 3x3 first layer with saved residual, three stages of two blocks
    (128 / 256 / 512 channels), stage-entry shortcut = 2x2 maximum of the previous residual into the
    first 128 / 256 channels."""
    B = batch
    spec = [dict(kind="inconv", name="Conv1", h=image, w=image, r=3, s=3, cin=3, cout=128, batch=B,
                 stride=1, padding=True, pool=1, save_residual=True)]
    h = image
    spec.append(_conv("L1B1C1", h, 128, 128, B, "Conv1"))
    spec.append(_conv("L1B1C2", h, 128, 128, B, "L1B1C1", save_residual=True, inject_residual=True,
                      residual_channels=128, res_src="Conv1"))
    spec.append(_conv("L1B2C1", h, 128, 128, B, "L1B1C2"))
    spec.append(_conv("L1B2C2", h, 128, 128, B, "L1B2C1", save_residual=True, inject_residual=True,
                      residual_channels=128, res_src="L1B1C2"))
    prev, cin = "L1B2C2", 128
    for stage, cout in ((2, 256), (3, 512)):
        n1, n2, n3, n4 = ("L%dB%dC%d" % (stage, b, c) for b in (1, 2) for c in (1, 2))
        spec.append(_conv(n1, h, cin, cout, B, prev, stride=2))
        h = _conv_out(h, 3, 2)
        spec.append(_conv(n2, h, cout, cout, B, n1, save_residual=True, inject_residual=True,
                          residual_channels=cin, residual_pool=True, res_src=prev))
        spec.append(_conv(n3, h, cout, cout, B, n2))
        last = stage == 3
        spec.append(_conv(n4, h, cout, cout, B, n3, ahead_fc=last, save_residual=not last,
                          inject_residual=True, residual_channels=cout, res_src=n2))
        prev, cin = n4, cout
    spec.append(dict(kind="fc", name="Fc1", batch=B, inp=h * h * 512, out=512, src=prev))
    spec.append(dict(kind="out", name="Fout", batch=B, inp=512, out=output_size, src="Fc1"))
    return spec


def imagenet_vgg_spec(batch=256, image=224, n_hidden=4096, output_size=1000):
    """imagenet_vgg.cu:217-286: VGG-16, 2x2 pooling after layers 2, 4, 7, 10 and 13."""
    spec = [dict(kind="inconv", name="Conv1", h=image, w=image, r=3, s=3, cin=3, cout=64, batch=batch,
                 stride=1, padding=True, pool=1, save_residual=False)]
    h, cin, prev = image, 64, "Conv1"
    plan = [(64, 2), (128, 1), (128, 2), (256, 1), (256, 1), (256, 2), (512, 1), (512, 1), (512, 2),
            (512, 1), (512, 1), (512, 2)]
    for i, (cout, pool) in enumerate(plan):
        name = "Conv%d" % (i + 2)
        spec.append(_conv(name, h, cin, cout, batch, prev, pool=pool, ahead_fc=i == len(plan) - 1))
        h = _conv_out(h, 3, 1, pool=pool)
        prev, cin = name, cout
    spec.append(dict(kind="fc", name="Fc1", batch=batch, inp=h * h * 512, out=n_hidden, src=prev))
    spec.append(dict(kind="fc", name="Fc2", batch=batch, inp=n_hidden, out=n_hidden, src="Fc1"))
    spec.append(dict(kind="out", name="Fout", batch=batch, inp=n_hidden, out=output_size, src="Fc2"))
    return spec


def imagenet_resnet_textbook_spec(batch=256, image=224, output_size=1000):
    """ResNet-18 BNN wired as the textbook network rather than as imagenet_resnet.cu:223-325 wires it:
    7x7 stride-2 first layer + 3x3 stride-2 max-pool (bits OR-pooled, residual max-pooled), a 1x1 stride-2
    binarized convolution as the shortcut at every stage entry (its pre-threshold sums are the injected
    residual), global average pool of the last residual + fp32 FC.  The reference has no such driver; the
    layers it needs beyond the reference's are Pool128 and AvgPoolFc."""
    B = batch
    spec = [dict(kind="inconv", name="Conv1", h=image, w=image, r=7, s=7, cin=3, cout=64, batch=B,
                 stride=2, padding=True, pool=1, save_residual=True)]
    h = _conv_out(image, 7, 2)
    spec.append(dict(kind="pool", name="Pool1", h=h, w=h, channels=64, batch=B, window=3, stride=2, pad=1,
                     src="Conv1", res_src="Conv1"))
    h = (h + 2 - 3) // 2 + 1
    spec.append(_conv("L1B1C1", h, 64, 64, B, "Pool1"))
    spec.append(_conv("L1B1C2", h, 64, 64, B, "L1B1C1", save_residual=True, inject_residual=True,
                      residual_channels=64, res_src="Pool1"))
    spec.append(_conv("L1B2C1", h, 64, 64, B, "L1B1C2"))
    spec.append(_conv("L1B2C2", h, 64, 64, B, "L1B2C1", save_residual=True, inject_residual=True,
                      residual_channels=64, res_src="L1B1C2"))
    prev, cin = "L1B2C2", 64
    for stage, cout in ((2, 128), (3, 256), (4, 512)):
        ds, n1, n2, n3, n4 = ["L%dDS" % stage] + ["L%dB%dC%d" % (stage, b, c) for b in (1, 2) for c in (1, 2)]
        spec.append(_conv(ds, h, cin, cout, B, prev, stride=2, save_residual=True, r=1))  # shortcut
        spec.append(_conv(n1, h, cin, cout, B, prev, stride=2))
        h = _conv_out(h, 3, 2)
        spec.append(_conv(n2, h, cout, cout, B, n1, save_residual=True, inject_residual=True,
                          residual_channels=cout, res_src=ds))
        spec.append(_conv(n3, h, cout, cout, B, n2))
        spec.append(_conv(n4, h, cout, cout, B, n3, save_residual=True, inject_residual=True,
                          residual_channels=cout, res_src=n2))
        prev, cin = n4, cout
    spec.append(dict(kind="avgfc", name="Fout", h=h, w=h, channels=512, batch=B, out=output_size, res_src=prev))
    return spec


SPECS = {"imagenet_resnet_textbook": imagenet_resnet_textbook_spec, "mnist_mlp": mnist_mlp_spec, "cifar10_vgg": cifar10_vgg_spec, "imagenet_resnet": imagenet_resnet_spec,
         "alexnet": alexnet_spec, "cifar10_resnet": cifar10_resnet_spec, "imagenet_vgg": imagenet_vgg_spec}


def binary_ops(spec):
    """Nominal binary operations (2 per +-1 multiply-accumulate, border taps included) of the
    bit layers, and fp32 operations (2 per tap-channel) of the first layer."""
    bops, flops = 0, 0
    for L in spec:
        if L["kind"] in ("fc", "out"):
            bops += 2 * L["batch"] * L["inp"] * L["out"]
        elif L["kind"] == "conv":
            oh = _conv_out(L["h"], L["r"], L["stride"]); ow = _conv_out(L["w"], L["s"], L["stride"])
            bops += 2 * L["batch"] * oh * ow * L["cout"] * L["cin"] * L["r"] * L["s"]
        elif L["kind"] == "inconv":
            oh = _conv_out(L["h"], L["r"], L["stride"]); ow = _conv_out(L["w"], L["s"], L["stride"])
            flops += 2 * L["batch"] * oh * ow * L["cout"] * L["cin"] * L["r"] * L["s"]
    return bops, flops


def synthetic_weights(spec, seed=0, fold_flips=True):
    """Seeded synthetic parameters in weight-file order: +-1 weights Bernoulli(0.5); BN
    thresholds N(0, sqrt(fan_in)); a random +-1 BN sign per neuron folded into the neuron's
    weights and threshold (x <= t  <=>  -x >= -t); output-layer scale N(1, 0.1), bias N(0, 1)."""
    rng = np.random.default_rng(seed)
    arrays = []
    for L in spec:
        k = L["kind"]
        if k in ("in", "pool"):
            continue
        if k == "avgfc":  # fp32 head: weights N(0, 1/sqrt(C)), bias N(0, 1)
            arrays += [rng.normal(0.0, 1.0 / np.sqrt(L["channels"]), (L["channels"], L["out"])).astype(np.float32),
                       rng.normal(0.0, 1.0, L["out"]).astype(np.float32)]
            continue
        if k in ("fc", "out"):
            w = rng.integers(0, 2, size=(L["inp"], L["out"])).astype(np.float32) * 2 - 1
            fan_in = L["inp"]
        else:
            w = rng.integers(0, 2, size=(L["r"], L["s"], L["cin"], L["cout"])).astype(np.float32) * 2 - 1
            fan_in = L["r"] * L["s"] * L["cin"]
        nout = w.shape[-1]
        if k == "out":
            arrays += [w, rng.normal(1.0, 0.1, nout).astype(np.float32),
                       rng.normal(0.0, 1.0, nout).astype(np.float32)]
            continue
        thr = rng.normal(0.0, np.sqrt(fan_in), nout).astype(np.float32)
        if fold_flips:
            flip = (rng.integers(0, 2, size=nout) * 2 - 1).astype(np.float32)
            w = w * flip
            thr = thr * flip
        arrays += [np.ascontiguousarray(w), thr]
    return arrays


def synthetic_input(spec, seed=0):
    """Seeded synthetic input batch for the first layer of `spec`."""
    rng = np.random.default_rng(seed + 7919)
    L = spec[0]
    if L["kind"] == "in":
        # pixels uniform [0,1), centred (the reference normalises MNIST, data.cpp:161)
        return (rng.random((L["batch"], L["features"]), dtype=np.float32) - 0.5).astype(np.float32)
    return rng.standard_normal((L["batch"], L["cin"], L["h"], L["w"]), dtype=np.float32)


class Network:
    """Layer objects of one network, wired as in the reference drivers."""

    def __init__(self, spec, weights, input, variant=_lib.VARIANT_AUTO, residual_format=None, input_layout=None):
        """residual_format: None = every saved residual in the narrowest format that is exact for its
        bound; _lib.RES_I32 keeps them all as int32 (the reference's type).  input_layout:
        _lib.INCONV_INPUT_PACKED = the first convolution reads a packed copy of the input that the upload makes."""
        self.spec = spec
        self.layers = {}
        self.order = []
        src = weights if hasattr(weights, "launch_array") else ArrayWeights(weights)
        for L in spec:
            k = L["kind"]
            if k == "in":
                layer = In128LayerParam(L["name"], L["batch"], L["features"]).initialize(input)
            elif k == "inconv":
                layer = InConv128LayerParam(L["name"], L["h"], L["w"], L["r"], L["s"], L["cin"], L["cout"],
                                            L["batch"], L["stride"], L["stride"], L["padding"], L["pool"],
                                            L["pool"], L["save_residual"], residual_format, input_layout).initialize(input, src)
            elif k == "conv":
                layer = Conv128LayerParam(L["name"], L["h"], L["w"], L["r"], L["s"], L["cin"], L["cout"],
                                          L["batch"], L["stride"], L["stride"], L["padding"], L["pool"],
                                          L["pool"], L["ahead_fc"], L["save_residual"], L["inject_residual"],
                                          L["residual_channels"], L["residual_pool"], variant=variant,
                                          residual_format=residual_format)
                res = self.layers[L["res_src"]].get_output_residual_gpu() if L["res_src"] else None
                layer.initialize(src, self.layers[L["src"]].get_output_gpu(), res)
            elif k == "pool":
                layer = Pool128LayerParam(L["name"], L["h"], L["w"], L["channels"], L["batch"], L["window"],
                                          L["stride"], L["pad"], pool_residual=L["res_src"] is not None)
                res = self.layers[L["res_src"]].get_output_residual_gpu() if L["res_src"] else None
                layer.initialize(self.layers[L["src"]].get_output_gpu(), res)
            elif k == "avgfc":
                layer = AvgPoolFcLayerParam(L["name"], L["h"], L["w"], L["channels"], L["batch"], L["out"])
                layer.initialize(src, self.layers[L["res_src"]].get_output_residual_gpu())
            elif k == "fc":
                layer = Fc128LayerParam(L["name"], L["batch"], L["inp"], L["out"], variant=variant)
                layer.initialize(src, self.layers[L["src"]].get_output_gpu())
            elif k == "out":
                layer = Out128LayerParam(L["name"], L["batch"], L["inp"], L["out"], variant=variant)
                layer.initialize(src, self.layers[L["src"]].get_output_gpu())
            else:
                raise ValueError(k)
            self.layers[L["name"]] = layer
            self.order.append(layer)

    def set_input(self, input):
        self.order[0].set_input(input)

    def forward(self, stream=None):
        for layer in self.order:
            layer.forward(stream)

    def logits(self):
        _lib.device_synchronize()
        return self.order[-1].download_output()

    def release(self):
        for layer in self.order:
            layer.release()
