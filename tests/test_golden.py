"""Known-answer fixture tests/golden/kat_small.npz (made by tests/golden/make_golden.py from numpy / torch
mathematics alone): the CPU oracle must reproduce it, and so must the HIP path through the C ABI."""
import os

import numpy as np
import pytest

from oracle import orc
from . import refmath as rm

KAT = np.load(os.path.join(os.path.dirname(__file__), "golden", "kat_small.npz"), allow_pickle=False)


def _bits(packed, n):
    """packed uint32 [..., W] -> bool [..., n]"""
    return orc.unpack_bits(packed, n) > 0


# ------------------------------------------------------------------------------- oracle (CPU)
def test_fixture_is_what_the_generator_writes(tmp_path, monkeypatch):
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden",
                                                                            "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    monkeypatch.setattr(mod, "HERE", str(tmp_path))
    mod.main()
    fresh = np.load(os.path.join(str(tmp_path), "kat_small.npz"), allow_pickle=False)
    assert sorted(fresh.files) == sorted(KAT.files)
    for k in KAT.files:
        np.testing.assert_array_equal(fresh[k], KAT[k], err_msg=k)


def test_oracle_bmm_kat():
    a = rm.packbits_msb(KAT["bmm_a"] >= 0, 3)
    b = rm.packbits_msb(KAT["bmm_b"].T >= 0, 3)
    np.testing.assert_array_equal(orc.bmm(a, b, 96), KAT["bmm_c"])


def test_oracle_bconv_kat():
    inp, filt = orc.pack_conv_input_nhwc(KAT["bconv_x"]), orc.pack_conv_filter(KAT["bconv_f"])
    np.testing.assert_array_equal(orc.bconv(inp, filt, 64, 32, 3, 3, 1, 1, 5, 5), KAT["bconv_s1"])
    np.testing.assert_array_equal(orc.bconv(inp, filt, 64, 32, 3, 3, 2, 1, 3, 3), KAT["bconv_s2"])


def test_oracle_fc_out_kat():
    inp, w = orc.in128(KAT["fc_x"]), orc.pack_fc_weight(KAT["fc_w"])
    np.testing.assert_array_equal(_bits(orc.fc128(inp, w, KAT["fc_bn"], 200, 40), 40), KAT["fc_bits"])
    np.testing.assert_array_equal(orc.out128(inp, w, KAT["out_scale"], KAT["out_bias"], 200, 40), KAT["out_y"])


def test_oracle_conv128_kat():
    inp, filt = orc.pack_conv_input_nhwc(KAT["conv_x"]), orc.pack_conv_filter(KAT["conv_f"])
    src = np.ascontiguousarray(KAT["conv_src"].transpose(1, 2, 0, 3))  # [2P][2Q][B][C]
    out, res = orc.conv128(inp, filt, KAT["conv_bn"], 64, 48, 3, 3, save_residual=True, inject_residual=True,
                           residual_channels=24, residual_pool=True, res_in=src)
    np.testing.assert_array_equal(res.transpose(2, 0, 1, 3), KAT["conv_res"])
    np.testing.assert_array_equal(_bits(out, 48).transpose(2, 0, 1, 3), KAT["conv_bits"])
    out, _ = orc.conv128(inp, filt, KAT["conv_bn"], 64, 48, 3, 3, pool=2)
    np.testing.assert_array_equal(_bits(out, 48).transpose(2, 0, 1, 3), KAT["conv_pool2_bits"])


def test_oracle_inconv_kat():
    out, res = orc.inconv128(KAT["inconv_x_nchw"], KAT["inconv_f"], KAT["inconv_bn"], 2, True, 1, True)
    np.testing.assert_array_equal(res.transpose(2, 0, 1, 3), KAT["inconv_res"])
    np.testing.assert_array_equal(_bits(out, 32).transpose(2, 0, 1, 3), KAT["inconv_bits"])


# ------------------------------------------------------------------------------- HIP path (GPU)
VARIANTS = ["popc", "mfma_i8", "mfma_f4"]


@pytest.mark.gpu
@pytest.mark.parametrize("variant", VARIANTS)
def test_gpu_bmm_bconv_kat(gpu, variant):
    from . import gpuops
    v = gpu.VARIANTS[variant]
    a = rm.packbits_msb(KAT["bmm_a"] >= 0, 3)
    b = rm.packbits_msb(KAT["bmm_b"].T >= 0, 3)
    np.testing.assert_array_equal(gpuops.bmm(a, b, 9, 32, 96, v), KAT["bmm_c"])
    inp, filt = gpuops.pack_conv_input(KAT["bconv_x"]), gpuops.pack_conv_filter(KAT["bconv_f"])
    np.testing.assert_array_equal(gpuops.bconv(inp, filt, 3, 5, 5, 64, 32, 3, 3, 1, 1, 5, 5, v), KAT["bconv_s1"])
    np.testing.assert_array_equal(gpuops.bconv(inp, filt, 3, 5, 5, 64, 32, 3, 3, 2, 1, 3, 3, v), KAT["bconv_s2"])


@pytest.mark.gpu
@pytest.mark.parametrize("variant", VARIANTS)
def test_gpu_fc_out_kat(gpu, variant):
    from . import gpuops
    v = gpu.VARIANTS[variant]
    inp, w = gpuops.in128(KAT["fc_x"]), gpuops.pack_fc_weight(KAT["fc_w"])
    np.testing.assert_array_equal(_bits(gpuops.fc128(inp, w, KAT["fc_bn"], 6, 200, 40, v), 40), KAT["fc_bits"])
    np.testing.assert_array_equal(gpuops.out128(inp, w, KAT["out_scale"], KAT["out_bias"], 6, 200, 40, v),
                                  KAT["out_y"])


@pytest.mark.gpu
@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("res_fmt", [0, 1])
def test_gpu_conv128_kat(gpu, variant, res_fmt):
    from . import gpuops
    from .test_gpu_parity import _residual_source
    v = gpu.VARIANTS[variant]
    x, f, bn = KAT["conv_x"], KAT["conv_f"], KAT["conv_bn"]
    src = np.ascontiguousarray(KAT["conv_src"].transpose(1, 2, 0, 3))
    layer = gpu.Conv128LayerParam("C", 6, 6, 3, 3, 64, 48, 4, 1, 1, True, 1, 1, False, True, True, 24, True,
                                  variant=v, residual_format=res_fmt)
    layer.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x), _residual_source(src, res_fmt))
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(layer.download_residual().transpose(2, 0, 1, 3), KAT["conv_res"])
    np.testing.assert_array_equal(_bits(layer.download_packed(), 48).transpose(2, 0, 1, 3), KAT["conv_bits"])
    layer.release()
    layer = gpu.Conv128LayerParam("C", 6, 6, 3, 3, 64, 48, 4, 1, 1, True, 2, 2, variant=v)
    layer.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x))
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(_bits(layer.download_packed(), 48).transpose(2, 0, 1, 3), KAT["conv_pool2_bits"])
    layer.release()


@pytest.mark.gpu
def test_gpu_inconv_kat(gpu):
    from . import gpuops
    layer = gpu.InConv128LayerParam("Conv1", 9, 9, 3, 3, 3, 32, 5, 2, 2, True, 1, 1, True)
    layer.initialize(KAT["inconv_x_nchw"], gpu.ArrayWeights([KAT["inconv_f"], KAT["inconv_bn"]]))
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(layer.download_residual().transpose(2, 0, 1, 3), KAT["inconv_res"])
    np.testing.assert_array_equal(_bits(layer.download_packed(), 32).transpose(2, 0, 1, 3), KAT["inconv_bits"])
    layer.release()
