"""TEST INFRASTRUCTURE — runs a network spec (tcbnn_amd.nets) through the CPU oracle, layer by
layer, keeping every intermediate so tests can compare packed activations layer by layer."""
import numpy as np

from . import orc


def run(spec, weights, x):
    """weights: list of arrays in weight-file order.  Returns dict name -> dict(out=..., res=...)."""
    it = iter(weights)
    outs = {}
    for L in spec:
        k = L["kind"]
        if k == "in":
            outs[L["name"]] = dict(out=orc.in128(x.reshape(L["batch"], L["features"])))
        elif k == "fc":
            w, bn = next(it), next(it)
            inp = outs[L["src"]]["out"].reshape(L["batch"], -1)
            outs[L["name"]] = dict(out=orc.fc128(inp, orc.pack_fc_weight(w.reshape(L["inp"], L["out"])), bn,
                                                 L["inp"], L["out"]))
        elif k == "out":
            w, sc, bi = next(it), next(it), next(it)
            inp = outs[L["src"]]["out"].reshape(L["batch"], -1)
            outs[L["name"]] = dict(out=orc.out128(inp, orc.pack_fc_weight(w.reshape(L["inp"], L["out"])),
                                                  sc, bi, L["inp"], L["out"]))
        elif k == "inconv":
            f, bn = next(it), next(it)
            o, r = orc.inconv128(x.reshape(L["batch"], 3, L["h"], L["w"]),
                                 f.reshape(L["r"], L["s"], 3, L["cout"]), bn, L["stride"], L["padding"],
                                 L["pool"], L["save_residual"])
            outs[L["name"]] = dict(out=o, res=r)
        elif k == "conv":
            f, bn = next(it), next(it)
            filt = orc.pack_conv_filter(f.reshape(L["r"], L["s"], L["cin"], L["cout"]))
            res_in = outs[L["res_src"]]["res"] if L["res_src"] else None
            o, r = orc.conv128(outs[L["src"]]["out"], filt, bn, L["cin"], L["cout"], L["r"], L["s"],
                               L["stride"], L["padding"], L["pool"], L["ahead_fc"], L["save_residual"],
                               L["inject_residual"], L["residual_channels"], L["residual_pool"], res_in)
            outs[L["name"]] = dict(out=o, res=r)
        elif k == "pool":
            res_in = outs[L["res_src"]]["res"] if L["res_src"] else None
            o, r = orc.pool128(outs[L["src"]]["out"], L["channels"], L["window"], L["stride"], L["pad"], res_in)
            outs[L["name"]] = dict(out=o, res=r)
        elif k == "avgfc":
            w, bias = next(it), next(it)
            outs[L["name"]] = dict(out=orc.avgpool_fc(outs[L["res_src"]]["res"],
                                                      w.reshape(L["channels"], L["out"]), bias))
        else:
            raise ValueError(k)
    return outs
