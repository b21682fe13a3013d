"""Independent numpy / torch statements of the mathematics the oracle must satisfy.
Nothing here shares code with oracle/ or with the product."""
import numpy as np
import torch
import torch.nn.functional as F


def pm1(rng, shape):
    return (rng.integers(0, 2, size=shape) * 2 - 1).astype(np.float32)


def packbits_msb(sign_ge0, words):
    """Boolean [..., n] -> uint32 [..., words], element e of a 32-group in bit 31-e, zero padded.
    Uses numpy.packbits (big bit order) + big-endian view: no shared code with the oracle."""
    b = np.asarray(sign_ge0, dtype=np.uint8)
    pad = words * 32 - b.shape[-1]
    b = np.concatenate([b, np.zeros(b.shape[:-1] + (pad,), np.uint8)], axis=-1)
    by = np.packbits(b, axis=-1, bitorder="big")
    return np.ascontiguousarray(by).view(">u4").astype(np.uint32).reshape(b.shape[:-1] + (words,))


def conv_pad_out(h, r, s, padding=True, pool=1):
    """Closed forms of param.h:719-728."""
    if padding:
        num = (((h + s - h % s) // s) - 1) * s + r - h
        pad = int(num / 2)  # C integer division truncates toward zero
        buf = -(-h // s)
    else:
        pad, buf = 0, (h - r) // s + 1
    return pad, buf, -(-buf // pool)


def xcorr_pm1(x_nhwc, f_hwio, stride, pad_h, pad_w, oh, ow):
    """Zero-padded cross-correlation with window origin (y*stride - pad): the quantity
    Cin*R*S - exclude*Cin - 2*popc equals (benchmark-bconv.cu:126-135, 694-697 validates the
    reference against cuDNN cross-correlation in the same way).  int64 [B][oh][ow][O]."""
    x = torch.from_numpy(np.ascontiguousarray(x_nhwc)).double().permute(0, 3, 1, 2)
    f = torch.from_numpy(np.ascontiguousarray(f_hwio)).double().permute(3, 2, 0, 1)
    B, C, H, W = x.shape
    R, S = f.shape[2], f.shape[3]
    need_h = (oh - 1) * stride + R
    need_w = (ow - 1) * stride + S
    xp = F.pad(x, (pad_w, max(0, need_w - W - pad_w), pad_h, max(0, need_h - H - pad_h)))
    y = F.conv2d(xp, f, stride=stride)[:, :, :oh, :ow]
    return y.permute(0, 2, 3, 1).round().long().numpy()


def maxpool_nhwc(v, ph, pw):
    """Max over non-overlapping windows with ceil-mode edges. v: [B][H][W][C]."""
    B, H, W, C = v.shape
    oh, ow = -(-H // ph), -(-W // pw)
    out = np.full((B, oh, ow, C), -np.inf)
    for i in range(ph):
        for j in range(pw):
            sub = v[:, i::ph, j::pw, :]
            out[:, :sub.shape[1], :sub.shape[2], :] = np.maximum(out[:, :sub.shape[1], :sub.shape[2], :], sub)
    return out


# ---- independent numpy versions of the reference's unpack kernels (layout definitions) ----
def unpack_fc_fmt(fmt, batch, k):
    """UnPackFcOutput128FMT, param.h:87-104: word of (row, 128-chunk c, word w) at
    ((row/8)*gdy + c)*32 + (row%8)*4 + w; element laneid is bit 31-laneid."""
    gdy = (k + 127) // 128
    out = np.zeros((batch, k), np.float32)
    for row in range(batch):
        for kk in range(k):
            c, w, lane = kk // 128, (kk % 128) // 32, kk % 32
            word = int(fmt[((row // 8) * gdy + c) * 32 + (row % 8) * 4 + w])
            out[row, kk] = 2.0 * ((word >> (31 - lane)) & 1) - 1.0
    return out


def unpack_conv_fmt(fmt, h, w, c, batch):
    """UnpackConvOutput32FMT, param.h:661-688 -> NHWC +-1."""
    ins = (c + 127) // 128
    b8 = ((batch + 7) // 8) * 8
    idx_c = np.arange(c)
    out = np.zeros((batch, h, w, c), np.float32)
    for by in range(h):
        for bx in range(w):
            for bz in range(batch):
                cw = idx_c // 32
                pos = by * w * b8 * ins * 4 + bx * b8 * ins * 4 + ((bz // 8) * ins + cw // 4) * 32 + (bz % 8) * 4 + cw % 4
                words = fmt[pos].astype(np.uint64)
                out[bz, by, bx, :] = 2.0 * ((words >> (31 - idx_c % 32).astype(np.uint64)) & 1) - 1.0
    return out
