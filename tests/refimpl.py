"""Independent numpy/torch statements of the op, used to pin the oracle (and, on the GPU box, to
cross-check the HIP path).  Written from the op's definition, not from the oracle's code:
gathers with index arrays and library convolutions instead of the reference's loop nests."""
import numpy as np
import torch


def quantize_np(v, nudged_min, scale):
    """trunc((v - min) * (1/scale) + 0.5) in float32, clamped to [0, 255]."""
    f32 = np.float32
    inv = f32(f32(1.0) / f32(scale))
    t = ((np.asarray(v, f32) - f32(nudged_min)).astype(f32) * inv).astype(f32) + f32(0.5)
    return np.clip(np.trunc(t), 0, 255).astype(np.uint8)


def same_or_valid_geometry(in_size, k, stride, dilation, padding):
    eff = (k - 1) * dilation + 1
    if padding == "VALID":
        out = (in_size - eff) // stride + 1 if in_size >= eff else 0
        return out, 0
    out = -(-in_size // stride)
    pad = max(0, (out - 1) * stride + eff - in_size)
    return out, pad // 2


def patch_indices(H, W, KH, KW, strides, padding, dilations):
    oh, ph = same_or_valid_geometry(H, KH, strides[0], dilations[0], padding)
    ow, pw = same_or_valid_geometry(W, KW, strides[1], dilations[1], padding)
    ih = (np.arange(oh)[:, None] * strides[0] - ph) + np.arange(KH)[None, :] * dilations[0]   # [oh, KH]
    iw = (np.arange(ow)[:, None] * strides[1] - pw) + np.arange(KW)[None, :] * dilations[1]   # [ow, KW]
    return oh, ow, ih, iw


def gather_patches(x, pad_value, KH, KW, strides, padding, dilations):
    """x [N,H,W,C] -> patches [N,oh,ow,KH,KW,C]; out-of-image taps hold pad_value."""
    N, H, W, C = x.shape
    oh, ow, ih, iw = patch_indices(H, W, KH, KW, strides, padding, dilations)
    big = np.full((N, H + 1, W + 1, C), pad_value, dtype=x.dtype)
    big[:, :H, :W, :] = x
    ihc = np.where((ih >= 0) & (ih < H), ih, H)
    iwc = np.where((iw >= 0) & (iw < W), iw, W)
    return big[:, ihc[:, None, :, None], iwc[None, :, None, :], :]


def lut_conv_numpy(table, x, f, qparams, strides=(1, 1), padding="SAME", dilations=(1, 1)):
    """Returns (acc int64 [N,oh,ow,Co], out float64).  qparams = (in_nmin, in_scale, f_nmin, f_scale)."""
    in_nmin, in_scale, f_nmin, f_scale = qparams
    KH, KW, C, Co = f.shape
    qa = quantize_np(x, in_nmin, in_scale)
    qb = quantize_np(f, f_nmin, f_scale)
    zp = quantize_np(np.zeros(1, np.float32), in_nmin, in_scale)[0]
    pa = gather_patches(qa, zp, KH, KW, strides, padding, dilations)          # codes
    px = gather_patches(x.astype(np.float64), 0.0, KH, KW, strides, padding, dilations)  # raw values
    N, oh, ow = pa.shape[:3]
    K = KH * KW * C
    A = pa.reshape(N * oh * ow, K).astype(np.int64)
    B = qb.reshape(K, Co).astype(np.int64)
    t = np.asarray(table, np.uint16).astype(np.int64)
    acc = np.zeros((A.shape[0], Co), np.int64)
    for j in range(Co):
        acc[:, j] = t[(A << 8) | B[None, :, j]].sum(axis=1)
    psum = px.reshape(N * oh * ow, K).sum(axis=1)
    fsum = f.astype(np.float64).reshape(K, Co).sum(axis=0)
    s1s2 = float(np.float32(in_scale)) * float(np.float32(f_scale))
    m1, m2 = float(np.float32(in_nmin)), float(np.float32(f_nmin))
    out = acc * s1s2 + m2 * psum[:, None] + m1 * fsum[None, :] - K * m1 * m2
    return acc.reshape(N, oh, ow, Co), out.reshape(N, oh, ow, Co)


def torch_conv2d_f64(x, f, strides=(1, 1), padding="SAME", dilations=(1, 1)):
    """Library convolution in float64 with TensorFlow's SAME/VALID padding rule."""
    N, H, W, C = x.shape
    KH, KW, _, Co = f.shape
    oh, ph = same_or_valid_geometry(H, KH, strides[0], dilations[0], padding)
    ow, pw = same_or_valid_geometry(W, KW, strides[1], dilations[1], padding)
    pad_h_total = max(0, (oh - 1) * strides[0] + (KH - 1) * dilations[0] + 1 - H) if padding == "SAME" else 0
    pad_w_total = max(0, (ow - 1) * strides[1] + (KW - 1) * dilations[1] + 1 - W) if padding == "SAME" else 0
    xt = torch.from_numpy(np.ascontiguousarray(x)).double().permute(0, 3, 1, 2)
    xt = torch.nn.functional.pad(xt, (pw, pad_w_total - pw, ph, pad_h_total - ph))
    ft = torch.from_numpy(np.ascontiguousarray(f)).double().permute(3, 2, 0, 1)
    y = torch.nn.functional.conv2d(xt, ft, stride=strides, dilation=dilations)
    return y.permute(0, 2, 3, 1).contiguous().numpy()


def linf_rel(a, b):
    """The reference test's norm: max|a-b| / max|b| (tf2/test/test_table_approx_conv_2d.py:62)."""
    den = np.max(np.abs(b))
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))) / (den if den > 0 else 1.0))


def grid_case(pkg, x_shape, f_shape, mm, seed, codes="uniform"):
    """On-grid float tensors from random codes."""
    rng = np.random.default_rng(seed)
    if codes == "uniform":
        qa = rng.integers(0, 256, size=x_shape)
        qb = rng.integers(0, 256, size=f_shape)
    else:  # half-normal activations, normal weights around the zero point
        qa = np.clip(np.rint(np.abs(rng.standard_normal(x_shape) * 48.0)), 0, 255)
        qb = np.clip(np.rint(128 + rng.standard_normal(f_shape) * 30.0), 0, 255)
    x = pkg.fake_quant.grid_value(qa.astype(np.uint8), mm[0], mm[1])
    f = pkg.fake_quant.grid_value(qb.astype(np.uint8), mm[2], mm[3])
    return x, f, qa.astype(np.uint8), qb.astype(np.uint8)
