"""Helpers for the GPU parity tests: run the op through the C ABI (via the ctypes binding) on cuda:0."""
import numpy as np
import torch


def dev():
    return torch.device("cuda:0")


def run_op(pkg, table, x, f, mm, strides=(1, 1), padding="SAME", dilations=(1, 1), depthwise=False):
    """Returns (float output, int32 accumulators) as numpy arrays."""
    op = pkg.ApproxConv2DWithMinMaxVars([1, strides[0], strides[1], 1], 8, table, padding,
                                        dilations=[1, dilations[0], dilations[1], 1], depthwise=depthwise)
    xd = torch.from_numpy(np.ascontiguousarray(x)).to(dev())
    fd = torch.from_numpy(np.ascontiguousarray(f)).to(dev())
    y = op(xd, fd, *mm)
    acc = op.accumulators(xd, fd, *mm)
    torch.cuda.synchronize()
    return y.cpu().numpy(), acc.cpu().numpy()
