"""Runs the float convolutions of the Bi-Real-18 stems at batch 256 a few times, for rocprofv3 runs; the two that a
MaxPool follows also as the one-pass kernel with the pool inside.

usage: python3 -m dabnn_amd.profile_fconv    (prints the shapes it launched, in launch order)
"""
import sys

import torch

import dabnn_amd as dab

SHAPES = [  # n, h = w, c, cout, k, pad, stride
    (256, 224, 3, 64, 7, 3, 2), (256, 224, 3, 32, 3, 1, 2), (256, 112, 32, 32, 3, 1, 1), (256, 112, 32, 64, 3, 1, 1),
    (256, 28, 64, 128, 1, 0, 1), (256, 1, 512, 1000, 1, 0, 1)]


def main():
    g = torch.Generator().manual_seed(5)
    for (n, h, c, cout, k, pad, stride) in SHAPES:
        x = torch.randn((n, h, h, c), generator=g).cuda()
        w = torch.randn((cout, k, k, c), generator=g).cuda()
        a, b = torch.randn(cout, generator=g).cuda(), torch.randn(cout, generator=g).cuda()
        for _ in range(3):
            dab.fconv_affine_relu(x, w, None, a, b, True, k, k, pad, pad, stride, stride)
        torch.cuda.synchronize()
        print("%dx%dx%dx%d -> %d, %dx%d stride %d" % (n, h, h, c, cout, k, k, stride))
        if (h + 2 * pad - k) // stride + 1 == 112 and cout == 64:
            # the last convolution of a stem with its MaxPool 3x3 stride 2 in one pass (no Relu in front of the pool
            # of the 7x7 stem, one behind the 3x3 one -- the same instructions either way)
            for _ in range(3):
                dab.fconv_maxpool(x, w, None, a, b, True, k, k, pad, pad, stride, stride, want_sign=True)
            torch.cuda.synchronize()
            print("  the same + MaxPool 3x3 stride 2 + sign bits, one pass")


if __name__ == "__main__":
    sys.exit(main())
