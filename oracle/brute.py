"""
Brute-force restatement of the operator formulas with explicit loops (float64 accumulation).

TEST INFRASTRUCTURE ONLY.  Deliberately slow and literal: every function is the defining formula
(reference src/ios/ios_runtime.cu:254-255,275-277 for convolution geometry and groups, :542-550 and
:1047-1057 for pooling modes) so that it can pin the library-backed oracle on tiny inputs.
"""
import math

import numpy as np


def out_size(size, kernel, pad, stride):
    return 1 + (size - kernel + 2 * pad) // stride


def conv2d(x, w, b, stride, padding, groups, act='identity'):
    n, ic, h, wd = x.shape
    oc, icg, kh, kw = w.shape
    assert ic == icg * groups and oc % groups == 0
    ocg = oc // groups
    oh, ow = out_size(h, kh, padding[0], stride[0]), out_size(wd, kw, padding[1], stride[1])
    y = np.zeros((n, oc, oh, ow), dtype=np.float64)
    for bi in range(n):
        for o in range(oc):
            g = o // ocg
            for p in range(oh):
                for q in range(ow):
                    acc = float(b[o])
                    for c in range(icg):
                        for i in range(kh):
                            ih = p * stride[0] - padding[0] + i
                            if ih < 0 or ih >= h:
                                continue
                            for j in range(kw):
                                iw = q * stride[1] - padding[1] + j
                                if iw < 0 or iw >= wd:
                                    continue
                                acc += float(x[bi, g * icg + c, ih, iw]) * float(w[o, c, i, j])
                    y[bi, o, p, q] = acc
    return activation(y, act)


def pool2d(x, pool_type, kernel, stride, padding):
    n, c, h, wd = x.shape
    if 'global' in pool_type:
        kernel, stride, padding = (h, wd), (1, 1), (0, 0)
    is_max = 'max' in pool_type
    oh, ow = out_size(h, kernel[0], padding[0], stride[0]), out_size(wd, kernel[1], padding[1], stride[1])
    y = np.zeros((n, c, oh, ow), dtype=np.float64)
    for bi in range(n):
        for ch in range(c):
            for p in range(oh):
                for q in range(ow):
                    best, total = -math.inf, 0.0
                    for i in range(kernel[0]):
                        ih = p * stride[0] - padding[0] + i
                        for j in range(kernel[1]):
                            iw = q * stride[1] - padding[1] + j
                            if 0 <= ih < h and 0 <= iw < wd:
                                v = float(x[bi, ch, ih, iw])
                                best = max(best, v)
                                total += v
                    y[bi, ch, p, q] = best if is_max else total / (kernel[0] * kernel[1])
    return y


def activation(x, act):
    if act == 'identity':
        return x
    if act == 'relu':
        return np.maximum(x, 0.0)
    if act == 'tanh':
        return np.tanh(x)
    if act == 'sigmoid':
        return 1.0 / (1.0 + np.exp(-x))
    raise ValueError(act)


def gather_input(inputs, outputs, multiply=False):
    terms = []
    for term in inputs:
        acc = None
        for name, begin, end in term:
            piece = outputs[name][:, begin:end].astype(np.float64)
            acc = piece if acc is None else (acc * piece if multiply else acc + piece)
        terms.append(acc)
    return np.concatenate(terms, axis=1)
