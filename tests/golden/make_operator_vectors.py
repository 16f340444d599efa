"""
Regenerates operator_vectors.npz: inputs, weights and expected outputs of a handful of small operators, computed
with the brute-force formulas of oracle/brute.py (explicit loops, float64 accumulation, rounded to float32 at the end).
The vectors pin the CPU oracle and the GPU runtime to fixed numbers that do not move when either of them changes.
    python tests/golden/make_operator_vectors.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, '..', '..'))

from oracle import brute  # noqa: E402

# name, input shape (N, C, H, W), out channels, kernel, stride, padding, groups, activation
CONVS = [
    ('conv3x3_same_relu', (2, 5, 7, 6), 8, (3, 3), (1, 1), (1, 1), 1, 'relu'),
    ('conv3x3_stride2_nopad', (1, 3, 9, 9), 4, (3, 3), (2, 2), (0, 0), 1, 'identity'),
    ('conv1x7_pad_tanh', (1, 6, 5, 9), 5, (1, 7), (1, 1), (0, 3), 1, 'tanh'),
    ('conv5x5_stride2_sigmoid', (1, 4, 11, 10), 6, (5, 5), (2, 2), (2, 2), 1, 'sigmoid'),
    ('conv1x1_odd_channels', (3, 19, 4, 4), 21, (1, 1), (1, 1), (0, 0), 1, 'relu'),
    ('conv_grouped', (1, 8, 6, 6), 12, (3, 3), (1, 1), (1, 1), 4, 'relu'),
    ('conv_depthwise5x5_stride2', (2, 6, 9, 8), 6, (5, 5), (2, 2), (2, 2), 6, 'identity'),
    ('conv_wide_padding', (1, 2, 4, 4), 3, (3, 3), (1, 1), (2, 2), 1, 'identity'),
]
# name, input shape, pool type, kernel, stride, padding
POOLS = [
    ('maxpool3x3_stride2', (2, 3, 9, 9), 'max', (3, 3), (2, 2), (0, 0)),
    ('maxpool3x3_same', (1, 4, 6, 7), 'max', (3, 3), (1, 1), (1, 1)),
    ('avgpool3x3_same_counts_padding', (1, 4, 6, 7), 'avg', (3, 3), (1, 1), (1, 1)),
    ('avgpool2x2', (2, 2, 8, 6), 'avg', (2, 2), (2, 2), (0, 0)),
    ('global_avg', (2, 5, 4, 3), 'global_avg', (1, 1), (1, 1), (0, 0)),
    ('global_max', (1, 3, 5, 5), 'global_max', (1, 1), (1, 1), (0, 0)),
]


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    for name, shape, oc, kernel, stride, padding, groups, act in CONVS:
        x = rng.standard_normal(shape).astype(np.float32)
        w = (rng.standard_normal((oc, shape[1] // groups, *kernel)) * 0.4).astype(np.float32)
        b = (rng.standard_normal(oc) * 0.5).astype(np.float32)
        y = brute.conv2d(x, w, b, stride, padding, groups, act).astype(np.float32)
        out[name + '.x'], out[name + '.w'], out[name + '.b'], out[name + '.y'] = x, w, b, y
    for name, shape, pool_type, kernel, stride, padding in POOLS:
        x = rng.standard_normal(shape).astype(np.float32)
        y = brute.pool2d(x, pool_type, kernel, stride, padding).astype(np.float32)
        out[name + '.x'], out[name + '.y'] = x, y
    np.savez_compressed(os.path.join(HERE, 'operator_vectors.npz'), **out)


if __name__ == '__main__':
    main()
