"""Measured tile / split-K choices for convolution shapes of the benchmark networks.

Key: (M = Cout, N = Ho*Wo, K = Cin*kh*kw, 1 if the filter is 1x1 else 0) -> (tile, split_k, microseconds).
Each entry is the fastest of every compiled tile x split-K factor for that shape, timed on an
MI355X as device durations (kernel trace) of the convolution plus its split-K reduce, inside one
long model whose weights are never reused, i.e. with cold caches as in a batch-1 inference.
Shapes that are not listed fall back to the analytic model in tiling.py.
"""
TUNED = {
    (64, 12544, 147, 0): ("64x64", 2, 16.8),
    (64, 3136, 64, 1): ("32x32k4", 1, 6.5),
    (64, 3136, 576, 0): ("64x32k2", 3, 16.6),
    (256, 3136, 64, 1): ("64x32k2", 1, 7.2),
    (64, 3136, 256, 1): ("32x32k4", 1, 7.1),
    (128, 784, 256, 1): ("128x32", 8, 10.3),
    (128, 784, 1152, 0): ("128x32", 8, 15.4),
    (512, 784, 256, 1): ("64x32k2", 1, 13.4),
    (512, 784, 128, 1): ("32x32k4", 1, 7.3),
    (128, 784, 512, 1): ("32x32k4", 1, 9.3),
    (256, 196, 512, 1): ("64x32k2", 8, 11.7),
    (256, 196, 2304, 0): ("64x32k2", 8, 18.1),
    (1024, 196, 512, 1): ("128x32", 4, 14.8),
    (1024, 196, 256, 1): ("32x32k4", 1, 8.1),
    (256, 196, 1024, 1): ("32x32k4", 4, 10.3),
    (512, 49, 1024, 1): ("64x32k2", 8, 13.4),
    (512, 49, 4608, 0): ("64x32k2", 12, 20.6),
    (2048, 49, 1024, 1): ("128x32", 8, 15.5),
    (2048, 49, 512, 1): ("64x64", 8, 12.9),
    (512, 49, 2048, 1): ("64x32k2", 16, 15.6),
}
