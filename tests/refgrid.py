"""Re-enumeration of the parameter grid the reference's own tests sweep
(tests/integration_tests.rs:885-923): 7 filters x {default, 2 paddings, 2 strides,
2 dilations}, output sizes {1,2,3,5}^2 mapped back to input sizes with
ConvOptions::input_shape (layer.rs:68-97), and the (batch, channels) list with
outputs == 1."""
import itertools

FILTERS = [(1, 1), (3, 3), (5, 5), (7, 7), (1, 3), (3, 5), (1, 7)]
PADDINGS = [(0, 1), (1, 1)]
STRIDES = [(1, 2), (2, 2)]
DILATIONS = STRIDES
OUTPUT_SIZES = [1, 2, 3, 5]
BATCH_CHANNELS = [(1, 1), (2, 1), (1, 2), (3, 1), (1, 3), (13, 1), (1, 13)]
# (batch, inputs, outputs) triples used by the conv2 tests (:911-919)
BATCH_IN_OUT = [(1, 1, 1)] + [t for x in (2, 3, 13) for t in ((x, 1, 1), (1, x, 1), (1, 1, x))]


def conv_options():
    for f in FILTERS:
        yield f, (0, 0), (1, 1), (1, 1)
        for p in PADDINGS:
            yield f, p, (1, 1), (1, 1)
        for s in STRIDES:
            yield f, (0, 0), s, (1, 1)
        for d in DILATIONS:
            yield f, (0, 0), (1, 1), d


def input_size(o, f, p, s, d):
    i = d * (f - 1) + 1 + s * (o - 1) - 2 * p
    return i if i > 0 else None


def input_shapes(f, p, s, d):
    for oh, ow in itertools.product(OUTPUT_SIZES, OUTPUT_SIZES):
        ih, iw = input_size(oh, f[0], p[0], s[0], d[0]), input_size(ow, f[1], p[1], s[1], d[1])
        if ih is not None and iw is not None:
            yield ih, iw


def cases():
    """(bs, c, ih, iw, filter, padding, stride, dilation) over the whole grid."""
    for f, p, s, d in conv_options():
        for ih, iw in input_shapes(f, p, s, d):
            for bs, c in BATCH_CHANNELS:
                yield bs, c, ih, iw, f, p, s, d


POOL_SHAPES = [(1, 1, 4, 4), (1, 1, 12, 12), (2, 3, 4, 4), (1, 1, 24, 24)]
DOT_SIZES = [2, 4, 5, 8, 16, 32, 64, 128]
