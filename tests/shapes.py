"""Shape matrix of the reference's own differential test
(reference test/gtest/test_convolution_compare_with_reference.cpp:82-217; its "Tf" groups
repeat the "Caffe" groups with the same formats, so each shape is listed once) and of its
bit-layout test (reference test/gtest/test_binarization.cpp:105-134).

Tuple order follows the reference's params_t: mb, ic, oc, ih, iw, kh, kw, sh, sw, ph, pw.
"""

TASK = [
    (1, 1, 32, 60, 61, 3, 3, 1, 1, 0, 0),
    (64, 1, 32, 60, 61, 3, 3, 1, 1, 0, 0),
    (1, 32, 32, 20, 20, 3, 3, 1, 1, 0, 0),
    (64, 32, 32, 20, 20, 3, 3, 1, 1, 0, 0),
]

SMALL = [
    (3, 24, 32, 27, 27, 5, 5, 1, 1, 2, 2),
    (3, 25, 32, 27, 27, 5, 5, 1, 1, 2, 2),
    (3, 26, 32, 27, 27, 5, 5, 1, 1, 2, 2),
    (3, 24, 24, 27, 27, 5, 5, 1, 1, 2, 2),
    (3, 24, 24, 13, 13, 3, 3, 1, 1, 1, 1),
    (3, 32, 32, 13, 13, 3, 3, 1, 1, 1, 1),
    (3, 24, 8, 13, 13, 3, 3, 1, 1, 1, 1),
    (3, 24, 16, 13, 13, 3, 3, 1, 1, 1, 1),
    (3, 8, 8, 13, 13, 3, 3, 1, 1, 1, 1),
    (3, 8, 16, 13, 13, 3, 3, 1, 1, 1, 1),
] + [(3, ic, 8, 13, 13, 3, 3, 1, 1, 1, 1) for ic in (9, 10, 11, 12, 13, 14, 15, 16, 3, 4, 5, 6, 7)]

ALEXNET = [
    (2, 3, 96, 227, 227, 11, 11, 4, 4, 0, 0),
    (2, 96, 256, 27, 27, 5, 5, 1, 1, 2, 2),
    (2, 256, 384, 13, 13, 3, 3, 1, 1, 1, 1),
    (2, 384, 384, 13, 13, 3, 3, 1, 1, 1, 1),
    (2, 384, 256, 13, 13, 3, 3, 1, 1, 1, 1),
]

ALEXNET_OUT_OF_TEMPLATE = [
    (2, 3, 64, 227, 227, 11, 11, 4, 4, 0, 0),
    (2, 96, 128, 27, 27, 5, 5, 1, 1, 2, 2),
    (2, 256, 256, 13, 13, 3, 3, 1, 1, 1, 1),
    (2, 12, 128, 13, 13, 3, 3, 1, 1, 1, 1),
    (2, 384, 64, 13, 13, 3, 3, 1, 1, 1, 1),
]

CIFAR10_TMP = [
    (2, 128, 128, 32, 32, 3, 3, 1, 1, 1, 1),
    (2, 128, 256, 16, 16, 3, 3, 1, 1, 1, 1),
    (2, 256, 256, 16, 16, 3, 3, 1, 1, 1, 1),
    (2, 256, 512, 8, 8, 3, 3, 1, 1, 1, 1),
    (2, 512, 512, 8, 8, 3, 3, 1, 1, 1, 1),
]

CIFAR10 = [
    (2, 3, 32, 32, 32, 5, 5, 1, 1, 2, 2),
    (2, 32, 32, 32, 32, 5, 5, 1, 1, 2, 2),
    (2, 32, 64, 32, 32, 5, 5, 1, 1, 2, 2),
]

MNIST = [
    (2, 1, 24, 28, 28, 5, 5, 1, 1, 0, 0),
    (2, 24, 48, 8, 8, 5, 5, 1, 1, 0, 0),
]

COMPARE_WITH_REFERENCE = (TASK + SMALL + ALEXNET + ALEXNET_OUT_OF_TEMPLATE + CIFAR10_TMP
                          + CIFAR10 + MNIST)

# reference test/gtest/test_binarization.cpp:105-134 (mb 256 rows trimmed to mb 4: the
# layout does not depend on mb)
BINARIZATION = [
    (1, 1, 32, 60, 61, 3, 3, 1, 1, 0, 0),
    (4, 1, 32, 60, 61, 3, 3, 1, 1, 0, 0),
    (1, 32, 32, 20, 20, 3, 3, 1, 1, 0, 0),
    (4, 32, 32, 20, 20, 3, 3, 1, 1, 0, 0),
] + ALEXNET


def as_dims(t):
    mb, ic, oc, ih, iw, kh, kw, sh, sw, ph, pw = t
    return dict(mb=mb, ic=ic, oc=oc, ih=ih, iw=iw, kh=kh, kw=kw, sh=sh, sw=sw, ph=ph, pw=pw)


def shape_id(t):
    return "mb%d_ic%d_oc%d_%dx%d_k%dx%d_s%d_p%d" % (t[0], t[1], t[2], t[3], t[4], t[5], t[6],
                                                     t[7], t[9])
