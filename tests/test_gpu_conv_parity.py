"""Convolution kernels against the CPU oracle on seeded inputs: odd shapes that exercise every
bounds check and the scalar-load paths, DCGAN layer shapes at a small batch, fused epilogues, and
split-K.  Tolerance: 1e-4 relative / 1e-5 absolute (fp32), scaled by the magnitude of the
reduction for the filter gradient whose sums run over the whole batch."""
import numpy as np
import pytest

from common import RTOL, ATOL, rand_conv_inputs, same_pad

pytestmark = pytest.mark.gpu

SHAPES = [  # N, H, W, C, kh, kw, O, stride
    (2, 8, 8, 3, 5, 5, 4, 2),
    (1, 7, 9, 2, 3, 3, 5, 2),
    (2, 6, 6, 4, 5, 5, 3, 1),
    (1, 9, 7, 2, 3, 5, 2, 3),
    (3, 4, 4, 8, 2, 2, 8, 2),
    (1, 5, 5, 1, 5, 5, 1, 2),
    (2, 11, 13, 12, 3, 3, 20, 1),
    (1, 10, 10, 16, 1, 1, 8, 3),      # 1x1 filter, stride 3: dx phases without any tap
    (5, 12, 12, 36, 5, 5, 72, 2),     # vector loads with partial tiles
    (2, 32, 32, 64, 5, 5, 128, 2),    # D1 at batch 2
    (2, 16, 16, 128, 5, 5, 256, 2),   # D2 at batch 2
    (4, 8, 8, 256, 5, 5, 512, 2),     # D3 at batch 4 (split-K)
    (2, 64, 64, 3, 5, 5, 64, 2),      # D0 at batch 2
]


@pytest.fixture(scope="module")
def be():
    import __graft_entry__ as ge
    return ge.load_package().HipBackend(0)


def close(got, exp, scale=1.0, what=""):
    np.testing.assert_allclose(got, exp, rtol=RTOL, atol=ATOL * scale, err_msg=what)


@pytest.mark.parametrize("shape", SHAPES)
def test_conv_fwd_dx_dk(be, orc, shape):
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(42, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    orc.set_threads(8)
    close(be.conv2d(x, k, (s, s)), orc.conv2d(x, k, (s, s)), what="fwd")
    close(be.conv2d_input_grad(dy, k, s, (H, W)), orc.conv2d_input_grad(dy, k, s, (H, W)), what="dx")
    exp = orc.conv2d_kernel_grad(dy, x, s, pads)
    # sums of N*Ho*Wo products of U(-1,1) values: absolute tolerance follows their magnitude
    close(be.conv2d_kernel_grad(dy, x, s, pads), exp, scale=max(1.0, float(np.abs(exp).max())), what="dk")


@pytest.mark.parametrize("shape", [(2, 4, 4, 512, 5, 5, 256, 2), (2, 32, 32, 64, 5, 5, 3, 2), (3, 5, 7, 6, 3, 3, 4, 2)])
def test_conv_transpose_and_grads(be, orc, shape):
    """Generator-style layers: x [N,Hi,Wi,Ci] -> [N,s*Hi,s*Wi,Co], filter [kh,kw,Co,Ci]."""
    print("shape", shape, flush=True)
    N, Hi, Wi, Ci, kh, kw, Co, s = shape
    rng = np.random.default_rng(17)
    x = rng.uniform(-1, 1, (N, Hi, Wi, Ci)).astype(np.float32)
    k = (rng.standard_normal((kh, kw, Co, Ci)) * 0.02).astype(np.float32)
    dy = rng.uniform(-1, 1, (N, Hi * s, Wi * s, Co)).astype(np.float32)
    orc.set_threads(8)
    close(be.conv2d_transpose(x, k, (Hi * s, Wi * s), s), orc.conv2d_transpose(x, k, (Hi * s, Wi * s), s))
    close(be.conv2d_transpose_input_grad(dy, k, s, (Hi, Wi)), orc.conv2d_transpose_input_grad(dy, k, s, (Hi, Wi)))
    exp = orc.conv2d_transpose_kernel_grad(dy, x, s, (kh, kw))
    close(be.conv2d_transpose_kernel_grad(dy, x, s, (kh, kw)), exp, scale=max(1.0, float(np.abs(exp).max())))


@pytest.mark.parametrize("act", ["none", "relu", "leaky", "tanh", "sigmoid"])
@pytest.mark.parametrize("shape", [(2, 16, 16, 32, 5, 5, 64, 2), (4, 8, 8, 256, 5, 5, 512, 2), (1, 7, 9, 2, 3, 3, 5, 2)])
def test_fused_epilogues(be, orc, act, shape):
    """conv + bias + activation in one call == the three reference operators in sequence;
    the second shape takes the split-K path, where the epilogue runs in the reduction."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(5, *shape)
    rng = np.random.default_rng(1)
    code = {"none": A.ACT_NONE, "relu": A.ACT_RELU, "leaky": A.ACT_LEAKY, "tanh": A.ACT_TANH, "sigmoid": A.ACT_SIGMOID}[act]
    f = {"none": lambda v: v, "relu": orc.relu, "leaky": lambda v: orc.relu_leaky(v, 0.2), "tanh": orc.tanh,
         "sigmoid": orc.sigmoid}[act]
    b = (rng.standard_normal(O) * 0.5).astype(np.float32)
    close(be.conv2d(x, k, (s, s), bias=b, act=code, alpha=0.2), f(orc.bias_add(orc.conv2d(x, k, (s, s)), b)))
    bc = (rng.standard_normal(C) * 0.5).astype(np.float32)
    close(be.conv2d_input_grad(dy, k, s, (H, W), bias=bc, act=code, alpha=0.2),
          f(orc.bias_add(orc.conv2d_input_grad(dy, k, s, (H, W)), bc)))


@pytest.mark.parametrize("shape", [(5, 12, 12, 36, 5, 5, 72, 2), (2, 32, 32, 64, 5, 5, 128, 2), (4, 8, 8, 256, 5, 5, 512, 2)])
def test_general_kernel_on_vector_shapes(be, orc, shape):
    """Shapes that normally take the 16-byte buffer-load kernel, forced through the general kernel
    (element-wise bounds checks), so that both code paths stay covered."""
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(11, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    orc.set_threads(8)
    be.lib.dh_debug_force_generic_conv(1)
    try:
        close(be.conv2d(x, k, (s, s)), orc.conv2d(x, k, (s, s)), what="fwd")
        close(be.conv2d_input_grad(dy, k, s, (H, W)), orc.conv2d_input_grad(dy, k, s, (H, W)), what="dx")
        exp = orc.conv2d_kernel_grad(dy, x, s, pads)
        close(be.conv2d_kernel_grad(dy, x, s, pads), exp, scale=max(1.0, float(np.abs(exp).max())), what="dk")
    finally:
        be.lib.dh_debug_force_generic_conv(0)


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (2, 64, 64, 3, 5, 5, 64, 2),     # the generator's last layer / discriminator's first, batch 2
    (3, 19, 13, 1, 5, 5, 8, 2),      # ragged patches on both axes, one channel
    (2, 17, 33, 2, 3, 3, 72, 2),     # 72 dy channels: a full 64-channel pass and a partial one
    (1, 20, 14, 4, 4, 4, 12, 2),     # even filter
    (2, 11, 16, 3, 5, 3, 16, 3),     # stride 3: nine phases, three passes over the wavefronts
    (1, 10, 10, 3, 2, 2, 4, 3),      # filter smaller than the stride: phases without any tap
])
def test_dx_onto_few_channels(be, orc, shape):
    """Input gradient onto 1-4 channels (vector-ALU kernel with the dy patch staged in LDS) with a
    fused bias + tanh, against the oracle and against the implicit-GEMM kernel on the same input."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(23, *shape)
    bias_c = np.linspace(-0.3, 0.3, C).astype(np.float32)
    orc.set_threads(8)
    exp = orc.tanh(orc.bias_add(orc.conv2d_input_grad(dy, k, s, (H, W)), bias_c))
    got = be.conv2d_input_grad(dy, k, s, (H, W), bias=bias_c, act=A.ACT_TANH)
    close(got, exp, what="few-channel kernel")
    be.lib.dh_debug_force_generic_conv(1)
    try:
        close(be.conv2d_input_grad(dy, k, s, (H, W), bias=bias_c, act=A.ACT_TANH), exp, what="implicit GEMM")
    finally:
        be.lib.dh_debug_force_generic_conv(0)


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (130, 64, 64, 3, 5, 5, 64, 2),     # strips of 16 rows: a row above and below each computed twice
    (264, 64, 64, 2, 5, 5, 64, 2),     # whole images, two channels
    (70, 20, 24, 1, 5, 5, 64, 2),      # strips of 4 of 10 rows, rows of 12 pixels, one channel
    (300, 20, 24, 3, 5, 5, 64, 2),     # whole images of 10 rows on eight wavefronts
    (40, 44, 64, 3, 5, 5, 64, 2),      # 22 rows in strips of 4: a last strip of 2
])
def test_dx_onto_three_channels_by_rows(be, orc, shape):
    """The matrix-core transposed convolution onto 1-3 channels (one dense product per dy row, sums over
    filter columns in registers, down the rows through LDS; wavefronts exchanging edge rows) at every
    strip height, with the fused bias + tanh and without, repeatable to the bit."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(47, *shape)
    bias_c = np.linspace(-0.3, 0.3, C).astype(np.float32)
    orc.set_threads(8)
    plain = orc.conv2d_input_grad(dy, k, s, (H, W))
    A.profile_enable(1)
    A.profile_reset()
    try:
        got = be.conv2d_input_grad(dy, k, s, (H, W))
        tags = [r["name"] for r in A.profile_read()]
    finally:
        A.profile_enable(0)
    assert tags == ["dx_col2im"], tags
    close(got, plain, what="no epilogue")
    np.testing.assert_array_equal(got, be.conv2d_input_grad(dy, k, s, (H, W)))
    close(be.conv2d_input_grad(dy, k, s, (H, W), bias=bias_c, act=A.ACT_TANH), orc.tanh(orc.bias_add(plain, bias_c)),
          what="bias + tanh")


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (2, 64, 64, 3, 5, 5, 64, 2),     # the discriminator's first layer, batch 2
    (3, 19, 13, 1, 5, 5, 16, 2),     # ragged tiles on both axes, one channel
    (2, 70, 37, 2, 3, 3, 48, 2),     # more than one tile along both axes, three blocks of output channels
    (1, 20, 40, 4, 4, 4, 32, 1),     # stride 1, even filter
    (2, 11, 50, 3, 5, 3, 16, 3),     # stride 3
    (3, 9, 9, 3, 5, 5, 60, 2),       # 60 output channels: the second 32-channel block is partial
    (2, 12, 10, 4, 5, 4, 8, 2),      # contraction of exactly 80
    (2, 15, 21, 3, 7, 3, 16, 2),     # seven filter rows: the contraction is not laid out by rows (4-byte loads)
    (2, 12, 14, 4, 4, 5, 24, 1),     # a filter row of 20 values: likewise
])
def test_fwd_from_few_channels(be, orc, shape):
    """Forward convolution from 1-4 input channels with a fused bias + leaky relu and without, against
    the oracle: through the kernel that loads MFMA operands straight from global memory (contraction
    of at most 80, at most 64 output channels) and through the implicit GEMM's scalar-gather path."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(29, *shape)
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    orc.set_threads(8)
    exp = orc.relu_leaky(orc.bias_add(orc.conv2d(x, k, (s, s)), bias), 0.2)
    close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), exp, what="with epilogue")
    close(be.conv2d(x, k, (s, s)), orc.conv2d(x, k, (s, s)), what="no epilogue")
    be.lib.dh_debug_force_generic_conv(1)
    try:
        close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), exp, what="implicit GEMM")
    finally:
        be.lib.dh_debug_force_generic_conv(0)


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (2, 64, 64, 3, 5, 5, 64, 2),       # one output row per task
    (130, 64, 64, 3, 5, 5, 16, 2),     # two output rows per task
    (264, 60, 64, 3, 5, 5, 64, 2),     # four, the last task of an image two; 30 output rows
    (64, 128, 32, 3, 5, 5, 32, 1),     # stride 1 (two pixels of padding), four rows per task
    (3, 20, 12, 3, 5, 5, 48, 2),       # rows of 6 output pixels, 48 channels
    (2, 64, 64, 1, 5, 15, 16, 2),      # one channel, a filter row of 15 taps
])
def test_fwd_from_three_channels_row_by_row(be, orc, shape):
    """The row-wise forward kernel (5 filter rows of 15 values; bias carried in the 16th slot of the
    contraction, input rows parked in LDS with zeros around them) against the oracle, with the fused
    bias + activation epilogues and without, at every number of output rows per task."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(37, *shape)
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    orc.set_threads(8)
    plain = orc.conv2d(x, k, (s, s))
    close(be.conv2d(x, k, (s, s)), plain, what="no epilogue")
    biased = orc.bias_add(plain, bias)
    close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), orc.relu_leaky(biased, 0.2), what="bias + leaky")
    close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=1.5), orc.relu_leaky(biased, 1.5), what="bias + leaky, slope > 1")
    if N <= 3:
        close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_TANH), orc.tanh(biased), what="bias + tanh")
        close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_RELU), orc.relu(biased), what="bias + relu")
        close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_SIGMOID), orc.sigmoid(biased), what="bias + sigmoid")
    A.profile_enable(1)
    A.profile_reset()
    try:
        be.conv2d(x, k, (s, s))
        tags = [r["name"] for r in A.profile_read()]
    finally:
        A.profile_enable(0)
    assert tags == ["fwd_rows"], tags


@pytest.mark.parametrize("shape", [(2, 64, 64, 3, 5, 5, 64, 2), (1, 9, 11, 3, 5, 5, 8, 2), (2, 12, 14, 4, 4, 5, 24, 1)])
def test_fwd_from_few_channels_reads_only_its_taps(be, orc, shape):
    """The thin forward kernel loads 16 bytes at a time and discards the elements that belong to no tap
    (the padding columns, the value after a filter row).  With NaNs planted in the input -- one pixel in
    the middle, the last pixel of the tensor -- exactly the outputs whose taps cover them may be NaN:
    the oracle's pattern, element for element."""
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(31, *shape)
    x[0, H // 2, W // 2, :] = np.nan
    x[N - 1, H - 1, W - 1, C - 1] = np.nan
    orc.set_threads(8)
    exp = orc.conv2d(x, k, (s, s))
    got = be.conv2d(x, k, (s, s))
    assert np.isnan(exp).any() and not np.isnan(exp).all()
    np.testing.assert_array_equal(np.isnan(got), np.isnan(exp))
    close(got, exp, what="thin forward with NaN inputs")


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (2, 64, 64, 3, 5, 5, 64, 2),     # the discriminator's first layer, batch 2
    (10, 38, 26, 1, 5, 5, 16, 2),    # one channel; 13 output columns: a ragged last segment
    (4, 70, 37, 2, 3, 3, 48, 2),     # 48 output channels: the second 32-channel tile is partial
    (4, 40, 40, 4, 4, 4, 32, 1),     # stride 1, even filter, 64 filter elements per output channel
    (6, 36, 36, 3, 5, 5, 60, 2),     # 60 output channels
    (4, 48, 40, 4, 5, 4, 8, 2),      # 80 filter elements, 8 output channels
    (4, 33, 50, 3, 5, 3, 16, 3),     # stride 3: the staged rows do not fit, the implicit GEMM takes it
])
def test_dk_from_few_channels(be, orc, shape):
    """Filter gradient of a thin input (the kernel that reads the gathered operand as a strided view
    of input rows staged in LDS) against the oracle and against the implicit GEMM, twice for
    repeatability."""
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(29, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    orc.set_threads(8)
    exp = orc.conv2d_kernel_grad(dy, x, s, pads)
    scale = max(1.0, float(np.abs(exp).max()))
    got = be.conv2d_kernel_grad(dy, x, s, pads)
    close(got, exp, scale=scale, what="thin filter gradient")
    np.testing.assert_array_equal(got, be.conv2d_kernel_grad(dy, x, s, pads))
    be.lib.dh_debug_force_generic_conv(1)
    try:
        close(be.conv2d_kernel_grad(dy, x, s, pads), exp, scale=scale, what="implicit GEMM")
    finally:
        be.lib.dh_debug_force_generic_conv(0)


@pytest.mark.parametrize("generic", [0, 1])
@pytest.mark.parametrize("shape", [(3, 12, 12, 36, 5, 5, 72, 2), (2, 16, 16, 128, 5, 5, 256, 2), (4, 9, 7, 3, 5, 5, 10, 2)])
def test_forced_split_counts(be, orc, shape, generic):
    """The contraction cut into 3, 7, 20 and 40 splits (32 and more take the reduction kernel that
    spreads the splits of one output over 16 lanes) on shapes that would not be split by themselves:
    all within tolerance of the oracle and each repeatable to the bit, for the forward and
    input-gradient products (bias and activation applied in the reduction) and the filter gradient."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(5, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    bias_c = np.linspace(-0.3, 0.3, C).astype(np.float32)
    orc.set_threads(8)
    exp_f = orc.relu_leaky(orc.bias_add(orc.conv2d(x, k, (s, s)), bias), 0.2)
    exp_x = orc.tanh(orc.bias_add(orc.conv2d_input_grad(dy, k, s, (H, W)), bias_c))
    exp_k = orc.conv2d_kernel_grad(dy, x, s, pads)
    be.lib.dh_debug_force_generic_conv(generic)
    try:
        for splits in (3, 7, 20, 40):
            be.lib.dh_debug_force_splitk(splits)
            for rep in range(2):
                got_f = be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2)
                got_x = be.conv2d_input_grad(dy, k, s, (H, W), bias=bias_c, act=A.ACT_TANH)
                got_k = be.conv2d_kernel_grad(dy, x, s, pads)
                if rep == 0:
                    first = (got_f, got_x, got_k)
                    close(got_f, exp_f, what="fwd splits=%d" % splits)
                    close(got_x, exp_x, what="dx splits=%d" % splits)
                    close(got_k, exp_k, scale=max(1.0, float(np.abs(exp_k).max())), what="dk splits=%d" % splits)
                else:
                    for a, b in zip(first, (got_f, got_x, got_k)):
                        np.testing.assert_array_equal(a, b)
    finally:
        be.lib.dh_debug_force_splitk(0)
        be.lib.dh_debug_force_generic_conv(0)


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (16, 8, 8, 16, 5, 5, 32, 2),     # one image slab per pixel; tiles span several pixels
    (32, 4, 4, 32, 5, 5, 16, 2),     # 2x2 outputs: every tap is padding for some pixel
    (16, 9, 7, 16, 5, 5, 16, 2),     # odd extents: one-sided padding differs between the axes
    (48, 5, 5, 16, 5, 5, 32, 2),     # 48 images: pixel boundaries fall inside row tiles
    (16, 6, 6, 16, 3, 3, 16, 1),     # stride 1: a single phase, taps skipped at all four borders
    (16, 7, 7, 16, 4, 4, 16, 3),     # stride 3, even filter
    (128, 4, 4, 16, 5, 5, 16, 2),    # one pixel per 128-row tile: the box of live taps is exact
    (16, 2, 2, 16, 5, 5, 16, 2),     # a single output pixel
    (16, 1, 1, 16, 5, 5, 16, 2),     # 1x1 image: one live tap
    (256, 4, 4, 16, 5, 5, 16, 2),    # two row tiles per pixel
    (64, 8, 8, 16, 5, 5, 32, 2),     # two pixels per tile: pixels taken in the order sorted by their tap box
    (64, 5, 5, 16, 5, 5, 16, 2),     # ... with an odd number of pixels
    (64, 16, 16, 16, 5, 5, 16, 2),   # ... 64 pixels per stride phase (the most the pixel table holds)
    (64, 6, 6, 16, 3, 3, 16, 1),     # ... stride 1
])
@pytest.mark.parametrize("splits", [0, 5])
def test_taps_in_the_padding_are_skipped(be, orc, shape, splits):
    """Shapes on which the buffer-load kernel leaves out the k-slabs whose taps fall into the
    padding (channel and image counts divisible by 16): forward, input gradient and filter gradient,
    single and paired, automatic split and a forced one, against the oracle."""
    padding_skip_case(be, orc, shape, splits)


@pytest.mark.parametrize("seed", range(16))
def test_seeded_random_geometries_with_skipped_taps(be, orc, seed):
    """The same checks on drawn geometries of that family (image counts 16 ... 80, small odd extents)."""
    rng = np.random.default_rng(7000 + seed)
    kh, kw = int(rng.integers(2, 6)), int(rng.integers(2, 6))
    shape = (16 * int(rng.integers(1, 6)), int(rng.integers(1, 11)), int(rng.integers(1, 11)), 16 * int(rng.integers(1, 4)),
             kh, kw, 16 * int(rng.integers(1, 6)), int(rng.integers(1, 3)))
    padding_skip_case(be, orc, shape, int(rng.integers(0, 7)))


def padding_skip_case(be, orc, shape, splits):
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, "splits", splits, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(31, *shape)
    x2, _, dy2 = rand_conv_inputs(32, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    orc.set_threads(8)
    exp_f = orc.relu_leaky(orc.bias_add(orc.conv2d(x, k, (s, s)), bias), 0.2)
    exp_x = orc.conv2d_input_grad(dy, k, s, (H, W))
    exp_k = orc.conv2d_kernel_grad(dy, x, s, pads)
    be.lib.dh_debug_force_splitk(splits)
    try:
        close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), exp_f, what="fwd")
        close(be.conv2d_input_grad(dy, k, s, (H, W)), exp_x, what="dx")
        kscale = max(1.0, float(np.abs(exp_k).max()))
        close(be.conv2d_kernel_grad(dy, x, s, pads), exp_k, scale=kscale, what="dk")
        if N <= 64:
            exp_f2 = orc.relu_leaky(orc.bias_add(orc.conv2d(x2, k, (s, s)), bias), 0.2)
            got1, got2 = be.conv2d_pair(x, x2, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2)
            close(got1, exp_f, what="fwd pair 1"), close(got2, exp_f2, what="fwd pair 2")
            got1, got2 = be.conv2d_input_grad_pair(dy, dy2, k, s, (H, W))
            close(got1, exp_x, what="dx pair 1")
            close(got2, orc.conv2d_input_grad(dy2, k, s, (H, W)), what="dx pair 2")
            exp_k2 = exp_k + orc.conv2d_kernel_grad(dy2, x2, s, pads)
            close(be.conv2d_kernel_grad_pair(dy, x, dy2, x2, s, pads), exp_k2, scale=2 * kscale, what="dk pair")
    finally:
        be.lib.dh_debug_force_splitk(0)


@pytest.mark.parametrize("case", [  # (N, H, W, C, kh, kw, O, stride), operator, tile the launch must take
    ((64, 64, 64, 16, 3, 3, 128, 2), "fwd", "128x128"),   # 512 square tiles fill the device unsplit
    ((64, 64, 64, 128, 3, 3, 16, 2), "dx", "measured"),   # 2048 square tiles, several rounds: the width is timed
    ((64, 32, 32, 16, 3, 3, 256, 2), "fwd", "128x64"),    # 256 square tiles: twice as many narrow ones need no split
    ((64, 8, 8, 64, 5, 5, 256, 2), "fwd", "128x64"),      # a small split launch: narrow tiles, pixels in sorted order
    ((64, 8, 8, 128, 5, 5, 64, 2), "dx", "128x64"),       # ... input gradient
    ((64, 8, 8, 64, 5, 5, 256, 2), "dk", "128x128"),      # the filter gradient keeps the square tile
])
def test_tile_width_follows_the_size_of_the_launch(be, orc, case):
    """Forward and input-gradient launches take 128x64 tiles where 128x128 tiles would need a split
    that the narrower ones avoid or make cheaper; a launch of more square tiles than the device holds at
    once takes whichever width the library measured to be faster on its first call (the measuring runs
    themselves are not recorded).  Which tile ran is read from the kernel tags of the profiling interface,
    the result is checked against the oracle."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    if A.device_info()["compute_units"] != 256:
        pytest.skip("the expected tiles are those of a device with 256 compute units")
    shape, op, tile = case
    print("case", case, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(41, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    orc.set_threads(8)
    A.profile_enable(1)
    A.profile_reset()
    try:
        if op == "fwd":
            got, exp, scale = be.conv2d(x, k, (s, s)), orc.conv2d(x, k, (s, s)), 1.0
        elif op == "dx":
            got, exp, scale = be.conv2d_input_grad(dy, k, s, (H, W)), orc.conv2d_input_grad(dy, k, s, (H, W)), 1.0
        else:
            got, exp = be.conv2d_kernel_grad(dy, x, s, pads), orc.conv2d_kernel_grad(dy, x, s, pads)
            scale = max(1.0, float(np.abs(exp).max()))
        tags = [r["name"] for r in A.profile_read()]
    finally:
        A.profile_enable(0)
    allowed = ("128x128", "128x64") if tile == "measured" else (tile,)
    assert tags in [["conv_igemm_fast<%s,%s>" % (op, t)] for t in allowed], tags
    close(got, exp, scale=scale, what=op)


def test_tile_width_does_not_change_an_unsplit_result(be):
    """Where the width is chosen by measurement the launch is unsplit with either width, so every output is
    the same sum in the same order: forward product and input gradient are identical to the bit with 128x128
    and 128x64 tiles, and so is the library's own choice."""
    shape = (64, 64, 64, 128, 3, 3, 128, 2)        # 512 x 1 and 4 x 512 square tiles, contraction of 72 slabs
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(43, *shape)
    results = {}
    try:
        for width in (128, 64, 0):
            print("width", width, flush=True)
            be.lib.dh_debug_force_tile_width(width)
            if width:
                be.lib.dh_debug_force_splitk(1)
            results[width] = (be.conv2d(x, k, (s, s)), be.conv2d_input_grad(dy, k, s, (H, W)))
            be.lib.dh_debug_force_splitk(0)
    finally:
        be.lib.dh_debug_force_tile_width(0)
        be.lib.dh_debug_force_splitk(0)
    for op in (0, 1):
        np.testing.assert_array_equal(results[64][op], results[128][op])
    # the input gradient's 2048 tiles are a measured launch: whichever width won, the bits are these
    np.testing.assert_array_equal(results[0][1], results[128][1])


def test_split_with_more_workgroups_than_the_table_holds(be, orc):
    """40 row tiles cut into 25 splits each are more workgroups than the kernel's workgroup table
    lists (640): the launch falls back to the nested grid in which every tile uses all its splits."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    shape = (80, 16, 16, 16, 5, 5, 16, 2)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(37, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    orc.set_threads(8)
    exp_f = orc.relu_leaky(orc.bias_add(orc.conv2d(x, k, (s, s)), bias), 0.2)
    exp_x = orc.conv2d_input_grad(dy, k, s, (H, W))
    exp_k = orc.conv2d_kernel_grad(dy, x, s, pads)
    be.lib.dh_debug_force_splitk(25)
    try:
        close(be.conv2d(x, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), exp_f, what="fwd")
        close(be.conv2d_input_grad(dy, k, s, (H, W)), exp_x, what="dx")
        close(be.conv2d_kernel_grad(dy, x, s, pads), exp_k, scale=max(1.0, float(np.abs(exp_k).max())), what="dk")
    finally:
        be.lib.dh_debug_force_splitk(0)


@pytest.mark.parametrize("shape", [  # N, H, W, C, kh, kw, O, stride
    (3, 12, 12, 48, 5, 5, 80, 2),     # partial tiles in m and n
    (2, 32, 32, 64, 5, 5, 128, 2),    # D1 at batch 2
    (4, 8, 8, 256, 5, 5, 512, 2),     # D3 at batch 4 (split-K)
    (2, 9, 7, 16, 3, 3, 32, 1),       # stride 1, odd extents
])
def test_paired_launches(be, orc, shape):
    """Two instances of a product in one launch (same filter, two sets of activations): forward and
    input gradient with a fused epilogue give each instance's oracle result; the paired filter
    gradient gives the sum of the two oracle filter gradients; all repeatable to the bit."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x1, k, dy1 = rand_conv_inputs(31, *shape)
    x2, _, dy2 = rand_conv_inputs(32, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    bias_c = np.linspace(-0.3, 0.3, C).astype(np.float32)
    orc.set_threads(8)
    for rep in range(2):
        y1, y2 = be.conv2d_pair(x1, x2, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2)
        g1, g2 = be.conv2d_input_grad_pair(dy1, dy2, k, s, (H, W), bias=bias_c, act=A.ACT_TANH)
        dk = be.conv2d_kernel_grad_pair(dy1, x1, dy2, x2, s, pads)
        if rep == 0:
            first = (y1, y2, g1, g2, dk)
        else:
            for a, b in zip(first, (y1, y2, g1, g2, dk)):
                np.testing.assert_array_equal(a, b)
    for got, x in ((y1, x1), (y2, x2)):
        close(got, orc.relu_leaky(orc.bias_add(orc.conv2d(x, k, (s, s)), bias), 0.2), what="paired forward")
    for got, dy in ((g1, dy1), (g2, dy2)):
        close(got, orc.tanh(orc.bias_add(orc.conv2d_input_grad(dy, k, s, (H, W)), bias_c)), what="paired input gradient")
    exp = orc.conv2d_kernel_grad(dy1, x1, s, pads).astype(np.float64) + orc.conv2d_kernel_grad(dy2, x2, s, pads)
    close(dk, exp.astype(np.float32), scale=max(1.0, float(np.abs(exp).max())), what="paired filter gradient")


@pytest.mark.parametrize("shape", [(64, 32, 32, 64, 5, 5, 128, 2), (64, 16, 16, 128, 5, 5, 256, 2), (64, 8, 8, 256, 5, 5, 512, 2)])
def test_paired_launches_at_batch_64_match_the_single_launches(be, shape):
    """At the benchmark's shapes, on inputs in the benchmark's distributions, with a fused epilogue: the
    paired launches against the single launches (test_gpu_layers_batch64.py compares both with the oracle
    at these shapes on standard-normal inputs)."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x1, k, dy1 = rand_conv_inputs(41, *shape)
    x2, _, dy2 = rand_conv_inputs(42, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    y1, y2 = be.conv2d_pair(x1, x2, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2)
    close(y1, be.conv2d(x1, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), what="forward, first instance")
    close(y2, be.conv2d(x2, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2), what="forward, second instance")
    g1, g2 = be.conv2d_input_grad_pair(dy1, dy2, k, s, (H, W))
    close(g1, be.conv2d_input_grad(dy1, k, s, (H, W)), what="input gradient, first instance")
    close(g2, be.conv2d_input_grad(dy2, k, s, (H, W)), what="input gradient, second instance")
    dk = be.conv2d_kernel_grad_pair(dy1, x1, dy2, x2, s, pads)
    exp = be.conv2d_kernel_grad(dy1, x1, s, pads).astype(np.float64) + be.conv2d_kernel_grad(dy2, x2, s, pads)
    close(dk, exp.astype(np.float32), scale=max(1.0, float(np.abs(exp).max())), what="filter gradient")


def test_paired_launch_refuses_what_it_cannot_take(be):
    """Channel counts that are not multiples of 4 -- or, for the channels a forward / input-gradient
    product contracts over, of 16 -- have no paired kernel: DH_ENOTSUP, not a wrong result."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    x, k, dy = rand_conv_inputs(1, 2, 8, 8, 3, 5, 5, 6, 2)
    with pytest.raises(A.HipError, match="10002"):
        be.conv2d_pair(x, x, k, (2, 2))
    with pytest.raises(A.HipError, match="10002"):
        be.conv2d_kernel_grad_pair(dy, x, dy, x, 2, (3, 3))
    x, k, dy = rand_conv_inputs(1, 2, 8, 8, 36, 5, 5, 72, 2)
    with pytest.raises(A.HipError, match="10002"):
        be.conv2d_pair(x, x, k, (2, 2))
    with pytest.raises(A.HipError, match="10002"):
        be.conv2d_input_grad_pair(dy, dy, k, 2, (8, 8))


def test_dk_is_reproducible(be):
    """Split-K partial sums are reduced in a fixed order: two runs give identical bits."""
    x, k, dy = rand_conv_inputs(3, 8, 16, 16, 128, 5, 5, 256, 2)
    a = be.conv2d_kernel_grad(dy, x, 2, (3, 3))
    b = be.conv2d_kernel_grad(dy, x, 2, (3, 3))
    np.testing.assert_array_equal(a, b)


def test_adjoint_at_full_batch(be):
    """Size-independent check at the benchmark's batch 64, beside the oracle comparison of
    test_gpu_layers_batch64.py: <conv(x,k), dy> = <x, dx(dy,k)> = <k, dk(x,dy)> for layer D2."""
    shape = (64, 16, 16, 128, 5, 5, 256, 2)
    x, k, dy = rand_conv_inputs(9, *shape)
    y = be.conv2d(x, k, (2, 2)).astype(np.float64)
    lhs = np.vdot(y, dy)
    a = np.vdot(x.astype(np.float64), be.conv2d_input_grad(dy, k, 2, (16, 16)))
    b = np.vdot(k.astype(np.float64), be.conv2d_kernel_grad(dy, x, 2, (3, 3)))
    assert abs(lhs - a) <= 1e-4 * abs(lhs) + 1e-2
    assert abs(lhs - b) <= 1e-4 * abs(lhs) + 1e-2


@pytest.mark.parametrize("shape", [
    (512, 32, 32, 64, 5, 5, 128, 2),    # layer D1 at batch 512: no split-K, 4096 row tiles
    (512, 8, 8, 256, 5, 5, 512, 2),     # layer D3 at batch 512
    (4096, 64, 64, 3, 5, 5, 64, 2),     # image layer at batch 4096: the largest tensor is [4096,32,32,64], 1.07 GB
])
def test_adjoint_at_large_batches(be, shape):
    """The batch-512 iteration and the batch-4096 generator: sizes where only properties can be checked.
    <conv(x,k), dy> = <x, dx(dy,k)> = <k, dk(x,dy)>, each inner product accumulated in float64; the
    filter gradient (a sum over up to 4 million pixels) additionally against a float64 sum of the
    same products over a sample of its entries."""
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    rng = np.random.default_rng(N + C)
    x = rng.uniform(-1, 1, (N, H, W, C)).astype(np.float32)
    k = (rng.standard_normal((kh, kw, C, O)) * 0.02).astype(np.float32)
    dy = rng.uniform(-1, 1, (N, H // s, W // s, O)).astype(np.float32)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    y = be.conv2d(x, k, (s, s))
    lhs = np.vdot(y.astype(np.float64).ravel(), dy.astype(np.float64).ravel())
    del y
    dx = be.conv2d_input_grad(dy, k, s, (H, W))
    a = np.vdot(x.astype(np.float64).ravel(), dx.astype(np.float64).ravel())
    del dx
    dk = be.conv2d_kernel_grad(dy, x, s, pads)
    b = np.vdot(k.astype(np.float64).ravel(), dk.astype(np.float64).ravel())
    # the three values are sums of ~1e9 products of magnitude <= 0.02..1: compare relative to the
    # root-sum-square scale of such a sum rather than to the (possibly cancelling) value itself
    scale = max(abs(lhs), 0.02 * np.sqrt(float(dy.size) * kh * kw * C / 3.0))
    assert abs(lhs - a) <= 1e-4 * scale, (lhs, a)
    assert abs(lhs - b) <= 1e-4 * scale, (lhs, b)
    # direct float64 evaluation of a few filter-gradient entries
    pt, pl = pads[0] // 2, pads[1] // 2
    for (di, dj, c, o) in [(0, 0, 0, 0), (kh - 1, kw - 1, C - 1, O - 1), (2, 3, C // 2, O // 3)]:
        xp = np.zeros((N, H + kh, W + kw), np.float64)
        xp[:, pt:pt + H, pl:pl + W] = x[:, :, :, c]
        win = xp[:, di:di + s * (H // s):s, dj:dj + s * (W // s):s]
        exp = float(np.sum(win * dy[:, :, :, o].astype(np.float64)))
        tol = 1e-4 * abs(exp) + 1e-5 * np.sqrt(float(N) * (H // s) * (W // s))
        assert abs(float(dk[di, dj, c, o]) - exp) <= tol, ((di, dj, c, o), float(dk[di, dj, c, o]), exp)


def test_bad_arguments_are_rejected(be):
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    x = A.Buf((1, 4, 4, 1))
    with pytest.raises(A.HipError):
        A.check(be.lib.dh_conv2d_fwd(x.ptr, x.ptr, x.ptr, 1, 4, 4, 1, 2, 2, 1, 2, 2, 5, 0, 2, 2, None, 0, 0.0, None))
    with pytest.raises(A.HipError):
        A.check(be.lib.dh_conv2d_fwd(None, x.ptr, x.ptr, 1, 4, 4, 1, 2, 2, 1, 2, 2, 0, 0, 2, 2, None, 0, 0.0, None))
    with pytest.raises(A.HipError):
        A.check(be.lib.dh_conv2d_dk(x.ptr, x.ptr, x.ptr, 0, 4, 4, 1, 2, 2, 1, 2, 2, 2, 2, 0, 0, None))


def test_plans_are_kept_per_geometry(be, orc):
    """The split plan and workgroup table of a launch are remembered per geometry and tuning switches.
    Launches of two shapes, interleaved and repeated, under changing forced split counts: every
    result is within tolerance of the oracle, and a repeated launch under the same switches equals
    its first run to the bit (a plan taken from the wrong entry would give other partial sums, or a
    table that does not cover the tiles)."""
    shapes = [(16, 16, 16, 32, 5, 5, 64, 2), (8, 8, 8, 64, 5, 5, 128, 2)]
    orc.set_threads(8)
    cases = []
    for seed, shape in enumerate(shapes):
        N, H, W, C, kh, kw, O, s = shape
        x, k, dy = rand_conv_inputs(40 + seed, *shape)
        pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
        exp = (orc.conv2d(x, k, (s, s)), orc.conv2d_input_grad(dy, k, s, (H, W)), orc.conv2d_kernel_grad(dy, x, s, pads))
        cases.append((shape, x, k, dy, pads, exp))

    def run(case):
        (N, H, W, C, kh, kw, O, s), x, k, dy, pads, exp = case
        got = (be.conv2d(x, k, (s, s)), be.conv2d_input_grad(dy, k, s, (H, W)), be.conv2d_kernel_grad(dy, x, s, pads))
        for g, e, what in zip(got, exp, ("fwd", "dx", "dk")):
            close(g, e, scale=max(1.0, float(np.abs(e).max())), what=what)
        return got

    first = {}
    try:
        for splits in (0, 3, 0, 5, 3, 0):
            be.lib.dh_debug_force_splitk(splits)
            for ci in (0, 1, 0):
                got = run(cases[ci])
                if (splits, ci) in first:
                    for a, b in zip(first[(splits, ci)], got):
                        np.testing.assert_array_equal(a, b)
                else:
                    first[(splits, ci)] = got
    finally:
        be.lib.dh_debug_force_splitk(0)


@pytest.mark.parametrize("shape", [(2, 64, 64, 3, 5, 5, 64, 2), (4, 70, 37, 2, 3, 3, 48, 2), (8, 36, 36, 3, 5, 5, 60, 2)])
def test_paired_filter_gradient_of_a_thin_input(be, orc, shape):
    """dk(x1, dy1) + dk(x2, dy2) of the image layer as one launch of the thin-input kernel (the second
    pair of operands are images N .. 2N-1 of its contraction), against the sum of the oracle's two
    gradients; the capability query says so beforehand, and says no for a shape the kernel refuses."""
    N, H, W, C, kh, kw, O, s = shape
    x1, k, dy1 = rand_conv_inputs(51, *shape)
    x2, _, dy2 = rand_conv_inputs(52, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    Ho, Wo = dy1.shape[1:3]
    assert be.lib.dh_conv2d_dk_pair_supported(N, H, W, C, Ho, Wo, O, kh, kw, s, s) == 1
    assert be.lib.dh_conv2d_dk_pair_supported(2, 8, 8, 3, 4, 4, 6, 5, 5, 2, 2) == 0
    orc.set_threads(8)
    exp = orc.conv2d_kernel_grad(dy1, x1, s, pads).astype(np.float64) + orc.conv2d_kernel_grad(dy2, x2, s, pads)
    got = be.conv2d_kernel_grad_pair(dy1, x1, dy2, x2, s, pads)
    close(got, exp.astype(np.float32), scale=max(1.0, float(np.abs(exp).max())), what="paired thin filter gradient")
    again = be.conv2d_kernel_grad_pair(dy1, x1, dy2, x2, s, pads)
    np.testing.assert_array_equal(got, again)


@pytest.mark.parametrize("shape", [(2, 64, 64, 3, 5, 5, 64, 2), (64, 64, 64, 3, 5, 5, 64, 2), (5, 60, 64, 3, 5, 5, 16, 2)])
def test_paired_forward_product_of_the_image_layer(be, orc, shape):
    """conv(x1, k) and conv(x2, k) of the image layer as one launch of the row-wise kernel (the second batch
    are images N .. 2N-1 of its tasks): each result is the single launch's to the bit, with and without the
    fused epilogue; the capability query says so beforehand."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x1, k, _ = rand_conv_inputs(61, *shape)
    x2, _, _ = rand_conv_inputs(62, *shape)
    bias = np.linspace(-0.5, 0.5, O).astype(np.float32)
    (ph, Ho), (pw, Wo) = same_pad(H, kh, s), same_pad(W, kw, s)
    assert be.lib.dh_conv2d_fwd_pair_supported(N, H, W, C, kh, kw, O, s, s, ph // 2, pw // 2, Ho, Wo) == 1
    assert be.lib.dh_conv2d_fwd_pair_supported(2, 8, 8, 3, 5, 5, 6, 2, 2, 1, 1, 4, 4) == 0
    A.profile_enable(1)
    A.profile_reset()
    try:
        y1, y2 = be.conv2d_pair(x1, x2, k, (s, s))
        tags = [r["name"] for r in A.profile_read()]
    finally:
        A.profile_enable(0)
    assert tags == ["fwd_rows"], tags
    np.testing.assert_array_equal(y1, be.conv2d(x1, k, (s, s)))
    np.testing.assert_array_equal(y2, be.conv2d(x2, k, (s, s)))
    y1, y2 = be.conv2d_pair(x1, x2, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2)
    np.testing.assert_array_equal(y1, be.conv2d(x1, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2))
    np.testing.assert_array_equal(y2, be.conv2d(x2, k, (s, s), bias=bias, act=A.ACT_LEAKY, alpha=0.2))
    if N <= 5:
        orc.set_threads(8)
        close(y2, orc.relu_leaky(orc.bias_add(orc.conv2d(x2, k, (s, s)), bias), 0.2), what="second batch")


def seeded_geometry(seed):
    """A geometry drawn from one of four families: any small shape (general kernel), channels in
    multiples of 16 / 4 (the vector-load kernels, partial tiles, often split), a thin input (at most
    4 channels) and a thin result (at most 4 output channels)."""
    rng = np.random.default_rng(1000 + seed)
    family = seed % 4
    kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    # (a stride larger than the filter can leave the last input pixels outside every window: the reference's
    # unsigned pad arithmetic wraps there, src/gpu/conv2d.cu:88-91, so such geometries have no defined result)
    s = int(rng.integers(1, min(kh, kw, 3) + 1))
    N = int(rng.integers(1, 7))
    H, W = int(rng.integers(3, 21)), int(rng.integers(3, 21))
    if family == 0:
        C, O = int(rng.integers(1, 41)), int(rng.integers(1, 41))
    elif family == 1:
        C, O = 16 * int(rng.integers(1, 9)), 4 * int(rng.integers(1, 41))
    elif family == 2:
        C, O = int(rng.integers(1, 5)), 4 * int(rng.integers(1, 17))
        H, W = int(rng.integers(8, 41)), int(rng.integers(8, 41))
    else:
        C, O = 16 * int(rng.integers(1, 5)), int(rng.integers(1, 5))
        H, W = int(rng.integers(8, 33)), int(rng.integers(8, 33))
    return (N, H, W, C, kh, kw, O, s)


@pytest.mark.parametrize("seed", range(48))
def test_seeded_random_geometries(be, orc, seed):
    """Forward, input gradient and filter gradient of a drawn geometry, with the automatic split and
    with a drawn forced one, against the oracle."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = A.load()
    shape = seeded_geometry(seed)
    print("seed", seed, "shape", shape, flush=True)
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(seed, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    orc.set_threads(8)
    exp_y = orc.conv2d(x, k, (s, s))
    exp_dx = orc.conv2d_input_grad(dy, k, s, (H, W))
    exp_dk = orc.conv2d_kernel_grad(dy, x, s, pads)
    forced = int(np.random.default_rng(seed).integers(2, 7))
    for splits in (0, forced):
        A.check(lib.dh_debug_force_splitk(splits))
        try:
            close(be.conv2d(x, k, (s, s)), exp_y, what="fwd, splits %d" % splits)
            close(be.conv2d_input_grad(dy, k, s, (H, W)), exp_dx, what="dx, splits %d" % splits)
            close(be.conv2d_kernel_grad(dy, x, s, pads), exp_dk, scale=max(1.0, float(np.abs(exp_dk).max())),
                  what="dk, splits %d" % splits)
        finally:
            A.check(lib.dh_debug_force_splitk(0))


@pytest.mark.parametrize("seed", range(24))
def test_seeded_random_transposed_geometries(be, orc, seed):
    """conv2d_transpose and its two gradients on drawn geometries (x [N,Hi,Wi,Ci] -> [N,s*Hi,s*Wi,Co],
    filter [kh,kw,Co,Ci]): any small shape, channel counts in multiples of 16 / 4, and the image end
    (at most 4 output channels)."""
    rng = np.random.default_rng(5000 + seed)
    kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    s = int(rng.integers(1, min(kh, kw, 3) + 1))
    N, Hi, Wi = int(rng.integers(1, 6)), int(rng.integers(2, 13)), int(rng.integers(2, 13))
    family = seed % 3
    if family == 0:
        Ci, Co = int(rng.integers(1, 33)), int(rng.integers(1, 33))
    elif family == 1:
        Ci, Co = 16 * int(rng.integers(1, 9)), 4 * int(rng.integers(1, 33))
    else:
        Ci, Co = 16 * int(rng.integers(1, 5)), int(rng.integers(1, 5))
    print("seed", seed, "shape", (N, Hi, Wi, Ci, kh, kw, Co, s), flush=True)
    x = rng.uniform(-1, 1, (N, Hi, Wi, Ci)).astype(np.float32)
    k = (rng.standard_normal((kh, kw, Co, Ci)) * 0.1).astype(np.float32)
    dy = rng.uniform(-1, 1, (N, Hi * s, Wi * s, Co)).astype(np.float32)
    orc.set_threads(8)
    close(be.conv2d_transpose(x, k, (Hi * s, Wi * s), s), orc.conv2d_transpose(x, k, (Hi * s, Wi * s), s), what="transpose")
    close(be.conv2d_transpose_input_grad(dy, k, s, (Hi, Wi)), orc.conv2d_transpose_input_grad(dy, k, s, (Hi, Wi)), what="dx")
    exp = orc.conv2d_transpose_kernel_grad(dy, x, s, (kh, kw))
    close(be.conv2d_transpose_kernel_grad(dy, x, s, (kh, kw)), exp, scale=max(1.0, float(np.abs(exp).max())), what="dk")
