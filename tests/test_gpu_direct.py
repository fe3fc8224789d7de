"""GPU parity of the direct-convolution kernels (stride 1, k = 3 or 5: forward, data gradient and
weight gradient without the lowered matrix) against the CPU oracle's lowering pipeline, and of the
ConvolutionBridge path levels against each other.  These kernels sum in another order than the
lowered GEMMs, so the bar is the fp32 one: max|gpu - ref| / max|ref| <= 1e-4."""
import numpy as np
import pytest

from gpu_util import dev, driver, empty, host, rel_err, tuning

pytestmark = pytest.mark.gpu
TOL = 1e-4

# b d n k p o  (stride is 1 throughout)
SHAPES = [
    (64, 1, 28, 5, 0, 20),    # LeNet conv1 (benchmark configuration 1)
    (8, 20, 12, 5, 0, 50),    # LeNet conv2: odd number of 32-row blocks, slabs not 16-byte aligned
    (3, 96, 27, 5, 2, 256),   # AlexNet conv2 geometry
    (2, 48, 27, 5, 2, 128),   # one group of CaffeNet conv2
    (3, 256, 13, 3, 1, 384),  # AlexNet conv3 geometry
    (2, 192, 13, 3, 1, 192),  # one group of conv4
    (2, 4, 8, 3, 1, 5),       # tiny: tiles straddle several images
    (3, 3, 12, 5, 2, 7),      # odd channel count in both directions
    (3, 5, 9, 5, 4, 6),       # full padding (p = k-1)
    (2, 6, 10, 3, 0, 40),     # no padding
    (1, 7, 5, 5, 2, 3),       # image as small as the filter
    (5, 9, 30, 3, 1, 33),     # padded width 32: the widest the image-pair weight-gradient kernels take
    (4, 5, 7, 3, 1, 4),       # 7x7 images: a 128-pixel tile spans four of them
    (3, 80, 13, 3, 1, 48),    # 48 maps forward, 80 maps in the data gradient: three and five 16-row blocks
    (2, 16, 27, 5, 2, 80),    # five 16-row blocks forward, one in the data gradient
    (2, 8, 56, 3, 1, 16),     # padded rows of 33..64 floats: 64-float patch rows, one image per weight-gradient step
    (2, 6, 40, 5, 2, 40),
    (3, 20, 62, 3, 1, 33),    # padded width 64: the widest the 16-row kernel takes
    (2, 3, 60, 5, 2, 8),
    (2, 6, 100, 3, 1, 24),    # padded rows above 64 floats: column bands (32-row kernel only); two bands of 50
    (1, 4, 126, 3, 1, 33),    # three bands
    (2, 3, 96, 5, 2, 9),
    (1, 5, 224, 3, 1, 8),     # VGG-sized planes: four bands of 56
    (1, 3, 150, 5, 0, 4),
    (1, 2, 254, 3, 1, 3),     # five bands of 51, the last one a column short
    (1, 40, 63, 3, 1, 2),     # 63 = 2 x 32: bands of 32-float patch rows (64-float rows would not fit a tile's patch)
    (1, 2, 330, 5, 3, 5),
    (3, 5, 20, 7, 3, 12),     # 7 x 7
    (2, 3, 33, 7, 0, 40),
    (2, 4, 9, 7, 6, 33),      # full padding
    (1, 3, 80, 7, 3, 70),     # 7 x 7 in column bands, two map blocks
    (3, 20, 14, 3, 1, 40),    # 14-, 7- and 28-pixel outputs of 3 x 3 layers: compile-time weight-gradient instances
    (3, 21, 7, 3, 1, 192),    # (four, twelve and eight wavefronts; an odd batch: the last step holds one image)
    (2, 64, 28, 3, 1, 250),
    (5, 64, 16, 3, 0, 33),    # 14-pixel outputs without padding
    (3, 16, 28, 5, 2, 40),    # 5 x 5 with 28- and 14-pixel outputs: compile-time weight-gradient instances
    (3, 32, 14, 5, 2, 250),
    (3, 12, 14, 5, 2, 40),    # 5 x 5 on padded rows of 18 and 24 floats: image-pair weight-gradient kernel
    (2, 7, 20, 5, 2, 130),
    (2, 6, 22, 5, 2, 260),    # 26 floats: image pairs with 256 maps or more, one image per step below
    (2, 6, 22, 5, 2, 70),
]


def _random_shapes(count, seed):
    """Seeded random geometries inside the kernels' range: k in {3, 5}, any padding 0..k-1, padded
    width up to 32, channel and map counts around the 4-channel steps and 32-row blocks."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        k = int(rng.choice([3, 5]))
        p = int(rng.integers(0, k))
        n = int(rng.integers(max(k - 2 * p, 2), 32 - 2 * p + 1))
        if n + 2 * p - k + 1 < 7:   # the kernels want outputs of at least 7x7
            continue
        b = int(rng.integers(1, 7))
        d = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 13, 16, 31]))
        o = int(rng.choice([1, 3, 16, 31, 32, 33, 47, 64, 65, 96, 100, 129]))
        out.append((b, d, n, k, p, o))
    return out


def _ids(s):
    return "b%d_d%d_n%d_k%d_p%d_o%d" % s


def _slabs(d_w, o, d, k):
    """Forward and data-gradient slab buffers of the device model d_w."""
    drv = driver()
    out = []
    for for_dgrad in (0, 1):
        buf = empty((drv.conv_direct_slab_floats(o, d, k, for_dgrad),))
        drv.conv_direct_slabs(buf, d_w, o, d, k, for_dgrad)
        out.append(buf)
    return out


def _tensors(shape, seed):
    b, d, n, k, p, o = shape
    m = n + 2 * p - k + 1
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    return x, w, bias, og, m


@pytest.mark.parametrize("shape", SHAPES + _random_shapes(24, 2024), ids=_ids)
def test_direct_kernels_match_oracle(oracle, shape):
    b, d, n, k, p, o = shape
    if shape not in SHAPES and not driver().conv_direct_supported(b, d, n, k, 1, p, o):
        pytest.skip("random geometry outside the direct kernels' range")
    x, w, bias, og, m = _tensors(shape, 4321 + sum(shape))
    drv = driver()
    assert drv.conv_direct_supported(b, d, n, k, 1, p, o)
    ref_out, lowered = oracle.conv_forward(x, w, bias, k, 1, p)
    ref_dx, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, k, 1, p)

    d_x, d_w, d_og = dev(x), dev(w), dev(og)
    slabs_f, slabs_b = _slabs(d_w, o, d, k)
    # slab layouts: [d][o][k*k] and [o][d][k*k] with reversed filters, zero-padded in both dimensions
    for buf, n_c, n_m, ref in ((slabs_f, d, o, w.reshape(o, d, k * k).transpose(1, 0, 2)),
                               (slabs_b, o, d, w.reshape(o, d, k * k)[:, :, ::-1])):
        pc = -(-n_c // 4) * 4
        got = host(buf).reshape(pc, -1, k * k)
        assert got.shape[1] >= n_m and got.shape[1] % 32 == 0
        np.testing.assert_array_equal(got[:n_c, :n_m], ref)
        assert not got[n_c:].any() and not got[:, n_m:].any()

    out = empty((b, o, m, m))
    drv.conv_direct_forward(out, d_x, slabs_f, dev(bias), b, d, n, k, p, o)
    assert rel_err(host(out), ref_out) <= TOL
    out_nb = empty((b, o, m, m))
    drv.conv_direct_forward(out_nb, d_x, slabs_f, None, b, d, n, k, p, o)
    assert rel_err(host(out_nb), ref_out - bias.reshape(1, o, 1, 1)) <= TOL
    # a following ReLU folded into the store: exactly max(x, 0) of the unfused result
    out_relu = empty((b, o, m, m))
    drv.conv_direct_forward(out_relu, d_x, slabs_f, dev(bias), b, d, n, k, p, o, relu=True)
    np.testing.assert_array_equal(host(out_relu), oracle.relu_forward(host(out)))
    assert (host(out) < 0).any()

    dx = empty((b, d, n, n))
    drv.conv_direct_backward_data(dx, d_og, slabs_b, b, d, n, k, p, o)
    assert rel_err(host(dx), ref_dx) <= TOL
    np.testing.assert_array_equal(host(d_og), og)  # the output gradient is read in place, not permuted
    # the backward of an in-place ReLU before the layer folded into the store: the same gradient
    # where the layer's input is positive, zero elsewhere
    dx_relu = empty((b, d, n, n))
    drv.conv_direct_backward_data(dx_relu, d_og, slabs_b, b, d, n, k, p, o, relu_data=d_x)
    np.testing.assert_array_equal(host(dx_relu), oracle.relu_backward(host(dx), x))

    dw, db = empty((o, d, k, k)), empty((o,))
    drv.conv_direct_backward_weights(dw, d_og, d_x, b, d, n, k, p, o, db=db)
    assert rel_err(host(dw), ref_dw) <= TOL
    # the same launch reduces the bias gradient; both the oracle's order and float64 must agree
    assert rel_err(host(db), ref_db) <= TOL
    assert rel_err(host(db), og.astype(np.float64).sum(axis=(0, 2, 3))) <= TOL
    # split-K partial sums are added in a fixed order: a second run gives the same bits, with or
    # without the bias gradient
    dw2 = empty((o, d, k, k))
    drv.conv_direct_backward_weights(dw2, d_og, d_x, b, d, n, k, p, o)
    np.testing.assert_array_equal(host(dw2), host(dw))
    db2 = empty((o,))
    drv.conv_direct_backward_weights(dw2, d_og, d_x, b, d, n, k, p, o, db=db2)
    np.testing.assert_array_equal(host(db2), host(db))


@pytest.mark.parametrize("tile", [11, 12, 21, 22, 31, 32, 41, 42])
@pytest.mark.parametrize("shape", [(3, 96, 27, 5, 2, 256), (3, 256, 13, 3, 1, 384), (2, 20, 12, 5, 0, 50)], ids=_ids)
def test_direct_every_tile_instance(oracle, shape, tile):
    """The library picks the tile (32*t1 maps x 128*t2 pixels) from an occupancy estimate; every
    instance must give the same convolution.  The tuning knob direct_tile=<t1><t2> pins the choice; a map
    tile that does not divide the padded map count is refused, never run."""
    b, d, n, k, p, o = shape
    x, w, bias, og, m = _tensors(shape, 99 + sum(shape))
    drv = driver()
    ref_out, lowered = oracle.conv_forward(x, w, bias, k, 1, p)
    ref_dx, _, _ = oracle.conv_backward(x.shape, w, og, lowered, k, 1, p)
    d_x, d_w, d_og = dev(x), dev(w), dev(og)
    slabs_f, slabs_b = _slabs(d_w, o, d, k)
    ran = 0
    with tuning("direct_tile", tile):
        for maps, call, ref in (
                (o, lambda t: drv.conv_direct_forward(t, d_x, slabs_f, dev(bias), b, d, n, k, p, o), ref_out),
                (d, lambda t: drv.conv_direct_backward_data(t, d_og, slabs_b, b, d, n, k, p, o), ref_dx)):
            padded = min(-(-maps // (32 * t)) * 32 * t for t in (2, 3, 4))
            got = empty(ref.shape)
            if padded % (32 * (tile // 10)):
                with pytest.raises(Exception, match="not covered"):
                    call(got)
                continue
            call(got)
            assert rel_err(host(got), ref) <= TOL
            ran += 1
    if tile // 10 == 1:
        assert ran == 2  # single-block map tiles fit every map count


@pytest.mark.parametrize("shape", [(4, 6, 13, 3, 1, 10), (3, 8, 27, 5, 2, 36), (2, 5, 44, 3, 1, 12)], ids=_ids)
def test_direct_kernels_on_channel_slices(oracle, shape):
    """Grouped convolution in place: each group reads its channel slice of the whole input and
    writes its slice of the whole output (image strides of the whole tensors); results equal the
    kernels run on gathered, contiguous slices bit for bit, and nothing outside a slice is touched."""
    b, d, n, k, p, o = shape
    groups = 2
    m = n + 2 * p - k + 1
    rng = np.random.default_rng(55 + sum(shape))
    x = rng.standard_normal((b, groups * d, n, n)).astype(np.float32)
    og = rng.standard_normal((b, groups * o, m, m)).astype(np.float32)
    ws = [(rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32) for _ in range(groups)]
    bias = rng.standard_normal(groups * o).astype(np.float32)
    drv = driver()
    d_x, d_og, d_bias = dev(x), dev(og), dev(bias)
    out_whole, dx_whole = empty((b, groups * o, m, m)), empty((b, groups * d, n, n))
    in_stride, out_stride = groups * d * n * n, groups * o * m * m
    for gi in range(groups):
        d_w = dev(ws[gi])
        sf, sb = _slabs(d_w, o, d, k)
        xs, ogs = d_x[:, gi * d:(gi + 1) * d], d_og[:, gi * o:(gi + 1) * o]   # views into the whole tensors
        outs, dxs = out_whole[:, gi * o:(gi + 1) * o], dx_whole[:, gi * d:(gi + 1) * d]
        bs = d_bias[gi * o:(gi + 1) * o]
        drv.conv_direct_forward(outs, xs, sf, bs, b, d, n, k, p, o, in_stride, out_stride)
        drv.conv_direct_backward_data(dxs, ogs, sb, b, d, n, k, p, o, in_stride, out_stride)
        dw, db = empty((o, d, k, k)), empty((o,))
        drv.conv_direct_backward_weights(dw, ogs, xs, b, d, n, k, p, o, db=db, in_stride=in_stride,
                                         out_stride=out_stride)
        # the same on contiguous copies of the slices
        xc, ogc = xs.contiguous(), ogs.contiguous()
        outc, dxc, dwc, dbc = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, d, k, k)), empty((o,))
        drv.conv_direct_forward(outc, xc, sf, bs, b, d, n, k, p, o)
        drv.conv_direct_backward_data(dxc, ogc, sb, b, d, n, k, p, o)
        drv.conv_direct_backward_weights(dwc, ogc, xc, b, d, n, k, p, o, db=dbc)
        np.testing.assert_array_equal(host(outs), host(outc))
        np.testing.assert_array_equal(host(dxs), host(dxc))
        np.testing.assert_array_equal(host(dw), host(dwc))
        np.testing.assert_array_equal(host(db), host(dbc))
        ref_out, _ = oracle.conv_forward(host(xc), ws[gi], bias[gi * o:(gi + 1) * o], k, 1, p)
        assert rel_err(host(outc), ref_out) <= TOL
    assert not np.isnan(host(out_whole)).any() and not np.isnan(host(dx_whole)).any()
    np.testing.assert_array_equal(host(d_x), x)
    np.testing.assert_array_equal(host(d_og), og)


GROUPED = [
    # b, d (all groups), n, k, p, o (all groups), groups, pinned tile
    (4, 12, 13, 3, 1, 20, 2, 11),
    (3, 16, 27, 5, 2, 72, 2, 21),
    (2, 15, 44, 3, 1, 36, 3, 11),     # padded rows of 46 floats: the one-image-per-step weight gradient, group by group
    (3, 96, 27, 5, 2, 32, 2, 161),    # 48 channels per group: the data gradient runs on 16-row tiles
    (2, 12, 9, 5, 4, 160, 4, 161),    # 40 maps per group forward (three 16-row blocks), 3 channels per group
    (2, 6, 100, 3, 1, 10, 2, 11),     # images in two column bands, weight-gradient rows in pieces, on channel slices
    (2, 8, 21, 7, 3, 12, 2, 21),      # 7 x 7
]


@pytest.mark.parametrize("cfg", GROUPED, ids=lambda c: "b%d_d%d_n%d_k%d_p%d_o%d_g%d_t%d" % c)
def test_grouped_launch_equals_per_group_launches(oracle, cfg):
    """A grouped convolution as ONE launch per product (group index inside the grid) against one launch per
    group on channel slices of the same tensors: with the tile and the step ranges pinned to the same
    choice both ways, every output element sees the same sums in the same order, so the results are
    identical bit for bit; unpinned, the one-launch form is held to the oracle run group by group."""
    b, d, n, k, p, o, groups, tile = cfg
    dg, og = d // groups, o // groups
    m = n + 2 * p - k + 1
    rng = np.random.default_rng(321 + sum(cfg))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    og_t = rng.standard_normal((b, o, m, m)).astype(np.float32)
    w = (rng.standard_normal((o, dg, k, k)) * 0.1).astype(np.float32)     # Caffe's blob of a grouped layer
    bias = rng.standard_normal(o).astype(np.float32)
    drv = driver()
    assert drv.conv_direct_supported(b, d, n, k, 1, p, o, groups)
    d_x, d_og, d_w, d_bias = dev(x), dev(og_t), dev(w), dev(bias)
    in_stride, out_stride = d * n * n, o * m * m

    def run_grouped():
        sf = empty((drv.conv_direct_slab_floats(o, d, k, 0, groups),))
        sb = empty((drv.conv_direct_slab_floats(o, d, k, 1, groups),))
        drv.conv_direct_slabs(sf, d_w, o, d, k, 0, groups)
        drv.conv_direct_slabs(sb, d_w, o, d, k, 1, groups)
        out, dx, dw, db = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, dg, k, k)), empty((o,))
        out_relu, dx_relu = empty((b, o, m, m)), empty((b, d, n, n))
        drv.conv_direct_forward(out, d_x, sf, d_bias, b, d, n, k, p, o, groups=groups)
        drv.conv_direct_forward(out_relu, d_x, sf, d_bias, b, d, n, k, p, o, relu=True, groups=groups)
        drv.conv_direct_backward_data(dx, d_og, sb, b, d, n, k, p, o, groups=groups)
        drv.conv_direct_backward_data(dx_relu, d_og, sb, b, d, n, k, p, o, relu_data=d_x, groups=groups)
        drv.conv_direct_backward_weights(dw, d_og, d_x, b, d, n, k, p, o, db=db, groups=groups)
        return [host(t) for t in (out, dx, dw, db, out_relu, dx_relu)], host(sf), host(sb)

    def run_per_group():
        out, dx, dw, db = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, dg, k, k)), empty((o,))
        slabs_f, slabs_b = [], []
        for gi in range(groups):
            wg = d_w[gi * og:(gi + 1) * og].contiguous()
            sf, sb = _slabs(wg, og, dg, k)
            slabs_f.append(host(sf))
            slabs_b.append(host(sb))
            xs, ogs = d_x[:, gi * dg:(gi + 1) * dg], d_og[:, gi * og:(gi + 1) * og]
            drv.conv_direct_forward(out[:, gi * og:(gi + 1) * og], xs, sf, d_bias[gi * og:(gi + 1) * og], b, dg, n, k, p,
                                    og, in_stride, out_stride)
            drv.conv_direct_backward_data(dx[:, gi * dg:(gi + 1) * dg], ogs, sb, b, dg, n, k, p, og, in_stride, out_stride)
            drv.conv_direct_backward_weights(dw[gi * og:(gi + 1) * og], ogs, xs, b, dg, n, k, p, og,
                                             db=db[gi * og:(gi + 1) * og], in_stride=in_stride, out_stride=out_stride)
        return [host(t) for t in (out, dx, dw, db)], np.concatenate(slabs_f), np.concatenate(slabs_b)

    with tuning("direct_tile", tile), tuning("direct_splits", 3):
        one, sf1, sb1 = run_grouped()
        per, sfg, sbg = run_per_group()
    np.testing.assert_array_equal(sf1, sfg)
    np.testing.assert_array_equal(sb1, sbg)
    for got, want, name in zip(one[:4], per, ("output", "input gradient", "weight gradient", "bias gradient")):
        np.testing.assert_array_equal(got, want, err_msg=name)
    np.testing.assert_array_equal(one[4], oracle.relu_forward(one[0]))
    np.testing.assert_array_equal(one[5], oracle.relu_backward(one[1], x))
    # unpinned (the library's own choice of tile and step ranges for the whole launch) against the oracle
    free, _, _ = run_grouped()
    for gi in range(groups):
        xs = np.ascontiguousarray(x[:, gi * dg:(gi + 1) * dg])
        ogs = np.ascontiguousarray(og_t[:, gi * og:(gi + 1) * og])
        wg, bg = w[gi * og:(gi + 1) * og], bias[gi * og:(gi + 1) * og]
        ref_out, lowered = oracle.conv_forward(xs, wg, bg, k, 1, p)
        ref_dx, ref_dw, ref_db = oracle.conv_backward(xs.shape, wg, ogs, lowered, k, 1, p)
        assert rel_err(free[0][:, gi * og:(gi + 1) * og], ref_out) <= TOL
        assert rel_err(free[1][:, gi * dg:(gi + 1) * dg], ref_dx) <= TOL
        assert rel_err(free[2][gi * og:(gi + 1) * og], np.asarray(ref_dw).reshape(og, dg, k, k)) <= TOL
        assert rel_err(free[3][gi * og:(gi + 1) * og], ref_db) <= TOL
    np.testing.assert_array_equal(host(d_x), x)
    np.testing.assert_array_equal(host(d_og), og_t)


def test_direct_exact_on_small_integers(oracle):
    """Small-integer tensors make every sum exact in fp32, so the direct kernels must reproduce the
    lowering pipeline bit for bit whatever the summation order."""
    b, d, n, k, p, o = 3, 6, 11, 5, 2, 9
    m = n + 2 * p - k + 1
    rng = np.random.default_rng(99)
    x = rng.integers(-3, 4, (b, d, n, n)).astype(np.float32)
    w = rng.integers(-2, 3, (o, d, k, k)).astype(np.float32)
    bias = rng.integers(-4, 5, o).astype(np.float32)
    og = rng.integers(-3, 4, (b, o, m, m)).astype(np.float32)
    ref_out, lowered = oracle.conv_forward(x, w, bias, k, 1, p)
    ref_dx, ref_dw, _ = oracle.conv_backward(x.shape, w, og, lowered, k, 1, p)
    drv = driver()
    d_x, d_w, d_og = dev(x), dev(w), dev(og)
    sf, sb = _slabs(d_w, o, d, k)
    out, dx, dw = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, d, k, k))
    drv.conv_direct_forward(out, d_x, sf, dev(bias), b, d, n, k, p, o)
    drv.conv_direct_backward_data(dx, d_og, sb, b, d, n, k, p, o)
    drv.conv_direct_backward_weights(dw, d_og, d_x, b, d, n, k, p, o)
    np.testing.assert_array_equal(host(out), ref_out)
    np.testing.assert_array_equal(host(dx), ref_dx)
    np.testing.assert_array_equal(host(dw).reshape(-1), np.asarray(ref_dw).reshape(-1))


@pytest.mark.parametrize("tile", [161, 162])
@pytest.mark.parametrize("shape", [(3, 48, 27, 5, 2, 128), (3, 80, 13, 3, 1, 48), (2, 7, 12, 5, 0, 16)], ids=_ids)
def test_direct_16_row_instances(oracle, shape, tile):
    """Map counts of an odd number of 16-row blocks (48 = one group of CaffeNet conv2's data gradient) run on
    the 16-row MFMA kernel; both of its pixel tiles (128 and 256 pixels) must give the same convolution as
    the oracle, bit for bit on small integers."""
    b, d, n, k, p, o = shape
    m = n + 2 * p - k + 1
    rng = np.random.default_rng(7)
    x = rng.integers(-3, 4, (b, d, n, n)).astype(np.float32)
    w = rng.integers(-2, 3, (o, d, k, k)).astype(np.float32)
    bias = rng.integers(-4, 5, o).astype(np.float32)
    og = rng.integers(-3, 4, (b, o, m, m)).astype(np.float32)
    ref_out, lowered = oracle.conv_forward(x, w, bias, k, 1, p)
    ref_dx, _, _ = oracle.conv_backward(x.shape, w, og, lowered, k, 1, p)
    drv = driver()
    d_x, d_w, d_og = dev(x), dev(w), dev(og)
    sf, sb = _slabs(d_w, o, d, k)
    out, dx = empty((b, o, m, m)), empty((b, d, n, n))
    from caffecontroll_amd import CctHipError
    with tuning("direct_tile", tile):
        ran = []
        try:
            if (o + 15) // 16 in (1, 3, 5):
                drv.conv_direct_forward(out, d_x, sf, dev(bias), b, d, n, k, p, o)
                ran.append(drv.lib.cct_hip_last_kernel().decode())
                np.testing.assert_array_equal(host(out), ref_out)
            if (d + 15) // 16 in (1, 3, 5):
                drv.conv_direct_backward_data(dx, d_og, sb, b, d, n, k, p, o)
                ran.append(drv.lib.cct_hip_last_kernel().decode())
                np.testing.assert_array_equal(host(dx), ref_dx)
        except CctHipError as e:
            # a pinned instance whose source patch does not fit is refused, never run
            assert tile == 162 and "not covered" in str(e)
            pytest.skip("the 256-pixel tile's four-channel patch does not fit for this geometry")
    assert ran and all(name.startswith("conv_direct16_kernel") for name in ran)


def test_direct_support_matrix_and_errors():
    from caffecontroll_amd import CctHipError
    drv = driver()
    assert drv.conv_direct_supported(256, 96, 27, 5, 1, 2, 256)
    assert drv.conv_direct_supported(256, 256, 13, 3, 1, 1, 384)
    assert not drv.conv_direct_supported(256, 3, 227, 11, 4, 0, 96)   # k = 11, stride 4
    assert not drv.conv_direct_supported(4, 3, 20, 5, 4, 2, 10)       # stride 4
    assert drv.conv_direct_supported(4, 3, 40, 5, 1, 2, 10)           # padded image 44 wide
    assert drv.conv_direct_supported(4, 3, 62, 5, 1, 2, 10)           # padded image 66 wide: two column bands
    assert drv.conv_direct_supported(2, 8, 224, 3, 1, 1, 16)          # VGG-sized planes
    assert all(drv.conv_direct_supported(1, 3, n, 3, 1, 1, 4) for n in range(8, 1700))   # every width in between
    assert drv.conv_direct_supported(1, 8, 4000, 5, 1, 2, 8)
    assert not drv.conv_direct_supported(1, 3, 9000, 3, 1, 1, 4)      # output rows beyond the weight gradient's 64 pieces
    assert not drv.conv_direct_supported(4, 3, 20, 5, 1, 5, 10)       # padding above k-1
    assert not drv.conv_direct_supported(1, 2, 3, 3, 1, 0, 2)         # 1x1 output: a tile would span 128 images
    # tensors read through buffer descriptors (2 GiB of addressable bytes each) must stay below 2^29 floats
    assert drv.conv_direct_supported(4660, 128, 30, 3, 1, 1, 16)
    assert not drv.conv_direct_supported(4661, 128, 30, 3, 1, 1, 16)      # input just above 2 GiB
    assert drv.conv_direct_supported(2330, 256, 30, 3, 1, 1, 16, 2)
    assert not drv.conv_direct_supported(2331, 256, 30, 3, 1, 1, 16, 2)   # the same as two groups
    assert drv.conv_strided_supported(1848, 3, 227, 11, 4, 0, 96)
    assert not drv.conv_strided_supported(1849, 3, 227, 11, 4, 0, 96)     # output gradient of 2 GiB and more
    assert not drv.conv_strided_backward_data_supported(1849, 3, 227, 11, 4, 0, 96)
    # groups must divide both depths
    assert drv.conv_direct_supported(4, 6, 13, 3, 1, 1, 8, 2)
    assert not drv.conv_direct_supported(4, 6, 13, 3, 1, 1, 9, 2)
    assert not drv.conv_direct_supported(4, 7, 13, 3, 1, 1, 8, 2)
    with pytest.raises(CctHipError):
        drv.conv_direct_forward(empty((4,)), empty((4,)), empty((4,)), None, 4, 3, 30, 9, 4, 10)   # no 9 x 9 instance
    with pytest.raises(CctHipError):
        drv.conv_direct_backward_weights(empty((1,)), empty((1,)), empty((1,)), 4, 3, 20, 9, 4, 10)
    w = empty((drv.conv_direct_slab_floats(10, 3, 5, 0),), fill=1.0)
    with pytest.raises(CctHipError):
        drv.conv_direct_slabs(w, w, 10, 3, 5, 0)


@pytest.mark.parametrize("shape", [(8, 96, 27, 5, 2, 256), (16, 20, 12, 5, 0, 50), (4, 256, 13, 3, 1, 384)],
                         ids=_ids)
def test_bridge_path_levels_agree(oracle, shape):
    """ConvolutionBridge at path levels 0..3 (separate passes, fused epilogues, direct data
    gradient, all direct): every level within 1e-4 of the oracle's CPU ConvolutionBridge."""
    from caffecontroll_amd.bridges import ConvolutionLayer
    b, d, n, k, p, o = shape
    x, w, bias, og, m = _tensors(shape, 777 + sum(shape))
    ref_out, lowered = oracle.conv_forward(x, w, bias, k, 1, p)
    ref_dx, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, k, 1, p)
    drv = driver()
    for level in (0, 1, 2, 3):
        in_data, in_grad = dev(x), empty((b, d, n, n))
        out_data, out_grad = empty((b, o, m, m)), dev(og)
        layer = ConvolutionLayer(b, d, n, k, 1, p, o, in_data, in_grad, out_data, out_grad)
        # default: all-direct where the kernels cover the geometry and the layer is not tiny
        gemm_flop = 2.0 * o * b * m * m * k * k * d
        assert layer.path() == (3 if gemm_flop >= 2e9 else 1)
        layer.set_options(fused=level)
        assert layer.path() == level
        drv.memcpy(layer.model_ptr(), w.ctypes.data, w.nbytes, 0)
        drv.memcpy(layer.bias_ptr(), bias.ctypes.data, bias.nbytes, 0)
        layer.forward()
        layer.backward(with_update=False)
        assert rel_err(host(out_data), ref_out) <= TOL, level
        assert rel_err(host(in_grad), ref_dx) <= TOL, level
        dw = np.empty((o, d, k, k), np.float32)
        db = np.empty((o,), np.float32)
        drv.memcpy(dw.ctypes.data, layer.model_grad_ptr(), dw.nbytes, 1)
        drv.memcpy(db.ctypes.data, layer.bias_grad_ptr(), db.nbytes, 1)
        assert rel_err(dw, np.asarray(ref_dw).reshape(dw.shape)) <= TOL, level
        assert rel_err(db, ref_db) <= TOL, level
        np.testing.assert_array_equal(host(out_grad), og)
        layer.close()


def test_bridge_falls_back_where_direct_does_not_apply():
    from caffecontroll_amd.bridges import ConvolutionLayer
    b, d, n, k, s, p, o = 2, 3, 20, 5, 4, 2, 10
    m = (n + 2 * p - k) // s + 1
    layer = ConvolutionLayer(b, d, n, k, s, p, o, empty((b, d, n, n), fill=0.0), empty((b, d, n, n)),
                             empty((b, o, m, m)), empty((b, o, m, m), fill=0.0))
    assert layer.path() == 1
    layer.set_options(fused=3)
    assert layer.path() == 1
    layer.close()


# full-size layers of the CaffeNet iteration (batch 256): conv2 whole and one group of it, conv3,
# one group of conv4; between them they run every compile-time specialised weight-gradient instance
# (8, 4 and 6 wavefronts)
FULL_SIZE = [(256, 96, 27, 5, 2, 256), (256, 48, 27, 5, 2, 128), (256, 256, 13, 3, 1, 384),
             (256, 192, 13, 3, 1, 192), (255, 192, 13, 3, 1, 128),
             # beyond CaffeNet: a VGG-sized 3 x 3 layer (four column bands, weight-gradient rows in four pieces), a
             # 112-wide one with an odd batch, a 7 x 7 stride-1 layer
             (32, 64, 224, 3, 1, 64), (17, 128, 112, 3, 1, 128), (32, 64, 56, 7, 3, 64),
             # 3 x 3 layers on 28-, 14- and 7-pixel maps (weight gradients by compile-time instances of their own)
             (64, 128, 28, 3, 1, 256), (255, 256, 14, 3, 1, 256), (256, 512, 7, 3, 1, 512),
             # 5 x 5 layers on 28- and 14-pixel maps (likewise)
             (128, 96, 28, 5, 2, 256), (127, 128, 14, 5, 2, 256)]


# the grouped layers of the CaffeNet iteration at batch 256, both groups in one launch: conv2, conv4, conv5
FULL_SIZE_GROUPED = [(256, 96, 27, 5, 2, 256, 2), (256, 384, 13, 3, 1, 384, 2), (256, 384, 13, 3, 1, 256, 2)]


@pytest.mark.parametrize("cfg", FULL_SIZE_GROUPED, ids=lambda c: "b%d_d%d_n%d_k%d_p%d_o%d_g%d" % c)
def test_full_size_grouped_vs_float64(cfg):
    """CaffeNet's grouped layers at full size, every group in the same launch, against torch's float64
    grouped convolution and its gradients."""
    import torch
    import torch.nn.functional as F
    b, d, n, k, p, o, groups = cfg
    m = n + 2 * p - k + 1
    drv = driver()
    g = torch.Generator(device="cuda").manual_seed(4321)
    x = torch.randn((b, d, n, n), device="cuda", generator=g)
    w = torch.randn((o, d // groups, k, k), device="cuda", generator=g) * 0.01
    bias = torch.full((o,), 0.1, device="cuda")
    og = torch.randn((b, o, m, m), device="cuda", generator=g)
    sf = empty((drv.conv_direct_slab_floats(o, d, k, 0, groups),))
    sb = empty((drv.conv_direct_slab_floats(o, d, k, 1, groups),))
    drv.conv_direct_slabs(sf, w, o, d, k, 0, groups)
    drv.conv_direct_slabs(sb, w, o, d, k, 1, groups)
    out, dx, dw, db = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, d // groups, k, k)), empty((o,))
    drv.conv_direct_forward(out, x, sf, bias, b, d, n, k, p, o, groups=groups)
    drv.conv_direct_backward_data(dx, og, sb, b, d, n, k, p, o, groups=groups)
    drv.conv_direct_backward_weights(dw, og, x, b, d, n, k, p, o, db=db, groups=groups)
    torch.cuda.synchronize()
    db_ref = og.double().sum(dim=(0, 2, 3))
    assert ((db.double() - db_ref).abs().max() / db_ref.abs().max()).item() <= TOL
    worst_out = worst_dx = scale_out = scale_dx = 0.0
    dw_ref = torch.zeros((o, d // groups, k, k), dtype=torch.float64, device="cuda")
    wd = w.double()
    for i in range(0, b, 32):
        xs, gs = x[i:i + 32].double(), og[i:i + 32].double()
        ro = F.conv2d(xs, wd, bias.double(), padding=p, groups=groups)
        rdx = torch.nn.grad.conv2d_input(xs.shape, wd, gs, padding=p, groups=groups)
        dw_ref += torch.nn.grad.conv2d_weight(xs, wd.shape, gs, padding=p, groups=groups)
        worst_out = max(worst_out, (out[i:i + 32].double() - ro).abs().max().item())
        worst_dx = max(worst_dx, (dx[i:i + 32].double() - rdx).abs().max().item())
        scale_out = max(scale_out, ro.abs().max().item())
        scale_dx = max(scale_dx, rdx.abs().max().item())
    assert worst_out / scale_out <= TOL
    assert worst_dx / scale_dx <= TOL
    assert ((dw.double() - dw_ref).abs().max() / dw_ref.abs().max()).item() <= TOL


@pytest.mark.parametrize("cfg", FULL_SIZE, ids=_ids)
def test_full_size_direct_vs_float64(cfg):
    """Full-size layers (benchmark configuration 2 first; the last one with an odd batch): the three direct
    kernels against torch's float64 convolution and its gradients (independent of this library
    and of the oracle)."""
    import torch
    import torch.nn.functional as F
    b, d, n, k, p, o = cfg
    m = n + 2 * p - k + 1
    drv = driver()
    g = torch.Generator(device="cuda").manual_seed(1235)
    x = torch.randn((b, d, n, n), device="cuda", generator=g)
    w = torch.randn((o, d, k, k), device="cuda", generator=g) * 0.01
    bias = torch.full((o,), 0.1, device="cuda")
    og = torch.randn((b, o, m, m), device="cuda", generator=g)
    sf, sb = _slabs(w, o, d, k)
    out, dx, dw = empty((b, o, m, m)), empty((b, d, n, n)), empty((o, d, k, k))
    drv.conv_direct_forward(out, x, sf, bias, b, d, n, k, p, o)
    drv.conv_direct_backward_data(dx, og, sb, b, d, n, k, p, o)
    db = empty((o,))
    drv.conv_direct_backward_weights(dw, og, x, b, d, n, k, p, o, db=db)
    torch.cuda.synchronize()
    db_ref = og.double().sum(dim=(0, 2, 3))
    assert ((db.double() - db_ref).abs().max() / db_ref.abs().max()).item() <= TOL

    def err(got, ref):
        return ((got.double() - ref).abs().max() / ref.abs().max()).item()

    # float64 references in chunks of 32 images to bound memory
    worst_out = worst_dx = 0.0
    dw_ref = torch.zeros((o, d, k, k), dtype=torch.float64, device="cuda")
    wd = w.double()
    scale_out = scale_dx = 0.0
    for i in range(0, b, 32):
        xs, gs = x[i:i + 32].double(), og[i:i + 32].double()
        ro = F.conv2d(xs, wd, bias.double(), padding=p)
        rdx = torch.nn.grad.conv2d_input(xs.shape, wd, gs, padding=p)
        dw_ref += torch.nn.grad.conv2d_weight(xs, wd.shape, gs, padding=p)
        worst_out = max(worst_out, (out[i:i + 32].double() - ro).abs().max().item())
        worst_dx = max(worst_dx, (dx[i:i + 32].double() - rdx).abs().max().item())
        scale_out = max(scale_out, ro.abs().max().item())
        scale_dx = max(scale_dx, rdx.abs().max().item())
    assert worst_out / scale_out <= TOL
    assert worst_dx / scale_dx <= TOL
    assert err(dw, dw_ref) <= TOL


# every specialised weight-gradient instance (8, 4, 6 x 2 wavefronts; 5x5 on 27, 28 and 14 rows, 3x3 on 13, 14, 7 and
# 28), with
# map counts that leave rows of the last tile empty, an odd batch (the last step holds one image) and two groups
STAGED_ROWS = [(256, 96, 27, 5, 2, 256, 1), (64, 48, 27, 5, 2, 100, 1), (33, 48, 27, 5, 2, 128, 2),
               (256, 256, 13, 3, 1, 384, 1), (255, 192, 13, 3, 1, 192, 1), (64, 64, 13, 3, 1, 250, 1),
               (63, 128, 13, 3, 1, 170, 2), (256, 192, 13, 3, 1, 192, 2),
               (128, 128, 14, 3, 1, 256, 1), (65, 192, 14, 3, 1, 192, 1), (31, 64, 16, 3, 0, 100, 2),
               (128, 128, 7, 3, 1, 250, 1), (64, 192, 7, 3, 1, 170, 2), (33, 64, 9, 3, 0, 128, 1),
               (32, 64, 28, 3, 1, 256, 1), (17, 128, 28, 3, 1, 192, 1), (9, 64, 30, 3, 0, 100, 2),
               (64, 32, 28, 5, 2, 100, 1), (33, 64, 28, 5, 2, 256, 1), (65, 32, 14, 5, 2, 128, 2),
               (32, 64, 18, 5, 0, 250, 1)]


@pytest.mark.parametrize("cfg", STAGED_ROWS, ids=lambda c: "b%d_d%d_n%d_k%d_p%d_o%d_g%d" % c)
def test_wgrad_rows_staged_in_lds_equal_rows_fetched_by_lanes(cfg):
    """The shape-specialised weight-gradient kernels feed the MFMAs' output-gradient operand either from rows each
    lane fetched itself or from rows staged in LDS: the same values in the same order of additions, so weight and
    bias gradients agree bit for bit (with the count of step ranges pinned: the default follows the LDS a workgroup
    takes, and another split of the steps is another order of additions)."""
    import torch
    b, d, n, k, p, o, groups = cfg
    m = n + 2 * p - k + 1
    drv = driver()
    g = torch.Generator(device="cuda").manual_seed(99)
    x = torch.randn((b, d * groups, n, n), device="cuda", generator=g)
    og = torch.randn((b, o * groups, m, m), device="cuda", generator=g)
    got = {}
    for mode in (1, 2):
        dw, db = empty((o * groups, d, k, k), fill=float("nan")), empty((o * groups,), fill=float("nan"))
        with tuning("direct_alds", mode), tuning("direct_splits", 5):
            drv.conv_direct_backward_weights(dw, og, x, b, d * groups, n, k, p, o * groups, db=db, groups=groups)
            names = drv.lib.cct_hip_last_kernel().decode()
        torch.cuda.synchronize()
        got[mode] = (host(dw), host(db), names)
    assert "wgrad_spec_kernel" in got[1][2] and got[1][2].endswith(",true>"), got[1][2]
    assert got[2][2].endswith(",false>"), got[2][2]
    assert not np.isnan(got[1][0]).any() and not np.isnan(got[1][1]).any()
    assert np.array_equal(got[1][0], got[2][0])
    assert np.array_equal(got[1][1], got[2][1])


# (batch, channels, size, kernel, pad, maps): LeNet's first layer, RGB inputs, every pad of a 3 x 3 and a 5 x 5 filter,
# one map, the most maps, batches that do not divide into the image groups of the weight-gradient launch
SMALL = [(64, 1, 28, 5, 0, 20), (7, 3, 17, 3, 1, 32), (5, 3, 12, 5, 2, 9), (3, 1, 9, 3, 2, 1), (33, 1, 8, 5, 4, 5),
         (1, 3, 5, 5, 0, 2), (600, 1, 6, 3, 0, 3)]


@pytest.mark.parametrize("shape", SMALL, ids=lambda c: "b%d_d%d_n%d_k%d_p%d_o%d" % c)
def test_small_convolution_kernels_match_oracle(oracle, shape):
    """The multiply-add kernels for layers of one or three channels and few maps: forward (with and without bias
    and ReLU) and weight / bias gradient against the oracle's lowering + GEMM; two runs bit-identical."""
    b, d, n, k, p, o = shape
    drv = driver()
    assert drv.conv_small_supported(b, d, n, k, 1, p, o)
    m = n + 2 * p - k + 1
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    w = (rng.standard_normal((o, d, k, k)) * 0.2).astype(np.float32)
    bias = rng.standard_normal(o).astype(np.float32)
    og = rng.standard_normal((b, o, m, m)).astype(np.float32)
    ref_out, low = oracle.conv_forward(x, w, bias, k, 1, p)
    _, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, low, k, 1, p, need_in_grad=False)
    dx_, dw_, dog = dev(x), dev(w), dev(og)
    out = empty((b, o, m, m), fill=float("nan"))
    drv.conv_small_forward(out, dx_, dw_, dev(bias), b, d, n, k, p, o)
    assert rel_err(host(out), ref_out) <= TOL
    drv.conv_small_forward(out, dx_, dw_, dev(bias), b, d, n, k, p, o, relu=True)
    assert rel_err(host(out), np.maximum(ref_out, 0)) <= TOL
    ref_nobias, _ = oracle.conv_forward(x, w, None, k, 1, p)
    drv.conv_small_forward(out, dx_, dw_, None, b, d, n, k, p, o)
    assert rel_err(host(out), ref_nobias) <= TOL
    runs = []
    for _ in range(2):
        gw, gb = empty((o, d, k, k), fill=float("nan")), empty((o,), fill=float("nan"))
        drv.conv_small_backward_weights(gw, dog, dx_, b, d, n, k, p, o, db=gb)
        runs.append((host(gw), host(gb)))
    assert rel_err(runs[0][0], ref_dw.reshape(o, d, k, k)) <= TOL
    assert rel_err(runs[0][1], ref_db.reshape(o)) <= TOL
    assert np.array_equal(runs[0][0], runs[1][0]) and np.array_equal(runs[0][1], runs[1][1])
    gw = empty((o, d, k, k), fill=float("nan"))
    drv.conv_small_backward_weights(gw, dog, dx_, b, d, n, k, p, o)    # no bias gradient wanted
    assert np.array_equal(host(gw), runs[0][0])


def test_small_convolution_support_and_errors():
    drv = driver()
    assert not drv.conv_small_supported(4, 2, 12, 5, 1, 0, 8)      # two channels
    assert not drv.conv_small_supported(4, 1, 12, 5, 2, 0, 8)      # strided
    assert not drv.conv_small_supported(4, 1, 12, 7, 1, 0, 8)      # 7 x 7
    assert not drv.conv_small_supported(4, 1, 12, 5, 1, 0, 33)     # too many maps
    assert not drv.conv_small_supported(4, 1, 3, 5, 1, 0, 8)       # filter larger than the padded image
    assert not drv.conv_small_supported(4, 1, 12, 5, 1, 5, 8)      # pad >= k
    from caffecontroll_amd import CctHipError
    with pytest.raises(CctHipError, match="not covered"):
        drv.conv_small_forward(empty((4, 8, 8, 8)), empty((4, 2, 12, 12)), empty((8, 2, 5, 5)), None, 4, 2, 12, 5, 0, 8)
