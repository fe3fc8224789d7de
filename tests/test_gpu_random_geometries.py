"""Seeded random geometries, beyond the hand-picked ones of the other files: the convolution bridge
on its all-direct and its lowering path, max pooling (both kernel families, with and without the
mask of a folded ReLU) and LRN, each against the CPU oracle.  The draws include what the fixed
lists tend to miss: trailing rows and columns no pooling window covers, paddings up to k - 1, map
and channel counts that are not multiples of any tile, planes whose size is not a multiple of four."""
import numpy as np
import pytest

from gpu_util import driver, dev, empty, host, rel_err, tuning

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _conv_geometries(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        k, s = [(3, 1), (5, 1), (1, 1), (7, 1), (11, 4), (7, 2), (5, 2), (3, 2)][rng.integers(0, 8)]
        p = int(rng.integers(0, k)) if rng.random() < 0.7 else (k - 1) // 2
        n = int(rng.integers(max(k - 2 * p, 1), 257 if rng.random() < 0.25 else 70 if s > 1 else 64))
        if n + 2 * p < k:
            continue
        m = (n + 2 * p - k) // s + 1
        b, d, o = int(rng.integers(1, 10)), int(rng.integers(1, 40)), int(rng.integers(1, 80))
        if 2.0 * b * m * m * k * k * d * o > 6e8 or b * m * m * k * k * d > 3e7:
            continue
        out.append((b, d, n, k, s, p, o))
    return out


def _direct_expected(shape):
    """Geometries that must not fall back to the lowering path, at any width up to 256: stride 1 with k = 1 (no
    padding), k = 3 or 5 from 5 x 5 outputs up, k = 7 from 6 x 6 outputs up (below that a tile of 128 pixels spans
    more images than its patch holds); stride 2 with k = 3, 5 or 7."""
    b, d, n, k, s, p, o = shape
    m = (n + 2 * p - k) // s + 1
    if s == 1:
        return (k == 1 and p == 0) or (k in (3, 5) and m >= 5) or (k == 7 and m >= 6)
    return s == 2 and k in (3, 5, 7)


@pytest.mark.parametrize("seed", [11, 12])
def test_convolution_bridge_random_geometries(oracle, seed):
    from caffecontroll_amd.bridges import ConvolutionLayer
    drv = driver()
    rng = np.random.default_rng(seed + 100)
    direct = 0
    for shape in _conv_geometries(seed, 40):
        b, d, n, k, s, p, o = shape
        m = (n + 2 * p - k) // s + 1
        x = rng.standard_normal((b, d, n, n)).astype(np.float32)
        w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
        bias = rng.standard_normal(o).astype(np.float32)
        og = rng.standard_normal((b, o, m, m)).astype(np.float32)
        ref_out, lowered = oracle.conv_forward(x, w, bias, k, s, p)
        ref_dx, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, k, s, p)
        for level in (3, 1):   # all direct where the kernels cover the geometry; lowering + GEMM + lifting
            in_grad, out_data = empty((b, d, n, n)), empty((b, o, m, m))
            layer = ConvolutionLayer(b, d, n, k, s, p, o, dev(x), in_grad, out_data, dev(og))
            layer.set_options(fused=level)
            direct += layer.path() == 3
            if level == 3 and _direct_expected(shape):
                assert layer.path() == 3, shape
            drv.memcpy(layer.model_ptr(), w.ctypes.data, w.nbytes, 0)
            drv.memcpy(layer.bias_ptr(), bias.ctypes.data, bias.nbytes, 0)
            layer.forward()
            layer.backward(with_update=False)
            dw, db = np.empty((o, d, k, k), np.float32), np.empty((o,), np.float32)
            drv.memcpy(dw.ctypes.data, layer.model_grad_ptr(), dw.nbytes, 1)
            drv.memcpy(db.ctypes.data, layer.bias_grad_ptr(), db.nbytes, 1)
            what = (shape, level, layer.path())
            assert rel_err(host(out_data), ref_out) <= TOL, what
            assert rel_err(host(in_grad), ref_dx) <= TOL, what
            assert rel_err(dw, np.asarray(ref_dw).reshape(dw.shape)) <= TOL, what
            assert rel_err(db, ref_db) <= TOL, what
            layer.close()
    assert direct >= 30   # most draws are inside the direct kernels' reach


@pytest.mark.parametrize("seed", [31, 32])
def test_wide_image_convolutions_stay_on_the_direct_kernels(oracle, seed):
    """Stride-1 layers with k = 3, 5 or 7 on images 61 to 400 pixels wide: forward and data gradient in column
    bands, the weight gradient with its output rows taken in pieces; all three against the oracle, and never the
    lowering path."""
    from caffecontroll_amd.bridges import ConvolutionLayer
    drv = driver()
    rng = np.random.default_rng(seed)
    done = 0
    while done < 8:
        k = int(rng.choice([3, 5, 7]))
        p = int(rng.integers(0, k))
        n = int(rng.integers(61, 401))
        m = n + 2 * p - k + 1
        b, d, o = int(rng.integers(1, 4)), int(rng.integers(1, 9)), int(rng.integers(1, 40))
        if 2.0 * b * m * m * k * k * d * o > 8e8:
            continue
        x = rng.standard_normal((b, d, n, n)).astype(np.float32)
        w = (rng.standard_normal((o, d, k, k)) * 0.1).astype(np.float32)
        bias = rng.standard_normal(o).astype(np.float32)
        og = rng.standard_normal((b, o, m, m)).astype(np.float32)
        ref_out, lowered = oracle.conv_forward(x, w, bias, k, 1, p)
        ref_dx, ref_dw, ref_db = oracle.conv_backward(x.shape, w, og, lowered, k, 1, p)
        assert drv.conv_direct_supported(b, d, n, k, 1, p, o), (b, d, n, k, p, o)
        in_grad, out_data = empty((b, d, n, n)), empty((b, o, m, m))
        layer = ConvolutionLayer(b, d, n, k, 1, p, o, dev(x), in_grad, out_data, dev(og))
        layer.set_options(fused=3)
        assert layer.path() == 3
        drv.memcpy(layer.model_ptr(), w.ctypes.data, w.nbytes, 0)
        drv.memcpy(layer.bias_ptr(), bias.ctypes.data, bias.nbytes, 0)
        layer.forward()
        layer.backward(with_update=False)
        dw, db = np.empty((o, d, k, k), np.float32), np.empty((o,), np.float32)
        drv.memcpy(dw.ctypes.data, layer.model_grad_ptr(), dw.nbytes, 1)
        drv.memcpy(db.ctypes.data, layer.bias_grad_ptr(), db.nbytes, 1)
        what = (b, d, n, k, p, o)
        assert rel_err(host(out_data), ref_out) <= TOL, what
        assert rel_err(host(in_grad), ref_dx) <= TOL, what
        assert rel_err(dw, np.asarray(ref_dw).reshape(dw.shape)) <= TOL, what
        assert rel_err(db, ref_db) <= TOL, what
        layer.close()
        done += 1


@pytest.mark.parametrize("seed", [21, 22])
def test_pooling_and_lrn_random_geometries(oracle, seed):
    import torch
    drv = driver()
    rng = np.random.default_rng(seed)
    uncovered = 0
    for case in range(60):
        B, D, n = int(rng.integers(1, 9)), int(rng.integers(1, 40)), int(rng.integers(2, 60))
        k, s = int(rng.integers(2, 5)), int(rng.integers(1, 4))
        if n >= k:
            oR = (n - k) // s + 1
            uncovered += (n - k) % s != 0
            x = rng.standard_normal((B, D, n, n)).astype(np.float32)
            x[rng.random(x.shape) < 0.3] = 0
            with tuning("pool_plane", int(rng.integers(0, 2))):
                idx, y = empty((B, D, oR, oR), dtype=torch.int32), empty((B, D, oR, oR))
                args = drv.pool_args(k, s, n, n, D, B, idx)
                drv.maxpool_forward(y, dev(x), args)
                ry, ridx = oracle.maxpool_forward(x, k, s)
                np.testing.assert_array_equal(host(y), ry)
                np.testing.assert_array_equal(host(idx), ridx)
                og = rng.standard_normal(ry.shape).astype(np.float32)
                g, gm = empty(x.shape), empty(x.shape)
                drv.maxpool_backward(g, dev(og), args)
                np.testing.assert_array_equal(host(g), oracle.maxpool_backward(og, ridx, n, n), err_msg=str((B, D, n, k, s)))
                # masked with (pooled > 0): windows whose maximum is not positive pass no gradient
                drv.maxpool_backward(gm, dev(og), args, pooled=y)
                want = oracle.maxpool_backward(np.where(ry > 0, og, 0).astype(np.float32), ridx, n, n)
                np.testing.assert_array_equal(host(gm), want, err_msg=str((B, D, n, k, s)))
        size = int(rng.choice([3, 5, 5, 5, 7]))
        alpha, beta = float(rng.choice([1e-4, 1e-2, 0.3])), float(rng.choice([0.75, 0.75, 0.5, 1.25]))
        n2 = int(rng.integers(1, 30))
        x = (rng.standard_normal((B, D, n2, n2)) * 3).astype(np.float32)
        og = rng.standard_normal((B, D, n2, n2)).astype(np.float32)
        y, den, g = empty(x.shape), empty(x.shape), empty(x.shape)
        dx = dev(x)
        drv.lrn_forward(y, dx, n2, n2, D, B, size, alpha, beta, den)
        ry, rden = oracle.lrn_forward(x, size, alpha, beta)
        what = (B, D, n2, size, alpha, beta)
        assert rel_err(host(den), rden) <= 1e-6, what
        assert rel_err(host(y), ry) <= 1e-5, what
        drv.lrn_backward(g, dev(og), dx, n2, n2, D, B, size, alpha, beta, den)
        assert rel_err(host(g), oracle.lrn_backward(og, x, rden, size, alpha, beta)) <= 1e-5, what
    assert uncovered >= 10


@pytest.mark.parametrize("seed", [31, 32])
def test_gemm_and_lowering_random_shapes(oracle, seed):
    """sgemm in every layout with ragged sizes, unaligned leading dimensions and the split over the
    contraction (against float64); lowering, lifting (+ bias gradient) bit for bit against the oracle,
    kernel sizes from 1 to 11, any stride and padding."""
    from caffecontroll_amd.driver import conv_pmap, lift_args
    RM, CM, N_, T_ = 101, 102, 111, 112
    drv = driver()
    rng = np.random.default_rng(seed)

    def store(mat, trans, order, pad):
        src = mat.T if trans == T_ else mat
        if order == CM:
            src = src.T
        buf = np.full((src.shape[0], src.shape[1] + pad), np.nan, np.float32)
        buf[:, :src.shape[1]] = src
        return buf, src.shape[1] + pad

    for case in range(40):
        kind = rng.integers(0, 4)
        if kind == 0:
            M, N, K = (int(rng.integers(1, 300)) for _ in range(3))
        elif kind == 1:
            M, N, K = int(rng.integers(1, 64)), int(rng.integers(1, 64)), int(rng.integers(256, 6000))
        elif kind == 2:
            M, N, K = int(rng.integers(1, 40)) * 16, int(rng.integers(1, 40)) * 4, int(rng.integers(1, 30)) * 16
        else:
            M, N, K = int(rng.integers(64, 700)), int(rng.integers(64, 2000)), int(rng.integers(1, 130))
        pad = int(rng.choice([0, 0, 1, 3, 4]))
        TA, TB, order = int(rng.choice([N_, T_])), int(rng.choice([N_, T_])), int(rng.choice([RM, CM]))
        alpha, beta = [(1.0, 0.0), (1.5, -0.5), (0.7, 1.0)][rng.integers(0, 3)]
        opA = rng.standard_normal((M, K)).astype(np.float32)
        opB = rng.standard_normal((K, N)).astype(np.float32)
        C0 = rng.standard_normal((M, N)).astype(np.float32)
        (A, lda), (B, ldb), (Cb, ldc) = store(opA, TA, order, pad), store(opB, TB, order, pad), store(C0, N_, order, pad)
        dC = dev(np.full_like(Cb, np.nan) if beta == 0.0 else Cb)
        drv.sgemm(order, TA, TB, M, N, K, alpha, dev(A), lda, dev(B), ldb, beta, dC, ldc)
        out = host(dC)
        got = out[:, :N] if order == RM else out[:, :M].T
        what = (M, N, K, pad, TA, TB, order, alpha, beta)
        assert rel_err(got, alpha * opA.astype(np.float64) @ opB.astype(np.float64) + beta * C0) <= TOL, what
        assert not pad or np.isnan(out[:, -pad:]).all(), what

        k, s = [(3, 1), (5, 1), (1, 1), (2, 2), (11, 4), (7, 2), (5, 2), (3, 2), (4, 3), (6, 1)][rng.integers(0, 10)]
        p, b, d = int(rng.integers(0, k)), int(rng.integers(1, 8)), int(rng.integers(1, 30))
        n = int(rng.integers(max(k - 2 * p, 1), 50))
        m = (n + 2 * p - k) // s + 1
        if n + 2 * p < k or b * m * m * k * k * d > 2e7:
            continue
        what = (b, d, n, k, s, p)
        x = rng.standard_normal((b, d, n, n)).astype(np.float32)
        low = empty((b * m * m, k * k * d))
        drv.lower_cube(low, dev(x), conv_pmap(b, d, n, k, s, p))
        np.testing.assert_array_equal(host(low), oracle.lower_cube(x, k, s, p), err_msg=str(what))
        y = rng.standard_normal((k * k * d, b * m * m)).astype(np.float32)
        o = int(rng.integers(1, 40))
        og = rng.standard_normal((b, o, m, m)).astype(np.float32)
        dx, db = empty((b, d, n, n)), empty((o,))
        drv.inverse_lower_cube_bias_backward(dx, dev(y), lift_args(b, d, n, k, s, p), db, dev(og), m * m, o, b)
        np.testing.assert_array_equal(host(dx), oracle.inverse_lower_cube(y, b, d, n, k, s, p), err_msg=str(what))
        assert rel_err(host(db), og.astype(np.float64).sum(axis=(0, 2, 3))) <= TOL, what


def _random_chain(rng):
    """A random layer chain: one to three convolutions (kernel sizes 1..11, strides, paddings, two
    groups) with ReLU / pooling / LRN between them, up to two inner-product layers with ReLU and
    dropout, a classifier and the loss."""
    from caffecontroll_amd import nets
    B, D, S = int(rng.integers(1, 9)), int(rng.choice([1, 2, 3, 4, 6])), int(rng.integers(12, 40))
    layers, d, n = [], D, S
    for _ in range(int(rng.integers(1, 4))):
        k, s = [(3, 1), (5, 1), (3, 1), (3, 2), (5, 2), (7, 2), (1, 1), (4, 1), (11, 4)][rng.integers(0, 9)]
        p = int(rng.integers(0, min(k, 3)))
        m = (n + 2 * p - k) // s + 1 if n + 2 * p >= k else 0
        if m < 2:
            break
        group = int(rng.choice([1, 1, 2])) if d % 2 == 0 else 1
        o = int(rng.integers(1, 24)) * group
        layers.append(nets.conv(o, k, stride=s, pad=p, group=group, lr_mult=(1.0, 2.0),
                                decay_mult=(1.0, float(rng.integers(0, 2)))))
        d, n = o, m
        if rng.random() < 0.8:
            layers.append(nets.relu())
        if rng.random() < 0.6:
            pk, ps = [(2, 2), (3, 2), (2, 1), (3, 3)][rng.integers(0, 4)]
            if n >= pk:
                layers.append(nets.maxpool(pk, ps))
                n = (n - pk) // ps + 1
        if rng.random() < 0.4:
            layers.append(nets.lrn(int(rng.choice([3, 5])), 1e-2, 0.75))
    for _ in range(int(rng.integers(0, 3))):
        layers.append(nets.fc(int(rng.integers(2, 70)), decay_mult=(1.0, 1.0)))
        if rng.random() < 0.8:
            layers.append(nets.relu())
        if rng.random() < 0.4:
            layers.append(nets.dropout(0.5))
    classes = int(rng.integers(2, 12))
    layers += [nets.fc(classes), nets.softmax_loss()]
    return B, D, S, classes, layers


@pytest.mark.parametrize("seed", [41, 42])
def test_random_layer_chains_train_like_the_oracle(oracle, seed):
    """Two training iterations of random layer chains, the convolution layers on a random path level
    (default, all direct, direct data gradient, staged passes): every layer's output, the loss, every
    gradient and every updated parameter against the oracle chain."""
    from caffecontroll_amd import nets
    from oracle.oracle_net import OracleNet
    import test_gpu_nets as T
    driver()
    rng = np.random.default_rng(seed)
    solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005)
    done = 0
    while done < 25:
        B, D, S, classes, layers = _random_chain(rng)
        if not any(L.type == nets.CONV for L in layers):
            continue
        net = nets.Net(B, D, S, layers, nets.solver_param(**solver))
        net.set_conv_path(int(rng.choice([-1, 3, 3, 2, 0])))
        ref = OracleNet(oracle, layers, B, D, S, solver)
        T._init_and_sync_params(net, ref, rng)
        net.freeze_dropout_masks(True)
        for li, L in enumerate(layers):
            if L.type == nets.DROPOUT:
                ptr, n = net.tensor(li, nets.AUX)
                mask = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
                T._up(ptr, mask)
                ref.masks[li] = mask
        for _ in range(2):
            x = rng.standard_normal((B, D, S, S)).astype(np.float32)
            labels = rng.integers(0, classes, B).astype(np.float32)
            T._up(net.input_ptr(), x)
            T._up(net.labels_ptr(), labels)
            net.forward()
            ref.forward(x, labels)
            T._check_forward_and_align_switches(net, ref, layers, TOL)
            assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
            net.backward()
            ref.backward()
            T._compare_params(net, ref, TOL)
        net.close()
        done += 1


@pytest.mark.parametrize("seed", [51, 52])
def test_random_tower_graphs_train_like_the_oracle(oracle, seed):
    """Random graphs of the two-tower kind (a stem whose output two or three towers read -- the
    reference's Split --, grouped and plain convolutions of kernel size 1, 3 and 5 in the towers,
    CONCAT, classifier): one training iteration on a random convolution path level against the
    oracle graph.  Weights are scaled by their fan-in so that the loss gradient is well conditioned."""
    from caffecontroll_amd import nets
    from oracle.oracle_net import OracleGraph
    import test_gpu_nets as T
    driver()
    rng = np.random.default_rng(seed)
    solver = dict(base_lr=0.05, momentum=0.9, weight_decay=0.001)

    def same_conv(o, group=1):
        k = int(rng.choice([1, 3, 5]))
        return nets.conv(o, k, pad=(k - 1) // 2, group=group)

    for case in range(20):
        B, D, S = int(rng.integers(1, 7)), int(rng.choice([1, 2, 3, 4])), int(rng.integers(8, 20))
        layers = [same_conv(int(rng.integers(1, 8)) * 2)]
        if rng.random() < 0.7:
            layers.append(nets.relu())
        if rng.random() < 0.5:
            layers.append(nets.maxpool(2, 2))
        if rng.random() < 0.4:
            layers.append(nets.lrn(3, 1e-2, 0.75))
        shared, ends, pool_towers = len(layers) - 1, [], rng.random() < 0.5
        for _ in range(int(rng.integers(2, 4))):
            g = int(rng.choice([1, 2]))
            layers.append(same_conv(int(rng.integers(2, 8)) * g + (g == 1), g).read_from(shared))
            if rng.random() < 0.7:
                layers.append(nets.relu())
            if rng.random() < 0.4:
                layers.append(same_conv(int(rng.integers(3, 10))))
                if rng.random() < 0.5:
                    layers.append(nets.relu())
            if pool_towers:
                layers.append(nets.maxpool(2, 2))
            ends.append(len(layers) - 1)
        layers.append(nets.concat(*ends))
        if rng.random() < 0.5:
            layers += [nets.fc(int(rng.integers(2, 40))), nets.relu()]
        classes = int(rng.integers(2, 8))
        layers += [nets.fc(classes), nets.softmax_loss()]
        net = nets.Net(B, D, S, layers, nets.solver_param(**solver))
        net.set_conv_path(int(rng.choice([-1, 3, 0])))
        ref = OracleGraph(oracle, layers, B, D, S, solver)
        T._init_and_sync_params(net, ref, rng)
        x = rng.standard_normal((B, D, S, S)).astype(np.float32)
        labels = rng.integers(0, classes, B).astype(np.float32)
        T._up(net.input_ptr(), x)
        T._up(net.labels_ptr(), labels)
        net.forward()
        ref.forward(x, labels)
        for li, L in enumerate(layers):
            if L.type == nets.RELU:
                continue
            ptr, n = net.tensor(li, nets.OUTPUT)
            want = ref.val[ref.blob[li]] if li != len(layers) - 1 else ref.out[li]
            assert rel_err(T._down(ptr, n), want.reshape(-1)) <= TOL, (case, li)
            if L.type == nets.MAXPOOL:   # route the gradients through the oracle's arg-max positions
                ptr, n = net.tensor(li, nets.AUX)
                T._up(ptr, ref.saved[(li, "idx")].reshape(-1).astype(np.int32))
        assert abs(net.loss() - ref.loss) <= TOL * max(1.0, abs(ref.loss))
        net.backward()
        ref.backward()
        for (li, gi), p in sorted(ref.params.items()):
            for which, k, key, hist in ((nets.MODEL_GRAD, 0, "w", "hw"), (nets.BIAS_GRAD, 1, "b", "hb")):
                ptr, n = net.tensor(li, which, gi)
                lam = np.float32(solver["weight_decay"] * layers[li].decay_mult[k])
                want = ref.grads[(li, gi)][k].reshape(-1) + lam * (p[key].reshape(-1) + p[hist])
                assert rel_err(T._down(ptr, n), want) <= TOL, (case, li, gi, k)
        net.close()
