"""CPU reference of a layer chain, composed from the oracle's per-layer functions in the order
DeepNet::run_forward_pass / run_backward_pass visit the bridges (src/DeepNet.h:171-266): ReLU and
dropout in place, the first weight layer without a data gradient, grouped convolutions as
independent convolutions on channel slices, one SGD update per weight layer per iteration.

TEST INFRASTRUCTURE ONLY, like the rest of this folder: the parity tests compare the device against
it, and the `cpu_baseline` leg of bench.py times it."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

CONV, FC, RELU, MAXPOOL, LRN, DROPOUT, SOFTMAXLOSS, CONCAT = 1, 2, 3, 4, 5, 6, 7, 8


class OracleNet:
    def __init__(self, O, layers, batch, depth, size, solver, partitions=1, fc_blas_threads=0):
        """solver: dict(base_lr, momentum, weight_decay); fixed learning-rate policy.
        partitions > 1: convolutions run the way the reference's ParallelizedBridge runs them on a
        CPU, the batch cut into that many contiguous partitions, one thread each, the partitions'
        weight and bias gradients added up in partition order
        (src/bridges/ParallelizedBridge_impl.hxx:888-955); pooling, LRN, ReLU and dropout are cut the
        same way (src/DeepNet.h:1397, 1455, 1516, 1842: per-image work, so the values do not depend on
        the cut).
        fc_blas_threads > 0 (needs OpenBLAS bound): the reference's policy for inner-product layers,
        ONE partition whose GEMMs use that many BLAS threads (src/DeepNet.h:1165-1167, half the
        hardware threads), while every partitioned layer runs one BLAS thread per partition."""
        self.O, self.layers, self.solver = O, layers, solver
        self.fc_blas_threads = fc_blas_threads
        self.partitions = max(1, min(partitions, batch))
        self.bounds = [(i * batch // self.partitions, (i + 1) * batch // self.partitions)
                       for i in range(self.partitions)]
        self.params = {}   # (layer, group) -> dict(w, b, hw, hb)
        self.shapes = []
        d, n = depth, size
        first = True
        self.first_weight = None
        for i, L in enumerate(layers):
            if L.type == CONV:
                g = max(L.group, 1)
                for gi in range(g):
                    self.params[(i, gi)] = dict(
                        w=np.zeros((L.num_output // g, d // g, L.kernel_size, L.kernel_size), np.float32),
                        b=np.zeros(L.num_output // g, np.float32))
                n = (n + 2 * L.pad - L.kernel_size) // L.stride + 1
                d = L.num_output
                if first:
                    self.first_weight, first = i, False
            elif L.type == FC:
                self.params[(i, 0)] = dict(w=np.zeros((L.num_output, d * n * n), np.float32),
                                           b=np.zeros(L.num_output, np.float32))
                d, n = L.num_output, 1
                if first:
                    self.first_weight, first = i, False
            elif L.type == MAXPOOL:
                n = (n - L.kernel_size) // L.stride + 1
            self.shapes.append((d, n))
        for p in self.params.values():
            p["hw"] = np.zeros(p["w"].size, np.float32)
            p["hb"] = np.zeros(p["b"].size, np.float32)
        self.masks = {}
        self.train = True   # False: dropout layers pass their input through (TEST phase)

    def _blas(self, for_fc):
        if self.fc_blas_threads > 0:
            self.O.bind_openblas(self.fc_blas_threads if for_fc else 1)

    def _cut(self, fn, *arrays):
        """fn(*slices) per batch partition, one thread each; returns the list of results (one entry when
        the net is not partitioned).  Every array has the batch as its first axis."""
        if self.partitions == 1:
            return [fn(*arrays)]
        with ThreadPoolExecutor(self.partitions) as ex:
            return list(ex.map(lambda lh: fn(*[a[lh[0]:lh[1]] for a in arrays]), self.bounds))

    @staticmethod
    def _join(parts, k=None):
        parts = [q if k is None else q[k] for q in parts]
        return parts[0] if len(parts) == 1 else np.concatenate(parts, axis=0)

    def forward(self, x, labels):
        O = self.O
        self.acts = [x]
        self.saved = {}
        cur = x
        for i, L in enumerate(self.layers):
            if L.type == CONV:
                self._blas(False)
                g = max(L.group, 1)
                dg = cur.shape[1] // g
                outs = []
                for gi in range(g):
                    p = self.params[(i, gi)]
                    xin = np.ascontiguousarray(cur[:, gi * dg:(gi + 1) * dg])
                    if self.partitions == 1:
                        out, low = O.conv_forward(xin, p["w"], p["b"], L.kernel_size, L.stride, L.pad)
                    else:
                        with ThreadPoolExecutor(self.partitions) as ex:
                            parts = list(ex.map(lambda lh: O.conv_forward(xin[lh[0]:lh[1]], p["w"], p["b"], L.kernel_size,
                                                                          L.stride, L.pad), self.bounds))
                        out = np.concatenate([q[0] for q in parts], axis=0)
                        low = [q[1] for q in parts]
                    self.saved[(i, gi)] = (xin.shape, low)
                    outs.append(out)
                cur = np.concatenate(outs, axis=1) if g > 1 else outs[0]
            elif L.type == FC:
                self._blas(True)
                p = self.params[(i, 0)]
                self.saved[(i, 0)] = cur.reshape(cur.shape[0], -1).copy()
                cur = O.fc_forward(self.saved[(i, 0)], p["w"], p["b"]).reshape(cur.shape[0], L.num_output, 1, 1)
            elif L.type == RELU:
                cur = self._join(self._cut(O.relu_forward, cur))
                self.acts[-1] = cur  # in place: the layer below now holds the rectified values
            elif L.type == MAXPOOL:
                self.saved[i] = cur.shape
                parts = self._cut(lambda a: O.maxpool_forward(np.ascontiguousarray(a), L.kernel_size, L.stride), cur)
                cur, idx = self._join(parts, 0), self._join(parts, 1)
                self.saved[(i, "idx")] = idx
            elif L.type == LRN:
                self.saved[i] = cur
                parts = self._cut(lambda a: O.lrn_forward(np.ascontiguousarray(a), L.lrn_local_size, L.lrn_alpha,
                                                          L.lrn_beta), cur)
                cur, den = self._join(parts, 0), self._join(parts, 1)
                self.saved[(i, "den")] = den
            elif L.type == DROPOUT:
                if self.train:
                    mask = np.asarray(self.masks[i]).reshape(cur.shape)
                    cur = self._join(self._cut(
                        lambda a, mk: O.dropout_forward(np.ascontiguousarray(a), np.ascontiguousarray(mk).reshape(-1),
                                                        L.dropout_ratio, threshold=True).reshape(a.shape), cur, mask))
                self.acts[-1] = cur
            elif L.type == SOFTMAXLOSS:
                cur, self.loss = O.softmax_loss_forward(cur, labels)
                self.labels = labels
            if L.type not in (RELU, DROPOUT):
                self.acts.append(cur)
        return cur

    def backward(self):
        O, s = self.O, self.solver
        grad = None
        self.grads = {}
        self.in_grads = {}  # layer -> gradient with respect to the layer's input, as it leaves the layer
        ai = len(self.acts) - 1  # index of the activation produced by the layer being visited
        for i in range(len(self.layers) - 1, -1, -1):
            L = self.layers[i]
            if i + 1 < len(self.layers) and grad is not None:
                self.in_grads[i + 1] = grad
            if L.type == SOFTMAXLOSS:
                grad = O.softmax_loss_backward(self.acts[ai], self.labels)
                ai -= 1
            elif L.type == RELU:
                grad = self._join(self._cut(lambda gq, a: O.relu_backward(np.ascontiguousarray(gq), np.ascontiguousarray(a)),
                                            grad, self.acts[ai].reshape(grad.shape)))
            elif L.type == DROPOUT:
                mask = np.asarray(self.masks[i]).reshape(grad.shape)
                grad = self._join(self._cut(
                    lambda a, mk: O.dropout_forward(np.ascontiguousarray(a), np.ascontiguousarray(mk).reshape(-1),
                                                    L.dropout_ratio, threshold=True).reshape(a.shape), grad, mask))
            elif L.type == MAXPOOL:
                shp = self.saved[i]
                grad = self._join(self._cut(
                    lambda gq, ix: O.maxpool_backward(np.ascontiguousarray(gq), np.ascontiguousarray(ix), shp[2], shp[3]),
                    grad, self.saved[(i, "idx")]))
                ai -= 1
            elif L.type == LRN:
                grad = self._join(self._cut(
                    lambda gq, a, dn: O.lrn_backward(np.ascontiguousarray(gq), np.ascontiguousarray(a),
                                                     np.ascontiguousarray(dn), L.lrn_local_size, L.lrn_alpha, L.lrn_beta),
                    grad, self.saved[i], self.saved[(i, "den")]))
                ai -= 1
            elif L.type == FC:
                self._blas(True)
                p = self.params[(i, 0)]
                need = i != self.first_weight
                xin = self.saved[(i, 0)]
                dx, dw, db = O.fc_backward(xin, p["w"], grad.reshape(grad.shape[0], -1), need_in_grad=need)
                self.grads[(i, 0)] = (dw.copy(), db.copy())
                self._update(p, L, dw, db)
                grad = dx.reshape(self.acts[ai - 1].shape) if need else None
                ai -= 1
            elif L.type == CONV:
                self._blas(False)
                g = max(L.group, 1)
                need = i != self.first_weight
                og_d = grad.shape[1] // g
                dxs = []
                for gi in range(g):
                    p = self.params[(i, gi)]
                    shp, low = self.saved[(i, gi)]
                    og = np.ascontiguousarray(grad[:, gi * og_d:(gi + 1) * og_d])
                    if self.partitions == 1:
                        dx, dw, db = O.conv_backward(shp, p["w"], og, low, L.kernel_size, L.stride, L.pad,
                                                     need_in_grad=need)
                    else:
                        def part(j):
                            lo, hi = self.bounds[j]
                            return O.conv_backward((hi - lo,) + tuple(shp[1:]), p["w"], og[lo:hi], low[j], L.kernel_size,
                                                   L.stride, L.pad, need_in_grad=need)
                        with ThreadPoolExecutor(self.partitions) as ex:
                            parts = list(ex.map(part, range(self.partitions)))
                        dx = np.concatenate([q[0] for q in parts], axis=0) if need else None
                        dw, db = parts[0][1].copy(), parts[0][2].copy()
                        for q in parts[1:]:
                            dw += q[1]
                            db += q[2]
                    self.grads[(i, gi)] = (dw.copy(), db.copy())
                    self._update(p, L, dw, db)
                    dxs.append(dx)
                grad = (np.concatenate(dxs, axis=1) if g > 1 else dxs[0]) if need else None
                ai -= 1
        return grad

    def _update(self, p, L, dw, db):
        s = self.solver
        w = p["w"].reshape(-1)
        self.O.sgd_update(w, dw.reshape(-1), p["hw"], s["base_lr"] * L.lr_mult[0], s["momentum"],
                          s["weight_decay"] * L.decay_mult[0])
        p["w"] = w.reshape(p["w"].shape)
        self.O.sgd_update(p["b"], db, p["hb"], s["base_lr"] * L.lr_mult[1], s["momentum"],
                          s["weight_decay"] * L.decay_mult[1])


class OracleGraph:
    """The same for layers that name their bottoms (`LayerSpec.read_from`): a tensor read by several
    layers is shared, each reader's gradient is kept apart and the gradients are added in reader
    order before the tensor's last writer runs its backward step (the reference's Split bridge,
    src/DeepNet.h:1924-2028); CONCAT stacks its bottoms along the depth (src/DeepNet.h:1700-1757).
    A layer computes an input gradient only if a layer with weights lies upstream of it."""

    def __init__(self, O, layers, batch, depth, size, solver):
        self.O, self.layers, self.solver = O, layers, solver
        n = len(layers)
        self.bottoms = [[L.bottoms[j] for j in range(L.n_bottoms)] if L.n_bottoms else [i - 1] for i, L in enumerate(layers)]
        self.in_place = [L.type in (RELU, DROPOUT) for L in layers]
        # the tensor a layer writes: its own, or its bottom's for an in-place layer (-1 = the input)
        self.blob = []
        for i in range(n):
            self.blob.append(self._blob_of(self.bottoms[i][0]) if self.in_place[i] else i)
        shape = {-1: (depth, size)}
        self.params, self.upstream = {}, {-1: False}
        for i, L in enumerate(layers):
            d, s = shape[self._blob_of(self.bottoms[i][0])]
            up = any(self.upstream[self._blob_of(b)] for b in self.bottoms[i])
            if L.type == CONV:
                g = max(L.group, 1)
                for gi in range(g):
                    self.params[(i, gi)] = dict(w=np.zeros((L.num_output // g, d // g, L.kernel_size, L.kernel_size), np.float32),
                                                b=np.zeros(L.num_output // g, np.float32))
                s = (s + 2 * L.pad - L.kernel_size) // L.stride + 1
                d = L.num_output
            elif L.type == FC:
                self.params[(i, 0)] = dict(w=np.zeros((L.num_output, d * s * s), np.float32), b=np.zeros(L.num_output, np.float32))
                d, s = L.num_output, 1
            elif L.type == MAXPOOL:
                s = (s - L.kernel_size) // L.stride + 1
            elif L.type == CONCAT:
                d = sum(shape[self._blob_of(b)][0] for b in self.bottoms[i])
            shape[self.blob[i]] = (d, s)
            self.upstream[self.blob[i]] = self.upstream.get(self.blob[i], False) or up or L.type in (CONV, FC)
        self.needs_in_grad = [any(self._up_before(i, b) for b in self.bottoms[i]) for i in range(n)]
        for p in self.params.values():
            p["hw"] = np.zeros(p["w"].size, np.float32)
            p["hb"] = np.zeros(p["b"].size, np.float32)
        self.masks = {}

    def _blob_of(self, layer_index):
        return -1 if layer_index < 0 else self.blob[layer_index]

    def _up_before(self, i, b):
        """True if a layer with weights lies at or above the producer of bottom `b` of layer `i`."""
        seen, todo = set(), [b]
        while todo:
            j = todo.pop()
            if j < 0 or j in seen:
                continue
            seen.add(j)
            if self.layers[j].type in (CONV, FC):
                return True
            todo.extend(self.bottoms[j])
        return False

    def forward(self, x, labels):
        O = self.O
        self.val = {-1: x}      # tensor -> current values (in-place layers replace them)
        self.out = {}           # layer -> what it wrote (for comparisons)
        self.saved = {}
        for i, L in enumerate(self.layers):
            ins = [self.val[self._blob_of(b)] for b in self.bottoms[i]]
            cur = ins[0]
            if L.type == CONV:
                g = max(L.group, 1)
                dg = cur.shape[1] // g
                outs = []
                for gi in range(g):
                    p = self.params[(i, gi)]
                    xin = np.ascontiguousarray(cur[:, gi * dg:(gi + 1) * dg])
                    out, low = O.conv_forward(xin, p["w"], p["b"], L.kernel_size, L.stride, L.pad)
                    self.saved[(i, gi)] = (xin.shape, low)
                    outs.append(out)
                res = np.concatenate(outs, axis=1) if g > 1 else outs[0]
            elif L.type == FC:
                p = self.params[(i, 0)]
                self.saved[(i, 0)] = cur.reshape(cur.shape[0], -1).copy()
                self.saved[(i, "shape")] = cur.shape
                res = O.fc_forward(self.saved[(i, 0)], p["w"], p["b"]).reshape(cur.shape[0], L.num_output, 1, 1)
            elif L.type == RELU:
                res = O.relu_forward(cur)
            elif L.type == MAXPOOL:
                self.saved[i] = cur.shape
                res, idx = O.maxpool_forward(cur, L.kernel_size, L.stride)
                self.saved[(i, "idx")] = idx
            elif L.type == LRN:
                self.saved[i] = cur
                res, den = O.lrn_forward(cur, L.lrn_local_size, L.lrn_alpha, L.lrn_beta)
                self.saved[(i, "den")] = den
            elif L.type == DROPOUT:
                res = O.dropout_forward(cur, self.masks[i], L.dropout_ratio, threshold=True)
            elif L.type == CONCAT:
                self.saved[i] = [a.shape[1] for a in ins]
                res = np.concatenate(ins, axis=1)
            elif L.type == SOFTMAXLOSS:
                res, self.loss = O.softmax_loss_forward(cur, labels)
                self.labels = labels
            self.val[self.blob[i]] = res
            self.out[i] = res
        return res

    def backward(self):
        O = self.O
        n = len(self.layers)
        contrib = {}            # tensor -> {reader layer: gradient}
        total = {}              # tensor -> gradient after the readers were added up
        self.grads, self.tensor_grads = {}, {}

        def grad_of(blob):
            if blob not in total:
                parts = contrib.get(blob, {})
                g = None
                for reader in sorted(parts):      # reader order, fp32 adds
                    g = parts[reader].copy() if g is None else g + parts[reader]
                total[blob] = g
            return total[blob]

        for i in range(n - 1, -1, -1):
            L = self.layers[i]
            blob = self.blob[i]
            bots = [self._blob_of(b) for b in self.bottoms[i]]
            need = self.needs_in_grad[i]
            if L.type == SOFTMAXLOSS:
                contrib.setdefault(bots[0], {})[i] = O.softmax_loss_backward(self.out[i], self.labels)
                continue
            g = grad_of(blob)
            if g is None:
                continue        # nothing with weights upstream and none here
            if L.type == RELU:
                total[blob] = O.relu_backward(g, self.val[blob])
            elif L.type == DROPOUT:
                total[blob] = O.dropout_forward(g, self.masks[i], L.dropout_ratio, threshold=True)
            elif L.type == MAXPOOL:
                shp = self.saved[i]
                if need:
                    contrib.setdefault(bots[0], {})[i] = O.maxpool_backward(g, self.saved[(i, "idx")], shp[2], shp[3])
            elif L.type == LRN:
                if need:
                    contrib.setdefault(bots[0], {})[i] = O.lrn_backward(g, self.saved[i], self.saved[(i, "den")],
                                                                          L.lrn_local_size, L.lrn_alpha, L.lrn_beta)
            elif L.type == CONCAT:
                off = 0
                for b, d in zip(bots, self.saved[i]):
                    contrib.setdefault(b, {})[i] = np.ascontiguousarray(g[:, off:off + d])
                    off += d
            elif L.type == FC:
                p = self.params[(i, 0)]
                dx, dw, db = O.fc_backward(self.saved[(i, 0)], p["w"], g.reshape(g.shape[0], -1), need_in_grad=need)
                self.grads[(i, 0)] = (dw.copy(), db.copy())
                self._update(p, L, dw, db)
                if need:
                    contrib.setdefault(bots[0], {})[i] = dx.reshape(self.saved[(i, "shape")])
            elif L.type == CONV:
                gn = max(L.group, 1)
                og_d = g.shape[1] // gn
                dxs = []
                for gi in range(gn):
                    p = self.params[(i, gi)]
                    shp, low = self.saved[(i, gi)]
                    og = np.ascontiguousarray(g[:, gi * og_d:(gi + 1) * og_d])
                    dx, dw, db = O.conv_backward(shp, p["w"], og, low, L.kernel_size, L.stride, L.pad, need_in_grad=need)
                    self.grads[(i, gi)] = (dw.copy(), db.copy())
                    self._update(p, L, dw, db)
                    dxs.append(dx)
                if need:
                    contrib.setdefault(bots[0], {})[i] = np.concatenate(dxs, axis=1) if gn > 1 else dxs[0]
        self.tensor_grads = dict(total)

    _update = OracleNet._update
