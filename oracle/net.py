"""Whole-network CPU oracle.  TEST INFRASTRUCTURE ONLY (see oracle/saga_oracle.c).

Executes a network description (saga_amd.networks.Net: a plain list of node records) with the
C oracle's operators: inference, training forward, backward and the Adam update, following the
op sequence the reference builds per node (src/cuda/cuda_dnn.cpp lowerings, cited in
oracle/saga_oracle.c) and its program semantics: gradients that fan in are summed
(src/cuda/cuda_program.cpp:429-453), the classifier scales its gradient by loss_scale/N for
fp16 (src/cuda/cuda_dnn.cpp:1297-1315), and the optimizer runs after backward
(src/cuda/cuda_optimizer.cpp).  For fp16 networks every stored tensor is rounded to fp16 as
the device does; arithmetic inside an operator stays in fp32/fp64.
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module.

Pinning: tests/test_oracle_net.py compares forward, every parameter gradient, the running statistics, the
loss_scale/N factor, five fp32 training steps and an overflowing mixed-precision run (skipped elements, flags,
loss-scale rule) with torch-CPU double autograd and a numpy Adam written from the reference kernel.
"""
import numpy as np

from . import ref

HALF_CODE = 1  # Tensor::DataType::HALF


class OracleNet:
    def __init__(self, net, lr=1e-4, l2=0.0, bn_expavg=0.1, loss_scale=None):
        self.net = net
        self.half = net.dtype == HALF_CODE
        self.lr, self.l2, self.bn_expavg = lr, l2, bn_expavg
        self.p = {}
        for k, v in net.params.items():
            v = np.array(v, np.float32)
            if self.half and not self._is_bn_param(k):
                v = ref.round_half(v)
            self.p[k] = v
        # reference default: initial loss scale = batch size (src/cuda/cuda_common.cpp:339-353)
        self.loss_scale = np.float32(loss_scale if loss_scale else net.batch)
        self.t = 0
        self.m = {k: np.zeros(self.p[k].size, np.float32) for k in net.trainable}
        self.v = {k: np.zeros(self.p[k].size, np.float32) for k in net.trainable}
        self.master = {k: self.p[k].reshape(-1).copy() for k in net.trainable}
        self.acts = {}
        self.saved = {}

    def _is_bn_param(self, k):
        return k.endswith(("-s", "-m", "-v")) or (k.endswith("-b") and k[:-2] + "-s" in self.net.params)

    def _r(self, a):
        return ref.round_half(a) if self.half else np.asarray(a, np.float32)

    # ------------------------------------------------------------------ forward
    def forward(self, x, training=False):
        a = self.acts = {self.net.input: self._r(x)}
        self.saved = {}
        get = lambda n: a[n] if n in a else self.p[n]
        for node in self.net.nodes:
            ty, i, at, out = node["type"], node["in"], node["attrs"], node["out"]
            if ty == "conv":
                x_, w = get(i["x"]), get(i["w"])
                pad, stride = at.get("pad", 0), at.get("stride", 1)
                if at.get("transpose"):
                    k = w.shape[2]
                    ho = ref.tconv_out(x_.shape[2], k, pad, stride, at.get("outputpad", 0))
                    wo = ref.tconv_out(x_.shape[3], k, pad, stride, at.get("outputpad", 0))
                    y = ref.conv2d_bwd_data(x_, w, (x_.shape[0], w.shape[1], ho, wo), pad, stride)
                else:
                    y = ref.conv2d_fwd(x_, w, pad, stride)
                if "b" in i:
                    y = ref.bias_add(self._r(y), get(i["b"]))
            elif ty == "batchnorm":
                x_ = get(i["x"])
                if training:
                    y, sm, sv, rm, rv = ref.bn_train_fwd(x_, get(i["s"]), get(i["b"]), get(i["m"]), get(i["v"]), 1e-5,
                                                         self.bn_expavg)
                    self.saved[out] = (sm, sv)
                    self.p[i["m"]] = rm.reshape(self.p[i["m"]].shape)
                    self.p[i["v"]] = rv.reshape(self.p[i["v"]].shape)
                else:
                    y = ref.bn_infer(x_, get(i["s"]), get(i["b"]), get(i["m"]), get(i["v"]), 1e-5)
            elif ty == "relu":
                y = ref.act_fwd(get(i["x"]), "relu")
            elif ty == "maxpool" or ty == "avgpool":
                x_ = get(i["x"])
                k = x_.shape[2] if at.get("global") else at.get("size", 1)
                fn = ref.maxpool_fwd if ty == "maxpool" else ref.avgpool_fwd
                y = fn(x_, k, at.get("pad", 0), at.get("stride", 1))
            elif ty == "sum":
                y = get(i["x0"]) + get(i["x1"])
            elif ty == "softmax":
                # over the channels at every pixel, inference only (src/cuda/cuda_dnn.cpp:1928-1964)
                if training:
                    raise NotImplementedError("softmax has no backward pass in the reference")
                y = ref.softmax(get(i["x"]))
            elif ty == "concat":
                y = np.concatenate([get(i[f"x{j}"]) for j in range(len(i))], axis=at.get("axis", 1))
            elif ty == "fc":
                x_ = get(i["x"])
                x2 = x_.reshape(x_.shape[0], -1)  # flatten in logical (C,H,W) order
                y = ref.fc_fwd(x2, get(i["w"]), bool(at.get("transW", False)))
                if "b" in i:
                    y = self._r(y) + get(i["b"]).reshape(1, -1)
            elif ty == "reshape":
                # elements keep their logical (N,C,H,W) order (src/cuda/cuda_dnn.cpp:2504-2540 aliases the storage)
                y = get(i["x"]).reshape([int(v) for v in at["shape"]])
            elif ty == "loss":
                # forward copies x (CudaLossFwd, src/cuda/cuda_dnn.cpp:1358-1393)
                y = get(i["x"])
            else:
                raise NotImplementedError(ty)
            a[out] = self._r(y)
        return a[self.net.output]

    def predict(self, x):
        return ref.catclassifier_fwd(self.forward(x, False))

    # ------------------------------------------------------------------ backward
    def backward(self, labels=None):
        """After forward(training=True).  Returns {param name: gradient}, per-sample loss, predictions;
        activation gradients stay in self.dacts.  A network that ends in an L2 loss node takes no labels: its
        backward pass starts at that node, the second return value is the node's mmss rows and the third None."""
        a = self.acts
        grads = {}
        if getattr(self.net, "loss", None) is None:
            logits = a[self.net.output]
            n = logits.shape[0]
            pred = ref.catclassifier_fwd(logits)
            scale = (1.0 / n) * (float(self.loss_scale) if self.half else 1.0)
            dlogits, loss = ref.catclassifier_bwd(logits, pred, labels, np.float32(scale))
            d = self.dacts = {self.net.output: self._r(dlogits)}
        else:
            d, loss, pred = {}, None, None
            self.dacts = d
        get = lambda name: a[name] if name in a else self.p[name]

        def acc(name, g):
            if name in self.p:
                return  # parameters are handled by the caller of acc
            g = self._r(g)
            d[name] = self._r(d[name] + g) if name in d else g

        for node in reversed(self.net.nodes):
            ty, i, at, out = node["type"], node["in"], node["attrs"], node["out"]
            if ty == "loss":
                # dx = (x - target) * strength / N * the program's loss scale, in EVERY precision
                # (CudaLossBwd, src/cuda/cuda_dnn.cpp:1395-1443; an fp32 program never divides it out again)
                x_ = get(i["x"])
                scale = np.float32(np.float32(at.get("strength", 1.0)) / np.float32(x_.shape[0])) * self.loss_scale
                dx, loss = ref.loss_bwd(x_, get(i["target"]), scale)
                acc(i["x"], dx)
                continue
            if out not in d:
                continue
            dy = d[out]
            if ty == "conv":
                x_, w = get(i["x"]), get(i["w"])
                pad, stride = at.get("pad", 0), at.get("stride", 1)
                if "b" in i:
                    grads[i["b"]] = self._r(ref.bias_bwd(dy)).reshape(self.p[i["b"]].shape)
                if at.get("transpose"):
                    grads[i["w"]] = self._r(ref.conv2d_bwd_filter(dy, x_, w.shape, pad, stride))
                    if i["x"] != self.net.input:
                        acc(i["x"], ref.conv2d_fwd(dy, w, pad, stride))
                else:
                    grads[i["w"]] = self._r(ref.conv2d_bwd_filter(x_, dy, w.shape, pad, stride))
                    if i["x"] != self.net.input:
                        acc(i["x"], ref.conv2d_bwd_data(dy, w, x_.shape, pad, stride))
            elif ty == "batchnorm":
                sm, sv = self.saved[out]
                dx, ds, db = ref.bn_bwd(get(i["x"]), dy, get(i["s"]), sm, sv)
                grads[i["s"]] = ds.reshape(self.p[i["s"]].shape)
                grads[i["b"]] = db.reshape(self.p[i["b"]].shape)
                acc(i["x"], dx)
            elif ty == "relu":
                acc(i["x"], ref.act_bwd(get(i["x"]), a[out], dy, "relu"))
            elif ty == "maxpool":
                x_ = get(i["x"])
                k = x_.shape[2] if at.get("global") else at.get("size", 1)
                acc(i["x"], ref.maxpool_bwd(x_, dy, k, at.get("pad", 0), at.get("stride", 1)))
            elif ty == "avgpool":
                x_ = get(i["x"])
                k = x_.shape[2] if at.get("global") else at.get("size", 1)
                acc(i["x"], ref.avgpool_bwd(dy, x_.shape, k, at.get("pad", 0), at.get("stride", 1)))
            elif ty == "sum":
                acc(i["x0"], dy)
                acc(i["x1"], dy)
            elif ty == "concat":
                off = 0
                for j in range(len(i)):
                    c = get(i[f"x{j}"]).shape[1]
                    acc(i[f"x{j}"], dy[:, off:off + c])
                    off += c
            elif ty == "fc":
                x_ = get(i["x"])
                x2 = x_.reshape(x_.shape[0], -1)
                tw = bool(at.get("transW", False))
                grads[i["w"]] = self._r(ref.fc_bwd_w(x2, dy, tw))
                if "b" in i:
                    grads[i["b"]] = self._r(dy.sum(0))
                if i["x"] != self.net.input:
                    acc(i["x"], ref.fc_bwd_x(dy, get(i["w"]), tw).reshape(x_.shape))
            elif ty == "reshape":
                acc(i["x"], dy.reshape(get(i["x"]).shape))
            else:
                raise NotImplementedError(ty)
        return grads, loss, pred

    # ------------------------------------------------------------------ optimizer
    def adam(self, grads):
        """One optimizer step (fp32 Adam for fp32 tensors, mixed Adam for fp16 ones) followed by the
        loss-scale rule.  Returns the flags [range, inf, nan]."""
        self.t += 1
        flags = np.zeros(3, np.uint32)
        for k in self.net.trainable:
            g = np.ascontiguousarray(grads[k], np.float32).reshape(-1)
            if self.half and not self._is_bn_param(k):
                w16 = self.p[k].astype(np.float16).reshape(-1).view(np.uint16).copy()
                with np.errstate(over="ignore"):
                    g16 = g.astype(np.float16).view(np.uint16)
                f = ref.adam_mixed(w16, g16, self.m[k], self.v[k], self.master[k], self.t, self.lr, self.loss_scale,
                                   self.l2)
                self.p[k] = w16.view(np.float16).astype(np.float32).reshape(self.p[k].shape)
            else:
                w = self.master[k]
                f = ref.adam_f32(w, g, self.m[k], self.v[k], self.t, self.lr, self.l2)
                self.p[k] = w.reshape(self.p[k].shape).copy()
            flags |= f
        if self.half:
            self.loss_scale = ref.loss_scale_update(self.loss_scale, flags)
        return flags

    def train_step(self, x, labels=None):
        self.forward(x, training=True)
        grads, loss, pred = self.backward(labels)
        flags = self.adam(grads)
        return loss, pred, grads, flags
