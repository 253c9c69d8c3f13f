"""Network descriptions for the benchmark configurations, and their construction as Saga graphs.

A network is a neutral list of node records (type, named inputs, attributes, output name) plus
a dict of explicitly seeded parameter arrays - never the front end's clock-seeded random
initialisation - so that the hip engine and a checker can be handed identical weights.
Node order inside the residual blocks is that of Graph::addResNet / addResNetBottleNeck
(reference: src/graph.cpp:273-425), the ResNet-50 stack that of test/test_classifier.cpp:427-474.
"""
import numpy as np

from . import api as S


class Net:
    def __init__(self, name, batch, in_shape, classes, dtype):
        self.name, self.batch, self.in_shape, self.classes, self.dtype = name, batch, in_shape, classes, dtype
        self.nodes = []      # dicts: type, name, in {slot: tensor name}, out, attrs
        self.params = {}     # tensor name -> float32 numpy array (logical dims)
        self.trainable = []  # parameter names updated by the optimizer, in creation order
        self._n = 0
        self.input = "input"
        self.rows = batch    # samples in the input tensor (the conv harness runs 2 rows at program batch size 1)
        self.loss = None     # output of an L2 loss node, when the network ends in one instead of a classifier
        self.output = None   # logits
        self.flops_fwd = 0   # multiply-add counted as 2

    def _t(self):
        self._n += 1
        return f"t{self._n}"

    def add(self, type_, inputs, attrs=None, name=None):
        out = self._t()
        self.nodes.append({"type": type_, "name": name, "in": dict(inputs), "out": out, "attrs": dict(attrs or {})})
        return out


class Builder:
    def __init__(self, net, seed):
        self.net = net
        self.rng = np.random.default_rng(seed)
        self.shape = {net.input: tuple(net.in_shape)}  # tensor name -> (C, H, W) or (F,)

    def he(self, shape, fan_in):
        return (self.rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)

    def conv(self, x, name, cout, size, stride=1, pad=0, bias=False, transpose=False, outputpad=0):
        net = self.net
        cin, h, w = self.shape[x]
        if transpose:
            wshape = (cin, cout, size, size)  # reference: src/node.cpp:99-110
            fan_in = cout * size * size
            ho = stride * (h - 1) + outputpad + size - 2 * pad
            wo = stride * (w - 1) + outputpad + size - 2 * pad
        else:
            wshape = (cout, cin, size, size)
            fan_in = cin * size * size
            ho = 1 + (h + 2 * pad - size) // stride
            wo = 1 + (w + 2 * pad - size) // stride
        net.params[name + "-w"] = self.he(wshape, fan_in)
        net.trainable.append(name + "-w")
        ins = {"x": x, "w": name + "-w"}
        attrs = {"size": size, "activations": cout, "stride": stride, "pad": pad}
        if bias:
            bname = name + ("-b" if transpose else "-bt")
            net.params[bname] = np.zeros((1, cout), np.float32)
            net.trainable.append(bname)
            ins["b"] = bname
            attrs["bias"] = True
        if transpose:
            attrs["transpose"] = True
            if outputpad:
                attrs["outputpad"] = outputpad
        y = net.add("conv", ins, attrs, name)
        self.shape[y] = (cout, ho, wo)
        macs = (ho * wo * cout * cin * size * size) if not transpose else (h * w * cin * cout * size * size)
        net.flops_fwd += 2 * macs
        return y

    def bn(self, x, name, random_stats=False):
        net = self.net
        c = self.shape[x][0]
        net.params[name + "-s"] = np.ones((1, c), np.float32)
        net.params[name + "-b"] = np.zeros((1, c), np.float32)
        if random_stats:  # running mean N(0, 0.1), running var U[0.5, 1.5]
            net.params[name + "-m"] = (self.rng.standard_normal((1, c)) * 0.1).astype(np.float32)
            net.params[name + "-v"] = self.rng.uniform(0.5, 1.5, (1, c)).astype(np.float32)
        else:
            net.params[name + "-m"] = np.zeros((1, c), np.float32)
            net.params[name + "-v"] = np.ones((1, c), np.float32)
        net.trainable += [name + "-s", name + "-b"]
        y = net.add("batchnorm", {"x": x, "s": name + "-s", "b": name + "-b", "m": name + "-m", "v": name + "-v"}, {},
                    name)
        self.shape[y] = self.shape[x]
        return y

    def unary(self, type_, x, attrs=None):
        y = self.net.add(type_, {"x": x}, attrs)
        self.shape[y] = self.shape[x]
        return y

    def relu(self, x):
        return self.unary("relu", x)

    def pool(self, type_, x, size=1, stride=1, pad=0, global_=False):
        c, h, w = self.shape[x]
        attrs = {"global": True} if global_ else {"size": size, "stride": stride, "pad": pad}
        k = h if global_ else size
        y = self.net.add(type_, {"x": x}, attrs)
        self.shape[y] = (c, 1 + (h + 2 * pad - k) // stride, 1 + (w + 2 * pad - k) // stride)
        return y

    def sum(self, a, b):
        y = self.net.add("sum", {"x0": a, "x1": b})
        self.shape[y] = self.shape[a]
        return y

    def concat(self, xs):
        y = self.net.add("concat", {f"x{i}": x for i, x in enumerate(xs)}, {"axis": 1})
        c = sum(self.shape[x][0] for x in xs)
        self.shape[y] = (c,) + tuple(self.shape[xs[0]][1:])
        return y

    def fc(self, x, name, outputs, bias=True, transW=False):
        net = self.net
        fin = int(np.prod(self.shape[x]))
        # transW = false: [in, out]; true: [out, in] (reference: src/node.cpp:266-275)
        net.params[name + "-w"] = self.he((outputs, fin) if transW else (fin, outputs), fin)
        net.trainable.append(name + "-w")
        ins = {"x": x, "w": name + "-w"}
        attrs = {"outputs": outputs}
        if transW:
            attrs["transW"] = True
        if bias:
            net.params[name + "-b"] = np.zeros((outputs,), np.float32)
            net.trainable.append(name + "-b")
            ins["b"] = name + "-b"
            attrs["bias"] = True
        y = net.add("fc", ins, attrs, name)
        self.shape[y] = (outputs,)
        net.flops_fwd += 2 * fin * outputs
        return y

    def reshape(self, x, shape):
        """shape: the new (C, H, W) of a sample; elements keep their logical order."""
        assert int(np.prod(shape)) == int(np.prod(self.shape[x]))
        y = self.net.add("reshape", {"x": x}, {"shape": S.Dims([self.net.rows, *shape])})
        self.shape[y] = tuple(shape)
        return y

    def loss(self, x, target, strength=1.0):
        """The L2 loss node against a target held like a parameter (not trained); its y copies x, its second
        output (per-sample min / max / mean / mean square of x - target) is named y + "-mmss"."""
        net = self.net
        net.params["target"] = np.asarray(target, np.float32)
        y = net.add("loss", {"x": x, "target": "target"}, {"strength": float(strength)})
        self.shape[y] = self.shape[x]
        net.loss = y
        return y

    # reference: Graph::addResNet, src/graph.cpp:384-425
    def basic_block(self, x, cout, downsample, name, random_stats=False):
        st = 2 if downsample else 1
        a = self.conv(x, name + "-conv-1", cout, 3, st, 1)
        a = self.relu(self.bn(a, name + "-bn-1", random_stats))
        a = self.conv(a, name + "-conv-2", cout, 3, 1, 1)
        a = self.bn(a, name + "-bn-2", random_stats)
        sc = x
        if self.shape[a] != self.shape[x]:
            sc = self.bn(self.conv(x, name + "-conv-p", cout, 1, st, 0), name + "-bn-p", random_stats)
        return self.relu(self.sum(a, sc))

    # reference: Graph::addResNetBottleNeck, src/graph.cpp:273-323 (stride on the 3x3: "v1.5")
    def bottleneck(self, x, squeeze, cout, downsample, name, random_stats=False):
        st = 2 if downsample else 1
        a = self.relu(self.bn(self.conv(x, name + "-conv-1", squeeze, 1, 1, 0), name + "-bn-1", random_stats))
        a = self.relu(self.bn(self.conv(a, name + "-conv-2", squeeze, 3, st, 1), name + "-bn-2", random_stats))
        a = self.bn(self.conv(a, name + "-conv-3", cout, 1, 1, 0), name + "-bn-3", random_stats)
        sc = x
        if self.shape[a] != self.shape[x]:
            sc = self.bn(self.conv(x, name + "-conv-p", cout, 1, st, 0), name + "-bn-p", random_stats)
        return self.relu(self.sum(a, sc))


def lenet(batch=64, seed=1):
    """LeNet-style CNN (config 1): 1x28x28 -> conv5x5x32 p2, relu, maxpool2 -> conv5x5x64 p2, relu,
    maxpool2 -> fc 3136->1024, relu -> fc 1024->10."""
    net = Net("lenet", batch, (1, 28, 28), 10, S.FLOAT)
    b = Builder(net, seed)
    x = b.relu(b.conv(net.input, "c1", 32, 5, 1, 2, bias=True))
    x = b.pool("maxpool", x, 2, 2)
    x = b.relu(b.conv(x, "c2", 64, 5, 1, 2, bias=True))
    x = b.pool("maxpool", x, 2, 2)
    x = b.relu(b.fc(x, "fc1", 1024))
    net.output = b.fc(x, "fc2", 10)
    return net


def resnet20(batch=128, seed=3, dtype=S.HALF):
    """ResNet-20-style CIFAR network (config 3): conv3x3x16, 3 stages x 3 basic blocks (16/32/64),
    global average pool, fc 64->10."""
    net = Net("resnet20", batch, (3, 32, 32), 10, dtype)
    b = Builder(net, seed)
    x = b.relu(b.bn(b.conv(net.input, "s1-conv", 16, 3, 1, 1), "s1-bn"))
    for stage, ch in enumerate((16, 32, 64)):
        for i in range(3):
            x = b.basic_block(x, ch, stage > 0 and i == 0, f"s{stage + 2}_{i}")
    x = b.pool("avgpool", x, global_=True)
    net.output = b.fc(x, "fc", 10)
    return net


def resnet50(batch=256, seed=4, dtype=S.HALF, image=224, classes=1000):
    """ResNet-50 v1.5 (config 4): 7x7/2 stem, maxpool 3/2/1, bottleneck stages [3,4,6,3] of widths
    64/128/256/512 (x4), global average pool, fc 2048->1000 with bias.  Running statistics are random
    (mean N(0,0.1), var U[0.5,1.5]) so that inference is not a no-op normalisation."""
    net = Net("resnet50", batch, (3, image, image), classes, dtype)
    b = Builder(net, seed)
    x = b.relu(b.bn(b.conv(net.input, "s1-conv", 64, 7, 2, 3), "s1-bn", True))
    x = b.pool("maxpool", x, 3, 2, 1)
    for stage, (blocks, width) in enumerate(((3, 64), (4, 128), (6, 256), (3, 512))):
        for i in range(blocks):
            x = b.bottleneck(x, width, width * 4, stage > 0 and i == 0, f"s{stage + 2}_{i + 1}", True)
    x = b.pool("avgpool", x, global_=True)
    net.output = b.fc(x, "fc3", classes)
    return net


def unet(batch=16, seed=5, dtype=S.HALF, image=256, classes=8, widths=(64, 128, 256, 512), bottleneck=1024,
         softmax=False):
    """U-Net-style encoder-decoder (config 5): 4 down stages (2 x conv3x3+bn+relu, maxpool 2), a
    bottleneck, 4 up stages (2x2/2 transposed conv, skip concat, 2 x conv3x3+bn+relu), 1x1 conv to
    `classes` channels.  The skip concats are realised by the engine as strided outputs.
    softmax: the per-pixel softmax over the classes on top (an inference-only node in the reference,
    src/cuda/cuda_dnn.cpp:1928-1964); net.output stays the class scores, net.softmax names the probabilities."""
    net = Net("unet", batch, (3, image, image), classes, dtype)
    b = Builder(net, seed)

    def double(x, ch, name):
        x = b.relu(b.bn(b.conv(x, name + "a", ch, 3, 1, 1), name + "a-bn"))
        return b.relu(b.bn(b.conv(x, name + "b", ch, 3, 1, 1), name + "b-bn"))

    skips = []
    x = net.input
    for i, ch in enumerate(widths):
        x = double(x, ch, f"down{i}")
        skips.append(x)
        x = b.pool("maxpool", x, 2, 2)
    x = double(x, bottleneck, "mid")
    for i, ch in reversed(list(enumerate(widths))):
        up = b.conv(x, f"up{i}-t", ch, 2, 2, 0, bias=True, transpose=True)
        x = double(b.concat([skips[i], up]), ch, f"up{i}")
    net.output = b.conv(x, "head", classes, 1, 1, 0, bias=True)
    net.softmax = b.unary("softmax", net.output) if softmax else None
    return net


def conv_harness(dtype=S.FLOAT, seed=6):
    """The training graph of the reference's `conv` command (test/test_conv.cpp:96-140): two 1x5x5 diagonal
    patterns -> 3x3 stride-2 conv to 5 channels + bias -> relu -> fc to 20 with transposed weights + bias -> relu
    -> reshape to 5x2x2 -> 3x3 stride-2 transposed conv to 1 channel + bias -> L2 loss against the input.
    The program's batch size is 1 although the tensors hold two samples, as in the harness, so the initial
    loss scale is 1.  Returns (net, x)."""
    net = Net("conv-harness", 1, (1, 5, 5), 0, dtype)
    net.rows = 2
    b = Builder(net, seed)
    x = np.stack([np.eye(5, dtype=np.float32), np.eye(5, dtype=np.float32)[:, ::-1]])[:, None]
    h = b.relu(b.conv(net.input, "node1", 5, 3, 2, 0, bias=True))
    h = b.relu(b.fc(h, "fc1", 20, transW=True))
    h = b.reshape(h, (5, 2, 2))
    net.output = b.conv(h, "node2", 1, 3, 2, 0, bias=True, transpose=True)
    b.loss(net.output, x)
    return net, x


def np_dtype(code):
    return np.float16 if code == S.HALF else np.float32


def build_graph(net, x, labels=None, with_classifier=True, param_dtype=None):
    """Builds the Saga graph of `net`.  x: numpy input batch (logical N,C,H,W).  Returns
    (graph, tensors) where tensors maps every name of the description (plus "labels", "pred",
    "loss") to its front-end Tensor."""
    g = S.Graph()
    dt = net.dtype
    t = {}
    t[net.input] = S.Tensor.from_numpy(np.asarray(x).astype(np_dtype(dt)))
    for name, a in net.params.items():
        is_bn = name.endswith(("-s", "-m", "-v")) or (name.endswith("-b") and name[:-2] + "-s" in net.params)
        pd = S.FLOAT if is_bn else (param_dtype if param_dtype is not None else dt)
        t[name] = S.Tensor.from_numpy(a.astype(np_dtype(pd)), name=name)
    for n in net.nodes:
        node = g.add_node(n["type"], {k: t[v] for k, v in n["in"].items()}, n["attrs"], n["name"])
        t[n["out"]] = node.y()
        if n["type"] == "loss":
            t[n["out"] + "-mmss"] = node.output("mmss")
    if with_classifier and net.loss is None:
        node = g.add_node("catclassifier", {"x": t[net.output]})
        t["pred"] = node.y()
        t["loss"] = node.output("loss")
        t["labels"] = t["pred"].grad()
    return g, t
