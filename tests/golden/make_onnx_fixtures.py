#!/usr/bin/env python3
"""Writes the ONNX loader's fixtures under tests/golden/onnx/, in the layout of the model zoo
directories the reference's `saga onnx` test walks (test/test_onnx.cpp:14-94):

    <model>/<model>.onnx  <model>/test_data_set_0/input_0.pb  <model>/test_data_set_0/output_0.pb

The reference's own models (squeezenet1.1, resnet50-v1-12, vgg19) are not in its repository, so
small networks with the same operator mix stand in for them:

  * mini_resnet, mini_squeezenet, mini_vgg are written by PyTorch's ONNX serializer (an independent
    producer of the wire format), and their expected outputs are PyTorch's own CPU fp32 results;
  * handmade is assembled field by field with the small encoder below and uses the encodings
    and operators the serializer never emits: unpacked repeated fields, float_data / int64_data
    instead of raw_data, a symbolic batch dimension, n-ary Sum, Dropout, MatMul + Add, Reshape
    with 0 / -1, LeakyRelu, AveragePool.  Its expected output comes from torch.nn.functional.

Run from the repository root:  python3 tests/golden/make_onnx_fixtures.py
The `onnx` Python package is not needed: the serializer's post-processing step that imports it
(it only matters for models with custom onnxscript functions) is bypassed.
"""
import io
import os
import struct
import warnings

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "onnx")


# ---------------------------------------------------------------- protobuf encoder (wire format)

def varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def key(num, wire):
    return varint((num << 3) | wire)


def f_varint(num, v):
    return key(num, 0) + varint(v)


def f_bytes(num, b):
    if isinstance(b, str):
        b = b.encode()
    return key(num, 2) + varint(len(b)) + b


def f_float(num, v):
    return key(num, 5) + struct.pack("<f", v)


FLOAT, UINT8, INT64, FLOAT16 = 1, 2, 7, 10


def tensor_proto(name, arr, style="raw", packed=True):
    """TensorProto: dims=1, data_type=2, float_data=4, int64_data=7, name=8, raw_data=9."""
    arr = np.asarray(arr)
    dt = {np.dtype(np.float32): FLOAT, np.dtype(np.int64): INT64, np.dtype(np.float16): FLOAT16,
          np.dtype(np.uint8): UINT8}[arr.dtype]
    out = b""
    if packed:
        out += f_bytes(1, b"".join(varint(d) for d in arr.shape))
    else:
        out += b"".join(f_varint(1, d) for d in arr.shape)
    out += f_varint(2, dt)
    if style == "raw":
        out += f_bytes(9, arr.tobytes())
    elif style == "float_data":
        flat = arr.reshape(-1)
        out += f_bytes(4, flat.tobytes()) if packed else b"".join(f_float(4, float(v)) for v in flat)
    elif style == "int64_data":
        flat = arr.reshape(-1)
        out += (f_bytes(7, b"".join(varint(int(v)) for v in flat)) if packed
                else b"".join(f_varint(7, int(v)) for v in flat))
    else:
        raise ValueError(style)
    if name:
        out += f_bytes(8, name)
    return out


def value_info(name, elem_type, dims):
    """ValueInfoProto{name=1, type=2{tensor_type=1{elem_type=1, shape=2{dim=1{dim_value=1|dim_param=2}}}}}."""
    shape = b""
    for d in dims:
        shape += f_bytes(1, f_bytes(2, d) if isinstance(d, str) else f_varint(1, d))
    tt = f_varint(1, elem_type) + f_bytes(2, shape)
    return f_bytes(1, name) + f_bytes(2, f_bytes(1, tt))


def attribute(name, v, packed=True):
    """AttributeProto: name=1, f=2, i=3, s=4, ints=8, type=20 (FLOAT 1, INT 2, STRING 3, INTS 7)."""
    out = f_bytes(1, name)
    if isinstance(v, float):
        return out + f_float(2, v) + f_varint(20, 1)
    if isinstance(v, int):
        return out + f_varint(3, v) + f_varint(20, 2)
    if isinstance(v, str):
        return out + f_bytes(4, v) + f_varint(20, 3)
    ints = (f_bytes(8, b"".join(varint(i) for i in v)) if packed else b"".join(f_varint(8, i) for i in v))
    return out + ints + f_varint(20, 7)


def node(op, inputs, outputs, packed=True, **attrs):
    """NodeProto: input=1, output=2, name=3, op_type=4, attribute=5."""
    out = b"".join(f_bytes(1, i) for i in inputs) + b"".join(f_bytes(2, o) for o in outputs)
    out += f_bytes(3, outputs[0] + "_node") + f_bytes(4, op)
    for k, v in attrs.items():
        out += f_bytes(5, attribute(k, v, packed))
    return out


def model(nodes, initializers, inputs, outputs, name="g"):
    """ModelProto{ir_version=1, producer_name=2, graph=7{node=1, name=2, initializer=5, input=11, output=12},
    opset_import=8{version=2}}."""
    g = b"".join(f_bytes(1, n) for n in nodes) + f_bytes(2, name)
    g += b"".join(f_bytes(5, t) for t in initializers)
    g += b"".join(f_bytes(11, v) for v in inputs) + b"".join(f_bytes(12, v) for v in outputs)
    return f_varint(1, 6) + f_bytes(2, "saga-amd-fixture") + f_bytes(7, g) + f_bytes(8, f_varint(2, 11))


# ---------------------------------------------------------------- writing one fixture directory

def write_case(name, model_bytes, x, y):
    d = os.path.join(OUT, name)
    os.makedirs(os.path.join(d, "test_data_set_0"), exist_ok=True)
    with open(os.path.join(d, name + ".onnx"), "wb") as f:
        f.write(model_bytes)
    with open(os.path.join(d, "test_data_set_0", "input_0.pb"), "wb") as f:
        f.write(tensor_proto("input_0", x.astype(np.float32)))
    with open(os.path.join(d, "test_data_set_0", "output_0.pb"), "wb") as f:
        f.write(tensor_proto("output_0", y.astype(np.float32)))
    print(f"{name}: model {len(model_bytes)} bytes, input {x.shape}, output {y.shape}")


def export(module, x):
    from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto
    buf = io.BytesIO()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.onnx.export(module, (x,), buf, dynamo=False, opset_version=11, input_names=["data"],
                          output_names=["out"], do_constant_folding=True,
                          # PRESERVE on a module in eval mode: inference-form operators, but without the
                          # serializer's conv + batch-norm folding, so BatchNormalization nodes stay
                          training=torch.onnx.TrainingMode.PRESERVE)
    return buf.getvalue()


def randomize_bn(module, gen):
    for m in module.modules():
        if isinstance(m, nn.BatchNorm2d):
            m.weight.data = torch.empty_like(m.weight).uniform_(0.5, 1.5, generator=gen)
            m.bias.data = torch.empty_like(m.bias).uniform_(-0.3, 0.3, generator=gen)
            m.running_mean.data = torch.empty_like(m.running_mean).uniform_(-0.2, 0.2, generator=gen)
            m.running_var.data = torch.empty_like(m.running_var).uniform_(0.5, 2.0, generator=gen)


class Block(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.c1 = nn.Conv2d(cin, cout, 3, stride, 1, bias=False)
        self.b1 = nn.BatchNorm2d(cout)
        self.c2 = nn.Conv2d(cout, cout, 3, 1, 1, bias=False)
        self.b2 = nn.BatchNorm2d(cout)
        self.proj = None
        if stride != 1 or cin != cout:
            self.proj = nn.Sequential(nn.Conv2d(cin, cout, 1, stride, 0, bias=False), nn.BatchNorm2d(cout))

    def forward(self, x):
        y = self.b2(self.c2(F.relu(self.b1(self.c1(x)))))
        return F.relu(y + (x if self.proj is None else self.proj(x)))


class MiniResNet(nn.Module):
    """Conv BatchNormalization Relu MaxPool Add GlobalAveragePool Flatten Gemm (as resnet50-v1-12)."""

    def __init__(self):
        super().__init__()
        self.stem = nn.Sequential(nn.Conv2d(3, 8, 3, 1, 1, bias=False), nn.BatchNorm2d(8), nn.ReLU(),
                                  nn.MaxPool2d(3, 2, 1))
        self.l1 = Block(8, 8, 1)
        self.l2 = Block(8, 16, 2)
        self.pool = nn.AdaptiveAvgPool2d(1)
        self.fc = nn.Linear(16, 10)

    def forward(self, x):
        return self.fc(torch.flatten(self.pool(self.l2(self.l1(self.stem(x)))), 1))


class Fire(nn.Module):
    def __init__(self, cin, s, e):
        super().__init__()
        self.s = nn.Conv2d(cin, s, 1)
        self.e1 = nn.Conv2d(s, e, 1)
        self.e3 = nn.Conv2d(s, e, 3, padding=1)

    def forward(self, x):
        x = F.relu(self.s(x))
        return torch.cat([F.relu(self.e1(x)), F.relu(self.e3(x))], 1)


class MiniSqueezeNet(nn.Module):
    """Conv(+bias) Relu MaxPool Concat GlobalAveragePool Reshape/Flatten Softmax (as squeezenet1.1)."""

    def __init__(self):
        super().__init__()
        self.features = nn.Sequential(nn.Conv2d(3, 8, 3, 2), nn.ReLU(), nn.MaxPool2d(3, 2), Fire(8, 4, 8),
                                      Fire(16, 4, 8), nn.MaxPool2d(3, 2), Fire(16, 8, 12))
        self.head = nn.Sequential(nn.Dropout(0.5), nn.Conv2d(24, 10, 1), nn.ReLU(), nn.AdaptiveAvgPool2d(1))

    def forward(self, x):
        return F.softmax(torch.flatten(self.head(self.features(x)), 1), dim=1)


class MiniVGG(nn.Module):
    """Conv(+bias) Relu MaxPool Flatten Gemm(transB) Relu Gemm (as vgg19)."""

    def __init__(self):
        super().__init__()
        self.features = nn.Sequential(nn.Conv2d(3, 8, 3, 1, 1), nn.ReLU(), nn.Conv2d(8, 8, 3, 1, 1), nn.ReLU(),
                                      nn.MaxPool2d(2, 2), nn.Conv2d(8, 16, 3, 1, 1), nn.ReLU(), nn.MaxPool2d(2, 2))
        self.classifier = nn.Sequential(nn.Linear(16 * 4 * 4, 32), nn.ReLU(), nn.Dropout(0.5), nn.Linear(32, 10))

    def forward(self, x):
        return self.classifier(torch.flatten(self.features(x), 1))


class Bottleneck(nn.Module):
    def __init__(self, cin, mid, cout, stride):
        super().__init__()
        self.c1, self.b1 = nn.Conv2d(cin, mid, 1, bias=False), nn.BatchNorm2d(mid)
        self.c2, self.b2 = nn.Conv2d(mid, mid, 3, stride, 1, bias=False), nn.BatchNorm2d(mid)  # v1.5: stride here
        self.c3, self.b3 = nn.Conv2d(mid, cout, 1, bias=False), nn.BatchNorm2d(cout)
        self.proj = None
        if stride != 1 or cin != cout:
            self.proj = nn.Sequential(nn.Conv2d(cin, cout, 1, stride, bias=False), nn.BatchNorm2d(cout))

    def forward(self, x):
        y = F.relu(self.b1(self.c1(x)))
        y = F.relu(self.b2(self.c2(y)))
        y = self.b3(self.c3(y))
        return F.relu(y + (x if self.proj is None else self.proj(x)))


class ResNet50(nn.Module):
    """ResNet-50 v1.5 with the operator sequence of the model zoo's resnet50-v1-12.onnx; used at full
    size by the GPU test, which exports it into a temporary directory (too large for a fixture)."""

    def __init__(self, classes=1000):
        super().__init__()
        self.stem = nn.Sequential(nn.Conv2d(3, 64, 7, 2, 3, bias=False), nn.BatchNorm2d(64), nn.ReLU(),
                                  nn.MaxPool2d(3, 2, 1))
        layers, cin = [], 64
        for mid, n, stride in [(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)]:
            for i in range(n):
                layers.append(Bottleneck(cin, mid, mid * 4, stride if i == 0 else 1))
                cin = mid * 4
        self.layers = nn.Sequential(*layers)
        self.pool = nn.AdaptiveAvgPool2d(1)
        self.fc = nn.Linear(2048, classes)

    def forward(self, x):
        return self.fc(torch.flatten(self.pool(self.layers(self.stem(x))), 1))


def torch_cases():
    cases = [("mini_resnet", MiniResNet, (2, 3, 16, 16)), ("mini_squeezenet", MiniSqueezeNet, (2, 3, 35, 35)),
             ("mini_vgg", MiniVGG, (2, 3, 16, 16))]
    for i, (name, cls, shape) in enumerate(cases):
        gen = torch.Generator().manual_seed(100 + i)
        torch.manual_seed(200 + i)
        m = cls().eval()
        randomize_bn(m, gen)
        x = torch.randn(*shape, generator=gen)
        with torch.no_grad():
            y = m(x)
        write_case(name, export(m, x), x.numpy(), y.numpy())


def handmade_case():
    rng = np.random.default_rng(7)
    f32 = lambda *s, scale=1.0: (rng.standard_normal(s) * scale).astype(np.float32)
    x = f32(3, 4, 8, 8)
    w1, b1 = f32(6, 4, 3, 3, scale=0.2), f32(6, scale=0.1)
    w2 = f32(6, 6, 1, 1, scale=0.3)
    w3 = f32(6, 4, 1, 1, scale=0.3)
    wm, bm = f32(6 * 2 * 2, 5, scale=0.2), f32(5, scale=0.1)
    shape = np.array([0, -1], np.int64)

    tx = torch.from_numpy(x)
    a = F.leaky_relu(F.conv2d(tx, torch.from_numpy(w1), torch.from_numpy(b1), 1, 1), 0.1)
    b = F.conv2d(a, torch.from_numpy(w2))
    c = F.conv2d(tx, torch.from_numpy(w3))
    s = a + b + c                                   # Sum with three inputs
    p = F.avg_pool2d(s, 4, 4)                       # Dropout in front is the identity at inference
    y = torch.flatten(p, 1) @ torch.from_numpy(wm) + torch.from_numpy(bm)

    nodes = [
        node("Conv", ["x", "w1", "b1"], ["c1"], packed=False, kernel_shape=[3, 3], pads=[1, 1, 1, 1],
             strides=[1, 1], dilations=[1, 1], group=1),
        node("LeakyRelu", ["c1"], ["a"], alpha=0.1),
        node("Conv", ["a", "w2"], ["b"], kernel_shape=[1, 1]),
        node("Conv", ["x", "w3"], ["c"], kernel_shape=[1, 1]),
        node("Sum", ["a", "b", "c"], ["s"]),
        node("Dropout", ["s"], ["d"], ratio=0.5),
        node("AveragePool", ["d"], ["p"], kernel_shape=[4, 4], strides=[4, 4]),
        node("Reshape", ["p", "shape"], ["r"]),
        node("MatMul", ["r", "wm"], ["m"]),
        node("Add", ["m", "bm"], ["y"]),
    ]
    inits = [
        tensor_proto("w1", w1, "float_data", packed=False), tensor_proto("b1", b1, "float_data"),
        tensor_proto("w2", w2), tensor_proto("w3", w3, packed=False), tensor_proto("wm", wm),
        tensor_proto("bm", bm, "float_data"), tensor_proto("shape", shape, "int64_data"),
    ]
    # old-style files also list the initializers as graph inputs: they must not count as inputs
    inputs = [value_info("x", FLOAT, ["N", 4, 8, 8]), value_info("w1", FLOAT, [6, 4, 3, 3]),
              value_info("shape", INT64, [2])]
    outputs = [value_info("y", FLOAT, ["N", 5])]
    # the symbolic batch dimension loads as 1, so the data set holds one sample
    write_case("handmade", model(nodes, inits, inputs, outputs), x[:1], y.numpy()[:1])


if __name__ == "__main__":
    torch_cases()
    handmade_case()
