#!/usr/bin/env python3
"""Writes tests/golden/torch_export/*.onnx and torch_export/expected.npz.

The .onnx files are real `torch.onnx.export` output (TorchScript exporter, opset 14,
constant folding on, static shapes) of small models with the topologies the reference's
scripts export (tests/full_test.py:21-41 MLP; tests/test_cnn.py conv stacks;
tests/test_resnet.py:45-71 torchvision ResNet-18: stem + BatchNorm-folded basic blocks
with 1x1 stride-2 projections), pruned like those scripts prune (random unstructured,
made permanent).  expected.npz holds the seeded inputs and PyTorch's own fp32 outputs.

The exporter's C++ serialiser writes the ModelProto bytes; only its last Python step,
which re-parses the bytes with the `onnx` package to splice in onnx-script functions
(there are none in these models), is skipped because that package is not installed.

    python tests/golden/make_torch_onnx.py
"""
import io
import os
import warnings

import numpy as np
import torch
import torch.nn as nn
import torch.nn.utils.prune as prune

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "torch_export")


def export_bytes(model, dummy):
    from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    keep = onnx_proto_utils._add_onnxscript_fn
    onnx_proto_utils._add_onnxscript_fn = lambda proto, custom_opsets: proto
    try:
        buf = io.BytesIO()
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            torch.onnx.export(model, dummy, buf, dynamo=False, opset_version=14, do_constant_folding=True,
                              input_names=["input"], output_names=["output"], dynamic_axes=None)
        return buf.getvalue()
    finally:
        onnx_proto_utils._add_onnxscript_fn = keep


def prune_all(model, amount):
    for m in model.modules():
        if isinstance(m, (nn.Conv2d, nn.Linear)):
            prune.random_unstructured(m, name="weight", amount=amount)
            prune.remove(m, "weight")


def randomise_bn(model, gen):
    for m in model.modules():
        if isinstance(m, nn.BatchNorm2d):
            m.weight.data = 0.5 + torch.rand(m.weight.shape, generator=gen)
            m.bias.data = 0.1 * torch.randn(m.bias.shape, generator=gen)
            m.running_mean.data = 0.1 * torch.randn(m.running_mean.shape, generator=gen)
            m.running_var.data = 0.5 + torch.rand(m.running_var.shape, generator=gen)


class BasicBlock(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.conv1 = nn.Conv2d(cin, cout, 3, stride, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(cout)
        self.relu = nn.ReLU(inplace=True)
        self.conv2 = nn.Conv2d(cout, cout, 3, 1, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(cout)
        self.down = None
        if stride != 1 or cin != cout:
            self.down = nn.Sequential(nn.Conv2d(cin, cout, 1, stride, bias=False), nn.BatchNorm2d(cout))

    def forward(self, x):
        idt = x if self.down is None else self.down(x)
        out = self.relu(self.bn1(self.conv1(x)))
        out = self.bn2(self.conv2(out))
        return self.relu(out + idt)


class TinyResNet(nn.Module):
    """torchvision's ResNet layout at small width: 7x7/2 stem, 3x3/2 max-pool, basic blocks."""

    def __init__(self, width=8, classes=10):
        super().__init__()
        self.conv1 = nn.Conv2d(3, width, 7, 2, 3, bias=False)
        self.bn1 = nn.BatchNorm2d(width)
        self.relu = nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(3, 2, 1)
        self.layer1 = nn.Sequential(BasicBlock(width, width, 1), BasicBlock(width, width, 1))
        self.layer2 = nn.Sequential(BasicBlock(width, 2 * width, 2), BasicBlock(2 * width, 2 * width, 1))
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(2 * width, classes)

    def forward(self, x):
        x = self.maxpool(self.relu(self.bn1(self.conv1(x))))
        x = self.layer2(self.layer1(x))
        return self.fc(torch.flatten(self.avgpool(x), 1))


def models():
    mlp = nn.Sequential(nn.Linear(20, 32), nn.ReLU(), nn.Linear(32, 16), nn.Sigmoid(),
                        nn.Linear(16, 8), nn.Tanh(), nn.Linear(8, 5))
    cnn_gap = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(), nn.MaxPool2d(2),
                            nn.Conv2d(8, 16, 3, stride=2, padding=1), nn.ReLU(),
                            nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(16, 10))
    cnn_flat = nn.Sequential(nn.Conv2d(2, 6, 3, padding=1), nn.ReLU(), nn.MaxPool2d(2),
                             nn.Conv2d(6, 4, 5, padding=2, dilation=1), nn.Tanh(),
                             nn.Flatten(), nn.Linear(4 * 5 * 6, 12), nn.ReLU(), nn.Linear(12, 7))
    return [
        ("mlp_gemm", mlp, (3, 20), 0.7),
        ("cnn_gap", cnn_gap, (2, 3, 16, 16), 0.6),
        ("cnn_flatten_fc", cnn_flat, (4, 2, 10, 12), 0.5),
        ("resnet_tiny", TinyResNet(), (2, 3, 40, 40), 0.6),
    ]


def main():
    os.makedirs(OUT, exist_ok=True)
    expected = {}
    for i, (name, model, shape, amount) in enumerate(models()):
        torch.manual_seed(100 + i)
        gen = torch.Generator().manual_seed(200 + i)
        for p in model.parameters():
            if p.dim() > 1:
                nn.init.kaiming_normal_(p, generator=gen)
            else:
                p.data = 0.1 * torch.randn(p.shape, generator=gen)
        randomise_bn(model, gen)
        model.eval()
        prune_all(model, amount)
        x = torch.randn(*shape, generator=gen)
        with torch.no_grad():
            y = model(x)
        payload = export_bytes(model, x)
        with open(os.path.join(OUT, name + ".onnx"), "wb") as f:
            f.write(payload)
        expected[name + "__input"] = x.numpy()
        expected[name + "__output"] = y.numpy()
        print("%-16s %7d bytes  in %s  out %s" % (name, len(payload), tuple(x.shape), tuple(y.shape)))
    np.savez_compressed(os.path.join(OUT, "expected.npz"), **expected)


if __name__ == "__main__":
    main()
