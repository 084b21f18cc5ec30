#!/usr/bin/env python3
"""The ResNet-18-shaped sparse conv stack against the vendor's DENSE convolution path.

    python sparse-ops_amd/bench/bench_cnn_vendor.py [--batch 32] [--hw 224] [--sparsity 0.8] [--runs 20]

Same network, same weights (80 % of the conv weights are zero), same input, on the same GPU:
  * SparseOnnxModel: this library's ELLPACK kernels (only the stored nonzeros are multiplied);
  * torch.nn.functional.conv2d on the GPU (MIOpen, fp32, dense: zeros are multiplied like any
    other weight) -- the analogue of the PyTorch / ONNX Runtime columns of the reference's
    tests/test_resnet.py, which time those runtimes on the CPU.
PyTorch is used for the vendor side only; nothing of the library depends on it.
"""
import argparse
import os
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
for p in (os.path.join(HERE, ".."), os.path.join(HERE, "..", "python")):
    sys.path.insert(0, os.path.abspath(p))

import numpy as np  # noqa: E402


def torch_forward(T, x, width):
    import torch.nn.functional as F
    x = F.relu(F.conv2d(x, T["stem_w"], T["stem_b"], stride=2, padding=3))
    x = F.max_pool2d(x, 3, 2, 1)
    cin = width
    for s, cout in enumerate((width, 2 * width, 4 * width, 8 * width)):
        for b in range(2):
            stride = 2 if (s > 0 and b == 0) else 1
            nm = "s%db%d" % (s, b)
            y = F.relu(F.conv2d(x, T[nm + "c1_w"], T[nm + "c1_b"], stride=stride, padding=1))
            y = F.conv2d(y, T[nm + "c2_w"], T[nm + "c2_b"], padding=1)
            skip = x if (stride == 1 and cin == cout) else F.conv2d(x, T[nm + "proj_w"], T[nm + "proj_b"], stride=stride)
            x, cin = F.relu(y + skip), cout
    return x.mean(dim=(2, 3)) @ T["fc_w"].T + T["fc_b"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--hw", type=int, default=224)
    ap.add_argument("--sparsity", type=float, default=0.8)
    ap.add_argument("--runs", type=int, default=20)
    args = ap.parse_args()

    import datagen
    import onnx_wire as ow
    import sparseops_backend as sb
    payload, t = datagen.resnet18_onnx(seed=47, batch=args.batch, hw=args.hw, sparsity=args.sparsity)
    X = np.random.default_rng(1).standard_normal((args.batch, 3, args.hw, args.hw)).astype(np.float32)

    with tempfile.TemporaryDirectory() as d:
        model = sb.SparseOnnxModel(ow.save(os.path.join(d, "r18.onnx"), payload))
    ours_ms = model.time_device(args.runs, 3)
    y_ours = model.run(X)
    gflop_nnz = model.nnz_flops_per_sample() * args.batch / 1e9
    print("sparse (this library)   : %8.3f ms per batch  %9.1f images/s  %6.2f nnz-TFLOP/s" %
          (ours_ms, args.batch / ours_ms * 1e3, gflop_nnz / ours_ms))

    # The vendor side runs in a child process: PyTorch brings its own HIP runtime, which must not
    # share a process with the one this library has already initialised.
    import subprocess
    with tempfile.TemporaryDirectory() as d:
        np.savez(os.path.join(d, "in.npz"), X=X, **t)
        r = subprocess.run([sys.executable, os.path.abspath(__file__), "--torch-child", d, "--runs", str(args.runs)],
                           capture_output=True, text=True)
        if r.returncode != 0 or not os.path.exists(os.path.join(d, "out.npz")):
            print("vendor side skipped:", (r.stdout + r.stderr).strip().splitlines()[-1] if (r.stdout + r.stderr).strip() else "no output")
            return
        out = np.load(os.path.join(d, "out.npz"))
        dense_ms, y_t = float(out["ms"]), out["y"]
    print("dense  (torch / MIOpen) : %8.3f ms per batch  %9.1f images/s" % (dense_ms, args.batch / dense_ms * 1e3))
    err = np.abs(y_ours.astype(np.float64) - y_t).max() / np.abs(y_t).max()
    print("max relative difference of the outputs: %.2e   sparse / dense time: %.2fx" % (err, ours_ms / dense_ms))


def torch_child(d, runs):
    import torch
    if not torch.cuda.is_available():
        sys.exit("torch sees no GPU")
    dev = torch.device("cuda:0")
    z = np.load(os.path.join(d, "in.npz"))
    T = {k: torch.from_numpy(z[k]).to(dev) for k in z.files if k != "X"}
    xt = torch.from_numpy(z["X"]).to(dev)
    with torch.no_grad():
        for _ in range(3):
            y = torch_forward(T, xt, 64)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(runs):
            y = torch_forward(T, xt, 64)
        e1.record()
        torch.cuda.synchronize()
        np.savez(os.path.join(d, "out.npz"), ms=e0.elapsed_time(e1) / runs, y=y.cpu().numpy())


if __name__ == "__main__":
    if len(sys.argv) >= 3 and sys.argv[1] == "--torch-child":
        torch_child(sys.argv[2], int(sys.argv[4]) if len(sys.argv) >= 5 else 20)
    else:
        main()
