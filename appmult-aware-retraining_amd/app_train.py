"""Synthetic-data AppMult-aware retraining loop (counterpart of the reference's ``micronet+/app_train.py``
minus datasets and checkpoints, which need the network): prepare -> calibrate -> train steps.

    python app_train.py --lut <table file> --bits 7 --batch 512 --steps 10 [--ste] [--optimizer sgd|adam] [--float-grad-window W]

Flow as in the reference (``app_train.py:231-266``): ``init_lookup_tables`` -> ``app_layers.prepare`` ->
one calibration pass in training mode without gradients -> optimiser steps of
forward / cross-entropy / backward / update.  The reference trains with Adam(lr=1e-3); SGD is offered
because the benchmark configuration names it.
"""
import argparse
import os
import sys
import time

import torch
import torch.nn as nn

_HERE = os.path.dirname(os.path.abspath(__file__))
if _HERE not in sys.path:
    sys.path.insert(0, _HERE)

import app_layers  # noqa: E402
import models  # noqa: E402
import self_ops  # noqa: E402


def build_model(arch, bits, use_ste_gradient, device, num_classes=10, approx_linear=False, fold_relu=True):
    net = models.resnet18(num_classes) if arch == "resnet18" else models.vgg16(num_classes)
    net = net.to(device)
    net = app_layers.prepare(net, inplace=True, a_bits=bits, w_bits=bits, use_ste_gradient=use_ste_gradient,
                             approx_linear=approx_linear)
    if fold_relu:
        app_layers.fold_relu(net)       # (ReLUs whose only reader is a quantised convolution go into that layer's quantiser)
    return net


@torch.no_grad()
def calibrate(model, batches):
    """Observers see data once before training (reference ``app_train.py:39-46``)."""
    model.train()
    for x in batches:
        model(x)


def train_steps(model, optimizer, batches, labels):
    """One optimiser step per batch; returns the losses (reference ``app_train.py:23-36``)."""
    criterion = nn.CrossEntropyLoss()
    model.train()
    losses = []
    for x, y in zip(batches, labels):
        optimizer.zero_grad()
        loss = criterion(model(x), y)
        loss.backward()
        optimizer.step()
        losses.append(loss.detach())
    return losses


def synthetic_batches(n, batch, device, seed=0):
    gen = torch.Generator(device=device).manual_seed(seed)
    xs = [torch.randn(batch, 3, 32, 32, device=device, generator=gen) for _ in range(n)]
    ys = [torch.randint(0, 10, (batch,), device=device, generator=gen) for _ in range(n)]
    return xs, ys


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--lut", required=True, help="table file with forward and gradient sections")
    ap.add_argument("--bits", type=int, default=7)
    ap.add_argument("--arch", default="resnet18", choices=["resnet18", "vgg16"])
    ap.add_argument("--batch", type=int, default=512)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--ste", action="store_true", help="straight-through gradients instead of the gradient tables")
    ap.add_argument("--optimizer", default="adam", choices=["adam", "sgd"])
    ap.add_argument("--approx-linear", action="store_true", help="run the classifier on the table as well (the reference keeps it exact)")
    ap.add_argument("--float-grad-window", type=int, default=0, metavar="W",
                    help="replace the file's int16 gradient tables by the float32 difference slopes of its forward table, "
                         "half window W (the float-table backward pass; no counterpart in the reference)")
    ap.add_argument("--eval-batches", type=int, default=0, metavar="N",
                    help="afterwards time N evaluation-mode forward passes of one batch (frozen ranges and weights, no graph)")
    args = ap.parse_args(argv)
    assert torch.cuda.is_available(), "a GPU is required"
    device = torch.device("cuda")
    torch.manual_seed(199608224)
    self_ops.init_lookup_tables(device, args.lut, args.bits)
    if args.float_grad_window > 0:
        import numpy as np
        import gen_bp_lut
        from self_ops.ops_py import approx_ops as P
        rows, cols, _ = P.lut_geometry(args.bits)
        n = 1 << args.bits
        flat = P.lut_appmult.cpu().numpy()
        fwd = flat[:rows * cols].reshape(rows, cols)[:n, :n]
        ga, gb = gen_bp_lut.gradient_tables(fwd, args.float_grad_window, rounded=False)
        pa, pb = np.zeros(flat.size, np.float32), np.zeros(flat.size, np.float32)
        idx = (np.arange(n)[:, None] * cols + np.arange(n)[None, :]).ravel()
        pa[idx], pb[idx] = ga.ravel(), gb.ravel()
        P.set_lookup_tables(device, flat, pa, pb)
    model = build_model(args.arch, args.bits, args.ste, device, approx_linear=args.approx_linear)
    xs, ys = synthetic_batches(args.steps + 1, args.batch, device)
    calibrate(model, xs[:1])
    opt = (torch.optim.Adam(model.parameters(), lr=1e-3, weight_decay=0.0) if args.optimizer == "adam"
           else torch.optim.SGD(model.parameters(), lr=1e-2, momentum=0.9))
    train_steps(model, opt, xs[:1], ys[:1])          # warm-up
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    losses = train_steps(model, opt, xs[1:], ys[1:])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    print(f"{args.arch} batch {args.batch}: {args.steps * args.batch / dt:.1f} img/s, {dt / args.steps * 1e3:.1f} ms/step, "
          f"loss {float(losses[0]):.4f} -> {float(losses[-1]):.4f}")
    if args.eval_batches > 0:
        model.eval()
        with torch.no_grad():
            for _ in range(2):
                model(xs[0])                            # (the first pass expands the tables of the frozen weights)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.eval_batches):
                model(xs[0])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        print(f"{args.arch} batch {args.batch}, evaluation mode: {args.eval_batches * args.batch / dt:.1f} img/s, "
              f"{dt / args.eval_batches * 1e3:.2f} ms per batch")


if __name__ == "__main__":
    main()
