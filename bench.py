#!/usr/bin/env python3
"""Benchmark of the LUT-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-train-step] [--no-8bit] [--layers] [--grad-tables f32] [--workload vgg16_b128_8bit] [--codes captured]

One "step" = forward + backward (gradA and gradB) LUT-GEMM of every conv layer and the fc layer of a
CIFAR-style ResNet-18 at batch 256, 7-bit tables (BASELINE.json configs[2]: 21 GEMMs,
426 564 648 960 LUT-MACs), called through the C ABI of libamr_lutgemm.so on torch's current stream.
Operands are uniform random codes (worst case for LDS bank conflicts), the forward table is
a*b + seeded error in [-64,64], the gradient tables are its difference-based slopes (half window 8)
in the reference's int16 x16 encoding.  All inputs and outputs are resident in HBM before the timed
region starts.  Prints ONE JSON line.

The rate is compared with the LDS-gather roofline: one table gather per LUT-MAC,
256 CUs x 2.4 GHz x 32 lanes/clk = 1.966e13 gathers/s (a wave64 ds_read_u16/b32 occupies the LDS pipe
for two clocks when conflict-free; measured on this device by the probe in the library).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "appmult-aware-retraining_amd")
for _p in (ROOT, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# (name, count, M, K, N) at batch 256: M = batch*oh*ow, K = cin*kh*kw, N = cout
RESNET18_B256 = [
    ("conv1", 1, 262144, 27, 64), ("conv2_x", 4, 262144, 576, 64),
    ("conv3_first", 1, 65536, 576, 128), ("conv3_x", 3, 65536, 1152, 128), ("conv3_short", 1, 65536, 64, 128),
    ("conv4_first", 1, 16384, 1152, 256), ("conv4_x", 3, 16384, 2304, 256), ("conv4_short", 1, 16384, 128, 256),
    ("conv5_first", 1, 4096, 2304, 512), ("conv5_x", 3, 4096, 4608, 512), ("conv5_short", 1, 4096, 256, 512),
    ("fc", 1, 256, 512, 10),
]
BATCH = 256
# VGG-16 conv stack on 32x32 inputs + fc at batch 128 (BASELINE.json configs[3], 8-bit tables): 120 269 438 976 LUT-MACs
VGG16_B128 = [
    ("conv1_1", 1, 131072, 27, 64), ("conv1_2", 1, 131072, 576, 64), ("conv2_1", 1, 32768, 576, 128), ("conv2_2", 1, 32768, 1152, 128),
    ("conv3_1", 1, 8192, 1152, 256), ("conv3_x", 2, 8192, 2304, 256), ("conv4_1", 1, 2048, 2304, 512), ("conv4_x", 2, 2048, 4608, 512),
    ("conv5_x", 3, 512, 4608, 512), ("fc", 1, 128, 512, 10),
]
N_CU, CLK = 256, 2.4e9                    # MI355X: compute units, published peak clock
LDS_GATHER_PEAK = N_CU * CLK * 32         # gathers/s of the one-gather-per-MAC formulation: conflict-free lanes served per clock
LDS_READ_PEAK = N_CU * CLK * 256          # bytes/s the LDS delivers with ds_read_b64 / ds_read_b128 (64 lanes x 8 B in 2 clk, x 16 B in 4)
VALU_ISSUE_PEAK = N_CU * CLK * 64         # lane-operations/s of unpacked VALU instructions: 4 SIMDs x 16 lanes per clock
HBM_PEAK = 8.0e12

PROFILES = os.path.join(ROOT, "profiles")
# the expanded-table kernel that runs the conv2_x launch of each phase (the launch the committed counter tables cover)
CONV2X_KERNEL = {"forward": "lutgemm_fwd_slab_kernel", "gradA": "lutgemm_gradA_slab_kernel<32", "gradB": "lutgemm_gradB_slab16_kernel"}


def profile_rows(name):
    """Rows of the markdown tables of a committed profile summary: {first cell without back-ticks: [cells]}; {} when the file is absent."""
    rows = {}
    try:
        with open(os.path.join(PROFILES, name)) as f:
            for line in f:
                if line.startswith("| `"):
                    cells = [c.strip() for c in line.strip().strip("|").split("|")]
                    rows[cells[0].strip("`")] = cells
    except OSError:
        pass
    return rows


def conv2x_counters(kind):
    """From the committed counter tables in profiles/ (NOT measured in this run; every field taken from them is labelled
    "source": "committed profile"): (bytes the L2s read + wrote for the conv2_x launch of this phase's kernel, VALU
    instructions per multiply-add of that kernel = counted wave instructions x 64 lanes / multiply-adds of the counted
    launches); None, with a warning on stderr, for what no committed table holds."""
    kernel = CONV2X_KERNEL[kind]
    traffic = valu_per_mac = None
    for k, cells in profile_rows("conv2x_hbm_traffic.md").items():
        if kernel in k:
            traffic = (int(cells[2]) + int(cells[4])) * 2**20          # scaled FETCH_SIZE + WRITE_SIZE, MiB
    for k, cells in profile_rows("conv2x_lds_counters.md").items():
        if kernel in k and len(cells) > 9:
            valu_per_mac = float(cells[9])
    if traffic is None or valu_per_mac is None:
        print(f"bench.py: no row for kernel '{kernel}' in profiles/conv2x_hbm_traffic.md / conv2x_lds_counters.md: "
              "counter-derived fields of this phase are null", file=sys.stderr)
    return traffic, valu_per_mac


def synth_tables(np, bits, err, half_ws, float_slopes=False):
    """The benchmark's tables from the package's own generator: forward table a*b + seeded error in [-err, err] clipped to
    uint16 (BASELINE.json configs[0]), gradient tables = its difference-based slopes (gen_bp_lut.gradient_tables), all three
    as the padded 1-D arrays of the boundary.  Returns (forward u16, grad_a, grad_b, 2-D forward table)."""
    import gen_bp_lut
    from self_ops.ops_py import approx_ops as ops
    rng = np.random.default_rng(0)
    n = 1 << bits
    a = np.arange(n, dtype=np.int64)
    T = np.clip(a[:, None] * a[None, :] + rng.integers(-err, err + 1, size=(n, n)), 0, 65535)
    gx, gy = gen_bp_lut.gradient_tables(T, half_ws, rounded=not float_slopes)
    gdt = np.float32 if float_slopes else np.int16
    return ops.pad_table(T, bits, np.uint16), ops.pad_table(gx, bits, gdt), ops.pad_table(gy, bits, gdt), T


def capture_codes(torch, dev, bits, tables, arch, batch):
    """Operand codes of every LUT GEMM of one training-mode forward pass of this package's network on N(0,1) images:
    {(M, K, N): (A codes, B codes)}, the first GEMM of each shape."""
    import app_train
    from self_ops.ops_py import approx_ops as ops
    ops.set_lookup_tables(dev, *tables)
    torch.manual_seed(0)
    model = app_train.build_model(arch, bits, False, dev, approx_linear=True)
    x = torch.randn(batch, 3, 32, 32, device=dev, generator=torch.Generator(device=dev).manual_seed(1))
    seen = {}
    # (the layers call the LUT GEMM through either of the native module's two forward functions; both take a, b first)
    names = ("approx_gemm_forward", "approx_conv_forward_dequant")
    natives = {n: getattr(ops.approx_ops, n) for n in names}

    def spy_on(fn):
        def spy(a, b, *rest, **kw):
            seen.setdefault((a.shape[0], a.shape[1], b.shape[1]), (a.clone(), b.clone()))
            return fn(a, b, *rest, **kw)
        return spy

    import app_layers
    for n in names:
        setattr(ops.approx_ops, n, spy_on(natives[n]))
    implicit, app_layers.IMPLICIT_FORWARD = app_layers.IMPLICIT_FORWARD, False      # (the GEMM operands are what is captured)
    try:
        model.train()
        with torch.no_grad():
            model(x)
    finally:
        app_layers.IMPLICIT_FORWARD = implicit
        for n in names:
            setattr(ops.approx_ops, n, natives[n])
    return seen


def training_step(torch, dev, tables, bits, batch=512, steps=10):
    """Forward + cross-entropy + backward + SGD update of this package's quantised ResNet-18 (LUT convolutions) on synthetic
    CIFAR-shaped data, after one calibration pass and one untimed step: wall-clock ms per step and images per second.
    The LUT GEMM's share of a step's GPU time is measured in this run, on three further steps outside the timed ones: HIP
    events on the launch stream around every call of the library's forward and backward LUT entry points (table expansion,
    header, finish and gated launches included; the forward call includes the dequantising store, the convolution-shaped
    gradA the finishing of the input gradient), summed, over the wall-clock time of a timed step (GPU-bound)."""
    import app_train
    import approx_ops as native
    from self_ops.ops_py import approx_ops as ops
    ops.set_lookup_tables(dev, *(t.cpu().numpy() for t in tables))
    torch.manual_seed(0)
    model = app_train.build_model("resnet18", bits, False, dev)
    share_steps = 3
    xs, ys = app_train.synthetic_batches(steps + 2 + share_steps, batch, dev)
    app_train.calibrate(model, xs[:1])
    opt = torch.optim.SGD(model.parameters(), lr=1e-2, momentum=0.9)
    app_train.train_steps(model, opt, xs[1:2], ys[1:2])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    losses = app_train.train_steps(model, opt, xs[2:2 + steps], ys[2:2 + steps])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    spans = []
    # (the layers reach the LUT kernels through these four functions of the native module; the last one, the convolution-shaped
    # gradA, finishes the input gradient of the quantiser in the same kernel)
    names = [n for n in ("approx_gemm_forward", "approx_gemm_backward", "approx_conv_forward_dequant", "approx_conv_input_grad") if hasattr(native, n)]
    originals = {n: getattr(native, n) for n in names}

    def timed_call(fn):
        def call(*a, **k):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = fn(*a, **k)
            e1.record()
            spans.append((e0, e1))
            return r
        return call

    for n in names:
        setattr(native, n, timed_call(originals[n]))
    try:
        s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s0.record()
        app_train.train_steps(model, opt, xs[2 + steps:], ys[2 + steps:])
        s1.record()
        torch.cuda.synchronize()
    finally:
        for n in names:
            setattr(native, n, originals[n])
    lut_ms = sum(a.elapsed_time(b) for a, b in spans)
    # the same network in evaluation mode (frozen ranges and weights, no graph): forward passes of one batch, wall clock
    model.eval()
    with torch.no_grad():
        for _ in range(2):
            model(xs[0])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            model(xs[0])
        torch.cuda.synchronize()
        eval_dt = time.perf_counter() - t0
    return {"workload": f"resnet18_cifar_b{batch}_{bits}bit full step: forward, cross-entropy, backward, SGD (BASELINE.json configs[4])",
            "steps": steps, "ms_per_step": dt / steps * 1e3, "images_per_s": batch * steps / dt,
            "loss_first_last": [float(losses[0]), float(losses[-1])],
            "lut_gemm_share_of_gpu_time": (lut_ms / share_steps) / (dt / steps * 1e3),
            "lut_gemm_ms_per_step": lut_ms / share_steps,
            "share_source": f"measured in this run: HIP events around the {len(spans) // share_steps} library GEMM calls of a step, {share_steps} steps, "
                            "over the wall-clock time of the timed steps (the step is bound by the GPU; the steps that carry the events run "
                            f"{s0.elapsed_time(s1) / share_steps:.1f} ms each, stretched by the event records, and are not the denominator)",
            "eval_forward": {"ms_per_batch": eval_dt / steps * 1e3, "images_per_s": batch * steps / eval_dt,
                             "note": "evaluation mode, no graph: expansions kept per layer, 3x3 layers without a window matrix"}}


def eight_bit_step(torch, np, dev, lib, O, stream, float_tables, steps=5):
    """The 8-bit stress configuration (BASELINE.json configs[3]: VGG-16 conv shapes at batch 128, forward error +-256, half
    window 16) as a secondary record of the default run, with the reference's int16 x16 gradient tables or with the float32
    slopes the configuration names: the same forward + backward GEMM step as the headline, timed over `steps` steps after two
    untimed ones.  (`--workload vgg16_b128_8bit [--grad-tables f32]` runs it as the main workload, with the per-kernel
    break-down.)"""
    bits = 8
    f16, ga_t, gb_t, _ = synth_tables(np, bits, 256, 16, float_slopes=float_tables)
    lut, lga, lgb = (torch.from_numpy(t).to(dev) for t in (f16, ga_t, gb_t))
    L = lut.numel()
    gen = torch.Generator(device=dev).manual_seed(0)
    bufs, ws_need = {}, 0
    ws_query = lib.amr_lut_gemm_backward_f32tab_workspace_bytes if float_tables else lib.amr_lut_gemm_backward_workspace_bytes
    for name, cnt, M, K, N in VGG16_B128:
        bufs[name] = (torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=gen),
                      torch.randint(0, 256, (K, N), dtype=torch.uint8, device=dev, generator=gen),
                      torch.empty((M, N), dtype=torch.int32, device=dev),
                      torch.randn((M, N), dtype=torch.float32, device=dev, generator=gen),
                      torch.empty((M, K), dtype=torch.float32, device=dev), torch.empty((K, N), dtype=torch.float32, device=dev))
        ws_need = max(ws_need, ws_query(M, K, N))
    ws = torch.empty(max(ws_need, 256), dtype=torch.uint8, device=dev)

    def step():
        for name, cnt, M, K, N in VGG16_B128:
            A, B, C = bufs[name][:3]
            for _ in range(cnt):
                assert lib.amr_lut_gemm_forward(A.data_ptr(), B.data_ptr(), C.data_ptr(), lut.data_ptr(), L, M, K, N, stream) == 0, lib.amr_last_error()
        for name, cnt, M, K, N in reversed(VGG16_B128):
            A, B, C, gC, gA, gB = bufs[name]
            for _ in range(cnt):
                if float_tables:
                    rc = lib.amr_lut_gemm_backward_f32tab(gC.data_ptr(), A.data_ptr(), B.data_ptr(), gA.data_ptr(), gB.data_ptr(), lga.data_ptr(),
                                                          lgb.data_ptr(), L, 1.0, M, K, N, 0, ws.data_ptr(), ws.numel(), stream)
                else:
                    rc = lib.amr_lut_gemm_backward(gC.data_ptr(), A.data_ptr(), B.data_ptr(), gA.data_ptr(), gB.data_ptr(), lga.data_ptr(),
                                                   lgb.data_ptr(), L, M, K, N, ws.data_ptr(), ws.numel(), stream)
                assert rc == 0, lib.amr_last_error()

    # parity guard on a row sample of one layer that takes the expanded tables (the parity suite proper is tests/ -m gpu)
    name, _, M, K, N = VGG16_B128[2]
    A, B, C, gC, gA, gB = bufs[name]
    step()
    torch.cuda.synchronize()
    rows = slice(100, 132)
    if float_tables:
        want_a, _ = O.backward_np(gC[rows].cpu().numpy(), A[rows].cpu().numpy(), B.cpu().numpy(), O.unpack_table(ga_t, bits),
                                  O.unpack_table(gb_t, bits), factor=1.0)
    else:
        want_a, _ = O.backward_c_f32(gC[rows].cpu().numpy(), A[rows].cpu().numpy(), B.cpu().numpy(), ga_t, gb_t, bits)
    got_a = gA[rows].cpu().numpy()
    assert np.abs(got_a - want_a).max() <= 1e-4 * np.abs(want_a).max(), "8-bit gradA parity guard failed"
    step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    macs = 3 * sum(c * M * K * N for _, c, M, K, N in VGG16_B128)
    # floors of this step: VALU issue, one multiply-add per backward LUT-MAC and half an addition per forward entry; LDS read
    # bandwidth, 2 bytes per table entry (4 for float32 gradient tables)
    floor_valu = (0.5 + 2.0) * (macs / 3) / VALU_ISSUE_PEAK
    floor_lds = (2 + (8 if float_tables else 4)) * (macs / 3) / LDS_READ_PEAK
    floor = max(floor_valu, floor_lds)
    return {"workload": "vgg16_cifar_b128_8bit_lutgemm_fwd_bwd (BASELINE.json configs[3]: 13 conv + 1 fc GEMMs), " +
                        ("float32 gradient tables (unrounded slopes)" if float_tables else "int16 x16 gradient tables"),
            "steps": steps, "ms_per_step": dt / steps * 1e3, "lut_mac_per_s": macs * steps / dt,
            "frac_of_lds_gather_roofline": macs * steps / dt / LDS_GATHER_PEAK,
            "own_bound": {"floor_ms": floor * 1e3, "binds": "valu_issue" if floor_valu >= floor_lds else "lds_read",
                          "frac": floor / (dt / steps)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-train-step", action="store_true", help="skip the full training step leg (ResNet-18, batch 512)")
    ap.add_argument("--no-8bit", action="store_true", help="skip the secondary 8-bit leg (VGG-16 conv shapes, batch 128)")
    ap.add_argument("--layers", action="store_true", help="also print a per-layer table to stderr")
    ap.add_argument("--calib", action="store_true", help="also run three plain 256 MiB device copies (reference for scaling FETCH_SIZE/WRITE_SIZE counters)")
    ap.add_argument("--only", default="", help="comma-separated layer names: restrict the step to them (profiling aid; the JSON line then describes that subset)")
    ap.add_argument("--grad-tables", choices=["i16", "f32"], default="i16",
                    help="i16: the reference's int16 x16 gradient tables (the headline metric); f32: the unrounded float32 slopes "
                         "through the float-table entry point")
    ap.add_argument("--workload", choices=["resnet18_b256_7bit", "vgg16_b128_8bit"], default="resnet18_b256_7bit",
                    help="resnet18_b256_7bit: the headline configuration; vgg16_b128_8bit: the 8-bit stress configuration "
                         "(forward error +-256, half window 16)")
    ap.add_argument("--codes", choices=["uniform", "captured"], default="uniform",
                    help="uniform: independent uniform random codes (the headline figure; worst case for LDS conflicts); captured: the "
                         "operand codes one forward pass of this package's network produces on N(0,1) images with random-init weights "
                         "(post-ReLU activations and bell-shaped weights: skewed codes)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures the one-GPU hot path only: every box of this build has one GPU; run with --gpus 1")

    import numpy as np
    import torch

    global RESNET18_B256, BATCH
    headline = args.workload == "resnet18_b256_7bit"
    BITS, ERR, HALF_WS = (7, 64, 8) if headline else (8, 256, 16)
    NCODE = 1 << BITS
    if not headline:
        RESNET18_B256, BATCH = VGG16_B128, 128      # the layer list of the step
    full = not args.only
    if args.only:
        keep = set(args.only.split(","))
        RESNET18_B256 = [l for l in RESNET18_B256 if l[0] in keep]
        assert RESNET18_B256, "no such layer"

    import approx_ops  # loads libamr_lutgemm.so, fails loudly when it is missing
    from oracle import lutgemm_oracle as O   # the parity guards and the CPU baseline leg only: every input comes from the package

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = approx_ops._lib
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    # tables (config 1 recipe), built by the package's own generator --------------------------------
    f32_tables = args.grad_tables == "f32"
    f16_np, ga_np, gb_np, _ = synth_tables(np, BITS, ERR, HALF_WS, float_slopes=f32_tables)
    lut, lga, lgb = (torch.from_numpy(t).to(dev) for t in (f16_np, ga_np, gb_np))
    L = lut.numel()

    # operands, resident in HBM --------------------------------------------------------------------
    gen = torch.Generator(device=dev).manual_seed(0)
    bufs = {}
    ws_need = 0
    for name, cnt, M, K, N in RESNET18_B256:
        bufs[name] = dict(
            A=torch.randint(0, NCODE, (M, K), dtype=torch.uint8, device=dev, generator=gen),
            B=torch.randint(0, NCODE, (K, N), dtype=torch.uint8, device=dev, generator=gen),
            C=torch.empty((M, N), dtype=torch.int32, device=dev),
            gC=torch.randn((M, N), dtype=torch.float32, device=dev, generator=gen),
            gA=torch.empty((M, K), dtype=torch.float32, device=dev),
            gB=torch.empty((K, N), dtype=torch.float32, device=dev))
        ws_need = max(ws_need, (lib.amr_lut_gemm_backward_f32tab_workspace_bytes if f32_tables else lib.amr_lut_gemm_backward_workspace_bytes)(M, K, N))
    ws = torch.empty(max(ws_need, 256), dtype=torch.uint8, device=dev)

    if args.codes == "captured":
        seen = capture_codes(torch, dev, BITS, (f16_np, ga_np, gb_np),
                             "resnet18" if headline else "vgg16", BATCH)
        for name, cnt, M, K, N in RESNET18_B256:
            assert (M, K, N) in seen, f"the network's forward pass ran no LUT GEMM of shape {(M, K, N)} ({name})"
            bufs[name]["A"], bufs[name]["B"] = seen[(M, K, N)]

    def fwd(name, M, K, N):
        b = bufs[name]
        rc = lib.amr_lut_gemm_forward(b["A"].data_ptr(), b["B"].data_ptr(), b["C"].data_ptr(), lut.data_ptr(), L, M, K, N, stream)
        assert rc == 0, lib.amr_last_error()

    def bwd(name, M, K, N, want_a=True, want_b=True):
        b = bufs[name]
        if f32_tables:
            rc = lib.amr_lut_gemm_backward_f32tab(b["gC"].data_ptr(), b["A"].data_ptr(), b["B"].data_ptr(),
                                                  b["gA"].data_ptr() if want_a else None, b["gB"].data_ptr() if want_b else None,
                                                  lga.data_ptr(), lgb.data_ptr(), L, 1.0, M, K, N, 0, ws.data_ptr(), ws.numel(), stream)
        else:
            rc = lib.amr_lut_gemm_backward(b["gC"].data_ptr(), b["A"].data_ptr(), b["B"].data_ptr(),
                                           b["gA"].data_ptr() if want_a else None, b["gB"].data_ptr() if want_b else None,
                                           lga.data_ptr(), lgb.data_ptr(), L, M, K, N, ws.data_ptr(), ws.numel(), stream)
        assert rc == 0, lib.amr_last_error()

    def step():
        for name, cnt, M, K, N in RESNET18_B256:
            for _ in range(cnt):
                fwd(name, M, K, N)
        for name, cnt, M, K, N in reversed(RESNET18_B256):
            for _ in range(cnt):
                bwd(name, M, K, N)

    macs_fwd = sum(c * M * K * N for _, c, M, K, N in RESNET18_B256)
    assert macs_fwd == (142188216320 if headline else 40089812992) or not full
    macs_step = 3 * macs_fwd

    # quick parity guard on a row sample of one layer (the full parity suite is tests/ -m gpu) ---------
    gname, _, gM, gK, gN = RESNET18_B256[-1] if not full else RESNET18_B256[4 if headline else 2]
    fwd(gname, gM, gK, gN)
    torch.cuda.synchronize()
    b = bufs[gname]
    rows = slice(100, 164)
    want = O.forward_c(b["A"][rows].cpu().numpy(), b["B"].cpu().numpy(), lut.cpu().numpy(), BITS)
    assert (b["C"][rows].cpu().numpy().view(np.uint32) == want).all(), "forward parity guard failed"

    if args.calib:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # timed region ------------------------------------------------------------------------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt / args.steps * 1e3
    rate = macs_step * args.steps / dt

    # per-kernel timing with events on the launch stream -------------------------------------------------
    def timed(fn, reps=3):
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / reps

    # forward pass with the table expansions kept between calls (frozen weights: inference, evaluation, calibration): one
    # amr_fwd_cache per layer, every timed call a hit
    caches = {name: approx_ops.ForwardCache() for name, *_ in RESNET18_B256}

    def fwd_cached(name, M, K, N):
        b = bufs[name]
        rc = lib.amr_lut_gemm_forward_cached(caches[name]._h, 1, b["A"].data_ptr(), b["B"].data_ptr(), b["C"].data_ptr(), 0, lut.data_ptr(),
                                             L, M, K, N, stream)
        assert rc == 0, lib.amr_last_error()

    kernels = {"forward": 0.0, "gradA": 0.0, "gradB": 0.0}
    fwd_frozen_ms = 0.0
    per_layer = []
    for name, cnt, M, K, N in RESNET18_B256:
        fwd_frozen_ms += cnt * timed(lambda: fwd_cached(name, M, K, N))
        tf = timed(lambda: fwd(name, M, K, N))
        ta = timed(lambda: bwd(name, M, K, N, True, False))
        tb = timed(lambda: bwd(name, M, K, N, False, True))
        kernels["forward"] += cnt * tf
        kernels["gradA"] += cnt * ta
        kernels["gradB"] += cnt * tb
        per_layer.append((name, cnt, M, K, N, tf, ta, tb))
    for c in caches.values():
        c.close()
    dominant = max(kernels, key=kernels.get)
    dom_ms = kernels[dominant]
    dom_rate = macs_fwd / (dom_ms * 1e-3)         # each kernel does M*K*N gathers per GEMM
    launches = sum(c for _, c, *_ in RESNET18_B256)
    if args.layers:
        print(f"{'layer':12s} cnt {'M':>7s} {'K':>5s} {'N':>4s}   fwd ms (GMAC/s)   gradA ms (GMAC/s)   gradB ms (GMAC/s)", file=sys.stderr)
        for name, cnt, M, K, N, tf, ta, tb in per_layer:
            w = M * K * N / 1e6
            print(f"{name:12s} {cnt:3d} {M:7d} {K:5d} {N:4d}   {tf:7.3f} ({w/tf:7.0f})   {ta:7.3f} ({w/ta:7.0f})   {tb:7.3f} ({w/tb:7.0f})", file=sys.stderr)
        print("kernel totals per step (ms):", {k: round(v, 3) for k, v in kernels.items()}, file=sys.stderr)

    # algorithmic HBM bytes of the dominant kernel over one step
    def hbm_bytes(kind, M, K, N):
        if kind == "forward":
            return M * K + K * N + 4 * M * N + 2 * L
        if kind == "gradA":
            return 4 * M * N + M * K + K * N + 4 * M * K + 2 * L
        return 4 * M * N + M * K + K * N + 4 * K * N + 2 * L
    dom_bytes = sum(c * hbm_bytes(dominant, M, K, N) for _, c, M, K, N in RESNET18_B256)

    probe_free = approx_ops.lds_gather_probe(0, 16, 4000)
    probe_row = approx_ops.lds_gather_probe(1, 16, 4000)
    probe_delivery = approx_ops.lds_gather_probe(2, 16, 4000)      # bytes/s of LDS-direct 32 KB chunk loads from the L2, all CUs

    # single-GEMM configuration (BASELINE configs[1]: M=4096, K=576, N=64 forward+backward) ---------------
    M1, K1, N1 = 4096, 576, 64
    bufs["single"] = dict(A=torch.randint(0, NCODE, (M1, K1), dtype=torch.uint8, device=dev, generator=gen),
                          B=torch.randint(0, NCODE, (K1, N1), dtype=torch.uint8, device=dev, generator=gen),
                          C=torch.empty((M1, N1), dtype=torch.int32, device=dev),
                          gC=torch.randn((M1, N1), dtype=torch.float32, device=dev, generator=gen),
                          gA=torch.empty((M1, K1), dtype=torch.float32, device=dev),
                          gB=torch.empty((K1, N1), dtype=torch.float32, device=dev))
    # (left out of a run restricted to some layers: a profiler run of such a subset then holds launches of those layers only)
    t_single = timed(lambda: (fwd("single", M1, K1, N1), bwd("single", M1, K1, N1)), reps=50) if full else float("nan")

    # Limits that are ceilings of this hardware for the work itself, whatever the formulation (no fraction of them can pass 1):
    # vector issue -- one multiply-add instruction lane per backward LUT-MAC, half an addition per forward table entry (two
    # 16-bit entries per 32-bit add), 64 lanes per clock and CU; LDS read bandwidth -- the table entry of every LUT-MAC (2 B;
    # 4 B from float32 gradient tables) at 256 B per clock and CU.
    entry_b = 4 if f32_tables else 2
    own = {"valu_issue_peak_lane_ops_per_s": VALU_ISSUE_PEAK, "lds_read_peak_Bps": LDS_READ_PEAK,
           "definition": "floor time = max(VALU-issue floor: 1 multiply-add per backward LUT-MAC, 0.5 additions per forward entry, 64 lanes/clk/CU; "
                         "LDS-read floor: one table entry per LUT-MAC at 256 B/clk/CU), 256 CU x 2.4 GHz; frac = floor time / measured time",
           "per_phase": {}}
    floor_step = 0.0
    for kind, ops_per_mac, bytes_per_mac in (("forward", 0.5, 2), ("gradA", 1.0, entry_b), ("gradB", 1.0, entry_b)):
        fv, fl = macs_fwd * ops_per_mac / VALU_ISSUE_PEAK * 1e3, macs_fwd * bytes_per_mac / LDS_READ_PEAK * 1e3
        floor_step += max(fv, fl)
        own["per_phase"][kind] = {"valu_floor_ms": fv, "lds_read_floor_ms": fl, "binds": "valu_issue" if fv >= fl else "lds_read",
                                  "measured_ms": kernels[kind], "frac": max(fv, fl) / kernels[kind]}
    own["step"] = {"floor_ms": floor_step, "measured_ms": ms_step, "frac": floor_step / ms_step}

    out = {
        "metric": "LUT-MAC/s fwd+bwd (ResNet-18 conv shapes, 7-bit)" if headline else "LUT-MAC/s fwd+bwd (VGG-16 conv shapes, 8-bit)",
        "value": rate, "unit": "LUT-MAC/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 codes; u16 table -> int32 sums (fwd); i16 table x f32 -> f32 sums (bwd)",
        "data": "synthetic",
        "config": {"workload": ("subset: " + args.only) if not full else
                   "resnet18_cifar_b256_7bit_lutgemm_fwd_bwd (BASELINE.json configs[2]: 20 conv + 1 fc GEMMs)" if headline else
                   "vgg16_cifar_b128_8bit_lutgemm_fwd_bwd (BASELINE.json configs[3]: 13 conv + 1 fc GEMMs)",
                   "batch": BATCH, "lut_macs_per_step": macs_step, "codes": "uniform random" if args.codes == "uniform" else "captured from one forward pass of the network (N(0,1) images, random-init weights, min/max quantisation)", "grad_tables": (f"float32 unrounded difference slopes, half window {HALF_WS}" if f32_tables else f"int16 x16 difference-based, half window {HALF_WS}")},
        "images_per_s": BATCH * args.steps / dt,
        # gather-equivalent: one table entry per LUT-MAC against the direct-gather peak; the expanded-table kernels read 8
        # entries per LDS instruction, so this figure can pass 1 -- `roofline.own_bound.step.frac` is the one that cannot
        "frac_of_lds_gather_roofline": rate / LDS_GATHER_PEAK,
        "kernel_ms_per_step": {k: round(v, 4) for k, v in kernels.items()},
        # not part of `value`: the forward pass when the weights do not change between calls and the table expansions stay in
        # an amr_fwd_cache per layer (inference, evaluation); the headline step expands for every call, as training must
        "forward_ms_per_step_frozen_weights": round(fwd_frozen_ms, 4),
        # The contract's roofline of this path: one LDS gather per LUT-MAC, 32 conflict-free lanes per clock and CU.  It is the
        # ceiling of the direct-gather formulation (the reference's), not of the hardware: the expanded-table kernels get 4 or
        # 8 multiply-adds out of one 64- or 128-bit LDS read, so a kernel can pass it; `kernel_bounds` below holds the limits
        # that do bound those kernels (LDS read bandwidth, VALU issue).
        "roofline": {"bound": "lds", "kernel": dominant, "achieved": dom_rate / 1e9, "peak": LDS_GATHER_PEAK / 1e9,
                     "unit": "Ggather/s", "frac": dom_rate / LDS_GATHER_PEAK,
                     "definition": "gather-equivalent rate (one table entry per LUT-MAC) against the direct-gather LDS peak, 256 CU x 2.4 GHz x 32 lanes/clk",
                     # bytes the L2s fetched + wrote for the conv2_x launch of that kernel (rocprofv3 FETCH_SIZE / WRITE_SIZE scaled
                     # against plain copies), read from the committed table profiles/conv2x_hbm_traffic.md
                     "traffic": conv2x_counters(dominant)[0] if headline and not f32_tables else None,
                     "traffic_source": "committed profile profiles/conv2x_hbm_traffic.md (rocprofv3 --pmc, not measured in this run)",
                     "traffic_launch": "conv2_x (M=262144,K=576,N=64)", "traffic_algorithmic": hbm_bytes(dominant, 262144, 576, 64),
                     "own_bound": own,
                     "avg_launch_ms": dom_ms / launches,
                     "hbm": {"achieved": dom_bytes / (dom_ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                             "frac": dom_bytes / (dom_ms * 1e-3) / HBM_PEAK},
                     "lds_probe_gathers_per_s": {"conflict_free": probe_free, "uniform_row_256B": probe_row},
                     "lds_direct_chunk_delivery_probe_GBps": probe_delivery / 1e9},
        "single_gemm": {"workload": f"M=4096 K=576 N=64 fwd+bwd, {BITS}-bit (BASELINE.json configs[1] shape)", "us": t_single * 1e3,
                        "lut_mac_per_s": 3 * M1 * K1 * N1 / (t_single * 1e-3),
                        "frac_of_lds_gather_roofline": 3 * M1 * K1 * N1 / (t_single * 1e-3) / LDS_GATHER_PEAK},
    }

    # Limits that bound the expanded-table kernels, for the conv2_x launch of each phase (the launch the committed counter
    # tables cover): bytes the kernel reads from LDS (2 per multiply-add: the table entry) against the LDS read bandwidth, and
    # VALU instructions (counted by the profiler) against the VALU issue rate.
    conv2x = [l for l in per_layer if l[0] == "conv2_x"]
    if headline and not f32_tables and conv2x:
        _, _, M2, K2, N2, *times = conv2x[0]
        kb = {"launch": f"conv2_x (M={M2},K={K2},N={N2})", "lds_read_peak_GBps": LDS_READ_PEAK / 1e9, "valu_issue_peak_Gops": VALU_ISSUE_PEAK / 1e9}
        for kind, ms in zip(("forward", "gradA", "gradB"), times):
            mac_rate = M2 * K2 * N2 / (ms * 1e-3)
            traffic, valu_per_mac = conv2x_counters(kind)
            entry = {"kernel": CONV2X_KERNEL[kind], "ms": round(ms, 4), "lut_mac_per_s": mac_rate,
                     "lds_read": {"achieved_GBps": 2 * mac_rate / 1e9, "frac": 2 * mac_rate / LDS_READ_PEAK},
                     "gather_equivalent_vs_direct_gather_peak": mac_rate / LDS_GATHER_PEAK,
                     "l2_traffic_bytes": traffic, "algorithmic_bytes": hbm_bytes(kind, M2, K2, N2)}
            # bytes the kernel has delivered from the L2 straight into LDS (expanded-table chunks of 32 KB per 4 k x 32 columns and
            # block of rows, plus the rows of gC / the codes of A that take the same road) against the rate the probe measures for
            # such loads alone; gradB streams its operands through registers instead
            if kind == "forward":
                direct_bytes = ((M2 + 1023) // 1024) * ((N2 + 31) // 32) * (K2 // 4) * 32768 + M2 * K2 * ((N2 + 31) // 32)
            elif kind == "gradA":
                direct_bytes = ((M2 + 511) // 512) * (N2 // 32) * (K2 // 4) * 32768 + ((M2 + 511) // 512) * (K2 // 32) * 512 * N2 * 4
            else:
                direct_bytes = 0
            if direct_bytes:
                entry["lds_direct_delivery"] = {"achieved_GBps": direct_bytes / (ms * 1e-3) / 1e9, "probe_GBps": probe_delivery / 1e9,
                                                "frac": direct_bytes / (ms * 1e-3) / probe_delivery}
            entry["l2_traffic_source"] = "committed profile profiles/conv2x_hbm_traffic.md"
            if valu_per_mac is not None:
                # utilisation of the issue slots by the instructions the kernel executes (counted: committed profile), not a
                # fraction of an algorithmic bound -- that is roofline.own_bound
                entry["valu_issue"] = {"valu_per_mac": round(valu_per_mac, 3), "frac": mac_rate * valu_per_mac / VALU_ISSUE_PEAK,
                                       "source": "committed profile profiles/conv2x_lds_counters.md"}
                entry["bounded_by"] = "valu_issue" if entry["valu_issue"]["frac"] > entry["lds_read"]["frac"] else "lds_read"
            kb[kind] = entry
        out["kernel_bounds"] = kb

    # The 8-bit configuration (BASELINE.json configs[3]) as a secondary record, outside the headline's timed region
    if headline and full and not args.no_8bit and not f32_tables and args.codes == "uniform":
        del bufs, ws
        torch.cuda.empty_cache()
        out["vgg16_b128_8bit"] = eight_bit_step(torch, np, dev, lib, O, stream, float_tables=False)
        torch.cuda.empty_cache()
        out["vgg16_b128_8bit_f32tab"] = eight_bit_step(torch, np, dev, lib, O, stream, float_tables=True)
        torch.cuda.empty_cache()

    # The full training step (BASELINE.json configs[4]): ResNet-18, batch 512, SGD, outside the headline's timed region
    if headline and full and not args.no_train_step and args.codes == "uniform":
        out["train_step"] = training_step(torch, dev, (lut, lga, lgb), BITS)

    # CPU baseline: the C oracle (port of the reference formulation) on the host cores ----------------------
    if not args.no_cpu:
        A, B, _, g = O.synth_gemm(M1, K1, N1, bits=BITS, err=ERR, seed=0)
        f16, a16, b16, _ = synth_tables(np, BITS, ERR, HALF_WS)
        O.forward_c(A, B, f16, BITS)
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0:
            O.forward_c(A, B, f16, BITS)
            O.backward_c_f32(g, A, B, a16, b16, BITS)
            reps += 1
        el = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": reps * 3 * M1 * K1 * N1 / el, "unit": "LUT-MAC/s", "cores": O.c_lib().oracle_num_threads(),
                               "kind": "port", "sample": f"{reps} x (M=4096,K=576,N=64 forward+backward), C/OpenMP restatement of the reference loops"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
