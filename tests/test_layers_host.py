"""CPU checks of the quantised-layer counterpart and the gradient-table generator (no LUT kernel runs)."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn


def test_gradient_table_generator_reproduces_shipped_tables(oracle, golden_dir):
    import gen_bp_lut as G
    for name, bits, hw in [("lut6_vert_trunc_bp2.txt.gz", 6, 2), ("lut7_resub_63_bp8.txt.gz", 7, 8), ("lut7_evo_081_bp16.txt.gz", 7, 16)]:
        fwd, ga, gb = oracle.parse_lut_file(os.path.join(golden_dir, name), bits)
        a16, b16 = G.gradient_tables(fwd, hw)
        assert (a16 == ga).all() and (b16 == gb).all()
    z = np.load(os.path.join(golden_dir, "lut8_resub_183.npz"))
    a16, b16 = G.gradient_tables(z["fwd"], int(z["half_window"]))
    assert (a16 == z["grad_a"]).all() and (b16 == z["grad_b"]).all()


def test_gradient_table_generator_equals_oracle_loops_on_random_table(oracle):
    import gen_bp_lut as G
    rng = np.random.default_rng(0)
    T = oracle.synth_lut(6, 40, rng)
    for hw in (1, 3, 8):
        a, b = G.gradient_tables(T, hw)
        ao, bo = oracle.gen_bp_lut(T, hw)
        assert (a == ao).all() and (b == bo).all()


def test_gradient_table_generator_float_slopes_equal_oracle_loops(oracle):
    import gen_bp_lut as G
    rng = np.random.default_rng(4)
    T = oracle.synth_lut(6, 16, rng)
    for hw in (1, 3, 8):
        a, b = G.gradient_tables(T, hw, rounded=False)
        a0, b0 = oracle.gen_bp_lut(T, hw, rounded=False)
        assert a.dtype == np.float32 and (a == a0).all() and (b == b0).all()
        a16, b16 = G.gradient_tables(T, hw)
        assert (a16 == np.round(a * np.float32(16))).all() and (b16 == np.round(b * np.float32(16))).all()


def test_generator_cli_round_trip(tmp_path, oracle, golden_dir, capsys):
    import gzip
    import gen_bp_lut as G
    src = tmp_path / "mul7u_test_lutfp.txt"     # bit-width is read off the file name, as in the reference
    text = gzip.open(os.path.join(golden_dir, "lut7_vert_trunc_fwdonly.txt.gz"), "rt").read()
    src.write_text(text)
    G.main(["-f", str(src), "-w", "2"])
    out = tmp_path / "mul7u_test_lutfp+bp_avg_2_2.txt"
    out.write_text(capsys.readouterr().out)
    fwd, ga, gb = oracle.parse_lut_file(str(out), 7)
    f0, _, _ = oracle.parse_lut_file(str(src), 7)
    a0, b0 = oracle.gen_bp_lut(f0, 2)
    assert (fwd == f0).all() and (ga == a0).all() and (gb == b0).all()


def test_observers_and_code_mapping():
    import app_layers as L
    mm, ema = L.MinMaxObserver("L", None), L.MovingAverageMinMaxObserver("L", None)
    for obs in (mm, ema):
        obs(torch.tensor([-1.0, 2.0]))
        assert float(obs.min_val) == -1.0 and float(obs.max_val) == 2.0
        obs(torch.tensor([-3.0, 1.0]))
    assert float(mm.min_val) == -3.0 and float(mm.max_val) == 2.0
    assert float(ema.min_val) == pytest.approx(0.9 * -1.0 + 0.1 * -3.0) and float(ema.max_val) == pytest.approx(0.9 * 2.0 + 0.1 * 1.0)
    x = torch.tensor([-0.5, 0.0, 0.26, 10.0], requires_grad=True)
    codes = L._to_codes(x, torch.tensor(0.1), torch.tensor(-5.0), torch.tensor(127.0))
    assert codes.tolist() == [0.0, 5.0, 8.0, 105.0]
    codes.sum().backward()
    assert x.grad.tolist() == [10.0, 10.0, 10.0, 10.0]      # straight-through: d(code)/dx = 1/scale inside the range


def test_quant_linear_and_prepare_on_cpu():
    import app_layers as L
    torch.manual_seed(0)
    net = nn.Sequential(nn.Linear(8, 6), nn.ReLU(), nn.Sequential(nn.Linear(6, 4)))
    q = L.prepare(net, inplace=False, a_bits=7, w_bits=7)
    assert isinstance(q[0], L.QuantLinear) and isinstance(q[2][0], L.QuantLinear) and isinstance(net[0], nn.Linear)
    assert q[0].weight.data_ptr() != net[0].weight.data_ptr() and torch.equal(q[0].weight, net[0].weight)
    x = torch.randn(16, 8)
    q.train()
    y = q(x)
    lin = q[0]
    s = (x.max() - x.min()) / 127
    assert float(lin.activation_scale) == pytest.approx(float(s))
    assert float(lin.activation_zp_neg) == float(torch.round(x.min() / s))
    # fake quantisation error is bounded by half a step per operand
    ref = net(x)
    assert (y - ref).abs().max() < 0.2
    y.sum().backward()
    assert lin.weight.grad is not None
    conv = L.prepare(nn.Sequential(nn.Conv2d(3, 4, 3, padding=1), nn.MaxPool2d(2), nn.AvgPool2d(2)), a_bits=7, w_bits=7)
    assert [type(m).__name__ for m in conv] == ["ApproxConv2d", "QuantMaxPool2d", "QuantAvgPool2d"]
    sd = conv.state_dict()
    assert "0.activation_scale" in sd and "0.weight_zp_neg" in sd and "1.activation_quantizer.scale" in sd


def test_benchmark_network_shapes():
    import models
    convs = [(m.in_channels * m.kernel_size[0] * m.kernel_size[1], m.out_channels) for m in models.resnet18().modules()
             if isinstance(m, nn.Conv2d)]
    assert len(convs) == 20
    assert sorted(set(convs)) == sorted({(27, 64), (576, 64), (576, 128), (1152, 128), (64, 128), (1152, 256), (2304, 256),
                                         (128, 256), (2304, 512), (4608, 512), (256, 512)})
    assert sum(isinstance(m, nn.Conv2d) for m in models.vgg16().modules()) == 13


def test_fold_relu_rewrites_only_relus_whose_reader_is_a_quantised_convolution():
    """app_layers.fold_relu on the package's networks (structure only: no kernel runs on the CPU)."""
    import app_layers as L
    import models
    net = L.prepare(models.resnet18(10), inplace=True, a_bits=7, w_bits=7)
    n_relu = sum(isinstance(m, nn.ReLU) for m in net.modules())
    assert L.fold_relu(net) == 8                                 # the ReLU between the two convolutions of each of the 8 blocks
    assert sum(isinstance(m, nn.ReLU) for m in net.modules()) == n_relu - 8
    flagged = [m for m in net.modules() if isinstance(m, L.ApproxConv2d) and m.pre_relu]
    assert len(flagged) == 8 and all(m.kernel_size == (3, 3) and m.stride == (1, 1) for m in flagged)
    for blk in (m for m in net.modules() if isinstance(m, models.BasicBlock)):
        mods = list(blk.residual_function)
        assert isinstance(mods[2], nn.Identity) and mods[3].pre_relu and not mods[0].pre_relu
    assert L.fold_relu(net) == 0                                 # nothing left to fold
    # the ReLU in front of a pooling layer stays
    seq = nn.Sequential(nn.Conv2d(3, 8, 3), nn.ReLU(), nn.MaxPool2d(2), nn.ReLU(), nn.Conv2d(8, 8, 3))
    q = L.prepare(seq, inplace=True, a_bits=7, w_bits=7)
    assert L.fold_relu(q) == 1 and isinstance(q[1], nn.ReLU) and isinstance(q[3], nn.Identity) and q[4].pre_relu
