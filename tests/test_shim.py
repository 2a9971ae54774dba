"""The training-script shim: state_dict keys as the reference's modules name them, the command
line, and (GPU) a short run with checkpoint save / load."""
import os

import pytest
import torch

BN_KEYS = ("weight", "bias", "running_mean", "running_var", "num_batches_tracked")


def expected_keys(convs, bns):
    keys = set()
    for c in convs:
        keys |= {f"{c}.weight", f"{c}.weight_org"}
    for b in bns:
        keys |= {f"{b}.{k}" for k in BN_KEYS}
    return keys


def test_state_dict_keys_match_the_reference_attribute_names():
    """network.py:134-143 (4-layer CNN) and :21-56 (VGG-16): parameter / buffer names are the
    attribute names of the reference's modules plus Conv2d_Add_Partial's ``weight_org`` buffer
    (utils_class.py:17); BatchNorm*_fixed's ``scale`` buffer is None until the first forward."""
    from geo_amd import network
    tiny = network.CONV_tiny_add_partial()
    assert set(tiny.state_dict()) == expected_keys(["conv1", "conv2", "conv3", "fc1"], ["bn1", "bn2", "bn3", "bn4"])
    assert tiny.conv1.weight.shape == (32, 3, 5, 5) and tiny.fc1.weight.shape == (10, 64, 4, 4)
    vgg = network.VGG16_add_partial()
    convs = [f"conv{i}" for i in range(1, 14)] + ["fc1"]
    bns = [f"bn{i}" for i in range(1, 14)] + ["bnfc1"]
    assert set(vgg.state_dict()) == expected_keys(convs, bns)
    shapes = {1: (64, 3), 2: (64, 64), 3: (128, 64), 5: (256, 128), 8: (512, 256), 13: (512, 512)}
    for i, (co, ci) in shapes.items():
        assert getattr(vgg, f"conv{i}").weight.shape == (co, ci, 3, 3)
    assert vgg.fc1.weight.shape == (10, 512, 1, 1)


def test_command_line_defaults_and_digit_strings():
    from geo_amd import main_conv
    a = main_conv.build_parser().parse_args([])
    assert (a.dataset, a.err, a.z_unit, a.load_unit, a.load_wait, a.batch, a.lr, a.generator, a.compute) == \
        ("CIFAR10", "7777", "3344", "2222", "2222", 256, 2e-3, "lfsr", "1d_bin")
    a = main_conv.build_parser().parse_args(["--err", "5557", "--compute", "yz_bin", "--relu", "1"])
    net = main_conv.build_model(a)
    assert net.err == [5, 5, 5, 7] and net.z_unit == [3, 3, 4, 4] and net.compute == "yz_bin" and net.relu
    a = main_conv.build_parser().parse_args(["--size", "1", "--err", "666666", "--z_unit", "555555",
                                             "--load_unit", "222222", "--load_wait", "222222"])
    assert type(main_conv.build_model(a)).__name__ == "VGG16_add_partial"
    with pytest.raises(SystemExit):
        main_conv.build_model(main_conv.build_parser().parse_args(["--size", "1"]))  # 4 digits for 6 groups


@pytest.mark.gpu
def test_short_training_run_and_checkpoint_round_trip(tmp_path, monkeypatch):
    from geo_amd import main_conv
    monkeypatch.chdir(tmp_path)
    os.makedirs(tmp_path / "work")
    monkeypatch.chdir(tmp_path / "work")     # the script saves under ../<save_dir>
    argv = ["--dataset", "SYNTHETIC", "--err", "6666", "--batch", "64", "--synthetic_size", "256", "--epochs", "2",
            "--save_dir", "ckpt"]
    out = main_conv.main(argv)
    assert len(out["history"]) == 2 and os.path.isfile(out["save_file"])
    sd = torch.load(out["save_file"], map_location="cpu", weights_only=True)
    assert "conv1.weight_org" in sd and "bn1.scale" in sd          # scale is set by the first forward
    assert sd["conv1.weight_org"].abs().max() <= 1.0
    val = main_conv.main(argv + ["--val", "1"])
    best = max(h["val_prec1"] for h in out["history"])
    assert abs(val["val_prec1"] - best) < 1e-6                     # the saved model reproduces its score
    assert main_conv.main(argv) is None                            # refuses to overwrite


@pytest.mark.gpu
def test_vgg16_forward_backward():
    from geo_amd import network
    torch.manual_seed(0)
    net = network.VGG16_add_partial().cuda()
    net.err = [6, 6, 6, 6, 6, 6]
    x = torch.rand(4, 3, 32, 32, device="cuda")
    y = net(x)
    assert y.shape == (4, 10) and torch.isfinite(y).all()
    y.square().mean().backward()
    for name in ("conv1", "conv7", "conv13", "fc1"):
        g = getattr(net, name).weight.grad
        assert g is not None and torch.isfinite(g).all()
    net.eval()
    with torch.no_grad():
        a, b = net(x.clone()), net(x.clone())
    assert torch.equal(a, b)


@pytest.mark.gpu
def test_vgg16_fused_blocks_match_module_chain():
    from geo_amd import network

    def run(fused):
        torch.manual_seed(0)
        net = network.VGG16_add_partial().cuda().train()
        net.err = [6, 6, 6, 6, 6, 6]
        net.fused_blocks = fused
        x = torch.rand(8, 3, 32, 32, generator=torch.Generator().manual_seed(1)).cuda()
        torch.manual_seed(5)                      # same dropout masks in both runs
        y = net(x)
        y.square().mean().backward()
        return y.detach(), {n: p.grad.clone() for n, p in net.named_parameters()}

    y_ref, g_ref = run(False)
    y_fused, g_fused = run(True)
    assert torch.equal(y_ref, y_fused)
    for name in g_ref:
        scale = g_ref[name].abs().max().item()
        if scale == 0.0:
            assert g_fused[name].abs().max().item() == 0.0, name
            continue
        assert (g_fused[name] - g_ref[name]).abs().max().item() / scale < 1e-4, name
