"""Training / validation driver with the command line of the reference's main_conv.py
(main_conv.py:23-44): the same flags and defaults, the same per-layer digit strings for
--err / --z_unit / --load_unit / --load_wait, the same model choice (--size 0: 4-layer CNN,
--size 1: VGG-16), optimiser, scheduler and checkpoint handling (``torch.save(net.state_dict())``
of the best epoch; ``--val 1`` loads it with ``strict=False``).

Datasets: CIFAR10 / SVHN through torchvision when that package and the data are available
(nothing is downloaded); ``--dataset SYNTHETIC`` (not in the reference) draws a fixed set of
random 3x32x32 images and labels, for smoke runs and timing where no dataset exists.  MNIST /
the LeNet model are not offered (that model is unfinished in the reference, network.py:204-206).
``--epochs`` and ``--iterations`` (not in the reference, which always runs 1000 epochs) bound a run.

    python -m geo_amd.main_conv --dataset SYNTHETIC --err 6666 --epochs 1 --iterations 4 --monitor 1
"""
from __future__ import annotations

import argparse
import os

import numpy as np
import torch
import torch.nn as nn
import torch.optim as optim

from . import network, utils_own


def build_parser():
    p = argparse.ArgumentParser(description="SC CNN training on MI355X (command line of the reference's main_conv.py)")
    p.add_argument("--save_dir", default="./training_data_sc/cifar_mid/", type=str)
    p.add_argument("--dataset", default="CIFAR10", type=str, help="CIFAR10, SVHN or SYNTHETIC")
    p.add_argument("--seed", default=0, type=int)
    p.add_argument("--device", default=0, type=int, help="GPU id (this build has no CPU path: -1 is refused)")
    p.add_argument("--optim", default="Adam", type=str, help="Adam, RMSprop or SGD")
    p.add_argument("--lr", default=2e-3, type=float)
    p.add_argument("--err", default="7777", type=str, help="stream length per layer as 2**digit")
    p.add_argument("--z_unit", default="3344", type=str, help="channels per OR group per layer as 2**digit (yz_bin)")
    p.add_argument("--load_unit", default="2222", type=str)
    p.add_argument("--load_wait", default="2222", type=str)
    p.add_argument("-b", "--batch", default=256, type=int)
    p.add_argument("--size", default=0, type=int, help="0: 4-layer CNN, 1: VGG-16")
    p.add_argument("--prec", default="7777", type=str)
    p.add_argument("--val", default=0, type=int, help="1: evaluate the saved model")
    p.add_argument("--uniform", default=0, type=int)
    p.add_argument("--generator", default="lfsr", type=str, help="lfsr, acc or rand")
    p.add_argument("--compute", default="1d_bin", type=str, help="1d_bin, z_bin, yz_bin or full_or")
    p.add_argument("--legacy", default=0, type=int)
    p.add_argument("--monitor", default=0, type=int)
    p.add_argument("--relu", default=0, type=int)
    p.add_argument("--epochs", default=1000, type=int)
    p.add_argument("--iterations", default=None, type=int, help="batches per epoch (default: all)")
    p.add_argument("--synthetic_size", default=2048, type=int, help="images in the SYNTHETIC set")
    p.add_argument("--fused", default=1, type=int,
                   help="1: conv + batch norm + pool + hardtanh blocks as fused autograd nodes in training (same "
                        "values as the module chain); 0: module by module")
    return p


def _loaders(args):
    b = args.batch
    if args.dataset == "SYNTHETIC":
        g = torch.Generator().manual_seed(args.seed)
        n = args.synthetic_size
        train = torch.utils.data.TensorDataset(torch.rand((n, 3, 32, 32), generator=g),
                                               torch.randint(10, (n,), generator=g))
        test = torch.utils.data.TensorDataset(torch.rand((n // 4, 3, 32, 32), generator=g),
                                              torch.randint(10, (n // 4,), generator=g))
        return (torch.utils.data.DataLoader(train, batch_size=b, shuffle=True),
                torch.utils.data.DataLoader(test, batch_size=b, shuffle=False))
    try:
        import torchvision
        import torchvision.transforms as transforms
    except ImportError as e:
        raise SystemExit(f"--dataset {args.dataset} needs torchvision, which is not installed here ({e}); "
                         "use --dataset SYNTHETIC") from e
    aug = transforms.Compose([transforms.RandomCrop(32, 4), transforms.RandomHorizontalFlip(), transforms.ToTensor()])
    if args.dataset == "CIFAR10":
        trainset = torchvision.datasets.CIFAR10(root="../data", train=True, download=False, transform=aug)
        testset = torchvision.datasets.CIFAR10(root="../data", train=False, download=False,
                                               transform=transforms.ToTensor())
    elif args.dataset == "SVHN":
        trainset = torchvision.datasets.SVHN(root="../data", split="train", download=False, transform=aug)
        testset = torchvision.datasets.SVHN(root="../data", split="test", download=False,
                                            transform=transforms.ToTensor())
    else:
        raise SystemExit(f"unknown dataset {args.dataset!r}: CIFAR10, SVHN or SYNTHETIC")
    return (torch.utils.data.DataLoader(trainset, batch_size=b, shuffle=True, num_workers=2),
            torch.utils.data.DataLoader(testset, batch_size=b, shuffle=False, num_workers=2))


def build_model(args):
    """Model and per-layer settings from the digit strings (main_conv.py:62-76, :113-122, :167-176)."""
    digits = lambda s: [int(c) for c in s]
    flags = dict(uniform=args.uniform == 1, sc_compute=args.compute, generator=args.generator,
                 legacy=args.legacy == 1)
    if args.size == 0:
        net, layers = network.CONV_tiny_add_partial(relu=args.relu == 1, **flags), 4
    elif args.size == 1:
        net, layers = network.VGG16_add_partial(**flags), 6
    else:
        raise SystemExit("--size must be 0 (4-layer CNN) or 1 (VGG-16)")
    for name in ("err", "z_unit", "load_unit", "load_wait"):
        if len(getattr(args, name)) != layers:
            raise SystemExit(f"Mismatch: --{name} needs {layers} digits for this model, got {getattr(args, name)!r}")
    net.prec = digits(args.prec)
    net.err = digits(args.err)
    net.z_unit = digits(args.z_unit)
    net.load_unit = digits(args.load_unit)
    net.load_wait = digits(args.load_wait)
    net.fused_blocks = args.fused == 1
    return net


def main(argv=None):
    args = build_parser().parse_args(argv)
    torch.manual_seed(args.seed)
    np.random.seed(args.seed)
    if args.device < 0 or not torch.cuda.is_available():
        raise SystemExit("this build runs the SC layers on the GPU only (no CPU code path): --device must be >= 0 "
                         "and a GPU must be visible")
    trainloader, testloader = _loaders(args)
    net = build_model(args).cuda(args.device)
    save_dir = os.path.join("../", args.save_dir)
    os.makedirs(save_dir, exist_ok=True)
    save_file = os.path.join(save_dir, "CONV_small.pt")
    criterion = nn.CrossEntropyLoss()
    if args.val == 1:
        net.load_state_dict(torch.load(save_file, map_location="cpu", weights_only=True), strict=False)
        net.eval()
        loss, p1, p5 = utils_own.validate(testloader, net, criterion, 0, verbal=True, monitor=args.monitor == 1,
                                          iteration=args.iterations)
        return dict(val_loss=loss, val_prec1=p1, val_prec5=p5)
    if os.path.exists(save_file):
        print("Save file already exists. Delete manually if want to overwrite")
        return None
    param_copy = [p.clone().cuda(args.device).float().detach().requires_grad_(True) for p in net.parameters()]
    if args.optim == "Adam":
        optimizer = optim.Adam(param_copy, lr=args.lr, weight_decay=0)
    elif args.optim == "RMSprop":
        optimizer = optim.RMSprop(param_copy, lr=args.lr, weight_decay=0)
    elif args.optim == "SGD":
        optimizer = optim.SGD(param_copy, lr=args.lr, weight_decay=0, momentum=0.01)
    else:
        raise SystemExit(f"unknown optimiser {args.optim!r}: Adam, RMSprop or SGD")
    scheduler = optim.lr_scheduler.ReduceLROnPlateau(optimizer=optimizer, factor=0.3, patience=150, threshold=0.05)
    best = -1.0
    history = []
    for epoch in range(args.epochs):
        tr = utils_own.train(trainloader, net, criterion, epoch, optimizer, param_copy=param_copy, modules=net,
                             monitor=args.monitor == 1, iteration=args.iterations)
        va = utils_own.validate(testloader, net, criterion, epoch, verbal=True, monitor=args.monitor == 1,
                                iteration=args.iterations)
        history.append(dict(epoch=epoch, train_loss=tr[0], train_prec1=tr[1], val_loss=va[0], val_prec1=va[1]))
        if va[1] > best:
            best = va[1]
            torch.save(net.state_dict(), save_file)
            print(f"\n Epoch: {epoch + 1}\tTraining Prec {tr[1]:.3f} \tBinary Prec {va[1]:.3f}")
        scheduler.step(va[0])
    print("\nTraining finished!")
    return dict(history=history, save_file=save_file)


if __name__ == "__main__":
    main()
