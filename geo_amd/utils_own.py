"""Training / validation loops with the reference's interface (utils_own.py): scaled loss,
full-precision master copies, ``weight_org`` refresh; ``AverageMeter`` and ``accuracy`` from the
reference's utils.py:86-160 (the logging / plotting helpers of that file need pandas and bokeh
and are not part of this build)."""
from __future__ import annotations

import time

import torch
import torch.nn as nn

# loss scale (utils_own.py:14); the step itself reads network.SCALE_FACTOR
scale_factor = 128.0


class AverageMeter:
    """Running value / average (utils.py:86-113)."""

    def __init__(self):
        self.reset()

    def reset(self):
        self.val = self.avg = self.sum = self.count = 0

    def update(self, val, n=1):
        self.val = val
        self.sum += val * n
        self.count += n
        self.avg = self.sum / self.count


def accuracy(output, target, topk=(1,)):
    """Precision@k in percent for each k (utils.py:142-160)."""
    maxk = max(topk)
    batch = target.size(0)
    _, pred = output.float().topk(maxk, 1, True, True)
    correct = pred.t().eq(target.view(1, -1).expand_as(pred.t()))
    return [correct[:k].reshape(-1).float().sum(0).mul_(100.0 / batch) for k in topk]


class _Progress:
    """Meters of one pass and the two line formats the loops print."""

    def __init__(self):
        self.loss, self.top1, self.top5, self.seconds = AverageMeter(), AverageMeter(), AverageMeter(), AverageMeter()
        self._tick = time.time()

    def record(self, loss, output, target, samples):
        p1, p5 = accuracy(output, target, topk=(1, 5))
        self.loss.update(float(loss), samples)
        self.top1.update(p1.item(), samples)
        self.top5.update(p5.item(), samples)
        now = time.time()
        self.seconds.update(now - self._tick)
        self._tick = now

    def batch_line(self, epoch, done, total):
        cells = [f"Epoch: [{epoch}][{done}/{total}]",
                 f"Time {self.seconds.val:.3f} ({self.seconds.avg:.6f})",
                 f"Loss {self.loss.val:.4f} ({self.loss.avg:.4f})",
                 f"Acc@1 {self.top1.val:.3f} ({self.top1.avg:.3f})",
                 f"Acc@5 {self.top5.val:.3f} ({self.top5.avg:.3f})"]
        return "\t".join(cells)

    def epoch_line(self, epoch):
        cells = [f"Epoch: [{epoch}]", f"Loss {self.loss.val:.4f} ({self.loss.avg:.4f})",
                 f"Prec@1 {self.top1.val:.3f} ({self.top1.avg:.3f})", f"Prec@5 {self.top5.val:.3f} ({self.top5.avg:.3f})"]
        return "\t".join(cells)


def forward(data_loader, model, criterion, epoch=0, training=True, optimizer=None, verbal=False, iteration=None,
            param_copy=None, modules=None, use_target=False, monitor=False):
    """One pass over ``data_loader`` with the reference's call (utils_own.py:31-140).  Training runs
    the step of ``network.apply_update`` (loss * 128, master copies, ``weight_org`` refresh) once at
    least 128 samples have been seen since the last update, on the gradients of the batch that
    completed them, as the reference does.  Returns (average scaled loss, prec@1, prec@5)."""
    from . import network

    net = model if modules is None else modules
    anchor = (model.module if isinstance(model, nn.DataParallel) else model).fc1.weight
    progress = _Progress()
    since_update = 0
    for done, (inputs, target) in enumerate(data_loader, start=1):
        if iteration is not None and done > iteration:
            break
        target = target.to(anchor.device, non_blocking=True)
        batch = inputs.to(anchor.device, anchor.dtype, non_blocking=True)
        output = model(batch, target) if use_target else model(batch)
        loss = criterion(output, target) * network.SCALE_FACTOR
        if training:
            for p in net.parameters():
                p.grad = None
            loss.backward()
            since_update += inputs.size(0)
            if since_update >= 128:
                network.apply_update(net, optimizer, param_copy)
                since_update = 0
        progress.record(loss.item(), output.detach(), target, inputs.size(0))
        if monitor:
            print(progress.batch_line(epoch, done, len(data_loader)))
    if training:
        for layer in model.modules():
            if isinstance(layer, (nn.Linear, nn.Conv2d)):
                layer.weight.data.clamp_(-1, 0.999)
    elif verbal:
        print(progress.epoch_line(epoch))
    return progress.loss.avg, progress.top1.avg, progress.top5.avg


def train(data_loader, model, criterion, epoch, optimizer, param_copy, iteration=None, modules=None, target=False,
          monitor=False):
    """utils_own.py:143-150"""
    model.train()
    optimizer.zero_grad()
    return forward(data_loader, model, criterion, epoch, training=True, optimizer=optimizer, iteration=iteration,
                   param_copy=param_copy, modules=modules, use_target=target, monitor=monitor)


def validate(data_loader, model, criterion, epoch, verbal=False, modules=None, target=False, monitor=False,
             iteration=None):
    """utils_own.py:153-161"""
    model.eval()
    with torch.no_grad():
        return forward(data_loader, model, criterion, epoch, training=False, verbal=verbal, iteration=iteration,
                       modules=modules, use_target=target, monitor=monitor)
