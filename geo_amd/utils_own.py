"""Training / validation loops with the reference's interface (utils_own.py): scaled loss,
full-precision master copies, ``weight_org`` refresh; ``AverageMeter`` and ``accuracy`` from the
reference's utils.py:86-160 (the logging / plotting helpers of that file need pandas and bokeh
and are not part of this build)."""
from __future__ import annotations

import time

import torch
import torch.nn as nn

# loss scale (utils_own.py:14)
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


def set_grad(params, params_with_grad):
    """Hand the model's gradients to the master copies (utils_own.py:19-24)."""
    for param, src in zip(params, params_with_grad):
        if param.grad is None:
            param.grad = torch.zeros_like(param.data)
        if src.grad is not None:
            param.grad.data.copy_(src.grad.data)


def forward(data_loader, model, criterion, epoch=0, training=True, optimizer=None, verbal=False, iteration=None,
            param_copy=None, modules=None, use_target=False, monitor=False):
    """One pass over ``data_loader`` (utils_own.py:31-140).  Training: loss * 128, backward,
    restore the full-precision weights, gradients to the master copies and / 128, optimiser step,
    copy back, ``weight_org = weight.clamp(-1, 0.999)``; the step is taken once at least 128
    samples have been accumulated.  Returns (average scaled loss, prec@1, prec@5)."""
    losses, top1, top5, batch_time = AverageMeter(), AverageMeter(), AverageMeter(), AverageMeter()
    end = time.time()
    acc = 0
    if modules is None:
        modules = model
    ref = model.module.fc1.weight if isinstance(model, nn.DataParallel) else model.fc1.weight
    for i, (inputs, target) in enumerate(data_loader):
        if iteration is not None and i >= iteration:
            break
        target = target.to(ref.device, non_blocking=True)
        input_var = inputs.to(dtype=ref.dtype).to(ref.device, non_blocking=True)
        output = model(input_var, target) if use_target else model(input_var)
        loss = criterion(output, target) * scale_factor
        prec1, prec5 = accuracy(output.data, target, topk=(1, 5))
        losses.update(loss.item(), inputs.size(0))
        top1.update(prec1.item(), inputs.size(0))
        top5.update(prec5.item(), inputs.size(0))
        acc += inputs.size(0)
        if training:
            for param in modules.parameters():
                param.grad = None
            loss.backward()
            if acc >= 128:
                for p in modules.modules():
                    if hasattr(p, "weight_org"):
                        p.weight.data.copy_(p.weight_org)
                set_grad(param_copy, list(modules.parameters()))
                if scale_factor != 1:
                    for param in param_copy:
                        param.grad.data = param.grad.data / scale_factor
                optimizer.step()
                for dst, src in zip(modules.parameters(), param_copy):
                    dst.data.copy_(src.data)
                for p in modules.modules():
                    if hasattr(p, "weight_org"):
                        p.weight_org.copy_(p.weight.data.clamp(-1, 0.999))
                optimizer.zero_grad()
                acc = 0
        batch_time.update(time.time() - end)
        end = time.time()
        if monitor:
            print(f"Epoch: [{epoch}][{i + 1}/{len(data_loader)}]\\tTime {batch_time.val:.3f} ({batch_time.avg:.6f})\\t"
                  f"Loss {losses.val:.4f} ({losses.avg:.4f})\\tAcc@1 {top1.val:.3f} ({top1.avg:.3f})\\t"
                  f"Acc@5 {top5.val:.3f} ({top5.avg:.3f})")
    if training:
        for p in model.modules():
            if isinstance(p, (nn.Linear, nn.Conv2d)):
                p.weight.data.clamp_(-1, 0.999)
    elif verbal:
        print(f"Epoch: [{epoch}]\\tLoss {losses.val:.4f} ({losses.avg:.4f})\\tPrec@1 {top1.val:.3f} ({top1.avg:.3f})\\t"
              f"Prec@5 {top5.val:.3f} ({top5.avg:.3f})")
    return losses.avg, top1.avg, top5.avg


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
