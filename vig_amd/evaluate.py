"""Evaluation-side callers of the ViG shell: checkpoint loading, top-k accuracy, validation and throughput loops.

Own code with the behaviour of classification/main.py:341-406 (validate, throughput) and of timm's `accuracy`
as used there; one process, one GPU (no reduce over ranks).  Forward only.
"""
from __future__ import annotations

import time
from typing import Iterable, Optional, Tuple

import torch
import torch.nn.functional as F

from .layers import invalidate_caches, resize_pos_embed


def load_checkpoint(model: torch.nn.Module, path: str, strict: bool = True, use_ema: bool = False):
    """Loads a reference checkpoint or a bare state_dict.  The reference keeps the weights under 'model' and, when it
    trained with an EMA copy, that copy's weights under 'model_ema' (classification/utils/utils.py:84-103);
    `use_ema=True` takes the EMA weights the way load_pretrained_ema fills its EMA model (utils.py:70-79: 'model_ema'
    if the file has it, else 'model').  Tensors only (`weights_only=True`): the reference's full training checkpoints
    also pickle their config object, which this loader refuses -- load their 'best' files (weights only, utils.py:85-86)
    or re-save the weights.  A position table of another grid is resized bicubically
    (classification/models/vig.py:915-958) when the model knows its patch grid.  The fp32 / stacked weight copies the
    layers keep are dropped, so the next forward reads the new values."""
    blob = torch.load(path, map_location="cpu", weights_only=True)
    state = blob
    if isinstance(blob, dict):
        key = "model_ema" if (use_ema and isinstance(blob.get("model_ema"), dict)) else "model"
        if isinstance(blob.get(key), dict):
            state = blob[key]
        elif use_ema and "model" not in blob and "model_ema" not in blob:
            state = blob  # a bare state_dict has no EMA copy to prefer
    state = dict(state)
    # timm's ModelEma wraps a deep copy of the model: same keys; a DataParallel-trained copy carries a 'module.' prefix
    if state and all(k.startswith("module.") for k in state):
        state = {k[len("module."):]: v for k, v in state.items()}
    own = model.state_dict()
    if "pos_embed" in state and "pos_embed" in own and state["pos_embed"].shape != own["pos_embed"].shape:
        n_src = state["pos_embed"].shape[1]
        side = int(round(n_src ** 0.5))
        if side * side != n_src or not hasattr(model, "patch_resolution"):
            raise ValueError("cannot resize pos_embed: source grid is not square or the model has no patch_resolution")
        state["pos_embed"] = resize_pos_embed(state["pos_embed"], (side, side), tuple(model.patch_resolution))
    res = model.load_state_dict(state, strict=strict)
    invalidate_caches(model)
    return res


def accuracy(output: torch.Tensor, target: torch.Tensor, topk: Tuple[int, ...] = (1,)):
    """Top-k accuracies in percent over a batch of logits."""
    maxk = min(max(topk), output.shape[1])
    _, pred = output.topk(maxk, dim=1, largest=True, sorted=True)
    correct = pred.eq(target.reshape(-1, 1))
    n = target.shape[0]
    return [correct[:, :min(k, maxk)].any(dim=1).float().sum() * (100.0 / n) for k in topk]


@torch.no_grad()
def validate(model: torch.nn.Module, data_loader: Iterable, dtype: torch.dtype = torch.bfloat16):
    """Weighted averages of top-1, top-5 and cross-entropy over a loader of (images, target) batches
    (classification/main.py:341-385).  Images are cast to `dtype`; the loss is taken on fp32 logits."""
    model.eval()
    dev = next(model.parameters()).device
    n_total, acc1_sum, acc5_sum, loss_sum = 0, 0.0, 0.0, 0.0
    for images, target in data_loader:
        images = images.to(dev, dtype, non_blocking=True)
        target = target.to(dev, non_blocking=True)
        logits = model(images).float()
        a1, a5 = accuracy(logits, target, topk=(1, 5))
        n = target.shape[0]
        n_total += n
        acc1_sum += a1.item() * n
        acc5_sum += a5.item() * n
        loss_sum += F.cross_entropy(logits, target).item() * n
    if n_total == 0:
        raise ValueError("empty data loader")
    return acc1_sum / n_total, acc5_sum / n_total, loss_sum / n_total


class GraphedForward:
    """One eval forward of `model` on a fixed input shape, captured as a HIP graph and replayed: the ~190 kernel
    launches of a ViG-S forward become one submission.  Everything the forward launches is a plain kernel on the
    current stream (this library's entry points allocate nothing and never synchronise), so it captures as is; the
    GEMM solution tuning, if on, has to have seen the shapes before (the warm-up forwards below do that)."""

    def __init__(self, model: torch.nn.Module, example: torch.Tensor, warmup: int = 3):
        self.model = model.eval()
        self.static_in = example.clone()
        side = torch.cuda.Stream(device=example.device)  # (default priority)
        side.wait_stream(torch.cuda.current_stream(example.device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                self.model(self.static_in)
        torch.cuda.current_stream(example.device).wait_stream(side)
        torch.cuda.synchronize(example.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self.static_out = self.model(self.static_in)

    def eval(self):
        return self

    def __call__(self, images: torch.Tensor) -> torch.Tensor:
        if images.data_ptr() != self.static_in.data_ptr():
            self.static_in.copy_(images)
        self.graph.replay()
        return self.static_out


def graphed_forward_checked(model: torch.nn.Module, images: torch.Tensor, replays: int = 4) -> Optional[GraphedForward]:
    """A GraphedForward that reproduced the eager logits bit for bit on `replays` replays with eager forwards and
    synchronisations in between, or None (capture refused, or a replay differed: a library call inside the forward
    may record nodes that do not replay faithfully)."""
    try:
        with torch.no_grad():
            want = model(images).clone()
        g = GraphedForward(model, images)
        for i in range(replays):
            got = g(images).clone()
            torch.cuda.synchronize(images.device)
            if not torch.equal(got, want):
                return None
            with torch.no_grad():
                model(images + float(i + 1))  # eager work on other data between the replays
            torch.cuda.synchronize(images.device)
        return g
    except Exception:  # noqa: BLE001 - capture is an optimisation; the eager forward is always there
        return None


def throughput(model: torch.nn.Module, images: torch.Tensor, warmup: int = 50, iters: int = 30) -> float:
    """Images per second of repeated forwards of one resident batch: `warmup` untimed and `iters` timed forwards
    between synchronisations (classification/main.py:388-406)."""
    model.eval()
    for _ in range(warmup):
        model(images)
    torch.cuda.synchronize(images.device)
    t0 = time.perf_counter()
    for _ in range(iters):
        model(images)
    torch.cuda.synchronize(images.device)
    return iters * images.shape[0] / (time.perf_counter() - t0)
