"""The training step the quantized linears run under: the caller-side loop of the reference, without its logging,
evaluation, checkpointing and data pipeline.

What is kept, because it fixes how the hot path is driven (src/optim/base.py:188-207, src/main.py:63-150,
src/models/base.py:313-360 of the reference):
  * every micro-step runs the forward pass *and* ``loss.backward()`` under bf16 autocast (the backward-side
    quantizers rely on it: gradients reach them in bf16 and their rotations run in bf16), with the loss divided by
    the number of accumulation steps;
  * the weights of a step are constant across its micro-steps (so each quantized linear quantizes its weight once per
    iteration, not once per micro-step): ``opt.step()`` comes after the last of them, preceded
    by gradient-norm clipping (``grad_clip``, 0 disables it) and followed by ``scheduler.step()`` and
    ``zero_grad(set_to_none=True)``;
  * AdamW (or SGD with momentum 0.9) over two parameter groups: weight decay on the weights of every linear layer
    (``QuantizedLinear`` included) except ``lm_head``, none on biases, norm gains, embeddings and ``lm_head``;
  * schedules: "cos" / "linear" = ``OneCycleLR`` from lr/100 up to lr over ``warmup_steps`` and down to lr/10,
    "cos_inf" and "wsd" (linear decay) as multiplicative ``LambdaLR`` schedules, "none".
"""
import contextlib
import math
import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch
import torch.nn as nn


@dataclass
class TrainConfig:
    """Defaults of the reference's command line (src/config/base.py:49-77)."""
    iterations: int = 15000
    warmup_steps: int = 300
    lr: float = 1e-3
    scheduler: str = "cos"
    cos_inf_steps: int = 0
    wsd_final_lr_scale: float = 0.0
    wsd_fract_decay: float = 0.1
    opt: str = "adamw"
    acc_steps: int = 4
    weight_decay: float = 0.1
    beta1: float = 0.9
    beta2: float = 0.95
    grad_clip: float = 1.0
    dtype: torch.dtype = torch.bfloat16
    log_interval: int = 0


@dataclass
class TrainStats:
    loss: List[float] = field(default_factory=list)        # mean loss of each iteration's micro-steps
    lr: List[float] = field(default_factory=list)          # learning rate the iteration's update used
    grad_norm: List[float] = field(default_factory=list)   # norm before clipping (nan when clipping is off)
    seconds: List[float] = field(default_factory=list)     # wall time per iteration


def parameter_groups(model: nn.Module) -> List[Dict]:
    """[decayed, not decayed] parameter groups, each sorted by parameter name."""
    decay, no_decay = {}, {}
    for mname, module in model.named_modules():
        for pname, p in module.named_parameters(recurse=False):
            full = f"{mname}.{pname}" if mname else pname
            if pname.endswith("weight") and isinstance(module, nn.Linear) and full != "lm_head.weight":
                decay[full] = p
            else:
                no_decay[full] = p
    named = dict(model.named_parameters())
    missing = set(named) - set(decay) - set(no_decay)
    assert not missing and not (set(decay) & set(no_decay)), f"parameters not placed in exactly one group: {missing}"
    # a tied parameter is reported once by named_parameters(); keep the first name only
    seen, groups = set(), []
    for bucket, extra in ((decay, {}), (no_decay, {"weight_decay": 0.0})):
        params = []
        for name in sorted(bucket):
            if id(bucket[name]) not in seen:
                seen.add(id(bucket[name]))
                params.append(bucket[name])
        groups.append({"params": params, **extra})
    return groups


def build_optimizer(model: nn.Module, cfg: TrainConfig) -> torch.optim.Optimizer:
    groups = parameter_groups(model)
    if cfg.opt == "adamw":
        return torch.optim.AdamW(groups, lr=cfg.lr, betas=(cfg.beta1, cfg.beta2), weight_decay=cfg.weight_decay)
    if cfg.opt == "sgd":
        return torch.optim.SGD(groups, lr=cfg.lr, momentum=0.9, weight_decay=cfg.weight_decay)
    raise ValueError(f"unknown optimizer {cfg.opt!r} (adamw, sgd)")


def cos_inf_schedule(n_iterations, n_warmup, div_factor, final_div_factor, n_inf) -> Callable[[int], float]:
    """Linear warm-up from 1/div_factor, cosine down to 1/(div_factor final_div_factor) over the steps before the
    last n_inf, constant afterwards (src/optim/utils.py:26-54)."""
    final = 1.0 / div_factor / final_div_factor
    n_anneal = n_iterations - n_inf

    def schedule(step):
        if step < n_warmup:
            return step / n_warmup + (1 - step / n_warmup) / div_factor
        if step < n_anneal:
            t = (step - n_warmup) / (n_anneal - n_warmup)
            return final + 0.5 * (1.0 - final) * (1 + math.cos(math.pi * t))
        return final
    return schedule


def wsd_schedule(n_iterations, final_lr_factor, n_warmup, init_div_factor, fract_decay) -> Callable[[int], float]:
    """Warm-up, hold at 1, then linear decay to final_lr_factor over the last fract_decay of the run
    (src/optim/utils.py:57-96, decay_type "linear")."""
    n_anneal = int(fract_decay * n_iterations)
    n_hold = n_iterations - n_anneal

    def schedule(step):
        if step < n_warmup:
            return step / n_warmup + (1 - step / n_warmup) / init_div_factor
        if step < n_hold:
            return 1.0
        if step < n_iterations:
            return final_lr_factor + (1 - final_lr_factor) * (1 - (step - n_hold) / n_anneal)
        return final_lr_factor
    return schedule


def build_scheduler(opt: torch.optim.Optimizer, cfg: TrainConfig):
    if cfg.scheduler == "none":
        return None
    if cfg.warmup_steps >= cfg.iterations:
        raise ValueError("warmup_steps must be smaller than iterations")
    if cfg.scheduler in ("cos", "linear"):
        return torch.optim.lr_scheduler.OneCycleLR(
            optimizer=opt, max_lr=[g.get("lr", cfg.lr) for g in opt.param_groups], total_steps=cfg.iterations,
            pct_start=cfg.warmup_steps / cfg.iterations, anneal_strategy=cfg.scheduler, cycle_momentum=False,
            div_factor=1e2, final_div_factor=0.1)
    if cfg.scheduler == "cos_inf":
        return torch.optim.lr_scheduler.LambdaLR(opt, cos_inf_schedule(cfg.iterations, cfg.warmup_steps, 1e2, 0.1, cfg.cos_inf_steps))
    if cfg.scheduler == "wsd":
        return torch.optim.lr_scheduler.LambdaLR(opt, wsd_schedule(cfg.iterations, cfg.wsd_final_lr_scale, cfg.warmup_steps, 1e2,
                                                                   cfg.wsd_fract_decay))
    raise ValueError(f"unknown scheduler {cfg.scheduler!r} (cos, linear, cos_inf, wsd, none)")


def train(model: nn.Module, get_batch: Callable[[], Tuple[torch.Tensor, torch.Tensor]], cfg: TrainConfig,
          opt: Optional[torch.optim.Optimizer] = None, scheduler=None,
          on_iteration: Optional[Callable[[int, TrainStats], None]] = None) -> TrainStats:
    """Run cfg.iterations optimizer steps of cfg.acc_steps micro-steps each.  ``get_batch()`` returns token ids and
    targets on the model's device; the model returns ``{"loss": ...}`` as ``quartet_amd.llama.Llama`` does."""
    device_type = next(model.parameters()).device.type
    opt = build_optimizer(model, cfg) if opt is None else opt
    scheduler = build_scheduler(opt, cfg) if scheduler is None else scheduler
    # fp32 "autocast" is no autocast at all
    autocast = (contextlib.nullcontext if cfg.dtype == torch.float32
                else lambda: torch.autocast(device_type=device_type, dtype=cfg.dtype))
    stats = TrainStats()
    model.train()
    if cfg.acc_steps > 1:
        # Q(W) is the same for every micro-step of an iteration: quantize it once per iteration
        from .linear import enable_packed_weight_cache
        enable_packed_weight_cache(model)
    from .linear import invalidate_packed_weights
    for it in range(cfg.iterations):
        t0 = time.perf_counter()
        total = 0.0
        for _ in range(cfg.acc_steps):
            x, y = get_batch()
            with autocast():
                loss = model(x, targets=y)["loss"] / cfg.acc_steps
            with autocast():
                loss.backward()
            total += float(loss.detach())
        norm = float("nan")
        if cfg.grad_clip != 0.0:
            norm = float(torch.nn.utils.clip_grad_norm_(model.parameters(), cfg.grad_clip))
        stats.lr.append(opt.param_groups[0]["lr"])
        opt.step()
        invalidate_packed_weights(model)
        if scheduler is not None:
            scheduler.step()
        opt.zero_grad(set_to_none=True)
        stats.loss.append(total)
        stats.grad_norm.append(norm)
        stats.seconds.append(time.perf_counter() - t0)
        if cfg.log_interval and (it + 1) % cfg.log_interval == 0:
            print(f"Train: Iter={it + 1} train_loss={total:.3f} iter_dt={stats.seconds[-1]:.2e}s lr={stats.lr[-1]:.2e}", flush=True)
        if on_iteration is not None:
            on_iteration(it, stats)
    return stats


def synthetic_batches(vocab_size: int, batch: int, seq_len: int, device, seed: int = 0):
    """Endless stream of (ids, targets) with structure a model can learn without a dataset: each sequence is an
    arithmetic progression modulo the vocabulary with a random start and a stride drawn from {1, 2, 3}; targets are
    the ids shifted by one."""
    g = torch.Generator().manual_seed(seed)

    def get_batch():
        start = torch.randint(0, vocab_size, (batch, 1), generator=g)
        stride = torch.randint(1, 4, (batch, 1), generator=g)
        seq = (start + stride * torch.arange(seq_len + 1)[None, :]) % vocab_size
        return seq[:, :-1].contiguous().to(device), seq[:, 1:].contiguous().to(device)
    return get_batch
