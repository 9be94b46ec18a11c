"""CPU tests of the training step around the quantized linears: parameter groups, schedules, accumulation
semantics and that a small model learns."""
import math

import pytest
import torch
import torch.nn as nn

from quartet_amd.llama import Llama, LlamaConfig, unquantized
from quartet_amd.train import (TrainConfig, build_optimizer, build_scheduler, cos_inf_schedule, parameter_groups,
                               synthetic_batches, train, wsd_schedule)


def tiny_model(seed=0, **kw):
    torch.manual_seed(seed)
    cfg = LlamaConfig(**unquantized(vocab_size=64, sequence_length=32, n_layer=2, n_head=2, n_embd=32, multiple_of=32, **kw))
    return Llama(cfg)


def test_parameter_groups_decay_only_linear_weights():
    model = tiny_model(bias=True)
    decay, no_decay = parameter_groups(model)
    names = {id(p): n for n, p in model.named_parameters()}
    decayed = {names[id(p)] for p in decay["params"]}
    kept = {names[id(p)] for p in no_decay["params"]}
    assert decayed | kept == set(names.values()) and not (decayed & kept)
    assert all(n.endswith(("c_attn.weight", "c_proj.weight", "w12.weight")) for n in decayed)
    assert len(decayed) == 4 * 2                      # four block linears per layer
    assert {"lm_head.weight", "transformer.wte.weight", "transformer.ln_f.weight"} <= kept
    assert all(n in kept for n in names.values() if n.endswith("bias") or ".ln_" in n)
    assert no_decay["weight_decay"] == 0.0 and "weight_decay" not in decay


def test_one_cycle_schedule_endpoints():
    model = tiny_model()
    cfg = TrainConfig(iterations=100, warmup_steps=10, lr=2e-3, scheduler="cos")
    opt = build_optimizer(model, cfg)
    sched = build_scheduler(opt, cfg)
    lrs = []
    for _ in range(cfg.iterations):
        lrs.append(opt.param_groups[0]["lr"])
        opt.step()
        sched.step()
    assert lrs[0] == pytest.approx(2e-3 / 100)        # initial = lr / div_factor
    assert max(lrs) == pytest.approx(2e-3) and lrs.index(max(lrs)) in (9, 10)
    assert lrs[-1] == pytest.approx(2e-3 / 100 / 0.1, rel=2e-2)   # final = initial / final_div_factor
    assert all(a >= b for a, b in zip(lrs[11:], lrs[12:]))


def test_lambda_schedules_closed_forms():
    s = cos_inf_schedule(n_iterations=100, n_warmup=10, div_factor=100, final_div_factor=0.1, n_inf=20)
    assert s(0) == pytest.approx(0.01) and s(10) == pytest.approx(1.0) and s(5) == pytest.approx(0.5 + 0.5 / 100)
    assert s(45) == pytest.approx(0.1 + 0.5 * 0.9 * (1 + math.cos(math.pi * 0.5))) and s(80) == s(99) == pytest.approx(0.1)
    w = wsd_schedule(n_iterations=100, final_lr_factor=0.0, n_warmup=10, init_div_factor=100, fract_decay=0.2)
    assert w(0) == pytest.approx(0.01) and w(10) == w(79) == 1.0 and w(90) == pytest.approx(0.5) and w(100) == 0.0
    with pytest.raises(ValueError):
        build_scheduler(build_optimizer(tiny_model(), TrainConfig()), TrainConfig(iterations=5, warmup_steps=5))


def test_accumulation_equals_one_large_batch():
    """acc_steps micro-batches with loss / acc_steps give the gradient of their concatenation (fp32, no autocast noise)."""
    batches = synthetic_batches(64, 2, 16, "cpu", seed=3)
    data = [batches() for _ in range(4)]
    results = []
    for acc in (4, 1):
        model = tiny_model(seed=1)
        cfg = TrainConfig(iterations=1, warmup_steps=0, scheduler="none", acc_steps=acc, opt="sgd", lr=0.1, weight_decay=0.0,
                          grad_clip=0.0, dtype=torch.float32)
        it = iter(data) if acc == 4 else iter([(torch.cat([d[0] for d in data]), torch.cat([d[1] for d in data]))])
        train(model, lambda: next(it), cfg)
        results.append(torch.cat([p.detach().flatten() for p in model.parameters()]))
    assert torch.allclose(results[0], results[1], atol=2e-6)


def test_a_small_model_learns_under_bf16_autocast():
    model = tiny_model(seed=2)
    cfg = TrainConfig(iterations=60, warmup_steps=5, lr=5e-3, acc_steps=2, scheduler="cos")
    stats = train(model, synthetic_batches(64, 8, 32, "cpu", seed=0), cfg)
    assert len(stats.loss) == 60 and all(math.isfinite(v) for v in stats.loss)
    first, last = sum(stats.loss[:5]) / 5, sum(stats.loss[-5:]) / 5
    assert first == pytest.approx(math.log(64), abs=0.3)
    assert last < first - 1.0, (first, last)
    assert stats.lr[0] == pytest.approx(5e-5) and all(g > 0 for g in stats.grad_norm)
    assert all(p.grad is None for p in model.parameters())  # zero_grad(set_to_none=True)


def test_quantized_linears_are_in_the_decayed_group():
    from quartet_amd import QuantizedLinear
    net = nn.ModuleDict({"lin": QuantizedLinear(32, 32, bias=True), "norm": nn.LayerNorm(32), "lm_head": nn.Linear(32, 8, bias=False)})
    decay, no_decay = parameter_groups(net)
    assert [id(p) for p in decay["params"]] == [id(net["lin"].weight)]
    assert {id(p) for p in no_decay["params"]} == {id(net["lin"].bias), id(net["norm"].weight), id(net["norm"].bias),
                                                   id(net["lm_head"].weight)}
