"""Synthetic parameter sets for the five benchmark/parity configurations.

Every generator is a pure function of its arguments: it returns an ordered list
of ``(name, shape)`` in *name-sorted* order, which is the order the reference
deploys parameters in (``src/comp/ParamStorage.cpp:23-31, 852`` sort by name)
and therefore the order gradient buckets are laid out in.

Nothing here touches a device; tensors are materialised by the caller.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Sequence, Tuple

import numpy as np

Shape = Tuple[int, ...]
NamedShapes = List[Tuple[str, Shape]]


def numel(shape: Sequence[int]) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


def _sorted(items: Dict[str, Shape]) -> NamedShapes:
    return [(k, items[k]) for k in sorted(items)]


def mlp_params(layers: int = 4, width: int = 1024) -> NamedShapes:
    """``c1_mlp``: ``layers`` x Linear(width, width) with biases (8 tensors, 4,198,400 elements)."""
    out: Dict[str, Shape] = {}
    for i in range(layers):
        out[f"layers.{i}.weight"] = (width, width)
        out[f"layers.{i}.bias"] = (width,)
    return _sorted(out)


def bert_params(layers: int, hidden: int, ffn: int, vocab: int = 30522,
                max_pos: int = 512, type_vocab: int = 2) -> NamedShapes:
    """BERT encoder parameter list (``c2_bert_large``: 24/1024/4096 -> 391 tensors, ~3.35e8;
    ``c3_bert_enlarged``: 48/2048/8192 -> 775 tensors, ~2.48e9)."""
    out: Dict[str, Shape] = {
        "bert.embeddings.word_embeddings.weight": (vocab, hidden),
        "bert.embeddings.position_embeddings.weight": (max_pos, hidden),
        "bert.embeddings.token_type_embeddings.weight": (type_vocab, hidden),
        "bert.embeddings.LayerNorm.weight": (hidden,),
        "bert.embeddings.LayerNorm.bias": (hidden,),
        "bert.pooler.dense.weight": (hidden, hidden),
        "bert.pooler.dense.bias": (hidden,),
    }
    for i in range(layers):
        p = f"bert.encoder.layer.{i}."
        for proj in ("query", "key", "value"):
            out[p + f"attention.self.{proj}.weight"] = (hidden, hidden)
            out[p + f"attention.self.{proj}.bias"] = (hidden,)
        out[p + "attention.output.dense.weight"] = (hidden, hidden)
        out[p + "attention.output.dense.bias"] = (hidden,)
        out[p + "attention.output.LayerNorm.weight"] = (hidden,)
        out[p + "attention.output.LayerNorm.bias"] = (hidden,)
        out[p + "intermediate.dense.weight"] = (ffn, hidden)
        out[p + "intermediate.dense.bias"] = (ffn,)
        out[p + "output.dense.weight"] = (hidden, ffn)
        out[p + "output.dense.bias"] = (hidden,)
        out[p + "output.LayerNorm.weight"] = (hidden,)
        out[p + "output.LayerNorm.bias"] = (hidden,)
    return _sorted(out)


def bert_large_params() -> NamedShapes:
    return bert_params(24, 1024, 4096)


def bert_enlarged_params() -> NamedShapes:
    return bert_params(48, 2048, 8192)


def resnet152_params(width_mult: int = 2, split: int = 2, num_classes: int = 1000) -> NamedShapes:
    """``c4_resnet152x2``: ResNet-152 bottleneck parameter list with channel widths multiplied by
    ``width_mult``; every tensor is then cut along dim 0 into ``split`` equal
    parts (the share layout of a x``split`` output-channel split), which gives
    934 tensors / ~2.3e8 elements with BN vectors of 64..2048 elements for the
    defaults."""
    out: Dict[str, Shape] = {}

    def add(name: str, shape: Shape) -> None:
        if split <= 1 or shape[0] % split != 0:
            out[name] = shape
            return
        part = (shape[0] // split,) + tuple(shape[1:])
        for s in range(split):
            out[f"{name}.part{s}"] = part

    def conv_bn(prefix_conv: str, prefix_bn: str, cout: int, cin: int, k: int) -> None:
        add(prefix_conv + ".weight", (cout, cin, k, k))
        add(prefix_bn + ".weight", (cout,))
        add(prefix_bn + ".bias", (cout,))

    w = width_mult
    conv_bn("conv1", "bn1", 64 * w, 3, 7)
    inplanes = 64 * w
    for li, (planes, blocks) in enumerate(zip((64, 128, 256, 512), (3, 8, 36, 3)), start=1):
        planes *= w
        for b in range(blocks):
            p = f"layer{li}.{b}."
            conv_bn(p + "conv1", p + "bn1", planes, inplanes, 1)
            conv_bn(p + "conv2", p + "bn2", planes, planes, 3)
            conv_bn(p + "conv3", p + "bn3", planes * 4, planes, 1)
            if b == 0:
                conv_bn(p + "downsample.0", p + "downsample.1", planes * 4, inplanes, 1)
            inplanes = planes * 4
    add("fc.weight", (num_classes, inplanes))
    add("fc.bias", (num_classes,))
    return _sorted(out)


def zero_segment_sizes(n_segments: int = 4096, total: int = 10_000_000_000,
                       lo: int = 1 << 10, hi: int = 1 << 26, seed: int = 0) -> List[int]:
    """ZeRO flat-buffer configuration: ``n_segments`` parameter sizes, log-uniform in [lo, hi], rescaled so the
    sum is close to ``total`` and forced odd (so every running offset in the flat
    buffer alternates parity and nothing is 16-byte aligned by luck)."""
    rng = np.random.default_rng(seed)
    raw = np.exp(rng.uniform(math.log(lo), math.log(hi), size=n_segments))
    sizes = np.maximum(1, np.floor(raw * (total / raw.sum()))).astype(np.int64)
    sizes |= 1
    return [int(s) for s in sizes]


@dataclass(frozen=True)
class StepConfig:
    """One fused-step workload: tensor list, gradient dtype/statistics, scaling."""
    key: str
    description: str
    params: NamedShapes
    grad_dtype: str          # "f32" | "f16" | "bf16": dtype of the incoming gradients
    bucket_dtype: str        # dtype of the packed destination bucket
    grad_std: float          # std of the unscaled gradient
    loss_scale: float        # gradients arrive multiplied by this
    max_norm: float
    inject_rate: float = 0.0  # fraction of elements replaced by +inf / NaN

    @property
    def inv_scale(self) -> float:
        return 1.0 / self.loss_scale

    @property
    def total_numel(self) -> int:
        return sum(numel(s) for _, s in self.params)


def step_config(key: str) -> StepConfig:
    if key == "c1_mlp":
        return StepConfig(key, "4x Linear(1024,1024) fp32 grads -> fp32 bucket", mlp_params(),
                          "f32", "f32", 1e-3, 1.0, 1.0)
    if key == "c2_bert_large":
        return StepConfig(key, "BERT-large stage, bf16 grads * 2^16 -> fp32 master bucket",
                          bert_large_params(), "bf16", "f32", 1e-2, 65536.0, 1.0)
    if key == "c3_bert_enlarged":
        return StepConfig(key, "48x2048x8192 BERT share, fp16 grads * 2^12 -> fp32 master bucket",
                          bert_enlarged_params(), "f16", "f32", 1e-3, 4096.0, 1.0)
    if key == "c3_bert_enlarged_overflow":
        return StepConfig(key, "as c3 with +inf/NaN injected at rate 1e-7",
                          bert_enlarged_params(), "f16", "f32", 1e-3, 4096.0, 1.0, 1e-7)
    if key == "c4_resnet152x2":
        return StepConfig(key, "ResNet-152 x2-wide, 934 tensors, fp32 grads -> fp32 bucket",
                          resnet152_params(), "f32", "f32", 1e-3, 1.0, 1.0)
    raise KeyError(key)


STEP_CONFIG_KEYS = ("c1_mlp", "c2_bert_large", "c3_bert_enlarged",
                    "c3_bert_enlarged_overflow", "c4_resnet152x2")


# --------------------------------------------------------------------------- seeded inputs

def make_grads(cfg: StepConfig, seed: int = 0, device: str = "cpu", scale_numel: float = 1.0):
    """Materialise the incoming gradients of ``cfg``: one generator seeded with ``seed``,
    tensors drawn in list order, each ``randn(shape) * grad_std`` in fp32, multiplied by the
    loss scale, then cast to the gradient dtype.  Non-finite values are injected afterwards
    at ``floor(inject_rate * N)`` positions drawn with ``randint(N)`` from the same
    generator, alternating +inf / NaN.  ``device != "cpu"`` draws on that device (a
    different stream of numbers; used for sizes the host cannot hold).

    ``scale_numel < 1`` shrinks dim 0 of every tensor (at least 1 row) so the same tensor
    *list* can be exercised at a fraction of the element count.
    Returns (list of tensors, list of injected (tensor index, flat index)).
    """
    import torch

    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[cfg.grad_dtype]
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    grads = []
    for _, shape in cfg.params:
        if scale_numel < 1.0:
            shape = (max(1, int(shape[0] * scale_numel)),) + tuple(shape[1:])
        g = torch.randn(shape, generator=gen, device=device, dtype=torch.float32)
        g.mul_(cfg.grad_std).mul_(cfg.loss_scale)
        grads.append(g.to(tdt))
    injected = []
    total = sum(int(g.numel()) for g in grads)
    n_inject = int(math.floor(cfg.inject_rate * total))
    if cfg.inject_rate > 0 and n_inject == 0:
        n_inject = 2
    if n_inject:
        cpu_gen = torch.Generator()
        cpu_gen.manual_seed(seed + 1)
        pos = torch.randint(0, total, (n_inject,), generator=cpu_gen).tolist()
        bounds = np.cumsum([0] + [int(g.numel()) for g in grads])
        for j, p in enumerate(pos):
            ti = int(np.searchsorted(bounds, p, side="right") - 1)
            fi = int(p - bounds[ti])
            grads[ti].view(-1)[fi] = float("inf") if j % 2 == 0 else float("nan")
            injected.append((ti, fi))
    return grads, injected
