"""Layered decoder models: a stack described layer by layer in ``config.json`` -- each layer names its sequence mixer, the
mixer's sizes and its feed-forward --, optionally with a span of layers that runs several times in a row with the same
weights.  Where model.py fixes ONE llama-shaped layer and a static geometry table, this file builds the stack from the
description, out of mixers that take a ragged step (executor/ragged.py) and keep their own kind of state in the
:class:`PagedStateCache`:

  * :class:`SinkAttention`     softmax attention, separate key / value widths, per-head q / k RMS norm, a position temperature
                               on the queries instead of a rotation, a learned sink in the denominator (kernels/attention.py)
  * :class:`GatedLinearMixer`  HGRN2: linear attention whose forget gate, bounded from below, also decides what is written
                               (kernels/recurrent.py)
  * :class:`DenseMLP`          ``down(act(up h))`` with the xIELU activation (kernels/activations.py)

The residual stream is fp32 throughout; every layer's residual add is fused into the norm that follows it
(kernels/norm_act.py::add_rmsnorm_shift), which also applies the token shift in front of a mixer.  Projections run through the
framework's linear layers (library GEMM for unquantised weights), with q|f|v and q|k|v fused into one launch at load time.
The first family built this way is Rakevik (``"architecture": "Rakevik"``).
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F

from .distributed.parallel_state import get_tp_world_size
from .kernels.activations import xielu
from .kernels.attention import qk_norm_cache, ragged_attention
from .kernels.norm_act import add_rmsnorm_shift, cast_pair, residual_set
from .kernels.recurrent import gated_linear_scan
from .linear import ReplicatedLinear


# ------------------------------------------------------------------------------------- #
# description
# ------------------------------------------------------------------------------------- #
@dataclass(frozen=True)
class MixerSpec:
    kind: str                   # "attention" | "hgrn2"
    heads: int
    dim: int                    # per-head query / key width
    vdim: int                   # per-head value width
    kv_heads: int = 0           # attention only
    scale: float = 1.0          # attention only
    temp_coef: float = 0.0      # attention only: q *= 1 + temp_coef ln(floor((p + 1) / temp_every) + 1)
    temp_every: int = 1


@dataclass(frozen=True)
class LayerSpec:
    mixer: MixerSpec
    ff: int = 0                 # 0: the layer has no feed-forward sublayer
    mlp_kind: str = "dense"


@dataclass(frozen=True)
class LayeredGeometry:
    name: str
    vocab_size: int
    width: int
    eps: float
    layers: tuple[LayerSpec, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    token_shift: bool = True
    extra: dict = field(default_factory=dict, compare=False)

    @property
    def looped(self) -> bool:
        return self.loop_stop > self.loop_start

    def run_order(self) -> list[tuple[int, int, bool]]:
        """``(layer index, pass number, first layer of a pass)`` per layer run."""
        n = len(self.layers)
        if not self.looped:
            return [(i, 0, False) for i in range(n)]
        order = [(i, 0, False) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            order += [(i, t, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        return order + [(i, 0, False) for i in range(self.loop_stop, n)]

    @staticmethod
    def from_config(config: Mapping, name: str = "rakevik") -> "LayeredGeometry":
        layers = []
        for entry in config["layers"]:
            m, kind = entry["mixer"], entry["type"]
            if kind == "attention":
                temp = m.get("q_temp") or {}
                spec = MixerSpec("attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                 kv_heads=int(m.get("kv_heads") or m["heads"]), scale=float(m["scale"]),
                                 temp_coef=float(temp.get("coef", 0.0)), temp_every=int(temp.get("every", 1)))
                if spec.heads % spec.kv_heads:
                    raise ValueError(f"{spec.heads} query heads do not divide over {spec.kv_heads} key/value heads")
            elif kind == "hgrn2":
                spec = MixerSpec("hgrn2", int(m["heads"]), int(m["dim"]), int(m["vdim"]))
            else:
                raise ValueError(f"unsupported mixer type {kind!r}; supported: attention, hgrn2")
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}; supported: dense")
            layers.append(LayerSpec(spec, ff=int(mlp["ff"]) if mlp is not None else 0))
        loop = config.get("loop") or {}
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        if stop > start and not (0 <= start < stop <= len(layers) and times >= 1):
            raise ValueError(f"loop {start}..{stop} x {times} does not fit {len(layers)} layers")
        return LayeredGeometry(name=name, vocab_size=int(config["vocab"]), width=int(config["width"]),
                               eps=float(config["norm"]["eps"]), layers=tuple(layers), loop_start=start, loop_stop=stop,
                               loop_times=times if stop > start else 1)


def _linear(inp: int, out: int) -> ReplicatedLinear:
    return ReplicatedLinear(inp, out)


def _vector(n: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(n, dtype=torch.float16), requires_grad=False)


# ------------------------------------------------------------------------------------- #
# mixers
# ------------------------------------------------------------------------------------- #
class SinkAttention(nn.Module):
    """``q|k|v`` in one projection, then per-head norm + temperature + cache write (one launch), attention with a sink over
    the paged cache (one launch), output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        self.q_size, self.k_size, self.v_size = spec.heads * spec.dim, spec.kv_heads * spec.dim, spec.kv_heads * spec.vdim
        self.qkv_proj = _linear(width, self.q_size + self.k_size + self.v_size)
        self.o_proj = _linear(spec.heads * spec.vdim, width)
        self.q_norm_weight = _vector(spec.dim)
        self.k_norm_weight = _vector(spec.dim)
        self.sink = _vector(spec.heads)

    def cache_run(self) -> dict:
        return {"kind": "attention", "kv_heads": self.spec.kv_heads, "dk": self.spec.dim, "dv": self.spec.vdim}

    def forward(self, h, step, cache, run: int, token_table):
        s = self.spec
        k_cache, v_cache = cache.kv_buffer[run]
        q = qk_norm_cache(self.qkv_proj(h), s.heads, s.kv_heads, s.dim, s.vdim, self.q_norm_weight, self.k_norm_weight, self.eps,
                          s.temp_coef, s.temp_every, step, k_cache, v_cache)
        o = ragged_attention(q, k_cache, v_cache, s.scale, step, token_table, sink=self.sink)
        return self.o_proj(o)


class GatedLinearMixer(nn.Module):
    """HGRN2.  ``q|f|v`` in one projection; gate, recurrence, read-out and the per-head output norm in one launch over the
    fp32 state slots; output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        self.qk_size, self.v_size = spec.heads * spec.dim, spec.heads * spec.vdim
        self.qfv_proj = _linear(width, 2 * self.qk_size + self.v_size)
        self.o_proj = _linear(self.v_size, width)
        self.f_bias = _vector(self.qk_size)
        self.lower = _vector(self.qk_size)
        self.out_norm_weight = _vector(spec.vdim)

    def cache_run(self) -> dict:
        return {"kind": "recurrent", "heads": self.spec.heads, "dk": self.spec.dim, "dv": self.spec.vdim}

    def forward(self, h, step, cache, run: int, token_table):
        s = self.spec
        o = gated_linear_scan(self.qfv_proj(h), s.heads, s.dim, s.vdim, self.f_bias, self.lower, self.out_norm_weight, self.eps,
                              step, cache.recurrent[run])
        return self.o_proj(o)


class DenseMLP(nn.Module):
    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up_proj = _linear(width, ff)
        self.down_proj = _linear(ff, width)
        self.act = _vector(2)

    def forward(self, h):
        return self.down_proj(xielu(self.up_proj(h), self.act))


MIXERS = {"attention": SinkAttention, "hgrn2": GatedLinearMixer}


class MixerLayer(nn.Module):
    def __init__(self, geo: LayeredGeometry, spec: LayerSpec):
        super().__init__()
        self.eps = geo.eps
        self.norm1_weight = _vector(geo.width)
        self.shift = _vector(geo.width) if geo.token_shift else None
        self.mixer = MIXERS[spec.mixer.kind](geo.width, spec.mixer, geo.eps)
        self.mlp = DenseMLP(geo.width, spec.ff) if spec.ff else None
        self.norm2_weight = _vector(geo.width) if spec.ff else None

    def forward(self, x, delta, step, cache, run: int, token_table):
        """``(x, delta)``: the fp32 residual and the update still to be added to it.  Returns the same pair."""
        h, x = add_rmsnorm_shift(x, delta, self.norm1_weight, self.eps, shift=self.shift, step=step, state=cache.shift[run])
        delta = self.mixer(h, step, cache, run, token_table)
        if self.mlp is not None:
            h, x = add_rmsnorm_shift(x, delta, self.norm2_weight, self.eps, x_out=x)
            delta = self.mlp(h)
        return x, delta


# ------------------------------------------------------------------------------------- #
# the model
# ------------------------------------------------------------------------------------- #
class LayeredLM(nn.Module):
    """Token ids of a ragged step -> logits of the asked rows."""

    def __init__(self, geo: LayeredGeometry, dtype=torch.bfloat16):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("layered models run on one GPU per replica (their projections are not sharded)")
        self.geo = geo
        self.embed_tokens = nn.Embedding(geo.vocab_size, geo.width, dtype=torch.float16)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(MixerLayer(geo, spec) for spec in geo.layers)
        if geo.looped:
            self.loop_in = _linear(2 * geo.width, geo.width)
            self.loop_step = nn.Parameter(torch.zeros(geo.loop_times, geo.width, dtype=torch.float16), requires_grad=False)
        self.norm_weight = _vector(geo.width)
        self.lm_head = _linear(geo.width, geo.vocab_size)
        self.run_order = geo.run_order()
        self.to(dtype)

    @property
    def dtype(self):
        return self.norm_weight.dtype

    def cache_runs(self) -> list[dict]:
        """What every layer run keeps per sequence (the constructor argument of :class:`PagedStateCache`)."""
        runs = []
        for index, _, _ in self.run_order:
            layer = self.layers[index]
            run = layer.mixer.cache_run()
            if layer.shift is not None:
                run["shift_width"] = self.geo.width
            runs.append(run)
        return runs

    @torch.no_grad()
    def forward(self, token_ids, step, cache, token_table, logits_rows=None, collect_layers: list | None = None):
        """``token_ids [n]`` int64 of the step's flat token array.  ``logits_rows``: int64 indices into it (``None``: no
        logits, the step only fills cache and state).  ``collect_layers``: a list that receives the fp32 residual stream after
        every layer run (diagnostics; costs one add per run)."""
        x0 = residual_set(F.embedding(token_ids, self.embed_tokens.weight))
        x, delta = (x0.clone() if self.geo.looped else x0), None  # (layers update the residual in place; x0 is read again)
        for run, (index, pass_no, first) in enumerate(self.run_order):
            if first:
                y = self.loop_in(cast_pair(x, x0, self.dtype, a_delta=delta))
                x, delta = residual_set(y, self.loop_step[pass_no]), None
            x, delta = self.layers[index](x, delta, step, cache, run, token_table)
            if collect_layers is not None:
                collect_layers.append(x + delta.float() if delta is not None else x.clone())
        if logits_rows is None:
            return None
        x = x[logits_rows].contiguous()
        delta = delta[logits_rows].contiguous() if delta is not None else None
        h, _ = add_rmsnorm_shift(x, delta, self.norm_weight, self.geo.eps, x_out=x)
        return self.lm_head(h)

    # --------------------------------------------------------------------------------- #
    # synthetic weights (benchmarks, tests): seeded, every tensor in a range that keeps the stack well-conditioned
    # --------------------------------------------------------------------------------- #
    @torch.no_grad()
    def init_synthetic(self, seed: int = 0, device="cuda") -> "LayeredLM":
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        self.to(device)

        def fill(p, std=None, mean=0.0, lo=None, hi=None):
            if lo is not None:
                v = torch.rand(p.shape, generator=g) * (hi - lo) + lo
            else:
                v = torch.randn(p.shape, generator=g) * std + mean
            p.data.copy_(v.to(p.dtype))

        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if name.endswith("proj.weight") or name.endswith("lm_head.weight"):
                fill(p, std=1.0 / (p.shape[1] ** 0.5))
            elif name == "embed_tokens.weight":
                fill(p, std=1.0)
            elif leaf in ("norm1_weight", "norm2_weight", "norm_weight", "q_norm_weight", "k_norm_weight", "out_norm_weight"):
                fill(p, std=0.1, mean=1.0)
            elif leaf in ("shift", "lower"):
                fill(p, lo=0.0, hi=0.9)
            elif leaf in ("f_bias", "sink", "act", "loop_step"):
                fill(p, std=0.5)
            else:
                raise RuntimeError(f"init_synthetic: no rule for {name}")
        return self
