"""Sefalorn: a decoder-only design of layer-normed, gated-residual layers.

Each layer is either a ``lightning`` layer (linear attention with a scalar
decay per head) or a ``parallel`` layer (a sliding-window softmax attention
with head mixing and a log-distance penalty next to a gated delta rule
behind a short convolution, their results added with fixed scales),
followed by an optional mixture-of-experts feed-forward. Every sublayer's
result is multiplied by sigmoid(W h + b) before it joins the fp32 residual
stream. The logits are scaled by a constant.

This module only ASSEMBLES the design from the reusable blocks in
``models/mixers.py``: it parses ``config.json`` (layer list, sizes,
constants), declares what cache/state each layer needs, and maps
checkpoint tensor names onto the merged parameters. The engine's block
manager, state-slot manager, scheduler and sampler serve it like any other
model.
"""

from __future__ import annotations

import dataclasses
import re
from typing import Dict, Iterable, List, Optional, Tuple, Union

import torch
import torch.nn as nn

from fusioninfer_amd.config import ModelConfig
from fusioninfer_amd.distributed import parallel_state as ps
from fusioninfer_amd.distributed.layers import ReplicatedLinear
from fusioninfer_amd.models.mixers import (
    DecayLinearAttention,
    DecayLinearAttentionConfig,
    GatedDeltaConfig,
    GatedDeltaMixer,
    GatedResidualLayer,
    RoutedExperts,
    TalkingWindowAttention,
    TalkingWindowAttentionConfig,
)
from fusioninfer_amd.ops import seqmix

ARCHITECTURE = "Sefalorn"


@dataclasses.dataclass
class ExpertsConfig:
    ff: int
    experts: int
    top: int
    scale: float


@dataclasses.dataclass
class ParallelPairConfig:
    left: TalkingWindowAttentionConfig
    right: GatedDeltaConfig
    left_scale: float
    right_scale: float


@dataclasses.dataclass
class SefalornLayerConfig:
    kind: str                                       # lightning | parallel
    mixer: Union[DecayLinearAttentionConfig, ParallelPairConfig]
    mlp: Optional[ExpertsConfig]


@dataclasses.dataclass
class SefalornConfig:
    width: int
    vocab: int
    eps: float
    logit_scale: float
    layers: List[SefalornLayerConfig]


def parse_config(raw: dict) -> SefalornConfig:
    """config.json -> SefalornConfig; every size and constant is read from
    the config."""
    layers = []
    for i, L in enumerate(raw["layers"]):
        kind, m = L.get("type"), L["mixer"]
        if kind == "lightning":
            mixer = DecayLinearAttentionConfig(
                heads=int(m["heads"]), dim=int(m["dim"]),
                vdim=int(m.get("vdim", m["dim"])),
                decay=tuple(float(d) for d in m["decay"]))
        elif kind == "parallel":
            lm, rm = m["left"], m["right"]
            left = TalkingWindowAttentionConfig(
                heads=int(lm["heads"]),
                kv_heads=int(lm.get("kv_heads", lm["heads"])),
                dim=int(lm["dim"]), vdim=int(lm.get("vdim", lm["dim"])),
                scale=float(lm["scale"]),
                window=int((lm.get("mask") or {}).get("size", 0)))
            right = GatedDeltaConfig(
                heads=int(rm["heads"]),
                kv_heads=int(rm.get("kv_heads", rm["heads"])),
                dim=int(rm["dim"]), vdim=int(rm.get("vdim", rm["dim"])),
                conv=int(rm.get("conv", 1)))
            mixer = ParallelPairConfig(
                left, right, float(m.get("left_scale", 1.0)),
                float(m.get("right_scale", 1.0)))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = L.get("mlp")
        experts = None
        if mlp:
            if mlp.get("kind") != "moe":
                raise ValueError(
                    f"layer {i}: unknown mlp kind {mlp.get('kind')!r}")
            r = mlp["router"]
            experts = ExpertsConfig(
                ff=int(mlp["expert"]["ff"]), experts=int(r["experts"]),
                top=int(r["top"]), scale=float(r.get("scale", 1.0)))
        layers.append(SefalornLayerConfig(kind, mixer, experts))
    return SefalornConfig(
        width=int(raw["width"]), vocab=int(raw["vocab"]),
        eps=float(raw["norm"]["eps"]),
        logit_scale=float(raw.get("logit_scale", 1.0)), layers=layers)


def model_config_from_dict(raw: dict, model_path: Optional[str] = None,
                           name: str = ARCHITECTURE) -> ModelConfig:
    """Engine-level ModelConfig for a Sefalorn config dict (the registry's
    architecture hook)."""
    arch = parse_config(raw)
    heads, kv_heads, dim = 1, 1, arch.width
    for L in arch.layers:
        if L.kind == "parallel":
            heads, kv_heads, dim = (L.mixer.left.heads,
                                    L.mixer.left.kv_heads, L.mixer.left.dim)
            break
        heads, kv_heads, dim = L.mixer.heads, L.mixer.heads, L.mixer.dim
    experts = [L.mlp for L in arch.layers if L.mlp is not None]
    return ModelConfig(
        name=name,
        architecture=ARCHITECTURE,
        arch=arch,
        hidden_size=arch.width,
        num_layers=len(arch.layers),
        num_heads=heads,
        num_kv_heads=kv_heads,
        head_dim=dim,
        intermediate_size=max((e.ff for e in experts), default=0),
        vocab_size=arch.vocab,
        rms_norm_eps=arch.eps,
        qk_norm=False,
        model_path=model_path,
        max_position_embeddings=1 << 24,
    )


_EXPERT = re.compile(r"^mlp\.e(\d+)\.(gate|up|down)$")


class SefalornLM(nn.Module):
    """embedding -> gated-residual layers -> final layer norm -> head.

    Engine interface (same as CausalLM): ``forward(ids, meta, caches)``
    returns the final-normed hidden rows, ``compute_logits`` applies the
    head and the logit scale. Declares per-layer cache/state needs
    (``allocate_caches``) and ``uses_state_slots`` so the runner builds
    sequence-grouped metadata and the scheduler hands out state slots."""

    uses_state_slots = True
    supports_prefix_caching = False   # recurrent state has no block form

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        assert ps.tp_world_size() == 1 and ps.pp_world_size() == 1, (
            "Sefalorn runs single-rank (TP/PP sharding of its mixers is "
            "not implemented)")
        self.cfg = cfg
        arch: SefalornConfig = cfg.arch
        self.arch = arch
        dtype = {"bfloat16": torch.bfloat16,
                 "float32": torch.float32}[cfg.dtype]
        self.dtype = dtype
        self.pp_first = self.pp_last = True
        W = arch.width
        base_seed = torch.initial_seed() % (2**62)
        torch.manual_seed(base_seed + 1000003)
        self.embed_tokens = nn.Parameter(
            torch.empty(arch.vocab, W, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        layers = []
        for i, L in enumerate(arch.layers):
            torch.manual_seed(base_seed + 1000003 * (i + 2))
            if L.kind == "lightning":
                mixers = [("", DecayLinearAttention(L.mixer, W, arch.eps,
                                                    dtype), 1.0)]
            else:
                mixers = [
                    ("left", TalkingWindowAttention(L.mixer.left, W,
                                                    arch.eps, dtype),
                     L.mixer.left_scale),
                    ("right", GatedDeltaMixer(L.mixer.right, W, arch.eps,
                                              dtype),
                     L.mixer.right_scale),
                ]
            mlp = None
            if L.mlp is not None:
                mlp = RoutedExperts(W, L.mlp.ff, L.mlp.experts, L.mlp.top,
                                    dtype, score="sigmoid", renorm=True,
                                    scale=L.mlp.scale)
            layers.append(GatedResidualLayer(mixers, mlp, W, arch.eps, dtype))
        self.layers = nn.ModuleList(layers)
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32),
                                       requires_grad=False)
        torch.manual_seed(base_seed + 1000003 * (len(arch.layers) + 2))
        self.lm_head = ReplicatedLinear(W, arch.vocab, dtype=dtype)
        torch.manual_seed(base_seed + 777)

    # ------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def kv_block_bytes(self, block_size: int) -> int:
        n = sum(m.block_bytes(block_size) for layer in self.layers
                for m in layer.mixers)
        return max(n, 1)     # a model of recurrent layers only pages nothing

    def allocate_caches(self, num_blocks: int, block_size: int,
                        num_slots: int, device) -> list:
        """One dict per layer: paged k/v of its windowed attention (model
        dtype) and the fp32 slot states of its recurrent mixers."""
        caches = []
        for layer in self.layers:
            cache = {}
            for m in layer.mixers:
                cache.update(m.state_tensors(num_blocks, block_size,
                                             num_slots, device))
            caches.append(cache)
        return caches

    # ----------------------------------------------------------- forward
    def forward(self, input_ids, meta, caches, hidden=None, residual=None):
        resid = self.embed_tokens[input_ids].float()
        h = seqmix.layer_norm(resid, self.layers[0].norm1, self.arch.eps,
                              self.dtype)
        n = len(self.layers)
        for i, (layer, cache) in enumerate(zip(self.layers, caches)):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            h = layer(resid, h, meta, cache, nxt)
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = self.lm_head(hidden).float()
        if self.arch.logit_scale != 1.0:
            logits = logits * self.arch.logit_scale
        return logits

    # ----------------------------------------------------------- weights
    def load_weights(self, tensors: Iterable[Tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names -> parameters. Input branches of a layer's
        mixers (and the first gate's matrix) land in the merged input
        projection, expert matrices in the stacked expert tensors; gains,
        biases of gates, decays and tables are kept in fp32."""
        n = 0
        seen = set()
        for name, t in tensors:
            self._load_one(name, t)
            seen.add(name)
            n += 1
        missing = [k for k in self.expected_tensor_names() if k not in seen]
        if missing:
            raise ValueError(f"checkpoint lacks tensors: {missing[:8]}"
                             f"{' ...' if len(missing) > 8 else ''}")
        for layer in self.layers:
            if layer.mlp is not None:
                layer.mlp.invalidate_packed()
        return n

    def expected_tensor_names(self) -> List[str]:
        return list(self._name_map())

    def _name_map(self) -> Dict[str, tuple]:
        """checkpoint name -> (parameter, row range or None)."""
        out: Dict[str, tuple] = {
            "embed": (self.embed_tokens, None),
            "head": (self.lm_head.weight, None),
            "final.norm": (self.final_norm, None),
        }
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = (layer.norm1, None)
            out[p + "rg1"] = (layer.in_proj.weight,
                              layer.in_proj_rows("", "rg1"))
            out[p + "rg1.b"] = (layer.rg1_bias, None)
            for name, mod in zip(layer.names, layer.mixers):
                mp = p + "mix." + (name + "." if name else "")
                for br in mod.in_names:
                    rows = layer.in_proj_rows(name, br)
                    out[mp + br] = (layer.in_proj.weight, rows)
                    if mod.has_bias:
                        out[mp + br + ".b"] = (layer.in_proj.bias, rows)
                out[mp + "o"] = (mod.o_proj.weight, None)
                if isinstance(mod, DecayLinearAttention):
                    out[mp + "norm"] = (mod.norm_w, None)
                elif isinstance(mod, TalkingWindowAttention):
                    out[mp + "o.b"] = (mod.o_bias, None)
                    out[mp + "r1"] = (mod.r1, None)
                    out[mp + "r2"] = (mod.r2, None)
                    out[mp + "talk"] = (mod.talk, None)
                elif isinstance(mod, GatedDeltaMixer):
                    nq = mod.cfg.kv_heads * mod.cfg.dim
                    nv = mod.cfg.heads * mod.cfg.vdim
                    out[mp + "q.conv"] = (mod.conv_w, (0, nq))
                    out[mp + "k.conv"] = (mod.conv_w, (nq, nq))
                    out[mp + "v.conv"] = (mod.conv_w, (2 * nq, nv))
                    out[mp + "A_log"] = (mod.a_log, None)
                    out[mp + "dt_bias"] = (mod.dt_bias, None)
                    out[mp + "norm"] = (mod.norm_w, None)
            if layer.mlp is not None:
                out[p + "norm2"] = (layer.norm2, None)
                out[p + "rg2"] = (layer.rg2.weight, None)
                out[p + "rg2.b"] = (layer.rg2_bias, None)
                out[p + "mlp.router"] = (layer.mlp.router, None)
                ff = layer.mlp.ff
                for e in range(layer.mlp.experts):
                    ep = f"{p}mlp.e{e}."
                    out[ep + "gate"] = (layer.mlp.gate_up, (e, 0, ff))
                    out[ep + "up"] = (layer.mlp.gate_up, (e, ff, ff))
                    out[ep + "down"] = (layer.mlp.down, (e, None, None))
        return out

    @staticmethod
    def _view(param, rows):
        dst = param.data
        if rows is None:
            return dst
        if len(rows) == 2:
            return dst[rows[0]: rows[0] + rows[1]]
        e, a, n = rows
        return dst[e] if a is None else dst[e, a: a + n]

    def _load_one(self, name: str, t: torch.Tensor) -> None:
        names = getattr(self, "_names", None)
        if names is None:
            names = self._names = self._name_map()
        if name not in names:
            raise ValueError(f"unknown tensor {name!r}")
        param, rows = names[name]
        dst = self._view(param, rows)
        if dst.shape != t.shape:
            raise ValueError(f"{name}: shape {tuple(t.shape)} does not fit "
                             f"{tuple(dst.shape)}")
        dst.copy_(t.to(dst.dtype))

    def export_weights(self) -> Dict[str, torch.Tensor]:
        """Inverse of load_weights (checkpoint naming), for writing
        random-init models to disk."""
        return {k: self._view(p, rows).detach().clone().contiguous()
                for k, (p, rows) in self._name_map().items()}

    def randomize_small_params(self, seed: int = 0) -> None:
        """Random-init use (benchmarks, tests): give gains, biases, decay
        inputs and tables non-trivial values so every branch contributes."""
        g = torch.Generator().manual_seed(seed)

        def rnd(p, lo, hi):
            p.data.copy_((torch.rand(p.shape, generator=g) * (hi - lo) + lo)
                         .to(device=p.device, dtype=p.dtype))

        rnd(self.final_norm, 0.8, 1.2)
        for layer in self.layers:
            rnd(layer.norm1, 0.5, 1.5)
            rnd(layer.rg1_bias, -1.0, 1.0)
            if layer.in_proj.bias is not None:
                rnd(layer.in_proj.bias, -0.1, 0.1)
                a, n = layer.in_proj_rows("", "rg1")
                layer.in_proj.bias.data[a: a + n] = 0
                for name, mod in zip(layer.names, layer.mixers):
                    if not mod.has_bias:
                        for br in mod.in_names:
                            a, n = layer.in_proj_rows(name, br)
                            layer.in_proj.bias.data[a: a + n] = 0
            if layer.mlp is not None:
                rnd(layer.norm2, 0.5, 1.5)
                rnd(layer.rg2_bias, -1.0, 1.0)
                rnd(layer.mlp.router, -0.5, 0.5)
            for mod in layer.mixers:
                if isinstance(mod, DecayLinearAttention):
                    rnd(mod.norm_w, 0.5, 1.5)
                elif isinstance(mod, TalkingWindowAttention):
                    rnd(mod.o_bias, -0.1, 0.1)
                    rnd(mod.r1, 0.0, 1.0)
                    rnd(mod.r2, 0.0, 2.0)
                    rnd(mod.talk, -0.3, 0.3)
                    mod.talk.data += torch.eye(mod.cfg.heads).to(
                        mod.talk.device)
                elif isinstance(mod, GatedDeltaMixer):
                    rnd(mod.conv_w, -0.5, 0.5)
                    rnd(mod.a_log, -2.0, 0.5)
                    rnd(mod.dt_bias, -1.0, 1.0)
                    rnd(mod.norm_w, 0.5, 1.5)
