"""Pinuvik: a decoder-only design of parallel-mixer layers.

Every layer runs a chunk-masked shared-key/value rotary attention and a
generalized-delta-rule recurrence side by side on a token-shifted input,
followed by an optional tanh-GELU gated MLP; all norms are scalar-gain RMS
norms on an fp32 residual stream. A contiguous range of layers may be run
several times in a row with the same weights; every run has its own paged
cache and state slots.

This module only ASSEMBLES the design from the reusable blocks in
``models/mixers.py``: it parses ``config.json`` (sizes, constants, layer
list, loop), declares what cache/state each layer run needs, and maps
checkpoint tensor names onto the merged parameters. The engine's block
manager, state-slot manager, scheduler and sampler serve it like any
other model.
"""

from __future__ import annotations

import dataclasses
import json
import os
import struct
from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from fusioninfer_amd.config import ModelConfig
from fusioninfer_amd.distributed import parallel_state as ps
from fusioninfer_amd.distributed.layers import ReplicatedLinear
from fusioninfer_amd.models.mixers import (
    DeltaRuleConfig,
    DeltaRuleMixer,
    GatedMLP,
    MixerLayer,
    ParallelMixer,
    SharedKVAttention,
    SharedKVAttentionConfig,
)
from fusioninfer_amd.ops import seqmix

ARCHITECTURE = "Pinuvik"


@dataclasses.dataclass
class PinuvikLayerConfig:
    left: SharedKVAttentionConfig
    right: DeltaRuleConfig
    ff: int = 0                      # 0 = no feed-forward sublayer


@dataclasses.dataclass
class PinuvikConfig:
    width: int
    vocab: int
    eps: float
    layers: List[PinuvikLayerConfig]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1

    def layer_runs(self) -> List[int]:
        """Layer index of every layer RUN, in execution order."""
        n = len(self.layers)
        a, b, t = self.loop_start, self.loop_stop, self.loop_times
        if not (0 <= a <= b <= n) or t < 0:
            raise ValueError(f"bad loop {a}..{b} x{t} over {n} layers")
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


def safetensors_shapes(path: str) -> Dict[str, Tuple[int, ...]]:
    """Tensor shapes from a safetensors header (8-byte little-endian
    length, then that many bytes of JSON) without touching the data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in header.items()
            if k != "__metadata__"}


def parse_config(raw: dict, shapes: Optional[Dict[str, tuple]] = None,
                 default_decay_rank: int = 32) -> PinuvikConfig:
    """config.json -> PinuvikConfig. Sizes the config does not carry (the
    inner size of the decay branch) come from the checkpoint's tensor
    shapes, or from an optional ``decay_rank`` key for random-init use."""
    shapes = shapes or {}
    layers = []
    for i, L in enumerate(raw["layers"]):
        if L.get("type") != "parallel":
            raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
        lm, rm = L["mixer"]["left"], L["mixer"]["right"]
        mask = lm.get("mask") or {}
        rot = lm.get("rot") or {}
        left = SharedKVAttentionConfig(
            heads=int(lm["heads"]),
            kv_heads=int(lm.get("kv_heads", lm["heads"])),
            dim=int(lm["dim"]),
            vdim=int(lm.get("vdim", lm["dim"])),
            scale=float(lm["scale"]),
            rot_dims=int(rot.get("dims", 0)),
            rot_base=float(rot.get("base", 10000.0)),
            chunk=int(mask.get("size", 0)),
        )
        w1 = shapes.get(f"l{i}.mix.right.w1")
        right = DeltaRuleConfig(
            heads=int(rm["heads"]),
            dim=int(rm["dim"]),
            decay_rank=int(w1[0] if w1 else
                           rm.get("decay_rank", default_decay_rank)),
        )
        mlp = L.get("mlp")
        ff = 0
        if mlp:
            if mlp.get("kind") != "dense":
                raise ValueError(
                    f"layer {i}: unknown mlp kind {mlp.get('kind')!r}")
            ff = int(mlp["ff"])
        layers.append(PinuvikLayerConfig(left, right, ff))
    loop = raw.get("loop") or {}
    return PinuvikConfig(
        width=int(raw["width"]),
        vocab=int(raw["vocab"]),
        eps=float(raw["norm"]["eps"]),
        layers=layers,
        loop_start=int(loop.get("start", 0)),
        loop_stop=int(loop.get("stop", loop.get("start", 0))),
        loop_times=int(loop.get("times", 1)),
    )


def model_config_from_dict(raw: dict, model_path: Optional[str] = None,
                           name: str = ARCHITECTURE) -> ModelConfig:
    """Engine-level ModelConfig for a Pinuvik config dict (the registry's
    architecture hook)."""
    shapes = None
    if model_path:
        files = sorted(f for f in os.listdir(model_path)
                       if f.endswith(".safetensors"))
        shapes = {}
        for f in files:
            shapes.update(safetensors_shapes(os.path.join(model_path, f)))
    arch = parse_config(raw, shapes)
    first = arch.layers[0].left
    return ModelConfig(
        name=name,
        architecture=ARCHITECTURE,
        arch=arch,
        hidden_size=arch.width,
        num_layers=len(arch.layer_runs()),
        num_heads=first.heads,
        num_kv_heads=first.kv_heads,
        head_dim=first.dim,
        intermediate_size=max((L.ff for L in arch.layers), default=0),
        vocab_size=arch.vocab,
        rope_theta=first.rot_base,
        rms_norm_eps=arch.eps,
        qk_norm=True,
        model_path=model_path,
        max_position_embeddings=1 << 24,
    )


class PinuvikLM(nn.Module):
    """embedding -> layer runs -> scalar-gain final norm -> head.

    Engine interface (same as CausalLM): ``forward(ids, meta, caches)``
    returns the final-normed hidden rows, ``compute_logits`` applies the
    head. Additionally declares per-run cache/state needs
    (``allocate_caches``/``allocate_state``) and ``uses_state_slots`` so
    the runner builds sequence-grouped metadata and the scheduler hands
    out state slots."""

    uses_state_slots = True
    supports_prefix_caching = False   # recurrent state has no block form

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        assert ps.tp_world_size() == 1 and ps.pp_world_size() == 1, (
            "Pinuvik runs single-rank (TP/PP sharding of the parallel "
            "mixers is not implemented)")
        self.cfg = cfg
        arch: PinuvikConfig = cfg.arch
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
            left = SharedKVAttention(L.left, W, arch.eps, dtype)
            right = DeltaRuleMixer(L.right, W, arch.eps, dtype)
            mixer = ParallelMixer(left, right, W, dtype)
            mlp = GatedMLP(W, L.ff, dtype) if L.ff else None
            layers.append(MixerLayer(mixer, mlp, W, arch.eps, dtype))
        self.layers = nn.ModuleList(layers)
        self.runs = arch.layer_runs()
        self.final_norm = nn.Parameter(torch.ones(1, dtype=torch.float32),
                                       requires_grad=False)
        torch.manual_seed(base_seed + 1000003 * (len(arch.layers) + 2))
        self.lm_head = ReplicatedLinear(W, arch.vocab, dtype=dtype)
        torch.manual_seed(base_seed + 777)

    # ------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.runs)

    def kv_block_bytes(self, block_size: int) -> int:
        esize = torch.empty((), dtype=self.dtype).element_size()
        n = 0
        for li in self.runs:
            c = self.arch.layers[li].left
            n += 2 * c.kv_heads * block_size * c.dim * esize
        return n

    def allocate_caches(self, num_blocks: int, block_size: int,
                        num_slots: int, device) -> list:
        """One cache dict per layer RUN: paged k (processed keys) and v
        (raw keys) in the model dtype; fp32 token-shift and delta-rule
        state per slot."""
        caches = []
        W = self.arch.width
        for li in self.runs:
            layer = self.layers[li]
            shape = layer.mixer.left.cache_shape(num_blocks, block_size)
            caches.append({
                "k": torch.zeros(shape, dtype=self.dtype, device=device),
                "v": torch.zeros(shape, dtype=self.dtype, device=device),
                "shift": torch.zeros((num_slots, W), dtype=torch.float32,
                                     device=device),
                "delta": torch.zeros(
                    (num_slots,) + layer.mixer.right.state_shape(),
                    dtype=torch.float32, device=device),
            })
        return caches

    # ----------------------------------------------------------- forward
    def forward(self, input_ids, meta, caches, hidden=None, residual=None):
        resid = self.embed_tokens[input_ids].float()
        for li, cache in zip(self.runs, caches):
            resid = self.layers[li](resid, meta, cache)
        return seqmix.scalar_rms_norm(resid, self.final_norm, self.arch.eps,
                                      self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden)

    # ----------------------------------------------------------- weights
    def load_weights(self, tensors: Iterable[Tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names -> parameters. ``l<i>.mix.{left,right}.<branch>``
        rows land in the merged input projection; gains and biases are kept
        in fp32."""
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
        return n

    def expected_tensor_names(self) -> List[str]:
        names = ["embed", "head", "final.norm"]
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            names += [p + "norm1", p + "norm1b", p + "shift"]
            names += [p + "mix.left." + x for x in ("q", "k", "o", "out")]
            names += [p + "mix.right." + x for x in (
                "r", "k", "v", "g", "a", "a.b", "w1", "w2", "w0", "norm",
                "o", "out")]
            if layer.mlp is not None:
                names += [p + "norm2", p + "norm2b", p + "mlp.gate",
                          p + "mlp.up", p + "mlp.down"]
        return names

    @staticmethod
    def _put(param, value, rows=None):
        dst = param.data if rows is None else \
            param.data[rows[0]: rows[0] + rows[1]]
        value = value.reshape(dst.shape) if value.numel() == dst.numel() \
            else value
        if dst.shape != value.shape:
            raise ValueError(f"shape mismatch {tuple(value.shape)} vs "
                             f"{tuple(dst.shape)}")
        dst.copy_(value.to(dst.dtype))

    def _load_one(self, name: str, t: torch.Tensor) -> None:
        if name == "embed":
            return self._put(self.embed_tokens, t)
        if name == "head":
            return self._put(self.lm_head.weight, t)
        if name == "final.norm":
            return self._put(self.final_norm, t)
        lname, _, rest = name.partition(".")
        if not (lname.startswith("l") and lname[1:].isdigit()):
            raise ValueError(f"unknown tensor {name!r}")
        layer: MixerLayer = self.layers[int(lname[1:])]
        if rest in ("norm1", "norm1b", "norm2", "norm2b", "shift"):
            return self._put(getattr(layer, rest), t)
        mixer = layer.mixer
        if rest.startswith("mix."):
            _, side, branch = rest.split(".", 2)
            if branch == "out":
                return self._put(getattr(mixer, side + "_out"), t)
            half = getattr(mixer, side)
            if branch == "o":
                return self._put(half.o_proj.weight, t)
            direct = {"a.b": "a_bias", "w0": "w0", "norm": "norm_w"}
            if side == "right" and branch in direct:
                return self._put(getattr(half, direct[branch]), t)
            if side == "right" and branch == "w2":
                return self._put(half.w2.weight, t)
            return self._put(mixer.in_proj.weight, t,
                             mixer.in_proj_rows(side, branch))
        if rest.startswith("mlp.") and layer.mlp is not None:
            which = rest[4:]
            ff = layer.mlp.down_proj.weight.shape[1]
            if which == "gate":
                return self._put(layer.mlp.gate_up_proj.weight, t, (0, ff))
            if which == "up":
                return self._put(layer.mlp.gate_up_proj.weight, t, (ff, ff))
            if which == "down":
                return self._put(layer.mlp.down_proj.weight, t)
        raise ValueError(f"unknown tensor {name!r}")

    def export_weights(self) -> Dict[str, torch.Tensor]:
        """Inverse of load_weights (checkpoint naming), for writing
        random-init models to disk."""
        out = {"embed": self.embed_tokens.data, "head": self.lm_head.weight.data,
               "final.norm": self.final_norm.data.reshape(())}
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            m = layer.mixer
            for nm in ("norm1", "norm1b", "norm2", "norm2b"):
                if getattr(layer, nm) is not None:
                    out[p + nm] = getattr(layer, nm).data.reshape(())
            out[p + "shift"] = layer.shift.data
            for side, half in (("left", m.left), ("right", m.right)):
                for br in half.in_names:
                    a, n = m.in_proj_rows(side, br)
                    out[f"{p}mix.{side}.{br}"] = m.in_proj.weight.data[a:a + n]
                out[f"{p}mix.{side}.o"] = half.o_proj.weight.data
                out[f"{p}mix.{side}.out"] = getattr(m, side + "_out").data
            out[p + "mix.right.a.b"] = m.right.a_bias.data
            out[p + "mix.right.w0"] = m.right.w0.data
            out[p + "mix.right.norm"] = m.right.norm_w.data
            out[p + "mix.right.w2"] = m.right.w2.weight.data
            if layer.mlp is not None:
                ff = layer.mlp.down_proj.weight.shape[1]
                out[p + "mlp.gate"] = layer.mlp.gate_up_proj.weight.data[:ff]
                out[p + "mlp.up"] = layer.mlp.gate_up_proj.weight.data[ff:]
                out[p + "mlp.down"] = layer.mlp.down_proj.weight.data
        return {k: v.detach().clone().contiguous() for k, v in out.items()}

    def randomize_small_params(self, seed: int = 0) -> None:
        """Random-init use (benchmarks, tests): give gains, shifts and
        biases non-trivial values so every branch contributes."""
        g = torch.Generator().manual_seed(seed)

        def rnd(p, lo, hi):
            p.data.copy_((torch.rand(p.shape, generator=g) * (hi - lo) + lo)
                         .to(p.device))

        rnd(self.final_norm, 0.8, 1.2)
        for layer in self.layers:
            for nm in ("norm1", "norm1b", "norm2", "norm2b"):
                if getattr(layer, nm) is not None:
                    rnd(getattr(layer, nm), 0.5, 1.5)
            rnd(layer.shift, 0.0, 1.0)
            m = layer.mixer
            rnd(m.left_out, 0.5, 1.5)
            rnd(m.right_out, 0.5, 1.5)
            rnd(m.right.w0, -1.0, 1.0)
            rnd(m.right.a_bias, -1.0, 1.0)
            rnd(m.right.norm_w, 0.5, 1.5)
