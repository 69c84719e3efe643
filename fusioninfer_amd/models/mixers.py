"""Sequence-mixer building blocks beyond plain causal softmax attention.

Each block is a mechanism with its constants as constructor parameters, so
model designs assemble them freely:

* ``SharedKVAttention``  rotary attention whose values ARE the projected
  keys (no value projection), interleaved-pair partial rotary, unit-RMS
  q/k, explicit score scale, chunk and/or sliding-window masks; reads and
  writes the engine's paged cache.
* ``DeltaRuleMixer``     generalized delta rule (per-channel decay from a
  low-rank branch, per-channel removal rate), fp32 recurrent state kept in
  the engine's state slots, per-head unit-RMS output with gain and gate.
* ``ParallelMixer``      two mixers side by side on one input with ONE
  merged input projection; the halves are width-normalized and averaged by
  the caller's fused residual kernel.
* ``GatedMLP``           act(gate) * up -> down with a chosen activation.

Activations run in the model dtype (bf16 or fp32); statistics, rotary
angles, scores, decays, gates of the recurrence and the state are fp32
inside the ops (fusioninfer_amd/ops/seqmix.py).
"""

from __future__ import annotations

import dataclasses
import math
from typing import List, Optional

import torch
import torch.nn as nn

from fusioninfer_amd.distributed.layers import (
    MergedColumnParallelLinear,
    ReplicatedLinear,
    RowParallelLinear,
)
from fusioninfer_amd.ops import seqmix


@dataclasses.dataclass
class SharedKVAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # per-head query/key size
    vdim: int                # per-head value size (== dim: values are keys)
    scale: float             # score multiplier
    rot_dims: int            # leading dims of each head that rotate
    rot_base: float
    chunk: int = 0           # >0: keys only from the query's own chunk
    window: int = 0          # >0: keys only from the last `window` positions

    def __post_init__(self):
        if self.vdim != self.dim:
            raise ValueError(
                "shared key/value attention needs vdim == dim "
                f"(got dim={self.dim}, vdim={self.vdim})")
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.dim:
            raise ValueError("rot.dims must be even and <= dim")


@dataclasses.dataclass
class DeltaRuleConfig:
    heads: int
    dim: int                 # per-head key = value size
    decay_rank: int          # inner size of the low-rank decay branch
    # decay w = exp(-decay_scale * sigmoid(.)): the design's fixed constant
    decay_scale: float = math.exp(-0.5)


def _f32_param(shape, fill: float = 1.0) -> nn.Parameter:
    """Small gains/biases stay fp32 whatever the model dtype (they enter
    32-bit statistics only)."""
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32),
                        requires_grad=False)


def rotary_inv_freq(dims: int, base: float) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, rounded once to fp32 (angles are
    position * f_i in fp32)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / max(dims, 1))).to(torch.float32)


class SharedKVAttention(nn.Module):
    """Attention half: consumes its slice of the merged projection."""

    def __init__(self, cfg: SharedKVAttentionConfig, width: int, eps: float,
                 dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.q_size = cfg.heads * cfg.dim
        self.k_size = cfg.kv_heads * cfg.dim
        self.in_sizes = [self.q_size, self.k_size]
        self.in_names = ["q", "k"]
        self.o_proj = RowParallelLinear(cfg.heads * cfg.vdim, width,
                                        dtype=dtype)
        self.register_buffer(
            "inv_freq", rotary_inv_freq(cfg.rot_dims, cfg.rot_base),
            persistent=False)

    def cache_shape(self, num_blocks: int, block_size: int):
        c = self.cfg
        return (num_blocks, c.kv_heads, block_size, c.dim)

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, k = parts
        c = self.cfg
        k_cache, v_cache = cache["k"], cache["v"]
        qn = seqmix.rope_unitnorm_cache_(
            q, k, meta.positions, self.inv_freq, self.eps, k_cache, v_cache,
            meta.slot_mapping, c.heads, c.kv_heads, c.dim)
        o = seqmix.ranged_paged_attention(
            qn, k_cache, v_cache, meta.seq_bt, meta.row_seq, meta.positions,
            c.scale, chunk=c.chunk, window=c.window, seq_cu=meta.seq_cu,
            tiles=meta.seq_tiles)
        return self.o_proj(o.view(o.shape[0], c.heads * c.vdim))


class DeltaRuleMixer(nn.Module):
    """Recurrent half: r/k/v/gate/removal/decay branches come from the
    merged projection; the decay branch is low-rank (tanh between)."""

    def __init__(self, cfg: DeltaRuleConfig, width: int, eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        n = cfg.heads * cfg.dim
        self.in_sizes = [n, n, n, n, n, cfg.decay_rank]
        self.in_names = ["r", "k", "v", "g", "a", "w1"]
        self.w2 = ReplicatedLinear(cfg.decay_rank, n, dtype=dtype)
        self.w0 = _f32_param((n,), 0.0)
        self.a_bias = _f32_param((n,), 0.0)
        self.norm_w = _f32_param((n,), 1.0)
        self.o_proj = RowParallelLinear(n, width, dtype=dtype)

    def state_shape(self):
        c = self.cfg
        return (c.heads, c.dim, c.dim)

    def forward(self, parts, meta, cache) -> torch.Tensor:
        r, k, v, g, a, w1 = parts
        c = self.cfg
        wlin = self.w2(torch.tanh(w1))
        o = seqmix.delta_rule(
            r, k, v, wlin, a, g, self.w0, self.a_bias, self.norm_w,
            cache["delta"], meta.seq_cu, meta.seq_slots, meta.positions,
            c.heads, c.dim, self.eps, c.decay_scale)
        return self.o_proj(o)


class ParallelMixer(nn.Module):
    """Two mixers reading the same input through one merged GEMM. Returns
    both halves' projected outputs and their width gains; the caller's
    fused kernel normalizes, averages and adds them to the residual."""

    def __init__(self, left: nn.Module, right: nn.Module, width: int, dtype):
        super().__init__()
        self.left = left
        self.right = right
        self.sizes: List[int] = list(left.in_sizes) + list(right.in_sizes)
        self.n_left = len(left.in_sizes)
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  dtype=dtype)
        self.left_out = _f32_param((width,), 1.0)
        self.right_out = _f32_param((width,), 1.0)

    def in_proj_rows(self, side: str, name: str):
        """(row offset, rows) of a named branch inside the merged weight."""
        names = [("left", n) for n in self.left.in_names] + \
                [("right", n) for n in self.right.in_names]
        off = 0
        for (s, n), size in zip(names, self.sizes):
            if (s, n) == (side, name):
                return off, size
            off += size
        raise KeyError((side, name))

    def forward(self, h, meta, cache):
        parts = self.in_proj(h).split(self.sizes, dim=-1)
        yl = self.left(parts[: self.n_left], meta, cache)
        yr = self.right(parts[self.n_left:], meta, cache)
        return yl, yr


class GatedMLP(nn.Module):
    """down(act(gate(x)) * up(x)); ``act`` names the fused activation."""

    def __init__(self, width: int, ff: int, dtype, act: str = "gelu_tanh"):
        super().__init__()
        if act != "gelu_tanh":
            raise ValueError(f"unsupported gated-MLP activation {act!r}")
        self.gate_up_proj = MergedColumnParallelLinear(width, [ff, ff],
                                                       dtype=dtype)
        self.down_proj = RowParallelLinear(ff, width, dtype=dtype)

    def forward(self, x):
        return self.down_proj(seqmix.gelu_tanh_and_mul(self.gate_up_proj(x)))


class MixerLayer(nn.Module):
    """Pre- and post-normed residual layer on an fp32 stream with
    scalar-gain RMS norms and a token shift in front of the mixer:

        x <- x + norm1b(mixer(shift(norm1(x))));  x <- x + norm2b(ff(norm2(x)))
    """

    def __init__(self, mixer: ParallelMixer, mlp: Optional[GatedMLP],
                 width: int, eps: float, dtype):
        super().__init__()
        self.mixer = mixer
        self.mlp = mlp
        self.eps = eps
        self.dtype = dtype
        self.norm1 = _f32_param((1,))
        self.norm1b = _f32_param((1,))
        self.norm2 = _f32_param((1,)) if mlp is not None else None
        self.norm2b = _f32_param((1,)) if mlp is not None else None
        self.shift = _f32_param((width,), 0.0)

    def forward(self, resid, meta, cache):
        h = seqmix.norm_token_shift(
            resid, self.norm1, self.shift, cache["shift"], meta.seq_cu,
            meta.row_seq, meta.positions, meta.seq_slots, self.eps,
            self.dtype)
        yl, yr = self.mixer(h, meta, cache)
        h2 = seqmix.dual_norm_combine_residual_(
            resid, yl, yr, self.mixer.left_out, self.mixer.right_out,
            self.norm1b, self.eps, self.norm2, self.dtype)
        if self.mlp is not None:
            seqmix.residual_add_scalar_norm_(
                resid, self.mlp(h2), self.norm2b, self.eps)
        return resid
