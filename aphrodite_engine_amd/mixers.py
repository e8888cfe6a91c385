"""Sequence-mixer building blocks beside the rotary softmax attention of ``attention/``: each is a mechanism with its
constants as parameters, says what cache it needs per layer run (``cache_spec``), and runs on a ``StepBatch`` -- prompt
portions and decoded tokens in one launch -- through the kernels of ``mixer_ops``.

  DistanceBiasAttention   grouped-query softmax attention over a token-major paged cache; no rotation: positions enter as
                          an additive per-head bias looked up by (bucketed) distance and as a query temperature that
                          grows with the logarithm of the position; optional per-head sigmoid output gate
  OuterProductMemory      a matrix state per head in a per-request slot: decay linear attention (fixed per-head decay) or
                          the mLSTM cell (exponential gating under a running maximum, normaliser vector)
  LayerNormParams, GatedMLP  the norm with weight and bias around an fp32 residual stream; gate * up feed-forward
  WindowedMapsAttention   softmax attention under a sliding window that keeps the sequence's first tokens, no rotation, with a
                          short causal convolution over time on q, k and v (its last inputs in a per-request slot) and
                          several maps per head over shared values, joined differentially (a_1 - lambda a_2), unit RMS per
                          head, elementwise sigmoid gate; may read another layer's keys and values instead of its own
  PolyNormMLP             down(a N(z) + b N(z^2) + c N(z^3) + e), z = up(x), N = division by the row's root mean square
  RoutedExperts           softmax router with a choice correction (or a sigmoid router whose choice is limited to the best groups
                          of neighbouring experts), clamped or plain gated experts, identity experts, gated shared expert
  HashedPairEmbedding     token embedding plus a row of a second table picked by a hash of (previous token, token); the previous
                          token of every live request in a per-request slot
  RotaryFrequencies       rotation frequencies with YaRN's blend of interpolated and original frequencies and its magnitude factor
  LatentAttention         softmax attention through a low-rank latent: a token caches one row [normed latent | one rotated key part
                          shared by all heads]; queries go through a latent of their own; elementwise sigmoid output gate
  ClampedGLUMLP           down(g * sigmoid(alpha g) * (u + 1)) with g and u clamped, biased projections
  StreamedResidual        a residual carried as several streams that sublayers read through a learned combination and write back
                          through a learned mixing matrix (hyper-connections), with a per-channel scale on every sublayer's result
  GatedDeltaMixer         the gated delta rule: a matrix state per head that forgets, corrects what it holds under the key and is
                          read after the write; short causal convolutions with silu on q, k and v; unit-norm q and k
  RotaryGQAttention       causal grouped-query softmax attention with a (partial) rotation, optional unit RMS of q and k after it
                          and optional blending of the values with an earlier layer's values of the same tokens
"""
import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
from torch import nn

from . import mixer_ops as mops
from .step_batch import StepBatch


@dataclass(frozen=True)
class PagedKVSpec:
    """A token-major paged key / value cache: K [blocks, block, kv_heads * maps, dim], V [blocks, block, kv_heads, vdim]
    (``maps`` key rows per kv head share one value row: the maps of differential attention)."""
    kv_heads: int
    dim: int
    vdim: int
    maps: int = 1

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return (torch.zeros(num_blocks, block_size, self.kv_heads * self.maps, self.dim, dtype=dtype, device=device),
                torch.zeros(num_blocks, block_size, self.kv_heads, self.vdim, dtype=dtype, device=device))


@dataclass(frozen=True)
class ConvStateSpec:
    """The last taps - 1 inputs of a short causal convolution over ``channels`` channels, one entry per request slot."""
    channels: int
    taps: int

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return torch.zeros(num_slots, max(self.taps - 1, 0), self.channels, dtype=dtype, device=device)


@dataclass(frozen=True)
class LatentCacheSpec:
    """A paged cache of one row per token that all heads share: [blocks, block, rank + rot_dim]."""
    rank: int
    rot_dim: int

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return torch.zeros(num_blocks, block_size, self.rank + self.rot_dim, dtype=dtype, device=device)


@dataclass(frozen=True)
class TokenStateSpec:
    """The last token of every live request, one int32 per request slot."""

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return torch.zeros(num_slots, dtype=torch.int32, device=device)


@dataclass(frozen=True)
class MemoryStateSpec:
    """fp32 state of an OuterProductMemory, one entry per request slot."""
    heads: int
    dim: int
    vdim: int
    mode: int

    def allocate(self, num_blocks: int, block_size: int, num_slots: int, dtype, device):
        return tuple(torch.zeros(s, dtype=torch.float32, device=device)
                     for s in mops.memory_state_shapes(num_slots, self.heads, self.dim, self.vdim, self.mode))


def log_distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of a [rows, heads] bias table for a key ``n`` positions back: exact rows below rows // 2, then rows that widen
    geometrically and reach the last one at distance ``far``."""
    half = rows // 2
    if n < half or rows == 1:
        return min(n, rows - 1)
    if far <= half:
        return rows - 1
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


class LayerNormParams(nn.Module):
    def __init__(self, width: int, dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(width, dtype=dtype), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(width, dtype=dtype), requires_grad=False)

    def pair(self) -> Tuple[torch.Tensor, torch.Tensor]:
        return self.weight, self.bias


class DistanceBiasAttention(nn.Module):
    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, bias_rows: int = 0,
                 bias_far: float = 0.0, temp_coef: float = 0.0, temp_every: int = 1):
        super().__init__()
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads over {kv_heads} key/value heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.bias_far = float(scale), float(bias_far)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        # the learned table stays fp32 (it is added to fp32 scores); ``finalize`` tabulates it by distance
        self.rel = nn.Parameter(torch.zeros(bias_rows, heads, dtype=torch.float32), requires_grad=False) if bias_rows else None
        self.bias_lut = None

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.kv_heads, self.dim, self.vdim)

    def finalize(self) -> None:
        """bias_lut[h, n] = rel[bucket(n), h] up to the first distance of the last row; farther keys clamp to it."""
        if self.rel is None:
            return
        rows = self.rel.shape[0]
        reach = max(rows // 2, int(math.ceil(self.bias_far))) + 1
        idx = torch.tensor([log_distance_bucket(n, rows, self.bias_far) for n in range(reach + 1)], device=self.rel.device)
        if int(idx[-1]) != rows - 1:
            raise ValueError("the distance bias does not reach its last row")
        self.bias_lut = self.rel.index_select(0, idx).t().contiguous()

    def forward(self, out: torch.Tensor, q, k, v, gate, cache, batch: StepBatch, out_scale: float = 1.0) -> None:
        k_cache, v_cache = cache
        mops.paged_kv_write(k_cache, v_cache, k, v, batch.slot_mapping)
        mops.distance_bias_attention(out, q, gate, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len,
                                     batch.ctx_len, batch.seq_of_token, (min(batch.q_lens), max(batch.q_lens)), self.heads,
                                     self.scale, self.bias_lut, self.temp_coef, self.temp_every, out_scale,
                                     max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))


class OuterProductMemory(nn.Module):
    def __init__(self, mode: int, heads: int, dim: int, vdim: int, decay: Optional[List[float]] = None,
                 q_scale: float = 1.0, gate_cap: float = 1.0):
        super().__init__()
        self.mode, self.heads, self.dim, self.vdim = mode, heads, dim, vdim
        self.q_scale, self.gate_cap = float(q_scale), float(gate_cap)
        if mode == mops.MEMORY_DECAY:
            if decay is None or len(decay) != heads:
                raise ValueError("decay linear attention takes one decay per head")
            self.register_buffer("decay", torch.tensor(decay, dtype=torch.float32), persistent=False)
        else:
            self.decay = None

    def cache_spec(self) -> MemoryStateSpec:
        return MemoryStateSpec(self.heads, self.dim, self.vdim, self.mode)

    def forward(self, q, k, v, state, batch: StepBatch, gate_i=None, gate_f=None) -> torch.Tensor:
        return mops.outer_memory_scan(q, k, v, state, batch.state_slots, batch.q_start, batch.q_len, batch.ctx_len,
                                      self.heads, self.mode, self.decay, gate_i, gate_f, self.q_scale, self.gate_cap,
                                      max_q_len=max(batch.q_lens))


class GatedMLP(nn.Module):
    """down(act(gate x) * (up x)) with gate and up as one product."""

    def __init__(self, width: int, ff: int, act: int, dtype, prefix: str = ""):
        super().__init__()
        from .model import QuantLinear
        self.act = act
        self.gate_up = QuantLinear(width, [ff, ff], None, dtype, prefix=prefix + "gate_up")
        self.down = QuantLinear(ff, [width], None, dtype, prefix=prefix + "down")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(mops.act_and_mul(self.gate_up(h), self.act))


class WindowedMapsAttention(nn.Module):
    """The mechanism only: takes the rows of the fused input product [q | k | v | ...] and leaves the gated, normed head
    outputs; the projections around it belong to the model.  ``own_kv`` False: the layer has queries only and attends over
    the cache another layer wrote (same head counts and sizes)."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, keep_first: int, taps: int,
                 diff: float, eps: float, dtype, maps: int = 2, own_kv: bool = True):
        super().__init__()
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads over {kv_heads} key/value heads")
        if maps not in (1, 2):
            raise ValueError("one map (plain attention) or two (differential attention)")
        if taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.heads, self.kv_heads, self.dim, self.vdim, self.maps = heads, kv_heads, dim, vdim, maps
        self.scale, self.window, self.keep_first, self.taps = float(scale), int(window), int(keep_first), int(taps)
        self.diff, self.eps, self.own_kv = float(diff), float(eps), own_kv
        self.cq = heads * maps * dim
        self.ck = kv_heads * maps * dim if own_kv else 0
        self.cv = kv_heads * vdim if own_kv else 0
        self.channels = self.cq + self.ck + self.cv
        self.conv = nn.Parameter(torch.zeros(self.channels, taps, dtype=dtype), requires_grad=False)
        # lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number per layer, fp32 (finalize)
        self.lq1, self.lk1, self.lq2, self.lk2 = (nn.Parameter(torch.zeros(dim, dtype=torch.float32), requires_grad=False)
                                                  for _ in range(4))
        self.lam = 0.0

    def kv_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.kv_heads, self.dim, self.vdim, self.maps)

    def state_spec(self) -> ConvStateSpec:
        return ConvStateSpec(self.channels, self.taps)

    def finalize(self) -> None:
        if self.maps == 2:
            self.lam = float(torch.exp(torch.dot(self.lq1.float(), self.lk1.float()))
                             - torch.exp(torch.dot(self.lq2.float(), self.lk2.float()))) + self.diff

    def forward(self, out: torch.Tensor, qkv: torch.Tensor, gate: Optional[torch.Tensor], kv_cache, conv_state,
                batch: StepBatch) -> None:
        """qkv [T, channels] rows of the input product (q only for a layer that shares another's cache); gate [T, heads * vdim]
        raw; out [T, heads * vdim]."""
        k_cache, v_cache = kv_cache
        q = mops.short_conv(qkv, self.conv, conv_state, batch.state_slots, batch.q_start, batch.q_len, batch.ctx_len,
                            batch.seq_of_token, self.cq, self.ck, self.cv, k_cache if self.own_kv else None,
                            v_cache if self.own_kv else None, batch.slot_mapping if self.own_kv else None)
        lens = (min(batch.q_lens), max(batch.q_lens))
        if self.maps == 2 and mops.differential_window_attention_supported(self.heads, self.kv_heads, self.dim, self.vdim, q.dtype) \
                and (gate is None or gate.stride(0) % 4 == 0):
            mops.differential_window_attention(out, q, gate, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len,
                                               batch.ctx_len, batch.seq_of_token, lens, self.heads, self.scale, self.window,
                                               self.keep_first, self.lam, 1.0 - self.diff, self.eps,
                                               max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))
            return
        a = mops.windowed_attention(q, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len, batch.ctx_len,
                                    batch.seq_of_token, (min(batch.q_lens), max(batch.q_lens)), self.heads, self.maps, self.scale,
                                    self.window, self.keep_first,
                                    max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))
        mops.differential_norm_gate(out, a, gate, self.heads, self.maps, self.vdim, self.lam,
                                    1.0 - self.diff if self.maps == 2 else 1.0, self.eps)


class PolyNormMLP(nn.Module):
    def __init__(self, width: int, ff: int, eps: float, dtype, prefix: str = ""):
        super().__init__()
        from .model import QuantLinear
        self.eps = float(eps)
        self.up = QuantLinear(width, [ff], None, dtype, prefix=prefix + "up")
        self.down = QuantLinear(ff, [width], None, dtype, prefix=prefix + "down")
        self.act = nn.Parameter(torch.zeros(4, dtype=torch.float32), requires_grad=False)
        self.coef = (0.0, 0.0, 0.0, 0.0)

    def finalize(self) -> None:
        self.coef = tuple(float(c) for c in self.act.tolist())

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(mops.poly_norm(self.up(h), self.coef, self.eps))


class RoutedExperts(nn.Module):
    """``experts`` clamped gated feed-forwards of which a token uses ``top``, chosen by softmax score plus a correction and
    weighted by the score itself; the last ``identity`` router outputs stand for experts that return their input; an optional
    shared expert runs for every token, times sigmoid of a one-row product.  The router runs in fp32."""

    def __init__(self, width: int, ff: int, experts: int, top: int, identity: int, limit: float, dtype, shared_ff: int = 0,
                 shared_limit: float = 0.0, alpha: float = 1.702, prefix: str = "", score: str = "softmax", groups: int = 1,
                 keep: int = 1, group_top: int = 2, route_scale: float = 1.0, shared_gate: bool = True):
        """``limit`` <= 0: experts of the plain gated form gate * sigmoid(alpha gate) * up (alpha 1: silu).  ``score``
        "sigmoid_grouped": scores are sigmoid(router output); the experts form ``groups`` equal groups of neighbours, a group's
        score is the sum of its ``group_top`` largest scores, only experts of the ``keep`` best groups can be chosen; the
        weights are the chosen scores times ``route_scale``.  ``score`` "topk_softmax": router output plus a learned bias; the
        ``top`` largest are chosen and weighted by the softmax over the chosen ones alone.  ``shared_gate`` False: the shared
        expert is added as it is."""
        super().__init__()
        from .model import QuantLinear
        self.width, self.ff, self.experts, self.top, self.identity = width, ff, experts, top, identity
        self.limit, self.alpha, self.shared_ff, self.shared_limit = float(limit), float(alpha), shared_ff, float(shared_limit)
        self.score, self.groups, self.keep, self.group_top, self.route_scale = score, int(groups), int(keep), int(group_top), float(route_scale)
        if not 0 < top <= experts + identity:
            raise ValueError(f"top {top} of {experts} + {identity} experts")
        if score not in ("softmax", "sigmoid_grouped", "topk_softmax"):
            raise ValueError(f"router score {score!r}")
        if score == "sigmoid_grouped":
            if identity or groups < 1 or experts % groups or not 0 < keep <= groups or top > keep * (experts // groups):
                raise ValueError(f"{experts} experts in {groups} groups of which {keep} are kept, top {top}")
        self.router = nn.Parameter(torch.zeros(experts + identity, width, dtype=torch.float32), requires_grad=False)
        self.correction = nn.Parameter(torch.zeros(experts + identity, dtype=torch.float32), requires_grad=False) \
            if score == "softmax" else None
        if score == "topk_softmax" and identity:
            raise ValueError("identity experts belong to the softmax router")
        self.router_bias = nn.Parameter(torch.zeros(experts, dtype=torch.float32), requires_grad=False) \
            if score == "topk_softmax" else None
        self.shared_gate = bool(shared_gate)
        self.w_gate_up = nn.Parameter(torch.zeros(experts, 2 * ff, width, dtype=dtype), requires_grad=False)
        self.w_down = nn.Parameter(torch.zeros(experts, width, ff, dtype=dtype), requires_grad=False)
        if shared_ff:
            # [gate | up | the one-row gate | zero rows up to a multiple of 8]: one product for everything that reads h
            self.shared_splits = [shared_ff, shared_ff, 1, (-(2 * shared_ff + 1)) % 8 or 8] if shared_gate else \
                [shared_ff, shared_ff] + ([-(2 * shared_ff) % 8] if (2 * shared_ff) % 8 else [])
            self.shared_in = QuantLinear(width, self.shared_splits, None, dtype, prefix=prefix + "shared.in")
            self.shared_in.weight.data.zero_()
            self.shared_down = QuantLinear(shared_ff, [width], None, dtype, prefix=prefix + "shared.down")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        z = torch.nn.functional.linear(h.float(), self.router)
        if self.score == "sigmoid_grouped":
            ids, w = mops.experts_route_grouped(z, self.top, self.groups, self.keep, self.route_scale, self.group_top)
        elif self.score == "topk_softmax":
            ids, w = mops.experts_route_topk(z, self.router_bias, self.top)
        else:
            ids, w = mops.experts_route(z, self.correction, self.top)
        shared = gate = None
        if self.shared_ff:
            s_in = self.shared_in(h)
            shared = self.shared_down(mops.clamped_glu(s_in, self.shared_ff, self.shared_limit, self.alpha))
            if self.shared_gate:
                gate = s_in[:, 2 * self.shared_ff:2 * self.shared_ff + 1]
        return mops.experts_forward(h, ids, w, self.w_gate_up, self.w_down, self.limit, self.alpha, shared, gate)


class HashedPairEmbedding(nn.Module):
    """x = table[token] + pair_table[(previous * mul_prev + token * mul_cur) mod buckets]; a sequence's first token takes the
    table's last row (number ``buckets``).  The previous token is state: one int32 per request slot (``state_spec``), read for
    the first row of a segment that continues a sequence and advanced to the segment's last token."""

    def __init__(self, vocab: int, width: int, buckets: int, mul_prev: int, mul_cur: int, dtype):
        super().__init__()
        if buckets < 1:
            raise ValueError("a hashed pair table needs at least one bucket")
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        self.table = nn.Parameter(torch.empty(vocab, width, dtype=dtype), requires_grad=False)
        self.pair_table = nn.Parameter(torch.empty(buckets + 1, width, dtype=dtype), requires_grad=False)

    def state_spec(self) -> TokenStateSpec:
        return TokenStateSpec()

    def forward(self, batch: StepBatch, token_state: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return mops.hashed_pair_embed(self.table, self.pair_table, batch.input_ids, token_state, batch.state_slots, batch.q_start,
                                      batch.q_len, batch.ctx_len, batch.seq_of_token, self.mul_prev, self.mul_cur, out=out)


class RotaryFrequencies:
    """Frequencies f_i = base^(-2 i / dims), i < dims / 2, of a rotation that pairs number i with number i + dims / 2, and the
    factor on cos and sin.  With YaRN scaling (factor, original length, fast and slow turn counts): a linear ramp over i between
    the numbers that turn ``fast`` and ``slow`` times over the original length blends f_i / factor (ramp 1) with f_i (ramp 0),
    and cos and sin are multiplied by 0.1 ln(factor) + 1."""

    def __init__(self, dims: int, base: float, factor: Optional[float] = None, original: Optional[float] = None,
                 fast: Optional[float] = None, slow: Optional[float] = None):
        if dims < 0 or dims % 2:
            raise ValueError(f"{dims} rotated numbers: pairs are needed")
        self.dims = int(dims)
        half = dims // 2
        f = [float(base) ** (-2.0 * i / dims) for i in range(half)]
        self.mscale = 1.0
        if factor is not None:
            def number_turning(turns: float) -> float:
                return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
            lo = max(math.floor(number_turning(fast)), 0)
            hi = min(math.ceil(number_turning(slow)), dims - 1)
            for i in range(half):
                ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
            self.mscale = 0.1 * math.log(factor) + 1.0
        self.inv_freq = torch.tensor(f, dtype=torch.float32)

    @staticmethod
    def wavelength_scaled(dims: int, base: float, factor: float, low: float, high: float, original: float) -> "RotaryFrequencies":
        """Frequencies scaled by wavelength l = 2 pi / f: kept where l < original / high, divided by ``factor`` where
        l > original / low, and between the two blended (1 - s) f / factor + s f with s = (original / l - low) / (high - low).
        cos and sin keep their magnitude."""
        rf = RotaryFrequencies(dims, base)
        f = rf.inv_freq.double()
        wave = 2.0 * math.pi / f
        s = ((original / wave - low) / (high - low)).clamp(0.0, 1.0) if high != low else torch.ones_like(f)
        blended = (1.0 - s) * f / factor + s * f
        out = torch.where(wave < original / high, f, torch.where(wave > original / low, f / factor, blended))
        rf.inv_freq = out.float()
        return rf

    def to(self, device) -> "RotaryFrequencies":
        self.inv_freq = self.inv_freq.to(device)
        return self


def interleaved_to_half(t: torch.Tensor, dims: int, at: int = 0) -> torch.Tensor:
    """Reorders ROWS at .. at + dims of a projection's weight so that a rotation that pairs number 2 i with number 2 i + 1
    becomes the one that pairs number i with number i + dims / 2: new row i is old row 2 i, new row dims / 2 + i is old row
    2 i + 1.  Scores are dot products of a query and a key part reordered alike, so they do not change."""
    idx = torch.arange(t.shape[0])
    idx[at:at + dims] = at + torch.cat([torch.arange(0, dims, 2), torch.arange(1, dims, 2)])
    return t.index_select(0, idx.to(t.device))


class LatentAttention(nn.Module):
    """Causal softmax attention whose keys and values are products of a cached low-rank latent.

      c_q = norm(W_dq h), q = W_uq c_q = per head [q_n (dim) | q_r (rot_dim)];   W_dkv h = [c (kv_rank) | k_r (rot_dim)], c normed
      key of head a = [W_uk,a c | rot(k_r)], value = W_uv,a c;  score = (q_n . W_uk,a c + rot(q_r) . rot(k_r)) * scale
      out = W_o (heads * sigmoid(W_g h))

    Every projection that reads h -- W_dq, W_dkv, W_g -- is one product.  The attention itself runs in the latent (the cache
    holds [c | rot(k_r)] per token and nothing per head): q_lat,a = W_uk,a^T q_n,a is a batched product over heads, the kernel
    returns sum_j p_ij c_j per head, and W_uv,a is applied to that, again batched over heads."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float,
                 rotary: RotaryFrequencies, eps: float, dtype, prefix: str = "", gate: bool = True, window: int = 0,
                 sink: bool = False):
        """``q_rank`` 0: queries are a plain projection of h (no query latent).  ``gate`` False: no output gate.  ``window`` > 0:
        a row sees itself and the window - 1 tokens before it.  ``sink``: a learned number per head whose exponential joins the
        softmax denominator."""
        super().__init__()
        from .loader import merged_plan
        from .model import QuantLinear
        if rotary.dims > rot_dim:
            raise ValueError(f"{rotary.dims} rotated numbers in a rotary part of {rot_dim}")
        self.heads, self.dim, self.rot_dim, self.vdim, self.q_rank, self.kv_rank = heads, dim, rot_dim, vdim, q_rank, kv_rank
        self.scale, self.eps, self.rotary = float(scale), float(eps), rotary
        self.window, self.gated = max(int(window), 0), bool(gate)
        self.names = ["dq" if q_rank else "q", "dkv"] + (["g"] if gate else [])
        self.splits = [q_rank if q_rank else heads * (dim + rot_dim), kv_rank + rot_dim] + ([heads * vdim] if gate else [])
        self.n_named = len(self.splits)
        pad = -sum(self.splits) % 8               # rows of the fused product stay 16-byte multiples
        if pad:
            self.splits.append(pad)
        self.in_proj = QuantLinear(width, self.splits, None, dtype, prefix=prefix + "in_proj", plan=merged_plan(self.splits))
        self.in_proj.weight.data.zero_()
        self.q_norm = nn.Parameter(torch.ones(q_rank, dtype=dtype), requires_grad=False) if q_rank else None
        self.kv_norm = nn.Parameter(torch.ones(kv_rank, dtype=dtype), requires_grad=False)
        self.uq = QuantLinear(q_rank, [heads * (dim + rot_dim)], None, dtype, prefix=prefix + "uq") if q_rank else None
        self.sink = nn.Parameter(torch.zeros(heads, dtype=torch.float32), requires_grad=False) if sink else None
        self.w_uk = nn.Parameter(torch.zeros(heads, dim, kv_rank, dtype=dtype), requires_grad=False)      # rows of W_uk, head by head
        self.w_uv = nn.Parameter(torch.zeros(heads, vdim, kv_rank, dtype=dtype), requires_grad=False)
        self.out_proj = QuantLinear(heads * vdim, [width], None, dtype, prefix=prefix + "out_proj")

    def cache_spec(self) -> LatentCacheSpec:
        return LatentCacheSpec(self.kv_rank, self.rot_dim)

    def finalize(self) -> None:
        self.rotary.to(self.w_uk.device)

    def forward(self, h: torch.Tensor, cache: torch.Tensor, batch: StepBatch) -> torch.Tensor:
        T, H, d, P, e, R = h.shape[0], self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        rot = self.rotary
        proj = self.in_proj(h)
        cq = mops.latent_prep(proj, 0, self.q_rank, self.splits[0], R, P, rot.dims, self.q_norm, self.kv_norm, cache,
                              batch.slot_mapping, batch.q_start, batch.ctx_len, batch.seq_of_token, rot.inv_freq, rot.mscale, self.eps)
        if self.q_rank:
            q = self.uq(cq).view(T, H, d + P)
        else:
            q = proj.as_strided((T, H, d + P), (proj.stride(0), d + P, 1))
        q_lat = torch.empty(T, H, R, dtype=h.dtype, device=h.device)
        torch.bmm(q[:, :, :d].transpose(0, 1), self.w_uk, out=q_lat.transpose(0, 1))
        o_lat = torch.empty(T, H, R, dtype=h.dtype, device=h.device)
        mops.latent_attention(o_lat, q_lat, q[:, :, d:] if P else None, cache, batch.block_tables, batch.q_start, batch.q_len,
                              batch.ctx_len, batch.seq_of_token, (min(batch.q_lens), max(batch.q_lens)), rot.inv_freq, rot.mscale,
                              rot.dims, self.scale, max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)),
                              window=self.window, sink=self.sink)
        o = torch.empty(T, H, e, dtype=h.dtype, device=h.device)
        torch.bmm(o_lat.transpose(0, 1), self.w_uv.transpose(1, 2), out=o.transpose(0, 1))
        o = o.view(T, H * e)
        if self.gated:
            g_at = self.splits[0] + R + P
            mops.sigmoid_gate_mul(o, proj[:, g_at:g_at + H * e], out=o)
        return self.out_proj(o)


class ClampedGLUMLP(nn.Module):
    """down(g * sigmoid(alpha g) * (u + 1)), g = min(gate h, limit), u = clamp(up h, +-limit); gate and up are one product;
    every projection may carry a bias."""

    def __init__(self, width: int, ff: int, limit: float, dtype, alpha: float = 1.702, bias: bool = True, prefix: str = ""):
        super().__init__()
        from .model import QuantLinear
        self.ff, self.limit, self.alpha = ff, float(limit), float(alpha)
        self.gate_up = QuantLinear(width, [ff, ff], None, dtype, prefix=prefix + "gate_up", bias=bias)
        self.down = QuantLinear(ff, [width], None, dtype, prefix=prefix + "down", bias=bias)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(mops.clamped_glu(self.gate_up(h), self.ff, self.limit, self.alpha))


class StreamedResidual:
    """Hyper-connections: the residual is ``streams`` copies x_1 .. x_n (all equal to the embedding at the start).  A sublayer
    reads u = sum_s a_in[s] x_s (through its norm) and writes, all streams at once from the old ones,
    x_t <- sum_s a_mix[s][t] x_s + mult * a_out[t] * (scale (.) y).  What leaves the stack is the sum of the streams.  One
    ``step`` is one launch: the write of the sublayer that has just run and the read (with the RMS norm) of the next one.
    With one stream and no coefficients this is the plain pre-norm residual x += mult * scale (.) y."""

    def __init__(self, streams: int, mult: float, eps: float, dtype):
        if streams < 1:
            raise ValueError("a residual has at least one stream")
        self.streams, self.mult, self.eps, self.dtype = int(streams), float(mult), float(eps), dtype

    def start(self, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """x fp32 [T, streams, W]: every stream is the embedding."""
        x = torch.empty(ids.shape[0], self.streams, table.shape[1], dtype=torch.float32, device=table.device)
        rows = ids if self.streams == 1 else ids.repeat_interleave(self.streams)       # row t * streams + s is token t
        mops.embed_scale(table, rows, 1.0, out=x.view(-1, table.shape[1]))
        return x

    def step(self, x: torch.Tensor, y: Optional[torch.Tensor], wrote, reads, weight: Optional[torch.Tensor], want_sum: bool = False):
        """``wrote``: the coefficient set (mix rows, out, scale tensor) of the sublayer whose result ``y`` is, or None;
        ``reads``: the in coefficients of the next sublayer (None: ones -- the sum of the streams)."""
        mix, out, scale = wrote if wrote is not None else (None, None, None)
        return mops.hyper_residual_rms_norm(x, y, scale, mix, out, self.mult, reads, weight, self.eps, dtype=self.dtype, want_sum=want_sum)


class GatedDeltaMixer(nn.Module):
    """The gated delta rule with its projections.  ONE input product gives q, k (kv_heads x dim), v and the output gate
    (heads x vdim each) and the two per-head numbers behind beta and the decay; q, k and v pass a short causal convolution over
    time with silu (its last inputs live in a per-request slot); q and k become unit vectors per head (q also times dim^-1/2);
    per head  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q  with beta = sigmoid(.), g = exp(-exp(A_log)
    softplus(. + dt_bias)); o is divided by its root mean square over the head, times a weight shared by the heads, times
    silu(gate); then the output product.  The state S is fp32 in a per-request slot and starts at zero."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, eps: float, dtype, prefix: str = "",
                 norm_eps: float = 1e-6):
        super().__init__()
        from .loader import merged_plan
        from .model import QuantLinear
        if heads % kv_heads:
            raise ValueError(f"{heads} value heads over {kv_heads} query/key heads")
        if taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps = heads, kv_heads, dim, vdim, int(taps)
        self.eps, self.norm_eps = float(eps), float(norm_eps)
        self.names = ["q", "k", "v", "g", "b", "a"]
        self.splits = [kv_heads * dim, kv_heads * dim, heads * vdim, heads * vdim, heads, heads]
        pad = -sum(self.splits) % 8               # rows of the fused product stay 16-byte multiples
        if pad:
            self.splits.append(pad)
        self.channels = sum(self.splits[:3])
        self.in_proj = QuantLinear(width, self.splits, None, dtype, prefix=prefix + "in_proj", plan=merged_plan(self.splits))
        self.in_proj.weight.data.zero_()
        self.conv = nn.Parameter(torch.zeros(self.channels, self.taps, dtype=dtype), requires_grad=False)
        self.a_log = nn.Parameter(torch.zeros(heads, dtype=torch.float32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(heads, dtype=torch.float32), requires_grad=False)
        self.out_norm = nn.Parameter(torch.ones(vdim, dtype=dtype), requires_grad=False)
        self.out_proj = QuantLinear(heads * vdim, [width], None, dtype, prefix=prefix + "out_proj")

    def cache_specs(self):
        """(convolution state, matrix state)"""
        return ConvStateSpec(self.channels, self.taps), MemoryStateSpec(self.heads, self.dim, self.vdim, mops.MEMORY_DECAY)

    def forward(self, h: torch.Tensor, conv_state: torch.Tensor, state, batch: StepBatch) -> torch.Tensor:
        H, G, d, e = self.heads, self.kv_heads, self.dim, self.vdim
        proj = self.in_proj(h)
        qkv = mops.short_conv(proj[:, :self.channels], self.conv, conv_state, batch.state_slots, batch.q_start, batch.q_len,
                              batch.ctx_len, batch.seq_of_token, self.channels, act=1)
        g_at = self.channels
        b_at = g_at + H * e
        o = mops.gated_delta_scan(qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:], proj[:, b_at:b_at + H],
                                  proj[:, b_at + H:b_at + 2 * H], self.a_log, self.dt_bias, state[0], batch.state_slots,
                                  batch.q_start, batch.q_len, batch.ctx_len, H, G, d ** -0.5, self.norm_eps, max_q_len=max(batch.q_lens))
        y = torch.empty(h.shape[0], H * e, dtype=h.dtype, device=h.device)
        mops.gated_head_rms_norm(y, o, self.out_norm, proj[:, g_at:g_at + H * e], H, self.eps, mops.GATE_SILU)
        return self.out_proj(y)


class RotaryGQAttention(nn.Module):
    """Causal grouped-query softmax attention over a token-major paged cache.  ONE input product gives q, k and v; one launch
    rotates the first ``rotary.dims`` numbers of every q and k head ("rotate half" pairs), brings q and k to unit RMS per head
    (``qk_norm``), blends the values with ``v_other`` -- an earlier layer's values of the same tokens -- by ``v_blend`` and
    writes keys and the blended values into the cache; the attention kernels are those of DistanceBiasAttention without bias."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, rotary: RotaryFrequencies,
                 eps: float, dtype, prefix: str = "", qk_norm: bool = True, v_blend: bool = False):
        super().__init__()
        from .loader import merged_plan
        from .model import QuantLinear
        if rotary.dims > dim:
            raise ValueError(f"{rotary.dims} rotated numbers in a head of {dim}")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.rotary, self.qk_norm = float(scale), float(eps), rotary, bool(qk_norm)
        self.attn = DistanceBiasAttention(heads, kv_heads, dim, vdim, scale)
        self.names = ["q", "k", "v"]
        self.splits = [heads * dim, kv_heads * dim, kv_heads * vdim]
        pad = -sum(self.splits) % 8
        if pad:
            self.splits.append(pad)
        self.in_proj = QuantLinear(width, self.splits, None, dtype, prefix=prefix + "in_proj", plan=merged_plan(self.splits))
        self.in_proj.weight.data.zero_()
        self.out_proj = QuantLinear(heads * vdim, [width], None, dtype, prefix=prefix + "out_proj")
        self.v_blend = nn.Parameter(torch.zeros((), dtype=torch.float32), requires_grad=False) if v_blend else None
        self.lam = 0.0

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.kv_heads, self.dim, self.vdim)

    def finalize(self) -> None:
        self.rotary.to(self.in_proj.weight.device)
        self.lam = float(self.v_blend) if self.v_blend is not None else 0.0

    def forward(self, h: torch.Tensor, cache, batch: StepBatch, v_other: Optional[torch.Tensor] = None):
        """Returns (output, this step's raw value rows [T, kv_heads * vdim] -- a view of the input product)."""
        H, G, d, e = self.heads, self.kv_heads, self.dim, self.vdim
        proj = self.in_proj(h)
        k_cache, v_cache = cache
        v = proj[:, (H + G) * d:(H + G) * d + G * e]
        q = mops.rotary_qk_norm_kv_write(proj[:, :H * d], proj[:, H * d:(H + G) * d], v, k_cache, v_cache, batch.slot_mapping,
                                         batch.q_start, batch.ctx_len, batch.seq_of_token, self.rotary.inv_freq, self.rotary.dims,
                                         mops.ROTARY_HALF, self.qk_norm, self.eps, v_other, self.lam if v_other is not None else 0.0)
        o = torch.empty(h.shape[0], H * e, dtype=h.dtype, device=h.device)
        mops.distance_bias_attention(o, q, None, k_cache, v_cache, batch.block_tables, batch.q_start, batch.q_len, batch.ctx_len,
                                     batch.seq_of_token, (min(batch.q_lens), max(batch.q_lens)), H, self.scale, None,
                                     max_kv_len=max(c + n for c, n in zip(batch.ctx_lens, batch.q_lens)))
        return self.out_proj(o), v
