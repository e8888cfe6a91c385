"""Fekotar: a decoder around an fp32 residual stream whose layers run their two sublayers side by side on ONE normed input.

  x_0 = embed[token] + bigram[hash(previous token, token)]           (HashedPairEmbedding; a sequence's first token: the last row)
  layer i:   h = norm1_i(x);  x += mixer_i(h) + ff_i(h)               (the feed-forward only if the layer has one)
  logits = head norm_final(x) * logit_scale

Every norm is an RMS norm with a per-channel weight.  The mixer is ``LatentAttention`` (mixers.py): queries through a normed
latent, keys and values as products of a cached normed latent plus one rotated key part shared by all heads (YaRN-scaled
frequencies), causal softmax, elementwise sigmoid output gate.  The feed-forward is ``ClampedGLUMLP`` (biased projections) or
``RoutedExperts`` with a sigmoid router limited to the best groups of experts and silu-gated experts.  Everything the
checkpoint's config.json can vary is read from it -- the layer list, every size, the rotation's constants, the hash's
constants -- and nothing here depends on particular values.  Norm statistics, angles, scores, the router and the residual are
fp32 also in a bfloat16 model.

One launch (``residual_add2_rms_norm``) folds both sublayers' residual add and the RMS norm that feeds the next layer."""
from dataclasses import dataclass
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn
from torch.nn import functional as F

from . import mixer_ops as mops
from .mixers import ClampedGLUMLP, HashedPairEmbedding, LatentAttention, RotaryFrequencies, RoutedExperts
from .step_batch import StepBatch


@dataclass
class FekotarConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    bigram: Optional[Dict[str, int]]
    layers: List[Dict[str, Any]]

    @staticmethod
    def from_dict(c: Dict[str, Any]) -> "FekotarConfig":
        big = (c.get("embedding") or {}).get("bigram")
        cfg = FekotarConfig(vocab=int(c["vocab"]), width=int(c["width"]), eps=float(c["norm"]["eps"]),
                            logit_scale=float(c.get("logit_scale", 1.0)),
                            bigram=None if big is None else {k: int(big[k]) for k in ("buckets", "mul_prev", "mul_cur")},
                            layers=list(c["layers"]))
        for i, lc in enumerate(cfg.layers):
            if lc["type"] != "latent_attention":
                raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        return cfg


def rotary_from_config(rot: Dict[str, Any]) -> RotaryFrequencies:
    sc = rot.get("scaling")
    if not sc:
        return RotaryFrequencies(int(rot["dims"]), float(rot["base"]))
    return RotaryFrequencies(int(rot["dims"]), float(rot["base"]), float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                             float(sc["slow"]))


class FekotarLayer(nn.Module):
    def __init__(self, cfg: FekotarConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        mc = lc["mixer"]
        pfx = f"l{index}."
        self.norm1 = nn.Parameter(torch.ones(cfg.width, dtype=dtype), requires_grad=False)
        self.mix = LatentAttention(cfg.width, int(mc["heads"]), int(mc["dim"]), int(mc["rot_dim"]), int(mc["vdim"]), int(mc["q_rank"]),
                                   int(mc["kv_rank"]), float(mc["scale"]), rotary_from_config(mc["rot"]), cfg.eps, dtype,
                                   prefix=pfx + "mix.")
        mlp = lc.get("mlp")
        self.mlp = None
        if mlp is not None and mlp["kind"] == "dense":
            self.mlp = ClampedGLUMLP(cfg.width, int(mlp["ff"]), float(mlp["limit"]), dtype, prefix=pfx + "mlp.")
        elif mlp is not None:
            r = mlp["router"]
            self.mlp = RoutedExperts(cfg.width, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), 0, 0.0, dtype, alpha=1.0,
                                     prefix=pfx + "mlp.", score="sigmoid_grouped", groups=int(r["groups"]["count"]),
                                     keep=int(r["groups"]["keep"]), group_top=2, route_scale=float(r.get("scale", 1.0)))


class FekotarForCausalLM(nn.Module):
    def __init__(self, cfg: FekotarConfig, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        from .distributed import get_tensor_model_parallel_world_size
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Fekotar runs on one rank")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Fekotar runs in bfloat16 or float32")
        self.cfg, self.dtype = cfg, dtype
        if cfg.bigram is not None:
            self.embed = HashedPairEmbedding(cfg.vocab, cfg.width, cfg.bigram["buckets"], cfg.bigram["mul_prev"], cfg.bigram["mul_cur"], dtype)
        else:
            self.embed = nn.Embedding(cfg.vocab, cfg.width, dtype=dtype)
            self.embed.weight.requires_grad_(False)
        self.layers = nn.ModuleList([FekotarLayer(cfg, i, dtype) for i in range(len(cfg.layers))])
        self.final_norm = nn.Parameter(torch.ones(cfg.width, dtype=dtype), requires_grad=False)
        self.head = nn.Parameter(torch.empty(cfg.vocab, cfg.width, dtype=dtype), requires_grad=False)
        # caches: the previous token of every request (if the embedding hashes pairs), then one latent cache per layer
        self.specs = [self.embed.state_spec()] if cfg.bigram is not None else []
        self.cache_index = []
        for layer in self.layers:
            self.cache_index.append(len(self.specs))
            self.specs.append(layer.mix.cache_spec())
        self.residual_trace: Optional[List[torch.Tensor]] = None     # set to [] to record x after every layer

    # ---- what the engine asks of a model ---------------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.cfg.vocab

    def make_caches(self, num_blocks: int, block_size: int, num_slots: int, device):
        return [s.allocate(num_blocks, block_size, num_slots, self.dtype, device) for s in self.specs]

    def finalize(self):
        for layer in self.layers:
            layer.mix.finalize()
        return self

    @torch.no_grad()
    def step(self, batch: StepBatch, caches, rows: torch.Tensor) -> torch.Tensor:
        """One engine step: run the batch's rows through every layer (caches and states advance), return the fp32 logits of
        ``rows`` (int64 indices into the batch)."""
        h = self.forward(batch, caches)
        return self.logits(h.index_select(0, rows))

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head).float() * self.cfg.logit_scale

    def forward(self, batch: StepBatch, caches) -> torch.Tensor:
        """The final norm's output for every row of the batch."""
        cfg, eps = self.cfg, self.cfg.eps
        L = len(self.layers)
        if cfg.bigram is not None:
            x = self.embed(batch, caches[0])
        else:
            x = mops.embed_scale(self.embed.weight, batch.input_ids, 1.0)
        h = mops.residual_add2_rms_norm(x, weight=self.layers[0].norm1 if L else self.final_norm, eps=eps, dtype=self.dtype)
        for i, layer in enumerate(self.layers):
            ya = layer.mix(h, caches[self.cache_index[i]], batch)
            yb = layer.mlp(h) if layer.mlp is not None else None
            w = self.layers[i + 1].norm1 if i + 1 < L else self.final_norm
            h = mops.residual_add2_rms_norm(x, ya, yb, weight=w, eps=eps)
            if self.residual_trace is not None:
                self.residual_trace.append(x.clone())
        return h

    # ---- checkpoint ----------------------------------------------------------------------------------------------------
    def expected_names(self) -> List[str]:
        names = ["embed", "head", "final.norm"] + (["bigram"] if self.cfg.bigram is not None else [])
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            names += [p + "norm1"] + [p + "mix." + n for n in ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o")]
            m = layer.mlp
            if isinstance(m, ClampedGLUMLP):
                names += [p + "mlp." + n for n in ("gate", "gate.b", "up", "up.b", "down", "down.b")]
            elif isinstance(m, RoutedExperts):
                names += [p + "mlp.router"] + [f"{p}mlp.e{e}.{n}" for e in range(m.experts) for n in ("gate", "up", "down")]
        return names

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names: embed, bigram, head, final.norm, l<i>.norm1, l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o},
        l<i>.mlp.{gate, up, down}[.b] or l<i>.mlp.{router, e<j>.{gate, up, down}}."""
        expected, seen = set(self.expected_names()), set()
        for name, t in weights:
            if name not in expected:
                raise ValueError(f"unexpected tensor {name!r} in a Fekotar checkpoint")
            seen.add(name)
            self._load_one(name, t)
        missing = expected - seen
        if "head" in missing:                    # no output matrix of its own: the embedding's
            self.head = self.embed.table if self.cfg.bigram is not None else self.embed.weight
            missing.discard("head")
        if missing:
            raise ValueError(f"checkpoint lacks {len(missing)} tensors, e.g. {sorted(missing)[:4]}")

    @staticmethod
    def _put(dst: torch.Tensor, t: torch.Tensor, name: str) -> None:
        if tuple(dst.shape) != tuple(t.shape):
            raise ValueError(f"{name}: checkpoint tensor {tuple(t.shape)} does not fit {tuple(dst.shape)}")
        dst.copy_(t.to(dst.dtype))

    def _load_one(self, name: str, t: torch.Tensor) -> None:
        put = self._put
        if name == "embed":
            return put((self.embed.table if self.cfg.bigram is not None else self.embed.weight).data, t, name)
        if name == "bigram":
            return put(self.embed.pair_table.data, t, name)
        if name == "head":
            return put(self.head.data, t, name)
        if name == "final.norm":
            return put(self.final_norm.data, t, name)
        first, rest = name.split(".", 1)
        layer = self.layers[int(first[1:])]
        if rest == "norm1":
            return put(layer.norm1.data, t, name)
        if rest.startswith("mix."):
            key, mix = rest[4:], layer.mix
            if key in mix.names:
                lin = mix.in_proj
                return lin.weight_loader(lin.weight, t.to(lin.weight.dtype), mix.names.index(key))
            if key == "dq.norm":
                return put(mix.q_norm.data, t, name)
            if key == "dkv.norm":
                return put(mix.kv_norm.data, t, name)
            if key == "uq":
                return mix.uq.weight_loader(mix.uq.weight, t.to(mix.uq.weight.dtype), 0)
            if key == "o":
                return mix.out_proj.weight_loader(mix.out_proj.weight, t.to(mix.out_proj.weight.dtype), 0)
            if key == "uk":
                return put(mix.w_uk.data.view(mix.heads * mix.dim, mix.kv_rank), t, name)
            return put(mix.w_uv.data.view(mix.heads * mix.vdim, mix.kv_rank), t, name)
        key, m = rest[4:], layer.mlp
        if isinstance(m, ClampedGLUMLP):
            part, is_bias = (key[:-2], True) if key.endswith(".b") else (key, False)
            lin = m.down if part == "down" else m.gate_up
            dst = lin.bias if is_bias else lin.weight
            return lin.weight_loader(dst, t.to(dst.dtype), {"gate": 0, "up": 1, "down": 0}[part])
        if key == "router":
            return put(m.router.data, t, name)
        who, part = key.split(".", 1)
        e = int(who[1:])
        if part == "down":
            return put(m.w_down.data[e], t, name)
        return put(m.w_gate_up.data[e, :m.ff] if part == "gate" else m.w_gate_up.data[e, m.ff:], t, name)

    @torch.no_grad()
    def init_synthetic(self, device, seed: int = 0):
        """Random weights of a checkpoint's scale on the device (benchmarks, tests)."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        self.to(device)
        for name, p in self.named_parameters():
            if p.dim() >= 2:
                std = 1.0 if name.startswith("embed") else p.shape[-1] ** -0.5
                p.copy_((torch.randn(p.shape, generator=g) * std).to(p.dtype))
            elif "norm" in name:
                p.copy_((1.0 + 0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
            else:
                p.copy_((0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
        for layer in self.layers:               # the fused product's padding rows stay zero
            layer.mix.in_proj.weight.data[sum(layer.mix.splits[:3]):].zero_()
        return self.finalize()


def load_fekotar(model_dir: str, hf: Dict[str, Any], dtype: torch.dtype, device, **_unused) -> FekotarForCausalLM:
    from .loader import iter_safetensors
    model = FekotarForCausalLM(FekotarConfig.from_dict(hf), dtype)
    model.load_weights(iter_safetensors(model_dir))
    model.to(device)
    return model.finalize()
