"""Pagulix: a pre-norm decoder whose residual is carried as several streams (hyper-connections) and whose layers pick their
mixer from three kinds.

  x_1 .. x_n = embed[token]                                           (n = ``streams`` copies)
  sublayer (mixer, then feed-forward):  u = sum_s in[s] x_s;  y = sublayer(norm(u)) * layer_scale;
                                        x_t <- sum_s mix[s, t] x_s + residual_mult * out[t] * y     (StreamedResidual)
  logits = softcap(embed . norm_final(sum_s x_s))                     (the output matrix is the embedding table)

Mixers, by the layer's ``type``:
  delta              GatedDeltaMixer: the gated delta rule behind short causal convolutions, state per request slot
  latent_attention   LatentAttention without a query latent and without an output gate, under a sliding window and with a
                     per-head sink in the softmax denominator; its rotation pairs neighbouring numbers (2 i, 2 i + 1) -- the
                     rows of the projections that make the rotated parts are reordered at load so that the kernels' pairing
                     (i, i + dims / 2) computes the same scores
  attention          RotaryGQAttention: partial rotation with wavelength-scaled frequencies, unit RMS of q and k after it, and
                     -- in every layer that says ``v_mix`` except the first such -- values blended with that first layer's
The feed-forward is RoutedExperts with a biased router whose weights are the softmax over the chosen logits, silu experts and
an ungated shared expert.  Every size and constant comes from config.json or a tensor's shape.  Norm statistics, angles,
scores, the router, the recurrent state and everything that enters it, and the residual streams are fp32 also in a bfloat16 model."""
from dataclasses import dataclass
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn
from torch.nn import functional as F

from . import mixer_ops as mops
from .mixers import (GatedDeltaMixer, LatentAttention, RotaryFrequencies, RotaryGQAttention, RoutedExperts, StreamedResidual,
                     interleaved_to_half)
from .step_batch import StepBatch

MIXER_TYPES = ("delta", "latent_attention", "attention")


@dataclass
class PagulixConfig:
    vocab: int
    width: int
    eps: float
    streams: int
    residual_mult: float
    logit_softcap: float
    layers: List[Dict[str, Any]]

    @staticmethod
    def from_dict(c: Dict[str, Any]) -> "PagulixConfig":
        cfg = PagulixConfig(vocab=int(c["vocab"]), width=int(c["width"]), eps=float(c["norm"]["eps"]), streams=int(c.get("streams", 1)),
                            residual_mult=float(c.get("residual_mult", 1.0)), logit_softcap=float(c.get("logit_softcap") or 0.0),
                            layers=list(c["layers"]))
        blended = None
        for i, lc in enumerate(cfg.layers):
            if lc["type"] not in MIXER_TYPES:
                raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            mc = lc["mixer"]
            if lc["type"] == "attention" and mc.get("v_mix"):
                shape = (int(mc["kv_heads"]), int(mc["vdim"]))
                if blended is not None and shape != blended:
                    raise ValueError(f"layer {i}: values of {shape} cannot be blended with the first such layer's {blended}")
                blended = blended or shape
        return cfg


def rotary_from_config(rot: Dict[str, Any]) -> RotaryFrequencies:
    sc = rot.get("scaling")
    if not sc:
        return RotaryFrequencies(int(rot["dims"]), float(rot["base"]))
    return RotaryFrequencies.wavelength_scaled(int(rot["dims"]), float(rot["base"]), float(sc["factor"]), float(sc["low"]),
                                               float(sc["high"]), float(sc["original"]))


class StreamCoefficients(nn.Module):
    """What one sublayer needs of the streamed residual: how it reads the streams, how its result is spread over them, how the
    streams mix, and the per-channel scale on its result.  Kept as fp32 parameters; ``finalize`` copies them to host numbers."""

    def __init__(self, streams: int, width: int, dtype):
        super().__init__()
        self.read = nn.Parameter(torch.ones(streams, dtype=torch.float32), requires_grad=False)
        self.write = nn.Parameter(torch.ones(streams, dtype=torch.float32), requires_grad=False)
        self.mix = nn.Parameter(torch.eye(streams, dtype=torch.float32), requires_grad=False)
        self.scale = nn.Parameter(torch.ones(width, dtype=dtype), requires_grad=False)
        self.reads = None
        self.wrote = None

    def finalize(self) -> None:
        self.reads = mops.host_floats(self.read.tolist())
        self.wrote = (mops.host_floats(self.mix.tolist()), mops.host_floats(self.write.tolist()), self.scale)


class PagulixLayer(nn.Module):
    def __init__(self, cfg: PagulixConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        mc, kind = lc["mixer"], lc["type"]
        pfx = f"l{index}."
        self.kind = kind
        self.norm1 = nn.Parameter(torch.ones(cfg.width, dtype=dtype), requires_grad=False)
        self.hc1 = StreamCoefficients(cfg.streams, cfg.width, dtype)
        if kind == "delta":
            self.mix = GatedDeltaMixer(cfg.width, int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"]),
                                       int(mc.get("conv", 1)), cfg.eps, dtype, prefix=pfx + "mix.")
        elif kind == "latent_attention":
            mask = mc.get("mask") or {}
            self.mix = LatentAttention(cfg.width, int(mc["heads"]), int(mc["dim"]), int(mc["rot_dim"]), int(mc["vdim"]), 0,
                                       int(mc["kv_rank"]), float(mc["scale"]), rotary_from_config(mc["rot"]), cfg.eps, dtype,
                                       prefix=pfx + "mix.", gate=False, window=int(mask.get("size", 0)), sink=True)
        else:
            self.mix = RotaryGQAttention(cfg.width, int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"]),
                                         float(mc["scale"]), rotary_from_config(mc["rot"]), cfg.eps, dtype, prefix=pfx + "mix.",
                                         qk_norm=True, v_blend=bool(mc.get("v_mix")))
        mlp = lc.get("mlp")
        self.mlp = self.norm2 = self.hc2 = None
        if mlp is not None:
            r, sh = mlp["router"], mlp.get("shared")
            self.norm2 = nn.Parameter(torch.ones(cfg.width, dtype=dtype), requires_grad=False)
            self.hc2 = StreamCoefficients(cfg.streams, cfg.width, dtype)
            self.mlp = RoutedExperts(cfg.width, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), 0, 0.0, dtype,
                                     shared_ff=int(sh["ff"]) if sh else 0, alpha=1.0, prefix=pfx + "mlp.", score="topk_softmax",
                                     shared_gate=False)


class PagulixForCausalLM(nn.Module):
    def __init__(self, cfg: PagulixConfig, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        from .distributed import get_tensor_model_parallel_world_size
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Pagulix runs on one rank")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Pagulix runs in bfloat16 or float32")
        self.cfg, self.dtype = cfg, dtype
        self.embed = nn.Parameter(torch.empty(cfg.vocab, cfg.width, dtype=dtype), requires_grad=False)
        self.layers = nn.ModuleList([PagulixLayer(cfg, i, dtype) for i in range(len(cfg.layers))])
        self.final_norm = nn.Parameter(torch.ones(cfg.width, dtype=dtype), requires_grad=False)
        self.residual = StreamedResidual(cfg.streams, cfg.residual_mult, cfg.eps, dtype)
        # caches: a delta layer owns a convolution state and a matrix state, the attentions a paged cache each
        self.specs, self.cache_index = [], []
        for layer in self.layers:
            self.cache_index.append(len(self.specs))
            if layer.kind == "delta":
                self.specs += list(layer.mix.cache_specs())
            else:
                self.specs.append(layer.mix.cache_spec())
        # the first layer that blends values keeps its own; the later ones blend with it
        blenders = [i for i, layer in enumerate(self.layers) if layer.kind == "attention" and layer.mix.v_blend is not None]
        self.first_blend = blenders[0] if blenders else -1
        self.residual_trace: Optional[List[torch.Tensor]] = None     # set to [] to record the streams' sum after every layer

    # ---- what the engine asks of a model ---------------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.cfg.vocab

    def make_caches(self, num_blocks: int, block_size: int, num_slots: int, device):
        return [s.allocate(num_blocks, block_size, num_slots, self.dtype, device) for s in self.specs]

    def finalize(self):
        for layer in self.layers:
            if layer.kind != "delta":
                layer.mix.finalize()
            layer.hc1.finalize()
            if layer.hc2 is not None:
                layer.hc2.finalize()
        return self

    @torch.no_grad()
    def step(self, batch: StepBatch, caches, rows: torch.Tensor) -> torch.Tensor:
        """One engine step: run the batch's rows through every layer (caches and states advance), return the fp32 logits of
        ``rows`` (int64 indices into the batch)."""
        h = self.forward(batch, caches, rows)
        return self.logits(h)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return mops.logit_softcap(F.linear(h, self.embed), 1.0, self.cfg.logit_softcap)

    def _sublayers(self):
        out = []
        for i, layer in enumerate(self.layers):
            out.append((i, layer, 1))
            if layer.mlp is not None:
                out.append((i, layer, 2))
        return out

    def forward(self, batch: StepBatch, caches, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The final norm's output for the rows asked for (all rows if ``rows`` is None)."""
        res = self.residual
        subs = self._sublayers()
        x = res.start(self.embed, batch.input_ids)
        v_first = None

        def reads_of(j):
            _, layer, q = subs[j]
            return (layer.hc1.reads, layer.norm1) if q == 1 else (layer.hc2.reads, layer.norm2)
        if not subs:
            h = res.step(x, None, None, None, self.final_norm)
            return h if rows is None else h.index_select(0, rows)
        h = res.step(x, None, None, *reads_of(0))
        for j, (i, layer, q) in enumerate(subs):
            if q == 2:
                y = layer.mlp(h)
            elif layer.kind == "delta":
                c = self.cache_index[i]
                y = layer.mix(h, caches[c], caches[c + 1], batch)
            elif layer.kind == "latent_attention":
                y = layer.mix(h, caches[self.cache_index[i]], batch)
            else:
                blend = layer.mix.v_blend is not None and i != self.first_blend
                y, v = layer.mix(h, caches[self.cache_index[i]], batch, v_first if blend else None)
                if i == self.first_blend:
                    v_first = v
            wrote = (layer.hc1 if q == 1 else layer.hc2).wrote
            last = j + 1 == len(subs)
            if not last:
                h = res.step(x, y, wrote, *reads_of(j + 1))
            elif rows is None:
                h = res.step(x, y, wrote, None, self.final_norm)
            else:                                # the last write runs on every row, the final norm on the wanted rows only
                mops.hyper_residual_rms_norm(x, y, wrote[2], wrote[0], wrote[1], res.mult, dtype=self.dtype, want_out=False)
                h = res.step(x.index_select(0, rows), None, None, None, self.final_norm)
            if self.residual_trace is not None and (last or subs[j + 1][0] != i):
                self.residual_trace.append(x.sum(1))
        return h

    # ---- checkpoint ----------------------------------------------------------------------------------------------------
    def expected_names(self) -> Tuple[List[str], List[str]]:
        """(names a checkpoint must hold, names it may hold)"""
        names, optional = ["embed", "final.norm"], []
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            names.append(p + "norm1")
            optional += [p + "ls1"] + [f"{p}hc1.{n}" for n in ("in", "out", "mix")]
            if layer.kind == "delta":
                names += [p + "mix." + n for n in ("q", "k", "v", "q.conv", "k.conv", "v.conv", "b", "a", "g", "o", "A_log", "dt_bias", "norm")]
            elif layer.kind == "latent_attention":
                names += [p + "mix." + n for n in ("q", "dkv", "dkv.norm", "uk", "uv", "sink", "o")]
            else:
                names += [p + "mix." + n for n in ("q", "k", "v", "o")]
                (names if layer.mix.v_blend is not None else optional).append(p + "mix.vmix")
            m = layer.mlp
            if m is None:
                optional += [p + "norm2", p + "ls2"] + [f"{p}hc2.{n}" for n in ("in", "out", "mix")]
                continue
            names += [p + "norm2", p + "mlp.router", p + "mlp.router.b"]
            optional += [p + "ls2"] + [f"{p}hc2.{n}" for n in ("in", "out", "mix")]
            names += [f"{p}mlp.e{e}.{n}" for e in range(m.experts) for n in ("gate", "up", "down")]
            if m.shared_ff:
                names += [p + "mlp.shared." + n for n in ("gate", "up", "down")]
        return names, optional

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names: embed, final.norm, l<i>.{norm1, norm2, ls1, ls2, hc1.{in,out,mix}, hc2.{in,out,mix}},
        l<i>.mix.* by the layer's type, l<i>.mlp.{router, router.b, e<j>.{gate,up,down}, shared.{gate,up,down}}."""
        names, optional = self.expected_names()
        expected, seen = set(names), set()
        allowed = expected | set(optional)
        for name, t in weights:
            if name not in allowed:
                raise ValueError(f"unexpected tensor {name!r} in a Pagulix checkpoint")
            seen.add(name)
            self._load_one(name, t)
        missing = expected - seen
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
            return put(self.embed.data, t, name)
        if name == "final.norm":
            return put(self.final_norm.data, t, name)
        first, rest = name.split(".", 1)
        layer = self.layers[int(first[1:])]
        if rest in ("norm1", "norm2"):
            dst = layer.norm1 if rest == "norm1" else layer.norm2
            return None if dst is None else put(dst.data, t, name)
        if rest in ("ls1", "ls2") or rest.startswith("hc"):
            hc = layer.hc1 if rest[2] == "1" else layer.hc2
            if hc is None:                       # coefficients of a feed-forward the layer does not have
                return None
            if rest.startswith("ls"):
                return put(hc.scale.data, t, name)
            return put({"in": hc.read, "out": hc.write, "mix": hc.mix}[rest[4:]].data, t, name)
        if rest.startswith("mix."):
            return self._load_mixer(layer, rest[4:], t, name)
        key, m = rest[4:], layer.mlp
        if key == "router":
            return put(m.router.data, t, name)
        if key == "router.b":
            return put(m.router_bias.data, t, name)
        who, part = key.split(".", 1)
        if who == "shared":
            lin = m.shared_down if part == "down" else m.shared_in
            return lin.weight_loader(lin.weight, t.to(lin.weight.dtype), {"gate": 0, "up": 1, "down": 0}[part])
        e = int(who[1:])
        if part == "down":
            return put(m.w_down.data[e], t, name)
        return put(m.w_gate_up.data[e, :m.ff] if part == "gate" else m.w_gate_up.data[e, m.ff:], t, name)

    def _load_mixer(self, layer: PagulixLayer, key: str, t: torch.Tensor, name: str) -> None:
        put, mix = self._put, layer.mix
        if key == "o":
            return mix.out_proj.weight_loader(mix.out_proj.weight, t.to(mix.out_proj.weight.dtype), 0)
        if layer.kind == "delta":
            if key.endswith(".conv"):
                at = sum(mix.splits[:mix.names.index(key[:-5])])
                return put(mix.conv.data[at:at + t.shape[0]], t, name)
            if key in ("A_log", "dt_bias", "norm"):
                return put({"A_log": mix.a_log, "dt_bias": mix.dt_bias, "norm": mix.out_norm}[key].data, t, name)
        elif layer.kind == "latent_attention":
            dims = mix.rotary.dims
            if key == "q":                       # every head's rotated part: neighbouring pairs -> pairs half the part apart
                for hd in range(mix.heads):
                    t = interleaved_to_half(t, dims, hd * (mix.dim + mix.rot_dim) + mix.dim)
            elif key == "dkv":
                t = interleaved_to_half(t, dims, mix.kv_rank)
            elif key == "dkv.norm":
                return put(mix.kv_norm.data, t, name)
            elif key == "sink":
                return put(mix.sink.data, t, name)
            elif key == "uk":
                return put(mix.w_uk.data.view(mix.heads * mix.dim, mix.kv_rank), t, name)
            elif key == "uv":
                return put(mix.w_uv.data.view(mix.heads * mix.vdim, mix.kv_rank), t, name)
        elif key == "vmix":
            return None if mix.v_blend is None else put(mix.v_blend.data, t.reshape(()), name)
        lin = mix.in_proj
        want = (mix.splits[mix.names.index(key)], lin.weight.shape[1])
        if tuple(t.shape) != want:
            raise ValueError(f"{name}: checkpoint tensor {tuple(t.shape)} does not fit {want}")
        return lin.weight_loader(lin.weight, t.to(lin.weight.dtype), mix.names.index(key))

    @torch.no_grad()
    def init_synthetic(self, device, seed: int = 0):
        """Random weights of a checkpoint's scale on the device (benchmarks, tests)."""
        g = torch.Generator(device="cpu").manual_seed(seed)
        self.to(device)
        n = self.cfg.streams
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf == "mix" and p.dim() == 2 and p.shape == (n, n):
                p.copy_(torch.eye(n) + 0.1 * torch.randn(n, n, generator=g))
            elif leaf in ("read", "write"):
                p.copy_(1.0 / n ** 0.5 + 0.1 * torch.randn(n, generator=g))
            elif leaf == "conv":
                p.copy_((torch.randn(p.shape, generator=g) * 0.5).to(p.dtype))
            elif p.dim() >= 2:
                std = 1.0 if name == "embed" else p.shape[-1] ** -0.5
                p.copy_((torch.randn(p.shape, generator=g) * std).to(p.dtype))
            elif "norm" in name or leaf == "scale":
                p.copy_((1.0 + 0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
            elif leaf == "v_blend":
                p.fill_(0.3)
            else:
                p.copy_((0.1 * torch.randn(p.shape, generator=g)).to(p.dtype))
        for layer in self.layers:               # the fused products' padding rows stay zero
            for lin, used in ((layer.mix.in_proj, sum(layer.mix.splits[:len(layer.mix.names)])),):
                lin.weight.data[used:].zero_()
            if layer.mlp is not None and layer.mlp.shared_ff:
                layer.mlp.shared_in.weight.data[2 * layer.mlp.shared_ff:].zero_()
        return self.finalize()


def load_pagulix(model_dir: str, hf: Dict[str, Any], dtype: torch.dtype, device, **_unused) -> PagulixForCausalLM:
    from .loader import iter_safetensors
    model = PagulixForCausalLM(PagulixConfig.from_dict(hf), dtype)
    model.load_weights(iter_safetensors(model_dir))
    model.to(device)
    return model.finalize()
