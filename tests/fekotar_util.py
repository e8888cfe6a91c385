"""Small random Fekotar checkpoints for the tests: a config dict, numpy weights named as in a checkpoint, and a writer of
config.json + model.safetensors.  Sizes are deliberately unlike one another (dim != rot_dim != vdim, ranks that differ, a width
that is no power of two, layers that differ in everything) so that a swapped size or a constant taken from the wrong layer shows."""
import json
import os

import numpy as np
import torch

from fatudra_util import bf16_round, logit_errors  # noqa: F401


def latent_layer(heads=3, dim=24, rot_dim=8, vdim=40, q_rank=56, kv_rank=48, scale=None, base=5000.0, scaling=(3.0, 64, 16.0, 2.0),
                 mlp="dense", ff=88, limit=1.5, experts=6, groups=3, keep=2, top=2, route_scale=2.5):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "rot": rot,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if mlp == "dense":
        f = {"kind": "dense", "ff": ff, "limit": limit}
    elif mlp == "moe":
        f = {"kind": "moe", "expert": {"ff": ff},
             "router": {"experts": experts, "top": top, "scale": route_scale, "groups": {"count": groups, "keep": keep}}}
    else:
        f = None
    return {"type": "latent_attention", "mixer": m, "mlp": f}


def make_config(layers, vocab=131, width=72, eps=1e-5, logit_scale=0.7, bigram=(61, 13, 5)):
    c = {"architecture": "Fekotar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale, "layers": layers}
    if bigram is not None:
        c["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return c


def make_weights(cfg, seed=0, round_bf16=True):
    rng = np.random.default_rng(seed)
    W, width = {}, cfg["width"]

    def mat(o, i, gain=1.0):
        return rng.standard_normal((o, i)) * gain / np.sqrt(i)

    def vec(n, mean=1.0, std=0.2):
        return mean + std * rng.standard_normal(n)

    W["embed"] = rng.standard_normal((cfg["vocab"], width))
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        W["bigram"] = rng.standard_normal((big["buckets"] + 1, width))
    W["head"] = mat(cfg["vocab"], width)
    W["final.norm"] = vec(width)
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = lc["mixer"]
        H, d, r, e, Rq, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
        W[p + "norm1"] = vec(width)
        W[p + "mix.dq"], W[p + "mix.dq.norm"] = mat(Rq, width), vec(Rq)
        W[p + "mix.uq"] = mat(H * (d + r), Rq, 2.0)
        W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = mat(R + r, width, 1.5), vec(R)
        W[p + "mix.uk"], W[p + "mix.uv"] = mat(H * d, R, 2.0), mat(H * e, R)
        W[p + "mix.g"], W[p + "mix.o"] = mat(H * e, width), mat(width, H * e)
        f = lc["mlp"]
        if f is not None and f["kind"] == "dense":
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = mat(f["ff"], width, 2.0), mat(f["ff"], width, 2.0), mat(width, f["ff"])
            W[p + "mlp.gate.b"], W[p + "mlp.up.b"], W[p + "mlp.down.b"] = vec(f["ff"], 0.0, 0.5), vec(f["ff"], 0.0, 0.5), vec(width, 0.0, 0.5)
        elif f is not None:
            W[p + "mlp.router"] = mat(f["router"]["experts"], width, 3.0)
            for j in range(f["router"]["experts"]):
                pe = f"{p}mlp.e{j}."
                W[pe + "gate"], W[pe + "up"] = mat(f["expert"]["ff"], width, 2.0), mat(f["expert"]["ff"], width, 2.0)
                W[pe + "down"] = mat(width, f["expert"]["ff"])
    if round_bf16:
        W = {k: bf16_round(v) for k, v in W.items()}
    return {k: np.asarray(v, np.float32) for k, v in W.items()}


def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.from_numpy(np.ascontiguousarray(v)).to(torch.bfloat16).contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return path


def assert_logits(got, want, sharp, what=""):
    """``sharp`` (float32 runs): every position within 2e-4 of the logits' spread.  bfloat16 against the unrounded restatement:
    the typical position within the rounding of a few bfloat16 layers and no more than a tenth of them far off -- with random
    weights a router's choice now and then rests on a margin smaller than that rounding, and the other expert's output is a
    different one; a bound on the worst position cannot tell that from a fault, the float32 run of the same test can."""
    e = logit_errors(got, want)
    assert np.isfinite(e).all(), what
    if sharp:
        assert e.max() < 2e-4, (what, float(e.max()), int(e.argmax()))
    else:
        assert np.median(e) < 0.04 and np.quantile(e, 0.9) < 0.15, (what, float(np.median(e)), float(np.quantile(e, 0.9)))
