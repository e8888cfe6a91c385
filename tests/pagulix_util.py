"""Small random Pagulix checkpoints for the tests: a config dict, numpy weights named as in a checkpoint, and a writer of
config.json + model.safetensors.  Sizes are deliberately unlike one another (dim != vdim, head counts that differ, a width that is
no power of two, layers that differ in everything) so that a swapped size or a constant taken from the wrong layer shows."""
import numpy as np

from fatudra_util import bf16_round, logit_errors  # noqa: F401
from fekotar_util import assert_logits, write_checkpoint  # noqa: F401


def moe(ff=40, experts=6, top=2, shared=56):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def delta_layer(heads=4, kv_heads=2, dim=24, vdim=40, conv=3, mlp="default"):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": moe() if mlp == "default" else mlp}


def latent_layer(heads=3, dim=24, rot_dim=8, vdim=40, kv_rank=48, window=13, base=5000.0, scale=None, mlp="default"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": {"base": base, "dims": rot_dim},
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": moe() if mlp == "default" else mlp}


def attn_layer(heads=6, kv_heads=2, dim=24, vdim=16, rot_dims=12, base=3000.0, scaling=(4.0, 1.0, 4.0, 64), scale=None, v_mix=True,
               mlp="default"):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale if scale is not None else dim ** -0.5}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": moe() if mlp == "default" else mlp}


def make_config(layers, vocab=131, width=72, eps=1e-5, streams=3, residual_mult=0.4, softcap=9.0):
    c = {"architecture": "Pagulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "streams": streams,
         "residual_mult": residual_mult, "layers": layers}
    if softcap:
        c["logit_softcap"] = softcap
    return c


def make_weights(cfg, seed=0, round_bf16=True):
    rng = np.random.default_rng(seed)
    W, width, n = {}, cfg["width"], cfg["streams"]

    def mat(o, i, gain=1.0):
        return rng.standard_normal((o, i)) * gain / np.sqrt(i)

    def vec(k, mean=1.0, std=0.2):
        return mean + std * rng.standard_normal(k)

    W["embed"] = rng.standard_normal((cfg["vocab"], width))
    W["final.norm"] = vec(width)
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        for q in (1, 2):
            if q == 2 and lc["mlp"] is None:
                continue
            W[f"{p}norm{q}"], W[f"{p}ls{q}"] = vec(width), vec(width, 1.0, 0.3)
            W[f"{p}hc{q}.in"], W[f"{p}hc{q}.out"] = vec(n, 1.0 / n, 0.2), vec(n, 1.0, 0.3)
            W[f"{p}hc{q}.mix"] = np.eye(n) + 0.15 * rng.standard_normal((n, n))
        if lc["type"] == "delta":
            H, G, d, e, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for nm, rows in (("q", G * d), ("k", G * d), ("v", H * e)):
                W[p + "mix." + nm] = mat(rows, width, 2.0)
                W[p + "mix." + nm + ".conv"] = rng.standard_normal((rows, taps)) * 0.6
            W[p + "mix.b"], W[p + "mix.a"] = mat(H, width, 2.0), mat(H, width, 2.0)
            W[p + "mix.A_log"], W[p + "mix.dt_bias"] = np.log(rng.uniform(0.3, 3.0, H)), vec(H, 0.0, 1.0)
            W[p + "mix.norm"] = vec(e)
            W[p + "mix.g"], W[p + "mix.o"] = mat(H * e, width, 2.0), mat(width, H * e)
        elif lc["type"] == "latent_attention":
            H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[p + "mix.q"] = mat(H * (d + r), width, 2.5)
            W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = mat(R + r, width, 1.5), vec(R)
            W[p + "mix.uk"], W[p + "mix.uv"] = mat(H * d, R, 2.0), mat(H * e, R)
            W[p + "mix.sink"] = vec(H, 0.5, 1.0)
            W[p + "mix.o"] = mat(width, H * e)
        else:
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = mat(H * d, width, 1.5), mat(G * d, width, 1.5), mat(G * e, width)
            W[p + "mix.o"] = mat(width, H * e)
            if m.get("v_mix"):
                W[p + "mix.vmix"] = np.asarray(rng.uniform(0.2, 0.7))
        f = lc["mlp"]
        if f is not None:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            W[p + "mlp.router"], W[p + "mlp.router.b"] = mat(E, width, 3.0), vec(E, 0.0, 0.5)
            for j in range(E):
                pe = f"{p}mlp.e{j}."
                W[pe + "gate"], W[pe + "up"], W[pe + "down"] = mat(ff, width, 2.0), mat(ff, width, 2.0), mat(width, ff)
            if f.get("shared"):
                sf = f["shared"]["ff"]
                W[p + "mlp.shared.gate"], W[p + "mlp.shared.up"] = mat(sf, width, 2.0), mat(sf, width, 2.0)
                W[p + "mlp.shared.down"] = mat(width, sf)
    if round_bf16:
        W = {k: bf16_round(v) for k, v in W.items()}
    return {k: np.asarray(v, np.float32) for k, v in W.items()}
