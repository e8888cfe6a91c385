"""``bench.py --mixers [--mixers-design fatudra|gipozen|fekotar|pagulix]``: prefill and decode throughput of a Fatudra (or Gipozen) stack at sizes that resemble a real model's layers
(random bf16 weights), beside a Llama stack of equal width / heads / feed-forward / layer count on the unquantised op path,
plus each mixer kernel alone against its roofline and against the like kernel of the Llama path.  Prints ONE JSON line;
the default workload of bench.py is untouched by it.  The Gipozen stack: windowed differential attention (two maps of half the
head size over shared values, window 1024 + 4 kept tokens, 4-tap convolutions), every second layer reading the previous
layer's keys and values and carrying 16 + 1 experts (top 4, a quarter of the dense feed-forward each, one shared expert)
instead of the PolyNorm feed-forward; its expert products are priced against the MFMA figure over the ACTIVE experts' flops.

The Fekotar stack: attention through a cached latent of rank 512 + 64 rotated numbers (queries through a latent of 3/8 of the
width), heads of 128 + 64 / 128, a dense clamped feed-forward in the first layer and 16 silu experts (top 4 of the 2 best of 4
groups, a quarter of the dense feed-forward each) in the others; it stands beside Llama AND beside the Gipozen stack (the
closest existing model: its own attention kernels plus routed experts) at equal width.

The Pagulix stack: a gated-delta layer (16 / 32 value heads of 128 x 128 state over 4 / 8 query-key heads, 4-tap convolutions), a
latent attention layer (rank 512 + 64 rotated numbers, window 1024, sinks), two rotary attention layers with unit-RMS q / k and
blended values, four residual streams, 16 silu experts (top 4, softmax over the chosen) plus a shared expert in every layer; it
stands beside the Fekotar stack (the closest existing model) and Llama.

Rooflines used: 8 TB/s HBM for the memory-bound kernels (norms, activations, decode attention, the decode step of the
memories: their state is read and written once), 2.5 PFLOP/s dense bf16 MFMA for prompt attention (4 d flops per visible
query-key pair and head), and for the prompt scan of the memories the same MFMA figure over 4 d e flops per token and head
(what a chunked matrix form would need; the scan kernel itself runs on the vector ALUs)."""
import json
import math
import time

import torch

HBM, MFMA = 8.0e12, 2.5e15

SIZES = {
    "w2048": dict(width=2048, ff=5632, heads=16, kv_heads=4, dim=128, mem_heads=8, mem_dim=64, mem_vdim=128, ml_heads=4,
                  ml_dim=128, ml_vdim=256),
    "w4096": dict(width=4096, ff=11008, heads=32, kv_heads=8, dim=128, mem_heads=16, mem_dim=64, mem_vdim=128, ml_heads=8,
                  ml_dim=128, ml_vdim=256),
}
LAYERS, VOCAB, BLOCK = 4, 32000, 16


def fatudra_config(s):
    par = {"type": "parallel",
           "mixer": {"left": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"], "bias_max": 4096,
                              "scale": s["dim"] ** -0.5, "q_temp": {"coef": 0.1, "every": 512}},
                     "right": {"heads": s["mem_heads"], "dim": s["mem_dim"], "vdim": s["mem_vdim"],
                               "decay": [1.0 - 2.0 ** -(2 + 6 * i / max(1, s["mem_heads"] - 1)) for i in range(s["mem_heads"])]},
                     "left_scale": 1.0, "right_scale": 1.0},
           "mlp": {"kind": "dense", "ff": s["ff"]}}
    ml = {"type": "mlstm", "mixer": {"heads": s["ml_heads"], "dim": s["ml_dim"], "vdim": s["ml_vdim"], "gate_cap": 15.0},
          "mlp": {"kind": "dense", "ff": s["ff"]}}
    return {"architecture": "Fatudra", "vocab": VOCAB, "width": s["width"], "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
            "layers": [par, ml, par, par][:LAYERS]}


def gipozen_config(s):
    d = s["dim"] // 2                       # two maps of half the head size: q is as wide as a plain head's
    mixer = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": d, "vdim": s["dim"], "conv": 4, "diff": 0.25,
             "mask": {"size": GIP_WINDOW, "keep_first": GIP_KEEP}, "scale": d ** -0.5}
    eff = s["ff"] // 4 // 32 * 32
    dense = {"kind": "dense", "ff": s["ff"]}
    moe = {"kind": "moe", "expert": {"ff": eff, "limit": 7.0}, "router": {"experts": GIP_EXPERTS, "identity": 1, "top": GIP_TOP},
           "shared": {"ff": eff, "limit": 7.0}}
    layers = []
    for i in range(LAYERS):
        m = dict(mixer)
        if i % 2:
            m["kv_from"] = i - 1
        layers.append({"type": "attention", "mixer": m, "mlp": moe if i % 2 else dense})
    return {"architecture": "Gipozen", "vocab": VOCAB, "width": s["width"], "norm": {"eps": 1e-6}, "logit_scale": 1.0, "layers": layers}


GIP_WINDOW, GIP_KEEP, GIP_EXPERTS, GIP_TOP = 1024, 4, 16, 4


FEK_RANK, FEK_ROT, FEK_EXPERTS, FEK_TOP, FEK_GROUPS, FEK_KEEP = 512, 64, 16, 4, 4, 2


def fekotar_config(s):
    mixer = {"heads": s["heads"], "dim": s["dim"], "rot_dim": FEK_ROT, "vdim": s["dim"], "q_rank": s["width"] * 3 // 8, "kv_rank": FEK_RANK,
             "scale": (s["dim"] + FEK_ROT) ** -0.5,
             "rot": {"base": 10000.0, "dims": FEK_ROT, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    eff = s["ff"] // 4 // 32 * 32
    dense = {"kind": "dense", "ff": s["ff"], "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": eff},
           "router": {"experts": FEK_EXPERTS, "top": FEK_TOP, "scale": 1.0, "groups": {"count": FEK_GROUPS, "keep": FEK_KEEP}}}
    layers = [{"type": "latent_attention", "mixer": dict(mixer), "mlp": dense if i == 0 else moe} for i in range(LAYERS)]
    return {"architecture": "Fekotar", "vocab": VOCAB, "width": s["width"], "norm": {"eps": 1e-6}, "logit_scale": 1.0,
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 131, "mul_cur": 3}}, "layers": layers}


def timed(fn, iters=10, warmup=3):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def batches(prompt_len, batch, ctx, device, vocab):
    from .step_batch import StepBatch
    g = torch.Generator().manual_seed(0)
    pages = (prompt_len + BLOCK - 1) // BLOCK
    pre = StepBatch.build([torch.randint(0, vocab, (prompt_len, ), generator=g).tolist()], [0], [list(range(pages))], [0], BLOCK,
                          device)
    per = (ctx + 1 + BLOCK - 1) // BLOCK
    perm = torch.randperm(batch * per, generator=g).view(batch, per).tolist()
    dec = StepBatch.build([[int(t)] for t in torch.randint(0, vocab, (batch, ), generator=g)], [ctx] * batch, perm,
                          list(range(batch)), BLOCK, device)
    return pre, dec, max(pages, batch * per)


def model_throughput(model, prompt_len, batch, ctx, device, vocab):
    pre, dec, pages = batches(prompt_len, batch, ctx, device, vocab)
    caches = model.make_caches(pages, BLOCK, batch, device)
    rows_p = torch.tensor([prompt_len - 1], device=device)
    rows_d = torch.arange(batch, device=device)
    tp = timed(lambda: model.step(pre, caches, rows_p), iters=5, warmup=2)
    td = timed(lambda: model.step(dec, caches, rows_d), iters=20, warmup=3)
    return {"prefill_tokens": prompt_len, "prefill_ms": round(tp * 1e3, 3), "prefill_tok_s": round(prompt_len / tp),
            "decode_batch": batch, "decode_ctx": ctx, "decode_ms": round(td * 1e3, 3), "decode_tok_s": round(batch / td)}


def kernel_section(s, prompt_len, batch, ctx, device):
    """Each mixer kernel alone at the stack's shapes, and the like kernel of the Llama path at the same shapes."""
    from . import _custom_ops as ops
    from . import mixer_ops as mops
    from .mixers import DistanceBiasAttention
    bf = torch.bfloat16
    H, G, d, W, ff = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"]
    pre, dec, pages = batches(prompt_len, batch, ctx, device, VOCAB)
    out = {}

    def rec(name, sec, bytes_=None, flops=None, like=None):
        r = {"us": round(sec * 1e6, 1)}
        if bytes_ is not None:
            r["frac_hbm"] = round(bytes_ / sec / HBM, 3)
        if flops is not None:
            r["frac_mfma"] = round(flops / sec / MFMA, 4)
        if like is not None:
            r["like"] = like
        out[name] = r
        return r

    # ---- attention --------------------------------------------------------------------------------------------------
    att = DistanceBiasAttention(H, G, d, d, d ** -0.5, bias_rows=32, bias_far=4096.0, temp_coef=0.1, temp_every=512).to(device)
    att.rel.normal_()
    att.finalize()
    kc, vc = att.cache_spec().allocate(pages, BLOCK, batch, bf, device)
    kc.normal_()
    vc.normal_()
    for name, b, T in (("prefill", pre, prompt_len), ("decode", dec, batch)):
        q = torch.randn(T, H * d, device=device, dtype=bf)
        gate = torch.randn(T, H, device=device, dtype=bf)
        o = torch.empty(T, H * d, device=device, dtype=bf)
        sec = timed(lambda: mops.distance_bias_attention(o, q, gate, kc, vc, b.block_tables, b.q_start, b.q_len, b.ctx_len,
                                                         b.seq_of_token, (min(b.q_lens), max(b.q_lens)), H, att.scale, att.bias_lut, att.temp_coef, att.temp_every,
                                                         max_kv_len=max(c + n for c, n in zip(b.ctx_lens, b.q_lens))))
        if name == "prefill":
            flops = 4.0 * d * H * T * (T + 1) / 2
            k = torch.randn(T, G, d, device=device, dtype=bf)
            v = torch.randn(T, G, d, device=device, dtype=bf)
            cu = torch.tensor([0, T], dtype=torch.int32, device=device)
            lsec = timed(lambda: ops.flash_attn_varlen(q.view(T, H, d), k, v, cu, T, d ** -0.5, causal=True))
            rec("attention_prefill", sec, flops=flops, like={"kernel": "flash_attn_varlen", "us": round(lsec * 1e6, 1),
                                                             "frac_mfma": round(flops / lsec / MFMA, 4)})
        else:
            nbytes = batch * (ctx + 1) * G * 2 * d * 2
            lk = torch.randn(pages, G, d // 8, BLOCK, 8, device=device, dtype=bf)
            lv = torch.randn(pages, G, d, BLOCK, device=device, dtype=bf)
            lens = torch.full((batch, ), ctx + 1, dtype=torch.int32, device=device)
            lo = torch.empty(T, H, d, device=device, dtype=bf)
            lsec = timed(lambda: ops.paged_attention_v1(lo, q.view(T, H, d), lk, lv, G, d ** -0.5, b.block_tables, lens, BLOCK,
                                                        ctx + 1, None, "auto", 1.0, 1.0))
            rec("attention_decode", sec, bytes_=nbytes, like={"kernel": "paged_attention_v1", "us": round(lsec * 1e6, 1),
                                                              "frac_hbm": round(nbytes / lsec / HBM, 3)})
    # ---- memories ---------------------------------------------------------------------------------------------------
    for tag, mode, Hm, dm, em in (("decay_memory", mops.MEMORY_DECAY, s["mem_heads"], s["mem_dim"], s["mem_vdim"]),
                                  ("mlstm_memory", mops.MEMORY_MLSTM, s["ml_heads"], s["ml_dim"], s["ml_vdim"])):
        state = tuple(torch.zeros(x, device=device) for x in mops.memory_state_shapes(batch, Hm, dm, em, mode))
        decay = torch.full((Hm, ), 0.99, device=device)
        for name, b, T in (("prefill", pre, prompt_len), ("decode", dec, batch)):
            q = torch.randn(T, Hm * dm, device=device, dtype=bf)
            k = torch.randn(T, Hm * dm, device=device, dtype=bf)
            v = torch.randn(T, Hm * em, device=device, dtype=bf)
            gi, gf = torch.randn(T, Hm, device=device, dtype=bf), torch.randn(T, Hm, device=device, dtype=bf) + 3
            sec = timed(lambda: mops.outer_memory_scan(q, k, v, state, b.state_slots, b.q_start, b.q_len, b.ctx_len, Hm, mode,
                                                       decay=decay, gate_i=gi, gate_f=gf, q_scale=dm ** -0.5, gate_cap=15.0,
                                                       max_q_len=max(b.q_lens)))
            if name == "prefill":
                rec(tag + "_prefill", sec, flops=4.0 * T * Hm * dm * em)
            else:
                rec(tag + "_decode", sec, bytes_=2.0 * batch * Hm * dm * em * 4)
    # ---- norm and activation ------------------------------------------------------------------------------------------
    for name, T in (("prefill", prompt_len), ("decode", batch)):
        res = torch.randn(T, W, device=device)
        y = torch.randn(T, W, device=device, dtype=bf)
        w = [torch.randn(W, device=device, dtype=bf) for _ in range(4)]
        sec = timed(lambda: mops.residual_layer_norm(res, y=y, post=(w[0], w[1]), pre=(w[2], w[3])))
        x16, r16 = torch.randn(T, W, device=device, dtype=bf), torch.randn(T, W, device=device, dtype=bf)
        lsec = timed(lambda: ops.fused_add_rms_norm(x16, r16, w[0], 1e-5))
        rec("residual_layer_norm_" + name, sec, bytes_=T * W * (4 + 4 + 2 + 2),
            like={"kernel": "fused_add_rms_norm", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * W * 8 / lsec / HBM, 3)})
        gu = torch.randn(T, 2 * ff, device=device, dtype=bf)
        sec = timed(lambda: mops.act_and_mul(gu, mops.ACT_GELU_TANH))
        lo = torch.empty(T, ff, device=device, dtype=bf)
        lsec = timed(lambda: ops.silu_and_mul(lo, gu))
        rec("act_and_mul_" + name, sec, bytes_=T * ff * 6,
            like={"kernel": "silu_and_mul", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * ff * 6 / lsec / HBM, 3)})
    return out


def gipozen_kernel_section(s, prompt_len, batch, ctx, device):
    """Each Gipozen kernel alone at the stack's shapes, and the like kernel of the Llama path at the same shapes."""
    from . import _custom_ops as ops
    from . import mixer_ops as mops
    from .mixers import PagedKVSpec
    bf = torch.bfloat16
    H, G, e, W, ff = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"]
    d = e // 2
    eff = ff // 4 // 32 * 32
    pre, dec, pages = batches(prompt_len, batch, ctx, device, VOCAB)
    out = {}

    def rec(name, sec, bytes_=None, flops=None, like=None):
        r = {"us": round(sec * 1e6, 1)}
        if bytes_ is not None:
            r["frac_hbm"] = round(bytes_ / sec / HBM, 3)
        if flops is not None:
            r["frac_mfma"] = round(flops / sec / MFMA, 4)
        if like is not None:
            r["like"] = like
        out[name] = r

    def visible_pairs(T):
        return sum(min(i + 1, GIP_WINDOW) + min(GIP_KEEP, max(0, i + 1 - GIP_WINDOW)) for i in range(T))

    # ---- attention: both maps, join, norm and gate in one launch ---------------------------------------------------------
    kc, vc = PagedKVSpec(G, d, e, 2).allocate(pages, BLOCK, batch, bf, device)
    kc.normal_()
    vc.normal_()
    for name, b, T in (("prefill", pre, prompt_len), ("decode", dec, batch)):
        q = torch.randn(T, H * 2 * d, device=device, dtype=bf)
        gate = torch.randn(T, H * e, device=device, dtype=bf)
        o = torch.empty(T, H * e, device=device, dtype=bf)
        sec = timed(lambda: mops.differential_window_attention(o, q, gate, kc, vc, b.block_tables, b.q_start, b.q_len, b.ctx_len,
                                                               b.seq_of_token, (min(b.q_lens), max(b.q_lens)), H, d ** -0.5, GIP_WINDOW,
                                                               GIP_KEEP, 0.2, 0.7, 1e-6,
                                                               max_kv_len=max(c + n for c, n in zip(b.ctx_lens, b.q_lens))))
        if name == "prefill":
            pairs = visible_pairs(T)
            flops = pairs * H * (4.0 * d + 4.0 * e)              # two maps: Q K^T over d, P V over e, each twice
            lq = torch.randn(T, H, e, device=device, dtype=bf)
            k = torch.randn(T, G, e, device=device, dtype=bf)
            v = torch.randn(T, G, e, device=device, dtype=bf)
            cu = torch.tensor([0, T], dtype=torch.int32, device=device)
            lsec = timed(lambda: ops.flash_attn_varlen(lq, k, v, cu, T, e ** -0.5, causal=True, window_size=(GIP_WINDOW - 1, 0)))
            lflops = pairs * H * 4.0 * e
            rec("attention_prefill", sec, flops=flops, like={"kernel": "flash_attn_varlen (window)", "us": round(lsec * 1e6, 1),
                                                             "frac_mfma": round(lflops / lsec / MFMA, 4)})
        else:
            nvis = min(ctx + 1, GIP_WINDOW) + min(GIP_KEEP, max(0, ctx + 1 - GIP_WINDOW))
            nbytes = batch * nvis * G * (2 * d + e) * 2
            lq = torch.randn(T, H, e, device=device, dtype=bf)
            lk = torch.randn(pages, G, e // 8, BLOCK, 8, device=device, dtype=bf)
            lv = torch.randn(pages, G, e, BLOCK, device=device, dtype=bf)
            lens = torch.full((batch, ), ctx + 1, dtype=torch.int32, device=device)
            lo = torch.empty(T, H, e, device=device, dtype=bf)
            lsec = timed(lambda: ops.paged_attention_v1(lo, lq, lk, lv, G, e ** -0.5, b.block_tables, lens, BLOCK, ctx + 1, None,
                                                        "auto", 1.0, 1.0))
            lbytes = batch * (ctx + 1) * G * 2 * e * 2
            rec("attention_decode", sec, bytes_=nbytes, like={"kernel": "paged_attention_v1", "us": round(lsec * 1e6, 1),
                                                              "frac_hbm": round(lbytes / lsec / HBM, 3)})
    # ---- convolution + cache write, norms, activation ---------------------------------------------------------------------
    C = H * 2 * d + G * 2 * d + G * e
    for name, b, T in (("prefill", pre, prompt_len), ("decode", dec, batch)):
        u = torch.randn(T, C + H * e, device=device, dtype=bf)
        w = torch.randn(C, 4, device=device, dtype=bf)
        state = torch.zeros(batch, 3, C, device=device, dtype=bf)
        sec = timed(lambda: mops.short_conv(u[:, :C], w, state, b.state_slots, b.q_start, b.q_len, b.ctx_len, b.seq_of_token,
                                            H * 2 * d, G * 2 * d, G * e, kc, vc, b.slot_mapping))
        k = torch.randn(T, G, e, device=device, dtype=bf)
        lkc = torch.zeros(pages, G, e // 8, BLOCK, 8, device=device, dtype=bf)
        lvc = torch.zeros(pages, G, e, BLOCK, device=device, dtype=bf)
        lq = torch.randn(T, H * e, device=device, dtype=bf)
        lk = torch.randn(T, G * e, device=device, dtype=bf)
        pos = b.positions
        cs = torch.randn(8192, e, device=device, dtype=bf)
        lsec = timed(lambda: (ops.rotary_embedding(pos, lq, lk, e, cs, True), ops.reshape_and_cache(k, k, lkc, lvc, b.slot_mapping, "auto", 1.0, 1.0)))
        rec("short_conv_cache_" + name, sec, bytes_=T * C * 4,
            like={"kernel": "rotary_embedding + reshape_and_cache", "us": round(lsec * 1e6, 1),
                  "frac_hbm": round(T * (H + 3 * G) * e * 4 / lsec / HBM, 3)})
        n_hist = LAYERS // 2
        hist = torch.randn(LAYERS + 1, T, W, device=device)
        x = torch.randn(T, W, device=device)
        y = torch.randn(T, W, device=device, dtype=bf)
        dw = torch.randn(n_hist + 1, device=device)
        sec = timed(lambda: mops.depth_residual_rms_norm(x, x_out=x, y=y, history=hist, n_hist=n_hist, depth_w=dw, gain=1.1))
        x16, r16 = torch.randn(T, W, device=device, dtype=bf), torch.randn(T, W, device=device, dtype=bf)
        w16 = torch.randn(W, device=device, dtype=bf)
        lsec = timed(lambda: ops.fused_add_rms_norm(x16, r16, w16, 1e-5))
        rec("depth_residual_rms_norm_" + name, sec, bytes_=T * W * (4 + 2 + 4 + 4 * n_hist + 4 + 2),
            like={"kernel": "fused_add_rms_norm", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * W * 8 / lsec / HBM, 3)})
        sec = timed(lambda: mops.depth_residual_rms_norm(x, x_out=x, y=y, gain=1.1))
        rec("residual_rms_norm_" + name, sec, bytes_=T * W * (4 + 2 + 4 + 2))
        z = torch.randn(T, ff, device=device, dtype=bf)
        sec = timed(lambda: mops.poly_norm(z, (0.7, 0.5, 0.3, 0.1), 1e-6))
        gu = torch.randn(T, 2 * ff, device=device, dtype=bf)
        lo = torch.empty(T, ff, device=device, dtype=bf)
        lsec = timed(lambda: ops.silu_and_mul(lo, gu))
        rec("poly_norm_" + name, sec, bytes_=T * ff * 4,
            like={"kernel": "silu_and_mul", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * ff * 6 / lsec / HBM, 3)})
        # ---- experts: route, sort, both products, combine -- against the dense feed-forward's library products of equal active size
        h = torch.randn(T, W, device=device, dtype=bf)
        R = GIP_EXPERTS + 1
        zr = torch.randn(T, R, device=device)
        ids, wts = mops.experts_route(zr, None, GIP_TOP)
        wgu = torch.randn(GIP_EXPERTS, 2 * eff, W, device=device, dtype=bf) * W ** -0.5
        wdn = torch.randn(GIP_EXPERTS, W, eff, device=device, dtype=bf) * eff ** -0.5
        sec = timed(lambda: mops.experts_forward(h, ids, wts, wgu, wdn, 7.0, 1.702))
        wl1 = torch.randn(2 * GIP_TOP * eff, W, device=device, dtype=bf)
        wl2 = torch.randn(W, GIP_TOP * eff, device=device, dtype=bf)
        act = torch.randn(T, GIP_TOP * eff, device=device, dtype=bf)
        lsec = timed(lambda: (torch.nn.functional.linear(h, wl1), torch.nn.functional.linear(act, wl2)))
        flops = 6.0 * T * GIP_TOP * eff * W
        wbytes = GIP_EXPERTS * 3 * eff * W * 2
        r = {"kernel": "library products of the dense feed-forward at the active size", "us": round(lsec * 1e6, 1)}
        if name == "prefill":
            r["frac_mfma"] = round(flops / lsec / MFMA, 4)
            rec("experts_" + name, sec, flops=flops, like=r)
        else:
            r["frac_hbm"] = round(3 * GIP_TOP * eff * W * 2 / lsec / HBM, 3)
            rec("experts_" + name, sec, bytes_=wbytes, like=r)
        sec = timed(lambda: mops.experts_route(zr, None, GIP_TOP))
        rec("experts_route_" + name, sec)
    return out


def fekotar_kernel_section(s, prompt_len, batch, ctx, device):
    """Each Fekotar kernel alone at the stack's shapes, and the like kernel of the Llama path at the same shapes."""
    from . import _custom_ops as ops
    from . import mixer_ops as mops
    from .mixers import LatentCacheSpec, RotaryFrequencies
    bf = torch.bfloat16
    H, G, d, W, ff = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"]
    R, P, Rq = FEK_RANK, FEK_ROT, s["width"] * 3 // 8
    eff = ff // 4 // 32 * 32
    pre, dec, pages = batches(prompt_len, batch, ctx, device, VOCAB)
    out = {}

    def rec(name, sec, bytes_=None, flops=None, like=None):
        r = {"us": round(sec * 1e6, 1)}
        if bytes_ is not None:
            r["frac_hbm"] = round(bytes_ / sec / HBM, 3)
        if flops is not None:
            r["frac_mfma"] = round(flops / sec / MFMA, 4)
        if like is not None:
            r["like"] = like
        out[name] = r

    rot = RotaryFrequencies(P, 10000.0, 4.0, 4096, 32.0, 1.0).to(device)
    cache = LatentCacheSpec(R, P).allocate(pages, BLOCK, batch, bf, device)
    cache.normal_()
    for name, b, T in (("prefill", pre, prompt_len), ("decode", dec, batch)):
        # ---- attention in the latent: every head over the shared rows -----------------------------------------------------------
        q_lat = torch.randn(T, H, R, device=device, dtype=bf) * R ** -0.5
        q = torch.randn(T, H, d + P, device=device, dtype=bf)
        o = torch.empty(T, H, R, device=device, dtype=bf)
        sec = timed(lambda: mops.latent_attention(o, q_lat, q[:, :, d:], cache, b.block_tables, b.q_start, b.q_len, b.ctx_len,
                                                  b.seq_of_token, (min(b.q_lens), max(b.q_lens)), rot.inv_freq, rot.mscale, P,
                                                  (d + P) ** -0.5, max_kv_len=max(c + n for c, n in zip(b.ctx_lens, b.q_lens))))
        lq = torch.randn(T, H, d, device=device, dtype=bf)
        if name == "prefill":
            pairs = T * (T + 1) / 2
            flops = pairs * H * (2.0 * (R + P) + 2.0 * R)
            k = torch.randn(T, G, d, device=device, dtype=bf)
            v = torch.randn(T, G, d, device=device, dtype=bf)
            cu = torch.tensor([0, T], dtype=torch.int32, device=device)
            lsec = timed(lambda: ops.flash_attn_varlen(lq, k, v, cu, T, d ** -0.5, causal=True))
            rec("attention_prefill", sec, flops=flops, like={"kernel": "flash_attn_varlen", "us": round(lsec * 1e6, 1),
                                                             "frac_mfma": round(pairs * H * 4.0 * d / lsec / MFMA, 4)})
        else:
            nbytes = batch * (ctx + 1) * (R + P) * 2
            lk = torch.randn(pages, G, d // 8, BLOCK, 8, device=device, dtype=bf)
            lv = torch.randn(pages, G, d, BLOCK, device=device, dtype=bf)
            lens = torch.full((batch, ), ctx + 1, dtype=torch.int32, device=device)
            lo = torch.empty(T, H, d, device=device, dtype=bf)
            lsec = timed(lambda: ops.paged_attention_v1(lo, lq, lk, lv, G, d ** -0.5, b.block_tables, lens, BLOCK, ctx + 1, None,
                                                        "auto", 1.0, 1.0))
            lbytes = batch * (ctx + 1) * G * 2 * d * 2
            rec("attention_decode", sec, bytes_=nbytes, like={"kernel": "paged_attention_v1", "us": round(lsec * 1e6, 1),
                                                              "frac_hbm": round(lbytes / lsec / HBM, 3)})
        # ---- norms of the latents + rotation + cache write -----------------------------------------------------------------------
        proj = torch.randn(T, Rq + R + P + H * d, device=device, dtype=bf)
        wq, wkv = torch.randn(Rq, device=device, dtype=bf), torch.randn(R, device=device, dtype=bf)
        sec = timed(lambda: mops.latent_prep(proj, 0, Rq, Rq, R, P, P, wq, wkv, cache, b.slot_mapping, b.q_start, b.ctx_len,
                                             b.seq_of_token, rot.inv_freq, rot.mscale, 1e-6))
        k = torch.randn(T, G, d, device=device, dtype=bf)
        lkc = torch.zeros(pages, G, d // 8, BLOCK, 8, device=device, dtype=bf)
        lvc = torch.zeros(pages, G, d, BLOCK, device=device, dtype=bf)
        lqq = torch.randn(T, H * d, device=device, dtype=bf)
        lkk = torch.randn(T, G * d, device=device, dtype=bf)
        cs = torch.randn(8192, d, device=device, dtype=bf)
        lsec = timed(lambda: (ops.rotary_embedding(b.positions, lqq, lkk, d, cs, True),
                              ops.reshape_and_cache(k, k, lkc, lvc, b.slot_mapping, "auto", 1.0, 1.0)))
        rec("latent_prep_" + name, sec, bytes_=T * (Rq + R + P) * 4,
            like={"kernel": "rotary_embedding + reshape_and_cache", "us": round(lsec * 1e6, 1),
                  "frac_hbm": round(T * (H + 3 * G) * d * 4 / lsec / HBM, 3)})
        # ---- output gate, both sublayers' residual add + norm, the dense activation, the embedding ----------------------------------
        og, gg = torch.randn(T, H * d, device=device, dtype=bf), torch.randn(T, H * d, device=device, dtype=bf)
        sec = timed(lambda: mops.sigmoid_gate_mul(og, gg, out=og))
        rec("sigmoid_gate_mul_" + name, sec, bytes_=T * H * d * 6)
        x = torch.randn(T, W, device=device)
        ya, yb = torch.randn(T, W, device=device, dtype=bf), torch.randn(T, W, device=device, dtype=bf)
        w16 = torch.randn(W, device=device, dtype=bf)
        sec = timed(lambda: mops.residual_add2_rms_norm(x, ya, yb, weight=w16))
        x16, r16 = torch.randn(T, W, device=device, dtype=bf), torch.randn(T, W, device=device, dtype=bf)
        lsec = timed(lambda: ops.fused_add_rms_norm(x16, r16, w16, 1e-5))
        rec("residual_add2_rms_norm_" + name, sec, bytes_=T * W * (4 + 4 + 2 + 2 + 2),
            like={"kernel": "fused_add_rms_norm", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * W * 8 / lsec / HBM, 3)})
        gu = torch.randn(T, 2 * ff, device=device, dtype=bf)
        sec = timed(lambda: mops.clamped_glu(gu, ff, 7.0, 1.702))
        lo2 = torch.empty(T, ff, device=device, dtype=bf)
        lsec = timed(lambda: ops.silu_and_mul(lo2, gu))
        rec("clamped_glu_" + name, sec, bytes_=T * ff * 6,
            like={"kernel": "silu_and_mul", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * ff * 6 / lsec / HBM, 3)})
        table, pair = torch.randn(VOCAB, W, device=device, dtype=bf), torch.randn(65522, W, device=device, dtype=bf)
        tstate = torch.zeros(batch, dtype=torch.int32, device=device)
        sec = timed(lambda: mops.hashed_pair_embed(table, pair, b.input_ids, tstate, b.state_slots, b.q_start, b.q_len, b.ctx_len,
                                                   b.seq_of_token, 131, 3))
        rec("hashed_pair_embed_" + name, sec, bytes_=T * W * 8)
        # ---- experts: route, sort, both products, combine -- against the dense feed-forward's library products of equal active size
        h = torch.randn(T, W, device=device, dtype=bf)
        zr = torch.randn(T, FEK_EXPERTS, device=device)
        ids, wts = mops.experts_route_grouped(zr, FEK_TOP, FEK_GROUPS, FEK_KEEP, 1.0)
        wgu = torch.randn(FEK_EXPERTS, 2 * eff, W, device=device, dtype=bf) * W ** -0.5
        wdn = torch.randn(FEK_EXPERTS, W, eff, device=device, dtype=bf) * eff ** -0.5
        sec = timed(lambda: mops.experts_forward(h, ids, wts, wgu, wdn, 0.0, 1.0))
        wl1 = torch.randn(2 * FEK_TOP * eff, W, device=device, dtype=bf)
        wl2 = torch.randn(W, FEK_TOP * eff, device=device, dtype=bf)
        act = torch.randn(T, FEK_TOP * eff, device=device, dtype=bf)
        lsec = timed(lambda: (torch.nn.functional.linear(h, wl1), torch.nn.functional.linear(act, wl2)))
        flops = 6.0 * T * FEK_TOP * eff * W
        r = {"kernel": "library products of the dense feed-forward at the active size", "us": round(lsec * 1e6, 1)}
        if name == "prefill":
            r["frac_mfma"] = round(flops / lsec / MFMA, 4)
            rec("experts_" + name, sec, flops=flops, like=r)
        else:
            r["frac_hbm"] = round(3 * FEK_TOP * eff * W * 2 / lsec / HBM, 3)
            rec("experts_" + name, sec, bytes_=FEK_EXPERTS * 3 * eff * W * 2, like=r)
        sec = timed(lambda: mops.experts_route_grouped(zr, FEK_TOP, FEK_GROUPS, FEK_KEEP, 1.0))
        rec("experts_route_grouped_" + name, sec)
    return out


PAG_RANK, PAG_ROT, PAG_WINDOW, PAG_EXPERTS, PAG_TOP, PAG_STREAMS, PAG_TAPS = 512, 64, 1024, 16, 4, 4, 4


def pagulix_config(s):
    """delta, windowed latent attention, two rotary attentions that blend values; four streams; 16 experts (top 4) + a shared one"""
    eff = s["ff"] // 4 // 32 * 32
    moe = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": PAG_EXPERTS, "top": PAG_TOP}, "shared": {"ff": eff}}
    rot = {"base": 500000.0, "dims": s["dim"] // 2, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    delta = {"type": "delta", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"], "conv": PAG_TAPS}}
    latent = {"type": "latent_attention",
              "mixer": {"heads": s["heads"], "dim": s["dim"], "rot_dim": PAG_ROT, "vdim": s["dim"], "kv_rank": PAG_RANK,
                        "scale": (s["dim"] + PAG_ROT) ** -0.5, "mask": {"size": PAG_WINDOW}, "rot": {"base": 10000.0, "dims": PAG_ROT}}}
    attn = {"type": "attention", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"], "rot": rot,
                                           "scale": s["dim"] ** -0.5, "v_mix": True}}
    layers = [dict(l, mlp=moe) for l in (delta, latent, attn, attn)][:LAYERS]
    return {"architecture": "Pagulix", "vocab": VOCAB, "width": s["width"], "norm": {"eps": 1e-6}, "streams": PAG_STREAMS,
            "residual_mult": 0.5, "logit_softcap": 30.0, "layers": layers}


def pagulix_kernel_section(s, prompt_len, batch, ctx, device):
    """Each kernel that Pagulix adds (or extends) alone at the stack's shapes, beside the like kernel of the closest existing path."""
    from . import _custom_ops as ops
    from . import mixer_ops as mops
    from .mixers import LatentCacheSpec, RotaryFrequencies
    bf = torch.bfloat16
    H, G, d, W, ff = s["heads"], s["kv_heads"], s["dim"], s["width"], s["ff"]
    R, P, n = PAG_RANK, PAG_ROT, PAG_STREAMS
    pre, dec, pages = batches(prompt_len, batch, ctx, device, VOCAB)
    out = {}

    def rec(name, sec, bytes_=None, flops=None, like=None):
        r = {"us": round(sec * 1e6, 1)}
        if bytes_ is not None:
            r["frac_hbm"] = round(bytes_ / sec / HBM, 3)
        if flops is not None:
            r["frac_mfma"] = round(flops / sec / MFMA, 4)
        if like is not None:
            r["like"] = like
        out[name] = r

    rot = RotaryFrequencies(P, 10000.0).to(device)
    rot_a = RotaryFrequencies.wavelength_scaled(d // 2, 500000.0, 8.0, 1.0, 4.0, 8192).to(device)
    cache = LatentCacheSpec(R, P).allocate(pages, BLOCK, batch, bf, device)
    cache.normal_()
    sink = torch.randn(H, device=device)
    kc = torch.randn(pages, BLOCK, G, d, device=device, dtype=bf)
    vc = torch.randn(pages, BLOCK, G, d, device=device, dtype=bf)
    for name, b, T in (("prefill", pre, prompt_len), ("decode", dec, batch)):
        lens = (min(b.q_lens), max(b.q_lens))
        kvmax = max(c + q for c, q in zip(b.ctx_lens, b.q_lens))
        # ---- the streamed residual: write of one sublayer + read and norm of the next -------------------------------------------
        x = torch.randn(T, n, W, device=device)
        y, ls, w16 = torch.randn(T, W, device=device, dtype=bf), torch.randn(W, device=device, dtype=bf), torch.randn(W, device=device, dtype=bf)
        mix = (torch.eye(n) + 0.1 * torch.randn(n, n)).tolist()
        oc, ic = [1.0] * n, [0.5] * n
        sec = timed(lambda: mops.hyper_residual_rms_norm(x, y, ls, mix, oc, 0.5, ic, w16, 1e-6))
        x16, r16 = torch.randn(T, W, device=device, dtype=bf), torch.randn(T, W, device=device, dtype=bf)
        lsec = timed(lambda: ops.fused_add_rms_norm(x16, r16, w16, 1e-5))
        rec("hyper_residual_rms_norm_" + name, sec, bytes_=T * W * (8 * n + 4),
            like={"kernel": "fused_add_rms_norm", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * W * 8 / lsec / HBM, 3)})
        # ---- the gated delta rule beside the decay memory of equal shape ------------------------------------------------------------
        q, k = torch.randn(T, G * d, device=device, dtype=bf), torch.randn(T, G * d, device=device, dtype=bf)
        v = torch.randn(T, H * d, device=device, dtype=bf)
        bb, aa = torch.randn(T, H, device=device, dtype=bf), torch.randn(T, H, device=device, dtype=bf)
        a_log, dtb = torch.zeros(H, device=device), torch.zeros(H, device=device)
        state = torch.zeros(batch, H, d, d, device=device)
        sec = timed(lambda: mops.gated_delta_scan(q, k, v, bb, aa, a_log, dtb, state, b.state_slots, b.q_start, b.q_len, b.ctx_len, H, G,
                                                  d ** -0.5, 1e-6, max_q_len=lens[1]))
        qh = torch.randn(T, H * d, device=device, dtype=bf)
        decay = torch.full((H, ), 0.97, device=device)
        lsec = timed(lambda: mops.outer_memory_scan(qh, qh, v, (state, ), b.state_slots, b.q_start, b.q_len, b.ctx_len, H, mops.MEMORY_DECAY,
                                                    decay, max_q_len=lens[1]))
        like = {"kernel": "outer_memory_scan (decay)", "us": round(lsec * 1e6, 1)}
        if name == "prefill":
            rec("gated_delta_scan_" + name, sec, flops=T * H * 4.0 * d * d, like=dict(like, frac_mfma=round(T * H * 4.0 * d * d / lsec / MFMA, 5)))
        else:
            nb = batch * H * d * d * 8
            rec("gated_delta_scan_" + name, sec, bytes_=nb, like=dict(like, frac_hbm=round(nb / lsec / HBM, 3)))
        o32, gate, wn = torch.randn(T, H * d, device=device), torch.randn(T, H * d, device=device, dtype=bf), torch.randn(d, device=device, dtype=bf)
        yo = torch.empty(T, H * d, device=device, dtype=bf)
        sec = timed(lambda: mops.gated_head_rms_norm(yo, o32, wn, gate, H, 1e-6, mops.GATE_SILU))
        wfull = wn.repeat(H)
        lsec = timed(lambda: mops.gated_group_rms_norm(yo, o32, wfull, gate, d, 1e-6))
        rec("gated_head_rms_norm_" + name, sec, bytes_=T * H * d * 8,
            like={"kernel": "gated_group_rms_norm", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * H * d * 8 / lsec / HBM, 3)})
        C = 2 * G * d + H * d
        u, cw = torch.randn(T, C, device=device, dtype=bf), torch.randn(C, PAG_TAPS, device=device, dtype=bf)
        cstate = torch.zeros(batch, PAG_TAPS - 1, C, device=device, dtype=bf)
        sec = timed(lambda: mops.short_conv(u, cw, cstate, b.state_slots, b.q_start, b.q_len, b.ctx_len, b.seq_of_token, C, act=1))
        lsec = timed(lambda: mops.short_conv(u, cw, cstate, b.state_slots, b.q_start, b.q_len, b.ctx_len, b.seq_of_token, C))
        rec("short_conv_silu_" + name, sec, bytes_=T * C * 4,
            like={"kernel": "short_conv (no activation)", "us": round(lsec * 1e6, 1), "frac_hbm": round(T * C * 4 / lsec / HBM, 3)})
        # ---- rotation + unit RMS + value blend + cache write ---------------------------------------------------------------------------
        pq, pk, pv = torch.randn(T, H * d, device=device, dtype=bf), torch.randn(T, G * d, device=device, dtype=bf), torch.randn(T, G * d, device=device, dtype=bf)
        vo = torch.randn(T, G * d, device=device, dtype=bf)
        sec = timed(lambda: mops.rotary_qk_norm_kv_write(pq, pk, pv, kc, vc, b.slot_mapping, b.q_start, b.ctx_len, b.seq_of_token,
                                                         rot_a.inv_freq, d // 2, mops.ROTARY_HALF, True, 1e-6, vo, 0.3))
        lkc = torch.zeros(pages, G, d // 8, BLOCK, 8, device=device, dtype=bf)
        lvc = torch.zeros(pages, G, d, BLOCK, device=device, dtype=bf)
        cs = torch.randn(8192, d, device=device, dtype=bf)
        k3 = pk.view(T, G, d)
        lsec = timed(lambda: (ops.rotary_embedding(b.positions, pq, pk, d, cs, True),
                              ops.reshape_and_cache(k3, k3, lkc, lvc, b.slot_mapping, "auto", 1.0, 1.0)))
        rec("rotary_qk_norm_kv_write_" + name, sec, bytes_=T * ((2 * H + 5 * G) * d) * 2,
            like={"kernel": "rotary_embedding + reshape_and_cache", "us": round(lsec * 1e6, 1),
                  "frac_hbm": round(T * (H + 3 * G) * d * 4 / lsec / HBM, 3)})
        # ---- causal attention on the kernels of the distance-biased attention, no bias ----------------------------------------------------
        o = torch.empty(T, H * d, device=device, dtype=bf)
        sec = timed(lambda: mops.distance_bias_attention(o, pq, None, kc, vc, b.block_tables, b.q_start, b.q_len, b.ctx_len, b.seq_of_token,
                                                         lens, H, d ** -0.5, None, max_kv_len=kvmax))
        lq = pq.view(T, H, d)
        if name == "prefill":
            pairs = T * (T + 1) / 2
            kk, vv = torch.randn(T, G, d, device=device, dtype=bf), torch.randn(T, G, d, device=device, dtype=bf)
            cu = torch.tensor([0, T], dtype=torch.int32, device=device)
            lsec = timed(lambda: ops.flash_attn_varlen(lq, kk, vv, cu, T, d ** -0.5, causal=True))
            rec("attention_prefill", sec, flops=pairs * H * 4.0 * d,
                like={"kernel": "flash_attn_varlen", "us": round(lsec * 1e6, 1), "frac_mfma": round(pairs * H * 4.0 * d / lsec / MFMA, 4)})
        else:
            lens_t = torch.full((batch, ), ctx + 1, dtype=torch.int32, device=device)
            lo = torch.empty(T, H, d, device=device, dtype=bf)
            lsec = timed(lambda: ops.paged_attention_v1(lo, lq, lkc, lvc, G, d ** -0.5, b.block_tables, lens_t, BLOCK, ctx + 1, None, "auto", 1.0, 1.0))
            nb = batch * (ctx + 1) * G * 2 * d * 2
            rec("attention_decode", sec, bytes_=nb, like={"kernel": "paged_attention_v1", "us": round(lsec * 1e6, 1), "frac_hbm": round(nb / lsec / HBM, 3)})
        # ---- attention in the latent under a window, with a sink -- beside the same launch without either ------------------------------
        q_lat = torch.randn(T, H, R, device=device, dtype=bf) * R ** -0.5
        qr = torch.randn(T, H, P, device=device, dtype=bf)
        ol = torch.empty(T, H, R, device=device, dtype=bf)
        la = lambda w, sk: mops.latent_attention(ol, q_lat, qr, cache, b.block_tables, b.q_start, b.q_len, b.ctx_len, b.seq_of_token, lens,
                                                 rot.inv_freq, 1.0, P, (d + P) ** -0.5, max_kv_len=kvmax, window=w, sink=sk)
        sec = timed(lambda: la(PAG_WINDOW, sink))
        lsec = timed(lambda: la(0, None))
        if name == "prefill":
            wpairs = sum(min(i + 1, PAG_WINDOW) for i in range(T))
            per = H * (2.0 * (R + P) + 2.0 * R)
            rec("latent_attention_window_prefill", sec, flops=wpairs * per,
                like={"kernel": "latent attention, causal, no sink", "us": round(lsec * 1e6, 1),
                      "frac_mfma": round(T * (T + 1) / 2 * per / lsec / MFMA, 4)})
        else:
            rec("latent_attention_window_decode", sec, bytes_=batch * min(ctx + 1, PAG_WINDOW) * (R + P) * 2,
                like={"kernel": "latent attention, causal, no sink", "us": round(lsec * 1e6, 1),
                      "frac_hbm": round(batch * (ctx + 1) * (R + P) * 2 / lsec / HBM, 3)})
        # ---- router ----------------------------------------------------------------------------------------------------------------------
        zr, rb = torch.randn(T, PAG_EXPERTS, device=device), torch.randn(PAG_EXPERTS, device=device)
        sec = timed(lambda: mops.experts_route_topk(zr, rb, PAG_TOP))
        lsec = timed(lambda: mops.experts_route_grouped(zr, PAG_TOP, 4, 2, 1.0))
        rec("experts_route_topk_" + name, sec, like={"kernel": "experts_route_grouped", "us": round(lsec * 1e6, 1)})
    z = torch.randn(batch, VOCAB, device=device, dtype=bf)
    sec = timed(lambda: mops.logit_softcap(z, 1.0, 30.0))
    lsec = timed(lambda: z.float() * 1.0)
    rec("logit_softcap_decode", sec, bytes_=batch * VOCAB * 6, like={"kernel": "cast and scale", "us": round(lsec * 1e6, 1),
                                                                     "frac_hbm": round(batch * VOCAB * 6 / lsec / HBM, 3)})
    return out


def main_pagulix(args) -> int:
    from . import _lib
    from .fekotar import FekotarConfig, FekotarForCausalLM
    from .model import LlamaConfig, LlamaForCausalLM
    from .pagulix import PagulixConfig, PagulixForCausalLM
    _lib.lib()
    _lib.mixers_lib()
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    prompt_len, batch, ctx = args.mixers_prompt, args.batch, args.ctx
    result = {"metric": "pagulix_vs_llama_bf16_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "n_gpus": 1, "layers": LAYERS, "sizes": {}}
    with torch.no_grad():
        for name, s in SIZES.items():
            if args.mixers_size and name != args.mixers_size:
                continue
            t0 = time.time()
            pag = PagulixForCausalLM(PagulixConfig.from_dict(pagulix_config(s)), torch.bfloat16).init_synthetic(device)
            r = {"pagulix": model_throughput(pag, prompt_len, batch, ctx, device, VOCAB)}
            del pag
            fek = FekotarForCausalLM(FekotarConfig.from_dict(fekotar_config(s)), torch.bfloat16).init_synthetic(device)
            r["fekotar"] = model_throughput(fek, prompt_len, batch, ctx, device, VOCAB)
            del fek
            lc = LlamaConfig(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=LAYERS,
                             num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], vocab_size=VOCAB,
                             max_position_embeddings=max(8192, prompt_len + 16))
            llama = LlamaForCausalLM(lc, None, torch.bfloat16).init_synthetic(device)
            llama.use_fused_decode = False
            r["llama"] = model_throughput(llama, prompt_len, batch, ctx, device, VOCAB)
            del llama
            r["kernels"] = pagulix_kernel_section(s, prompt_len, batch, ctx, device)
            r["seconds"] = round(time.time() - t0, 1)
            result["sizes"][name] = r
            torch.cuda.empty_cache()
    print(json.dumps(result), flush=True)
    return 0


def main(args) -> int:
    from . import _lib
    if getattr(args, "mixers_design", "fatudra") == "pagulix":
        return main_pagulix(args)
    if getattr(args, "mixers_design", "fatudra") == "gipozen":
        return main_gipozen(args)
    if getattr(args, "mixers_design", "fatudra") == "fekotar":
        return main_fekotar(args)
    from .fatudra import FatudraConfig, FatudraForCausalLM
    from .model import LlamaConfig, LlamaForCausalLM
    _lib.lib()
    _lib.mixers_lib()
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    prompt_len, batch, ctx = args.mixers_prompt, args.batch, args.ctx
    result = {"metric": "fatudra_vs_llama_bf16_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "n_gpus": 1, "layers": LAYERS, "sizes": {}}
    with torch.no_grad():
        for name, s in SIZES.items():
            if args.mixers_size and name != args.mixers_size:
                continue
            t0 = time.time()
            fat = FatudraForCausalLM(FatudraConfig.from_dict(fatudra_config(s)), torch.bfloat16).init_synthetic(device)
            r = {"fatudra": model_throughput(fat, prompt_len, batch, ctx, device, VOCAB)}
            del fat
            lc = LlamaConfig(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=LAYERS,
                             num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], vocab_size=VOCAB,
                             max_position_embeddings=max(8192, prompt_len + 16))
            llama = LlamaForCausalLM(lc, None, torch.bfloat16).init_synthetic(device)
            llama.use_fused_decode = False
            r["llama"] = model_throughput(llama, prompt_len, batch, ctx, device, VOCAB)
            del llama
            r["kernels"] = kernel_section(s, prompt_len, batch, ctx, device)
            r["seconds"] = round(time.time() - t0, 1)
            result["sizes"][name] = r
            torch.cuda.empty_cache()
    print(json.dumps(result), flush=True)
    return 0


def main_gipozen(args) -> int:
    from . import _lib
    from .gipozen import GipozenConfig, GipozenForCausalLM
    from .model import LlamaConfig, LlamaForCausalLM
    _lib.lib()
    _lib.mixers_lib()
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    prompt_len, batch, ctx = args.mixers_prompt, args.batch, args.ctx
    result = {"metric": "gipozen_vs_llama_bf16_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "n_gpus": 1, "layers": LAYERS, "sizes": {}}
    with torch.no_grad():
        for name, s in SIZES.items():
            if args.mixers_size and name != args.mixers_size:
                continue
            t0 = time.time()
            gip = GipozenForCausalLM(GipozenConfig.from_dict(gipozen_config(s)), torch.bfloat16).init_synthetic(device)
            r = {"gipozen": model_throughput(gip, prompt_len, batch, ctx, device, VOCAB)}
            del gip
            lc = LlamaConfig(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=LAYERS,
                             num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], vocab_size=VOCAB,
                             max_position_embeddings=max(8192, prompt_len + 16))
            llama = LlamaForCausalLM(lc, None, torch.bfloat16).init_synthetic(device)
            llama.use_fused_decode = False
            r["llama"] = model_throughput(llama, prompt_len, batch, ctx, device, VOCAB)
            del llama
            r["kernels"] = gipozen_kernel_section(s, prompt_len, batch, ctx, device)
            r["seconds"] = round(time.time() - t0, 1)
            result["sizes"][name] = r
            torch.cuda.empty_cache()
    print(json.dumps(result), flush=True)
    return 0


def main_fekotar(args) -> int:
    from . import _lib
    from .fekotar import FekotarConfig, FekotarForCausalLM
    from .gipozen import GipozenConfig, GipozenForCausalLM
    from .model import LlamaConfig, LlamaForCausalLM
    _lib.lib()
    _lib.mixers_lib()
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    prompt_len, batch, ctx = args.mixers_prompt, args.batch, args.ctx
    result = {"metric": "fekotar_vs_llama_bf16_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
              "n_gpus": 1, "layers": LAYERS, "sizes": {}}
    with torch.no_grad():
        for name, s in SIZES.items():
            if args.mixers_size and name != args.mixers_size:
                continue
            t0 = time.time()
            fek = FekotarForCausalLM(FekotarConfig.from_dict(fekotar_config(s)), torch.bfloat16).init_synthetic(device)
            r = {"fekotar": model_throughput(fek, prompt_len, batch, ctx, device, VOCAB)}
            del fek
            gip = GipozenForCausalLM(GipozenConfig.from_dict(gipozen_config(s)), torch.bfloat16).init_synthetic(device)
            r["gipozen"] = model_throughput(gip, prompt_len, batch, ctx, device, VOCAB)
            del gip
            lc = LlamaConfig(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=LAYERS,
                             num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], vocab_size=VOCAB,
                             max_position_embeddings=max(8192, prompt_len + 16))
            llama = LlamaForCausalLM(lc, None, torch.bfloat16).init_synthetic(device)
            llama.use_fused_decode = False
            r["llama"] = model_throughput(llama, prompt_len, batch, ctx, device, VOCAB)
            del llama
            r["kernels"] = fekotar_kernel_section(s, prompt_len, batch, ctx, device)
            r["seconds"] = round(time.time() - t0, 1)
            result["sizes"][name] = r
            torch.cuda.empty_cache()
    print(json.dumps(result), flush=True)
    return 0
