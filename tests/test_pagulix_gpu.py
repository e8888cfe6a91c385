"""Pagulix on the GPU against the plain restatement (oracle/pagulix.py, float64): every kernel alone, then the model through the
engine -- whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages and slots, long
decoding past every window, greedy generation through the scheduler, the trace replay command.  Small random configurations made
here; sizes are unlike one another and unlike any shipped model.  Unused cache memory is poisoned with NaN so that a read outside
a sequence's own keys or of a stale state shows."""
import numpy as np
import pytest
import torch

import pagulix_util as U
from oracle import pagulix as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def mops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    torch.backends.cuda.matmul.allow_tf32 = False
    from aphrodite_engine_amd import mixer_ops
    return mixer_ops


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(DEV).to(dtype)


def rounded(a, dtype):
    return U.bf16_round(a).astype(np.float64) if dtype == torch.bfloat16 else np.asarray(a, np.float32).astype(np.float64)


def tol_of(dtype):
    return 3e-5 if dtype == torch.float32 else 2e-2


def batch_of(segs, tables, slots, block):
    """segs: [(ctx, tokens)] -> StepBatch"""
    from aphrodite_engine_amd.step_batch import StepBatch
    return StepBatch.build([list(t) for _, t in segs], [c for c, _ in segs], tables, slots, block, DEV)


def run_cut(fn, T, cuts, slot=1, block=16, tables=None):
    """Calls fn(batch, lo, hi) for consecutive portions of one sequence of T tokens."""
    at, out = 0, []
    for n in cuts:
        b = batch_of([(at, [0] * n)], [tables or list(range((T + block - 1) // block))], [slot], block)
        out.append(fn(b, at, at + n))
        at += n
    assert at == T
    return out


# ---------------------------------------------------------------------------------------------------------------------
# the streamed residual
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("streams,width", [(1, 72), (2, 75), (3, 200), (4, 1032), (5, 64), (9, 40)])
def test_streamed_residual_write_then_read(mops, dtype, streams, width):
    rng = np.random.default_rng(streams)
    T, mult, eps = 7, 0.37, 1e-5
    x = rng.standard_normal((T, streams, width))
    y, scale, weight = (rounded(rng.standard_normal(s), dtype) for s in ((T, width), (width,), (width,)))
    mix, out_c, in_c = rng.standard_normal((streams, streams)), rng.standard_normal(streams), rng.standard_normal(streams)
    f32 = lambda a: np.asarray(a, np.float32).astype(np.float64)
    mix, out_c, in_c, xr = f32(mix), f32(out_c), f32(in_c), f32(x)
    new = np.einsum("st,nsw->ntw", mix, xr) + np.float32(mult) * out_c[None, :, None] * (y * scale)[:, None, :]
    u = np.einsum("s,nsw->nw", in_c, new)
    want = O.rms_norm(u, weight, eps)
    xd = dev(x)
    got, total = mops.hyper_residual_rms_norm(xd, dev(y, dtype), dev(scale, dtype), mix.tolist(), out_c.tolist(), mult, in_c.tolist(),
                                              dev(weight, dtype), eps, want_sum=True)
    np.testing.assert_allclose(xd.cpu().numpy(), new, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(total.cpu().numpy(), u, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=tol_of(dtype), atol=tol_of(dtype))
    # the read alone leaves the streams as they are; no coefficients: the plain residual and the sum of the streams
    before = xd.clone()
    got = mops.hyper_residual_rms_norm(xd, None, None, None, None, mult, None, None, eps, dtype=dtype)
    assert torch.equal(xd, before)
    np.testing.assert_allclose(got.float().cpu().numpy(), O.rms_norm(new.sum(1), None, eps), rtol=tol_of(dtype), atol=tol_of(dtype))
    mops.hyper_residual_rms_norm(xd, dev(y, dtype), None, None, None, mult, want_out=False)
    np.testing.assert_allclose(xd.cpu().numpy(), new + np.float32(mult) * y[:, None, :], rtol=2e-5, atol=2e-5)


def test_logit_softcap(mops):
    z = np.linspace(-40, 40, 333)
    got = mops.logit_softcap(dev(z), 1.0, 7.5).cpu().numpy()
    np.testing.assert_allclose(got, 7.5 * np.tanh(z / 7.5), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(mops.logit_softcap(dev(z), 0.5, 0.0).cpu().numpy(), 0.5 * z, rtol=1e-6)


# ---------------------------------------------------------------------------------------------------------------------
# the gated delta rule
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,channels", [(4, 64), (3, 52), (1, 24), (7, 40)])
def test_short_convolution_with_silu_cut_anywhere(mops, dtype, taps, channels):
    rng = np.random.default_rng(taps)
    T = 45
    u, w = rounded(rng.standard_normal((T, channels)), dtype), rounded(rng.standard_normal((channels, taps)), dtype)
    want = O.silu(O.causal_conv(u, w))
    state = torch.full((3, max(taps - 1, 0), channels), float("nan"), dtype=dtype, device=DEV)
    ud, wd = dev(u, dtype), dev(w, dtype)

    def part(b, lo, hi):
        return mops.short_conv(ud[lo:hi], wd, state, b.state_slots, b.q_start, b.q_len, b.ctx_len, b.seq_of_token, channels, act=1)
    for cuts in ([T], [1] * T, [2, 1, 1, 9, 2, 30], [40, 1, 1, 1, 2]):
        got = torch.cat(run_cut(part, T, cuts)).float().cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=tol_of(dtype), atol=tol_of(dtype))


def delta_inputs(rng, T, H, G, d, e, dtype, loud=None):
    q, k = rounded(rng.standard_normal((T, G, d)), dtype), rounded(rng.standard_normal((T, G, d)), dtype)
    v = rounded(rng.standard_normal((T, H, e)), dtype)
    b, a = rounded(rng.standard_normal((T, H)) * 2, dtype), rounded(rng.standard_normal((T, H)) * 2, dtype)
    a_log, dt_bias = np.float32(np.log(rng.uniform(0.2, 3.0, H))).astype(np.float64), np.float32(rng.standard_normal(H)).astype(np.float64)
    return q, k, v, b, a, a_log, dt_bias


def delta_oracle(q, k, v, b, a, a_log, dt_bias):
    T, G, d = q.shape
    H = v.shape[1]
    qn = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    kn = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta, g = O.sigmoid(b), np.exp(-np.exp(a_log) * O.softplus(a + dt_bias))
    return np.stack([O.delta_rule(qn[:, h // (H // G)], kn[:, h // (H // G)], v[:, h], beta[:, h], g[:, h]) for h in range(H)], 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e", [(4, 2, 24, 40), (3, 3, 64, 64), (2, 1, 100, 72), (6, 2, 16, 130), (1, 1, 200, 8)])
def test_delta_rule_in_segments_of_every_size(mops, dtype, H, G, d, e):
    rng = np.random.default_rng(H * 100 + d)
    T = 90
    q, k, v, b, a, a_log, dt_bias = delta_inputs(rng, T, H, G, d, e, dtype)
    want = delta_oracle(q, k, v, b, a, a_log, dt_bias).reshape(T, H * e)
    qd, kd, vd = dev(q.reshape(T, -1), dtype), dev(k.reshape(T, -1), dtype), dev(v.reshape(T, -1), dtype)
    bd, ad = dev(b, dtype), dev(a, dtype)
    state = torch.full((3, H, d, e), float("nan"), dtype=torch.float32, device=DEV)       # poison: a first portion must not read it

    def part(bt, lo, hi):
        return mops.gated_delta_scan(qd[lo:hi], kd[lo:hi], vd[lo:hi], bd[lo:hi], ad[lo:hi], dev(a_log), dev(dt_bias), state, bt.state_slots,
                                     bt.q_start, bt.q_len, bt.ctx_len, H, G, d ** -0.5, 1e-6, max_q_len=hi - lo)
    tol = 2e-4 if dtype == torch.float32 else 2e-4      # inputs are rounded alike on both sides; the recurrence is fp32
    for cuts in ([T], [1] * T, [2] * 45, [40, 1, 1, 33, 2, 13], [3, 50, 1, 36]):      # both work splits write what the other reads
        got = torch.cat(run_cut(part, T, cuts)).cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol)


def test_delta_rule_batch_of_unequal_segments_and_a_slot_taken_over(mops):
    rng = np.random.default_rng(5)
    H, G, d, e, dtype = 4, 2, 32, 48, torch.float32
    lens = [50, 1, 7]
    data = [delta_inputs(rng, n, H, G, d, e, dtype) for n in lens]
    a_log, dt_bias = data[0][5], data[0][6]
    want = [delta_oracle(*x[:5], a_log, dt_bias).reshape(n, H * e) for x, n in zip(data, lens)]
    state = torch.full((2, H, d, e), float("nan"), dtype=torch.float32, device=DEV)
    # sequence 1 (one token) ends after the first step and sequence 2 takes its slot
    plan = [[(0, 20), (1, 1)], [(0, 1), (2, 3)], [(2, 1), (0, 29)], [(2, 3)]]
    slot_of, at, got = {0: 1, 1: 0, 2: 0}, [0, 0, 0], [[], [], []]
    for step in plan:
        b = batch_of([(at[i], [0] * n) for i, n in step], [[0]] * len(step), [slot_of[i] for i, _ in step], 64)
        cat = lambda j: dev(np.concatenate([data[i][j][at[i]:at[i] + n].reshape(n, -1) for i, n in step]))
        out = mops.gated_delta_scan(cat(0), cat(1), cat(2), cat(3), cat(4), dev(a_log), dev(dt_bias), state, b.state_slots, b.q_start,
                                    b.q_len, b.ctx_len, H, G, d ** -0.5, 1e-6, max_q_len=max(n for _, n in step)).cpu().numpy()
        r = 0
        for i, n in step:
            got[i].append(out[r:r + n])
            r += n
            at[i] += n
    for i in range(3):
        np.testing.assert_allclose(np.concatenate(got[i]), want[i], rtol=2e-4, atol=2e-4)


def test_delta_rule_overwrites_what_a_key_held(mops):
    """With beta = 1, no decay and orthogonal unit keys the state holds exactly the last value written under each key: a second
    write under the same key REPLACES the first (plain linear attention would add them)."""
    H = G = 1
    d, e = 16, 8
    keys = np.eye(d)[[0, 1, 0, 2]] * 3.0
    vals = np.arange(4 * e, dtype=np.float64).reshape(4, e) / 10
    q = np.eye(d)[[0, 0, 0, 0]]
    big = np.full((4, 1), 30.0)                                  # sigmoid -> 1
    a = np.full((4, 1), -60.0)                                   # softplus -> 0: g = 1
    state = torch.zeros(1, 1, d, e, device=DEV)
    b = batch_of([(0, [0] * 4)], [[0]], [0], 16)
    out = mops.gated_delta_scan(dev(q), dev(keys), dev(vals), dev(big), dev(a), dev(np.zeros(1)), dev(np.zeros(1)), state, b.state_slots,
                                b.q_start, b.q_len, b.ctx_len, H, G, 1.0, 1e-6, max_q_len=4).cpu().numpy()
    np.testing.assert_allclose(out[1], vals[0], atol=1e-4)       # key 0 still holds the first value
    np.testing.assert_allclose(out[2], vals[2], atol=1e-4)       # ... and then only the third
    np.testing.assert_allclose(out[3], vals[2], atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim", [(4, 40), (1, 200), (5, 8)])
def test_head_norm_with_shared_weight_and_silu_gate(mops, dtype, heads, vdim):
    rng = np.random.default_rng(vdim)
    T = 9
    x = np.float32(rng.standard_normal((T, heads, vdim)) * 0.01).astype(np.float64)      # small: eps matters
    w, g = rounded(rng.standard_normal(vdim), dtype), rounded(rng.standard_normal((T, heads, vdim)), dtype)
    for act, f in ((mops.GATE_SILU, O.silu), (mops.GATE_SIGMOID, O.sigmoid)):
        out = torch.empty(T, heads * vdim + 8, dtype=dtype, device=DEV)[:, :heads * vdim]
        mops.gated_head_rms_norm(out, dev(x.reshape(T, -1)), dev(w, dtype), dev(g.reshape(T, -1), dtype), heads, 1e-5, act)
        want = (O.rms_norm(x, w, 1e-5) * f(g)).reshape(T, -1)
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=tol_of(dtype), atol=tol_of(dtype))


# ---------------------------------------------------------------------------------------------------------------------
# rotation, unit RMS and value blending on the way into the cache
# ---------------------------------------------------------------------------------------------------------------------
ROT_S = {"base": 3000.0, "dims": 12, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
ROT_P = {"base": 100.0, "dims": 40}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e,rot,layout", [(6, 2, 24, 16, ROT_S, "half"), (2, 2, 40, 72, ROT_P, "interleaved"), (3, 1, 130, 8, ROT_P, "half"),
                                                (4, 2, 64, 32, {"base": 100.0, "dims": 32}, "half")])
@pytest.mark.parametrize("norm,blend", [(True, True), (False, False)])
def test_rotation_norm_blend_and_cache_write(mops, dtype, H, G, d, e, rot, layout, norm, blend):
    from aphrodite_engine_amd.mixers import RotaryFrequencies
    rng = np.random.default_rng(d)
    ctx, n, block, eps, lam = 1003, 9, 16, 1e-5, 0.3
    q, k = rounded(rng.standard_normal((n, H, d)), dtype), rounded(rng.standard_normal((n, G, d)), dtype)
    v, vo = rounded(rng.standard_normal((n, G, e)), dtype), rounded(rng.standard_normal((n, G, e)), dtype)
    pos = np.arange(ctx, ctx + n)
    qw, kw = O.rotate(q, pos, rot, layout), O.rotate(k, pos, rot, layout)
    if norm:
        qw, kw = O.rms_norm(qw, None, eps), O.rms_norm(kw, None, eps)
    vw = (1 - np.float32(lam)) * v + np.float32(lam) * vo if blend else v
    pages = (ctx + n + block - 1) // block
    table = list(rng.permutation(pages + 3)[:pages])
    kc = torch.full((pages + 3, block, G, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((pages + 3, block, G, e), float("nan"), dtype=dtype, device=DEV)
    b = batch_of([(ctx, [0] * n)], [table], [0], block)
    sc = rot.get("scaling")
    rf = RotaryFrequencies.wavelength_scaled(rot["dims"], rot["base"], sc["factor"], sc["low"], sc["high"], sc["original"]) if sc else \
        RotaryFrequencies(rot["dims"], rot["base"])
    np.testing.assert_allclose(rf.inv_freq.numpy(), O.rotary_frequencies(rot), rtol=1e-6)
    got = mops.rotary_qk_norm_kv_write(dev(q.reshape(n, -1), dtype), dev(k.reshape(n, -1), dtype), dev(v.reshape(n, -1), dtype), kc, vc,
                                       b.slot_mapping, b.q_start, b.ctx_len, b.seq_of_token, rf.inv_freq.to(DEV), rot["dims"],
                                       mops.ROTARY_HALF if layout == "half" else mops.ROTARY_INTERLEAVED, norm, eps,
                                       dev(vo.reshape(n, -1), dtype) if blend else None, lam)
    tol = 2e-4 if dtype == torch.float32 else 2e-2           # fp32 angles at position 1000
    np.testing.assert_allclose(got.float().cpu().numpy(), qw.reshape(n, -1), rtol=tol, atol=tol)
    slots = b.slot_mapping.cpu().numpy()
    kf, vf = kc.view(-1, G, d).float().cpu().numpy(), vc.view(-1, G, e).float().cpu().numpy()
    np.testing.assert_allclose(kf[slots], kw, rtol=tol, atol=tol)
    np.testing.assert_allclose(vf[slots], vw, rtol=tol_of(dtype), atol=tol_of(dtype))
    rest = np.setdiff1d(np.arange(kf.shape[0]), slots)
    assert np.isnan(kf[rest]).all() and np.isnan(vf[rest]).all()           # no other row was touched


# ---------------------------------------------------------------------------------------------------------------------
# attention through the latent: window and sink
# ---------------------------------------------------------------------------------------------------------------------
def latent_oracle(q_lat, q_rot, rows, rot, scale, R, window, sink):
    """sum_j p_ij c_j per head with the query's rotary part rotated ("half" pairs, as the kernels do) at its position."""
    T, H = q_lat.shape[:2]
    qr = O.rotate(q_rot, np.arange(T), rot, "half")
    out = np.zeros((T, H, R))
    for a in range(H):
        qa = np.concatenate([q_lat[:, a], qr[:, a]], -1)
        out[:, a] = O.masked_attention(qa, rows, rows[:, :R], scale, window, None if sink is None else float(sink[a]))
    return out


def attend(mops, q_lat, q_rot, rows, cuts, dtype, rot, scale, window, sink, block=16, plain=False, seed=0):
    """Runs one sequence cut into portions over shuffled, poisoned pages; returns [T, H, R]."""
    T, H, R = q_lat.shape
    P = q_rot.shape[2]
    rng = np.random.default_rng(seed)
    pages = (T + block - 1) // block
    table = list(rng.permutation(pages + 4)[:pages])
    cache = torch.full((pages + 4, block, R + P), float("nan"), dtype=dtype, device=DEV)
    flat = cache.view(-1, R + P)
    inv = dev(O.rotary_frequencies(rot))
    sk = None if sink is None else dev(sink)
    ql, qr, rw = dev(q_lat, dtype), dev(q_rot, dtype), dev(rows, dtype)

    def part(b, lo, hi):
        flat[b.slot_mapping] = rw[lo:hi]
        out = torch.empty(hi - lo, H, R, dtype=dtype, device=DEV)
        mops.latent_attention(out, ql[lo:hi], qr[lo:hi], cache, b.block_tables, b.q_start, b.q_len, b.ctx_len, b.seq_of_token,
                              (hi - lo, hi - lo), inv, 1.0, rot["dims"], scale, max_kv_len=hi, plain=plain, window=window, sink=sk)
        return out
    return torch.cat(run_cut(part, T, cuts, block=block, tables=table)).float().cpu().numpy()


LA_SHAPES = [(3, 48, 8, {"base": 5000.0, "dims": 8}), (5, 128, 32, {"base": 100.0, "dims": 32}), (16, 128, 16, {"base": 900.0, "dims": 16}),
             (2, 256, 64, {"base": 10000.0, "dims": 64})]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", LA_SHAPES)
@pytest.mark.parametrize("window", [0, 1, 13, 45, 100])
def test_latent_attention_window_and_sink_in_portions_and_decoded(mops, dtype, shape, window):
    H, R, P, rot = shape
    rng = np.random.default_rng(R + window)
    T, scale = 150, (R / 4 + P) ** -0.5
    q_lat, q_rot = rounded(rng.standard_normal((T, H, R)) * 0.5, dtype), rounded(rng.standard_normal((T, H, P)), dtype)
    rows = rounded(rng.standard_normal((T, R + P)), dtype)
    rows[:, R:] = rounded(O.rotate(rows[:, R:], np.arange(T), rot, "half"), dtype)       # the cache holds rotated key parts
    sink = np.float32(rng.standard_normal(H) * 2).astype(np.float64)
    want = latent_oracle(q_lat, q_rot, rows, rot, scale, R, window, sink)
    tol = 3e-4 if dtype == torch.float32 else 3e-2
    for cuts in ([T], [100] + [1] * 50, [2, 62, 1, 33, 2, 50], [37, 64, 49]):
        for plain in ((True, False) if dtype == torch.bfloat16 else (True,)):
            got = attend(mops, q_lat, q_rot, rows, cuts, dtype, rot, scale, window, sink, plain=plain)
            np.testing.assert_allclose(got, want, rtol=tol, atol=tol, err_msg=f"{cuts} plain={plain}")
    # without a sink the weights sum to one; a sink far above every score empties the output
    got = attend(mops, q_lat, q_rot, rows, [T], dtype, rot, scale, window, None)
    np.testing.assert_allclose(got, latent_oracle(q_lat, q_rot, rows, rot, scale, R, window, None), rtol=tol, atol=tol)
    got = attend(mops, q_lat, q_rot, rows, [T], dtype, rot, scale, window, np.full(H, 80.0))
    assert np.abs(got).max() < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("shape", [(3, 48, 8, {"base": 5000.0, "dims": 8}), (4, 128, 32, {"base": 100.0, "dims": 32})])
def test_one_loud_key_just_inside_and_just_outside_the_window(mops, dtype, decoded, shape):
    """Among 700 quiet keys one carries a large component that the query picks up: the row's output is that key's latent when the
    key is the oldest one the window still holds, and nothing of it one row later."""
    H, R, P, rot = shape
    window, T = 37, 700
    rng = np.random.default_rng(11)
    for loud in (0, 15, 16, 333, T - window, T - window - 1, T - 1 - 5):
        rows = rounded(rng.standard_normal((T, R + P)) * 0.05, dtype)
        rows[:, R:] = 0.0
        rows[loud, 0] = 30.0
        q_lat = np.zeros((T, H, R))
        q_lat[:, :, 0] = 8.0
        q_rot = np.zeros((T, H, P))
        cuts = [T - 60] + [1] * 60 if decoded else [T - 60, 33, 27]
        got = attend(mops, q_lat, q_rot, rows, cuts, dtype, rot, 1.0, window, np.zeros(H), seed=loud)
        want = latent_oracle(q_lat, q_rot, rows, rot, 1.0, R, window, np.zeros(H))
        tol = 3e-4 if dtype == torch.float32 else 3e-2
        np.testing.assert_allclose(got[T - 60:], want[T - 60:], rtol=tol, atol=tol, err_msg=str(loud))
        for i in range(max(loud, T - 60), T):
            seen = i - loud < window
            assert (abs(got[i, 0, 0] - 30.0) < 0.5) == seen, (loud, i)


def test_decoded_rows_under_a_window_beside_long_ones(mops):
    """bf16 matrix-core kernel: decoded rows with 1100, 515 and 3 keys in one batch, windows that start in the middle of a tile."""
    H, R, P, rot, dtype = 4, 128, 32, {"base": 100.0, "dims": 32}, torch.bfloat16
    rng = np.random.default_rng(3)
    lens, block, scale = [1100, 515, 3], 16, 0.11
    inv = dev(O.rotary_frequencies(rot))
    for window in (0, 50, 600):
        seqs, tables, nb = [], [], 0
        for n in lens:
            rows = rounded(rng.standard_normal((n, R + P)), dtype)
            seqs.append((rounded(rng.standard_normal((n, H, R)) * 0.3, dtype), rounded(rng.standard_normal((n, H, P)), dtype), rows))
            pages = (n + block - 1) // block
            tables.append(list(range(nb, nb + pages)))
            nb += pages
        cache = torch.full((nb, block, R + P), float("nan"), dtype=dtype, device=DEV)
        flat = cache.view(-1, R + P)
        for (ql, qr, rows), tb in zip(seqs, tables):
            idx = torch.tensor([tb[j // block] * block + j % block for j in range(len(rows))], device=DEV)
            flat[idx] = dev(rows, dtype)
        b = batch_of([(n - 1, [0]) for n in lens], tables, [0, 1, 2], block)
        sink = np.float32(rng.standard_normal(H)).astype(np.float64)
        out = torch.empty(3, H, R, dtype=dtype, device=DEV)
        mops.latent_attention(out, dev(np.stack([s[0][-1] for s in seqs]), dtype), dev(np.stack([s[1][-1] for s in seqs]), dtype), cache,
                              b.block_tables, b.q_start, b.q_len, b.ctx_len, b.seq_of_token, (1, 1), inv, 1.0, rot["dims"], scale,
                              max_kv_len=max(lens), window=window, sink=dev(sink))
        for r, (ql, qr, rows) in enumerate(seqs):
            want = latent_oracle(ql, qr, rows, rot, scale, R, window, sink)[-1]
            np.testing.assert_allclose(out[r].float().cpu().numpy(), want, rtol=3e-2, atol=3e-2, err_msg=f"{window} {r}")


# ---------------------------------------------------------------------------------------------------------------------
# router and experts
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("experts,top", [(6, 2), (9, 4), (130, 7), (5, 5), (3, 1), (70, 66)])
def test_router_softmax_over_the_chosen_logits(mops, experts, top):
    rng = np.random.default_rng(experts)
    z = np.float32(rng.standard_normal((37, experts)) * 3)
    z[3, :] = 1.25                                              # ties go to the lower index
    bias = np.float32(rng.standard_normal(experts))
    ids, w = mops.experts_route_topk(dev(z), dev(bias), top)
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    for t in range(z.shape[0]):
        chosen, weights = O.route(z[t].astype(np.float64) + bias, top)
        assert ids[t].tolist() == chosen, t
        np.testing.assert_allclose(w[t], weights, rtol=1e-5, atol=1e-6)
        assert abs(w[t].sum() - 1.0) < 1e-5
    ids2, _ = mops.experts_route_topk(dev(z), None, top)
    assert ids2.cpu().numpy()[3].tolist() == list(range(top))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(72, 40, 6, 2, 56, 45), (96, 64, 12, 3, 0, 300), (75, 24, 4, 4, 17, 9), (64, 32, 8, 1, 32, 70)])
def test_routed_experts_against_the_restatement_and_alone(mops, dtype, shape):
    from aphrodite_engine_amd.mixers import RoutedExperts
    width, ff, experts, top, shared, T = shape
    rng = np.random.default_rng(width + T)
    mlp = U.moe(ff, experts, top, shared)
    W = {k[len("l0.mlp."):]: rounded(v, dtype) for k, v in U.make_weights(U.make_config([U.delta_layer(mlp=mlp)], width=width), seed=T).items()
         if k.startswith("l0.mlp.")}
    h = rounded(rng.standard_normal((T, width)), dtype)
    want = O.moe_ff(h, W, "", mlp)
    m = RoutedExperts(width, ff, experts, top, 0, 0.0, dtype, shared_ff=shared, alpha=1.0, score="topk_softmax", shared_gate=False).to(DEV)
    m.router.data.copy_(dev(W["router"]))
    m.router_bias.data.copy_(dev(W["router.b"]))
    for j in range(experts):
        m.w_gate_up.data[j, :ff].copy_(dev(W[f"e{j}.gate"], dtype))
        m.w_gate_up.data[j, ff:].copy_(dev(W[f"e{j}.up"], dtype))
        m.w_down.data[j].copy_(dev(W[f"e{j}.down"], dtype))
    if shared:
        m.shared_in.weight.data[:shared].copy_(dev(W["shared.gate"], dtype))
        m.shared_in.weight.data[shared:2 * shared].copy_(dev(W["shared.up"], dtype))
        m.shared_down.weight.data.copy_(dev(W["shared.down"], dtype))
    got = m(dev(h, dtype)).float().cpu().numpy()
    if dtype == torch.float32:
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    else:
        assert np.median(np.abs(got - want)) < 0.02 and np.quantile(np.abs(got - want), 0.99) < 0.15
    alone = m(dev(h[3:4], dtype)).float().cpu().numpy()
    np.testing.assert_allclose(alone[0], got[3], rtol=tol_of(dtype), atol=tol_of(dtype))


# ---------------------------------------------------------------------------------------------------------------------
# the model through the engine
# ---------------------------------------------------------------------------------------------------------------------
D, L, A = U.delta_layer, U.latent_layer, U.attn_layer
CONFIGS = {
    # every mixer kind, layers that differ in everything, one without a feed-forward, the first blending layer not the first
    # attention layer, a window of 13
    "mixed": lambda: U.make_config([A(v_mix=False, heads=4, kv_heads=4, dim=16, vdim=24, rot_dims=16, scaling=None, mlp=None), D(), L(),
                                    A(), D(heads=3, kv_heads=3, dim=16, vdim=24, conv=2, mlp=U.moe(32, 4, 1, 0)),
                                    A(rot_dims=24, base=50.0, scaling=(2.0, 2.0, 8.0, 32)), L(heads=2, dim=16, rot_dim=12, vdim=24, kv_rank=36,
                                                                                             window=44, mlp=None), A()]),
    # sizes the matrix-core kernels serve in bfloat16; one stream, no layer scale surprises, no soft cap
    "wide": lambda: U.make_config([L(heads=5, dim=24, rot_dim=32, vdim=40, kv_rank=128, window=50, mlp=U.moe(64, 4, 2, 64)),
                                   D(heads=4, kv_heads=2, dim=64, vdim=64, conv=4, mlp=U.moe(64, 8, 3, 0)),
                                   A(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, v_mix=False), A(heads=6, kv_heads=3, dim=128, vdim=64, rot_dims=32)],
                                  width=128, vocab=211, streams=1, residual_mult=1.0, softcap=0.0),
    # a window longer than anything it sees, five taps, one head
    "plain": lambda: U.make_config([D(heads=1, kv_heads=1, dim=40, vdim=20, conv=5), L(heads=1, dim=32, rot_dim=16, vdim=32, kv_rank=32, window=4000),
                                    A(heads=1, kv_heads=1, dim=32, vdim=32, rot_dims=32, v_mix=True, mlp=None)], width=96, streams=2),
}


def build(tmp_path, name, dtype, seed=0, **engine_args):
    from aphrodite_engine_amd.engine import LLMEngine
    cfg = CONFIGS[name]() if isinstance(name, str) else name
    W = U.make_weights(cfg, seed=seed)
    path = U.write_checkpoint(str(tmp_path / f"m-{seed}"), cfg, W)
    args = dict(max_tokens=512, max_num_seqs=4)
    args.update(engine_args)
    eng = LLMEngine.from_pretrained(path, dtype=dtype, device=DEV, **args)
    for c in eng.runner.caches:                   # poison: nothing may be read before it is written
        for t in (c if isinstance(c, (tuple, list)) else [c]):
            t.fill_(float("nan") if t.is_floating_point() else -12345)
    return cfg, W, eng


def prompts(cfg, lens, seed=0):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_and_layer_trace(mops, tmp_path, name, dtype):
    cfg, W, eng = build(tmp_path, name, dtype)
    toks = prompts(cfg, [83])[0]
    trace = []
    want = O.forward(cfg, W, toks, trace)
    model = eng.runner.model
    model.residual_trace = []
    got = eng.run_segments([("a", toks, list(range(len(toks))))]).cpu().numpy()
    U.assert_logits(got, want, dtype == torch.float32)
    assert len(model.residual_trace) == len(trace)
    for x, w in zip(model.residual_trace, trace):
        x = x.cpu().numpy()
        assert np.isfinite(x).all()
        if dtype == torch.float32:
            assert np.abs(x - w).max() < 2e-4 * max(1.0, np.abs(w).max() / 10)
    model.residual_trace = None
    eng.release("a")
    again = eng.run_segments([("b", toks, list(range(len(toks))))]).cpu().numpy()      # reused pages and slot
    U.assert_logits(again, want, dtype == torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_portions_and_token_by_token_equal_the_whole_prompt(mops, tmp_path, name, dtype):
    cfg, W, eng = build(tmp_path, name, dtype)
    toks = prompts(cfg, [70], seed=1)[0]
    want = O.forward(cfg, W, toks)
    whole = eng.run_segments([("whole", toks, list(range(70)))]).cpu().numpy()
    eng.release("whole")
    for rid, sizes in (("tok", [1] * 70), ("two", [2] * 35), ("mix", [2, 15, 1, 16, 2, 17, 3, 1, 1, 12]), ("tail", [38] + [1] * 32)):
        got, a = [], 0
        for n in sizes:
            got.append(eng.run_segments([(rid, toks[a:a + n], list(range(n)))]).cpu().numpy())
            a += n
        eng.release(rid)
        assert a == 70
        U.assert_logits(np.concatenate(got), want, dtype == torch.float32, rid)
        # how a prompt is cut changes nothing beyond rounding -- in bfloat16 too
        assert np.quantile(U.logit_errors(np.concatenate(got), whole), 0.9) < (2e-4 if dtype == torch.float32 else 0.04), rid


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_requests_in_one_batch_equal_each_alone(mops, tmp_path, dtype):
    cfg, W, eng = build(tmp_path, "mixed", dtype, max_tokens=320)
    ps = prompts(cfg, [90, 1, 23, 47], seed=2)
    want = [O.forward(cfg, W, p) for p in ps]
    # a schedule with portions beside single tokens; request 1 ends early and request 3 takes its pages and slot
    plan = [[(0, 2), (1, 1)], [(0, 30), (2, 3)], [(0, 1), (2, 1), (3, 2)], [(0, 1), (2, 17), (3, 16)], [(2, 2), (3, 1), (0, 20)],
            [(3, 28), (0, 1)], [(0, 35)]]
    at, got = [0] * 4, [[] for _ in ps]
    for step in plan:
        entries = [(str(i), ps[i][at[i]:at[i] + n], list(range(n))) for i, n in step]
        out = eng.run_segments(entries).cpu().numpy()
        a = 0
        for i, n in step:
            got[i].append(out[a:a + n])
            a += n
            at[i] += n
            if at[i] == len(ps[i]):
                eng.release(str(i))
    for i in range(4):
        assert at[i] == len(ps[i])
        U.assert_logits(np.concatenate(got[i]), want[i], dtype == torch.float32, i)
    assert eng.pages.num_free == eng.pages.total and eng.slots.num_free == 4


def test_pages_and_slots_taken_over_from_a_finished_request(mops, tmp_path):
    cfg, W, eng = build(tmp_path, "plain", torch.float32, max_tokens=64, max_num_seqs=1)
    a, b = prompts(cfg, [60, 50], seed=3)
    eng.run_segments([("a", a, [])])
    with pytest.raises(Exception):
        eng.run_segments([("b", b, [])])             # neither pages nor a slot are left
    eng.requests.pop("b", None)
    eng.release("a")
    # the new request starts with single tokens in the slot the old one left: neither its state nor its convolution may see a's
    got = [eng.run_segments([("b", b[:1], [0])]), eng.run_segments([("b", b[1:3], [0, 1])]), eng.run_segments([("b", b[3:31], list(range(28)))]),
           eng.run_segments([("b", b[31:], list(range(19)))])]
    U.assert_logits(torch.cat(got).cpu().numpy(), O.forward(cfg, W, b), True)


def test_a_far_key_decides_and_a_window_forgets(mops, tmp_path):
    """One sharp attention layer (large score scale, no feed-forward): a marker token 340 positions back still changes every later
    row, in a prompt and decoded; through a latent layer with a window of 64 it changes the next 63 rows and none after."""
    for kind in ("attention", "latent_attention"):
        layer = A(heads=2, kv_heads=1, dim=16, vdim=16, rot_dims=0, scaling=None, v_mix=False, mlp=None, scale=4.0) if kind == "attention" else \
            L(heads=2, dim=16, rot_dim=4, vdim=16, kv_rank=24, window=64, mlp=None, scale=4.0)
        cfg = U.make_config([layer], vocab=50, width=32, streams=1, residual_mult=1.0, softcap=0.0)
        W = U.make_weights(cfg, seed=7)
        toks = prompts(cfg, [400], seed=8)[0]
        toks = [t if t != 7 else 8 for t in toks]
        toks[60] = 7                                               # the marker
        want = O.forward(cfg, W, toks)
        from aphrodite_engine_amd.engine import LLMEngine
        path = U.write_checkpoint(str(tmp_path / kind), cfg, W)
        eng = LLMEngine.from_pretrained(path, dtype=torch.float32, device=DEV, max_tokens=512, max_num_seqs=2)
        whole = eng.run_segments([("w", toks, list(range(400)))]).cpu().numpy()
        U.assert_logits(whole, want, True, kind)
        eng.release("w")
        got = [eng.run_segments([("d", toks[:350], [349])])] + [eng.run_segments([("d", [t], [0])]) for t in toks[350:]]
        U.assert_logits(torch.cat(got).cpu().numpy(), want[349:], True, kind)
        # the marker matters to later rows exactly when the mixer can still see it
        other = list(toks)
        other[60] = 9
        diff = np.abs(O.forward(cfg, W, other) - want).max(-1)
        assert diff[60] > 1e-3
        if kind == "attention":
            assert (diff[61:] > 0).mean() > 0.9 and diff[360:].max() > 1e-3      # (a weight can underflow at this sharpness)
        else:
            assert diff[60 + 64:].max() == 0 and diff[60 + 63] > 0


def test_long_decoding_past_every_window(mops, tmp_path):
    cfg, W, eng = build(tmp_path, "mixed", torch.float32)
    toks = prompts(cfg, [180], seed=4)[0]
    want = O.forward(cfg, W, toks)
    got = [eng.run_segments([("a", toks[:5], [4])])]
    for t in toks[5:]:
        got.append(eng.run_segments([("a", [t], [0])]))
    U.assert_logits(torch.cat(got).cpu().numpy(), want[4:], True)


def test_greedy_generation_through_the_scheduler(mops, tmp_path):
    from aphrodite_engine_amd.engine import SamplingParams
    cfg, W, eng = build(tmp_path, "mixed", torch.float32, max_num_seqs=2, max_num_batched_tokens=24, max_tokens=192)
    ps = prompts(cfg, [40, 3, 1, 29], seed=5)
    outs = eng.generate(ps, SamplingParams(max_tokens=8))
    for p, out in zip(ps, outs):
        seq = list(p)
        for _ in range(8):
            seq.append(int(np.argmax(O.forward(cfg, W, seq)[-1])))
        assert out == seq[len(p):]
    assert eng.pages.num_free == eng.pages.total and eng.slots.num_free == 2 and not eng.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command_on_an_unseen_shape(mops, tmp_path, dtype):
    """bin/trace_run end to end: a checkpoint of sizes no other test uses, a schedule with portions beside single tokens and a
    request that ends, the logits files against the restatement."""
    import json
    import os
    import subprocess
    cfg = U.make_config([L(heads=2, dim=48, rot_dim=16, vdim=80, kv_rank=50, window=21, mlp=U.moe(48, 9, 3, 24)),
                         A(heads=6, kv_heads=3, dim=40, vdim=16, rot_dims=20, scaling=(8.0, 1.0, 2.0, 40), v_mix=True, mlp=None),
                         D(heads=6, kv_heads=2, dim=48, vdim=24, conv=4, mlp=U.moe(100, 5, 5, 0)),
                         A(heads=3, kv_heads=3, dim=8, vdim=16, rot_dims=8, scaling=None, v_mix=True)],
                        vocab=300, width=104, streams=5, residual_mult=0.25, softcap=20.0)
    W = U.make_weights(cfg, seed=21)
    model_dir = U.write_checkpoint(str(tmp_path / "m"), cfg, W)
    ps = prompts(cfg, [75, 20, 2], seed=9)
    want = [O.forward(cfg, W, p) for p in ps]
    plan = [[(0, 40), (1, 2)], [(0, 1), (1, 1), (2, 2)], [(0, 20), (1, 17)], [(0, 14)]]
    at, lines, rows = [0, 0, 0], [], []
    for n, step in enumerate(plan):
        entries, end = [], []
        for i, k in step:
            w = list(range(0, k, 2)) if k > 2 else list(range(k))
            entries.append({"id": "q%d" % i, "tokens": ps[i][at[i]:at[i] + k], "want": w})
            rows.append([(i, at[i] + x) for x in w])
            at[i] += k
            if at[i] == len(ps[i]):
                end.append("q%d" % i)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done %d" % n for n in range(len(plan))]
    got, exp, k = [], [], 0
    for n, step in enumerate(plan):
        g = np.fromfile(str(out / ("%d.f32" % n)), dtype="<f4").reshape(-1, cfg["vocab"])
        need = sum(len(rows[k + j]) for j in range(len(step)))
        assert g.shape[0] == need
        got.append(g)
        for j in range(len(step)):
            exp += [want[i][pos] for i, pos in rows[k + j]]
        k += len(step)
    U.assert_logits(np.concatenate(got), np.stack(exp), dtype == "float32")
