"""Fekotar on the GPU against the plain restatement (oracle/fekotar.py, float64): every kernel alone, then the model through the
engine -- whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages and slots, long
decoding, greedy generation through the scheduler, the trace replay command.  Small random configurations made here; sizes are
unlike one another and unlike any shipped model.  Unused cache memory is poisoned with NaN so that a read outside a sequence's
own keys or of a stale state shows."""
import numpy as np
import pytest
import torch

import fekotar_util as U
from oracle import fekotar as O

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


def i32(a):
    return torch.tensor(list(a), dtype=torch.int32, device=DEV)


def rounded(a, dtype):
    return U.bf16_round(a).astype(np.float64) if dtype == torch.bfloat16 else np.asarray(a, np.float32).astype(np.float64)


def tol_of(dtype):
    return 3e-5 if dtype == torch.float32 else 2e-2


def batch_of(segs, tables, slots, block):
    """segs: [(ctx, tokens)] -> StepBatch"""
    from aphrodite_engine_amd.step_batch import StepBatch
    return StepBatch.build([list(t) for _, t in segs], [c for c, _ in segs], tables, slots, block, DEV)


# ---------------------------------------------------------------------------------------------------------------------
# embedding with hashed token pairs, the two-branch residual norm, the gate
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hashed_pair_embed_in_steps_with_slots_taken_over(mops, dtype):
    rng = np.random.default_rng(0)
    vocab, width, buckets, mp, mc = 90, 40, 17, 1000003, 7919          # products that overflow 32 bits
    table, pair = rounded(rng.standard_normal((vocab, width)), dtype), rounded(rng.standard_normal((buckets + 1, width)), dtype)
    hashing = {"buckets": buckets, "mul_prev": mp, "mul_cur": mc}
    state = torch.full((3,), -12345, dtype=torch.int32, device=DEV)    # poison: a first token must not read it
    seqs = [rng.integers(0, vocab, n).tolist() for n in (11, 1, 6)]
    want = [O.embed(s, table, pair, hashing) for s in seqs]
    # steps: (sequence, how many tokens); sequence 1 ends and sequence 2 takes its slot afterwards
    plan = [[(0, 1), (1, 1)], [(0, 4)], [(0, 1), (2, 2)], [(2, 1), (0, 2)], [(2, 3), (0, 3)]]
    slot_of = {0: 2, 1: 0, 2: 0}
    at, got = [0, 0, 0], [[], [], []]
    for step in plan:
        segs = [(at[i], seqs[i][at[i]:at[i] + n]) for i, n in step]
        b = batch_of(segs, [[0]] * len(step), [slot_of[i] for i, _ in step], 64)
        x = mops.hashed_pair_embed(dev(table, dtype), dev(pair, dtype), b.input_ids, state, b.state_slots, b.q_start, b.q_len, b.ctx_len,
                                   b.seq_of_token, mp, mc).cpu().numpy()
        a = 0
        for i, n in step:
            got[i].append(x[a:a + n])
            a += n
            at[i] += n
    for i in range(3):
        np.testing.assert_allclose(np.concatenate(got[i]), want[i], rtol=1e-6, atol=1e-6)
    assert state.tolist()[2] == seqs[0][-1] and state.tolist()[0] == seqs[2][-1]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 75, 200, 1032])      # 75: rows that cannot be read 16 bytes at a time
def test_residual_add2_rms_norm(mops, dtype, width):
    rng = np.random.default_rng(width)
    T, eps = 5, 1e-5
    x0 = (rng.standard_normal((T, width)) * 3).astype(np.float32)
    ya, yb = rounded(rng.standard_normal((T, width + 8)) * 2 + 0.5, dtype), rounded(rng.standard_normal((T, width)), dtype)
    bias, weight = rounded(rng.standard_normal(width), dtype), rounded(1 + 0.3 * rng.standard_normal(width), dtype)
    for use_a, use_b, use_bias in ((1, 1, 1), (1, 0, 0), (0, 1, 0), (1, 1, 0), (0, 0, 0)):
        x = dev(x0)
        out = mops.residual_add2_rms_norm(x, dev(ya, dtype)[:, :width] if use_a else None, dev(yb, dtype) if use_b else None,
                                          dev(bias, dtype) if use_bias else None, dev(weight, dtype), eps=eps, dtype=dtype)
        r = x0.astype(np.float64) + use_a * ya[:, :width] + use_b * yb + use_bias * bias
        np.testing.assert_allclose(x.cpu().numpy(), r, rtol=2e-6, atol=2e-6)
        np.testing.assert_allclose(out.float().cpu().numpy(), O.rms_norm(r, weight, eps), rtol=tol_of(dtype), atol=tol_of(dtype))
    x = dev(x0)
    assert mops.residual_add2_rms_norm(x, dev(ya, dtype)[:, :width], want_out=False) is None
    np.testing.assert_allclose(x.cpu().numpy(), x0 + ya[:, :width], rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sigmoid_gate_mul_in_place_on_strided_rows(mops, dtype):
    rng = np.random.default_rng(1)
    x, g = rounded(rng.standard_normal((7, 300)), dtype), rounded(rng.standard_normal((7, 333)) * 3, dtype)
    xt = dev(x, dtype)
    mops.sigmoid_gate_mul(xt, dev(g, dtype)[:, 20:320], out=xt)
    np.testing.assert_allclose(xt.float().cpu().numpy(), x * O.sigmoid(g[:, 20:320]), rtol=tol_of(dtype), atol=tol_of(dtype))


# ---------------------------------------------------------------------------------------------------------------------
# the latent's way into the cache
# ---------------------------------------------------------------------------------------------------------------------
ROT_A = {"base": 5000.0, "dims": 8, "scaling": {"factor": 3.0, "original": 64, "fast": 16.0, "slow": 2.0}}
ROT_B = {"base": 100.0, "dims": 16}


def rotary_of(rot):
    from aphrodite_engine_amd.fekotar import rotary_from_config
    return rotary_from_config(rot).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank,kv_rank,rot_dim,rot", [(56, 48, 8, ROT_A), (0, 33, 16, ROT_B), (260, 300, 12, ROT_A)])
def test_latent_prep_norms_rotates_and_writes_the_slots(mops, dtype, q_rank, kv_rank, rot_dim, rot):
    rng = np.random.default_rng(q_rank + kv_rank)
    eps, block = 1e-5, 4
    segs = [(5, [0] * 6), (0, [0] * 3), (1022, [0])]
    tables = [[7, 1, 4], [2], list(range(10, 10 + 256))]
    b = batch_of(segs, tables, [0, 1, 2], block)
    T = b.num_tokens
    proj = rounded(rng.standard_normal((T, 5 + q_rank + kv_rank + rot_dim)) * 2, dtype)
    wq, wkv = rounded(1 + 0.3 * rng.standard_normal(max(q_rank, 1)), dtype), rounded(1 + 0.3 * rng.standard_normal(kv_rank), dtype)
    cache = torch.full((270, block, kv_rank + rot_dim), float("nan"), dtype=dtype, device=DEV)
    r = rotary_of(rot)
    cq = mops.latent_prep(dev(proj, dtype), 5, q_rank, 5 + q_rank, kv_rank, rot_dim, rot["dims"], dev(wq, dtype) if q_rank else None,
                          dev(wkv, dtype), cache, b.slot_mapping, b.q_start, b.ctx_len, b.seq_of_token, r.inv_freq, r.mscale, eps)
    tol = tol_of(dtype)
    if q_rank:
        np.testing.assert_allclose(cq.float().cpu().numpy(), O.rms_norm(proj[:, 5:5 + q_rank], wq[:q_rank], eps), rtol=tol, atol=tol)
    else:
        assert cq is None
    pos = b.positions.cpu().numpy()
    rows = cache.view(-1, kv_rank + rot_dim)[b.slot_mapping].float().cpu().numpy()
    np.testing.assert_allclose(rows[:, :kv_rank], O.rms_norm(proj[:, 5 + q_rank:5 + q_rank + kv_rank], wkv, eps), rtol=tol, atol=tol)
    np.testing.assert_allclose(rows[:, kv_rank:], O.rotate(proj[:, 5 + q_rank + kv_rank:], pos, rot), rtol=tol, atol=2 * tol)
    assert int(torch.isnan(cache.view(-1, kv_rank + rot_dim)[:, 0]).sum()) == 270 * block - T        # nothing else was written


# ---------------------------------------------------------------------------------------------------------------------
# attention in the latent
# ---------------------------------------------------------------------------------------------------------------------
def latent_oracle(q_lat, q_rot, rows, rot, scale, R, only=None):
    """q_lat [T, H, R], q_rot [T, H, P] raw, rows [T, R + P] (latent | rotated key part): sum_j p_ij c_j per head, for every
    row i (or the rows ``only``; the others stay zero)."""
    T, H, _ = q_lat.shape
    q = np.concatenate([q_lat, O.rotate(q_rot, np.arange(T), rot)], -1)
    out = np.zeros((T, H, R))
    for a in range(H):
        for i in (range(T) if only is None else only):
            s = rows[:i + 1] @ q[i, a] * scale
            w = np.exp(s - s.max())
            out[i, a] = (w / w.sum()) @ rows[:i + 1, :R]
    return out


def attend(mops, q_lat, q_rot, rows, cuts, dtype, rot, scale, block=16, plain=False, seed=0):
    """One sequence cut into segments of the given sizes, the pages shuffled and poisoned; returns out [T, H, R]."""
    T, H, R = q_lat.shape
    P = q_rot.shape[2]
    pages = (T + block - 1) // block
    perm = np.random.default_rng(seed).permutation(pages + 3)[:pages].tolist()
    cache = torch.full((pages + 3, block, R + P), float("nan"), dtype=dtype, device=DEV)
    r = rotary_of(rot)
    out, a = [], 0
    ql, qr, rw = dev(q_lat, dtype), dev(np.concatenate([np.zeros((T, H, 8)), q_rot], -1), dtype)[:, :, 8:], dev(rows, dtype)
    for n in cuts:
        b = batch_of([(a, [0] * n)], [perm], [0], block)
        cache.view(-1, R + P)[b.slot_mapping] = rw[a:a + n]
        o = torch.zeros(n, H, R, dtype=dtype, device=DEV)
        mops.latent_attention(o, ql[a:a + n], qr[a:a + n], cache, b.block_tables, b.q_start, b.q_len, b.ctx_len, b.seq_of_token, (n, n),
                              r.inv_freq, r.mscale, rot["dims"], scale, max_kv_len=a + n, plain=plain)
        out.append(o.float().cpu().numpy())
        a += n
    assert a == T
    return np.concatenate(out)


# (heads, kv_rank, rot_dim, rot): the last three are sizes of the matrix-core kernel; 650 is past its widest latent
ATT_SHAPES = [(3, 48, 8, ROT_A), (1, 200, 16, ROT_B), (5, 33, 8, ROT_A), (2, 650, 16, ROT_B), (5, 128, 16, ROT_B),
              (16, 256, 32, dict(ROT_B, dims=32)), (2, 512, 64, dict(ROT_A, dims=64))]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", ATT_SHAPES)
def test_attention_prompt_portions_and_decode(mops, dtype, shape):
    H, R, P, rot = shape
    rng = np.random.default_rng(R + H)
    T, scale = 90, 0.3
    q_lat, q_rot = rounded(rng.standard_normal((T, H, R)) * 0.4, dtype), rounded(rng.standard_normal((T, H, P)), dtype)
    rows = rounded(rng.standard_normal((T, R + P)), dtype)
    want = latent_oracle(q_lat, q_rot, rows, rot, scale, R)
    tol = 3e-5 if dtype == torch.float32 else 2.5e-2
    for cuts in ([T], [1] * T, [2] * 45, [37, 1, 1, 17, 2, 30, 2], [70] + [1] * 20):
        for plain in (False, True):
            got = attend(mops, q_lat, q_rot, rows, cuts, dtype, rot, scale, plain=plain)
            np.testing.assert_allclose(got, want, rtol=tol, atol=tol, err_msg=f"{cuts[:3]} plain={plain}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("shape", [(3, 48, 8, ROT_A), (4, 128, 32, dict(ROT_B, dims=32))])
def test_one_loud_key_far_back_at_page_borders_and_at_the_start(mops, dtype, decoded, shape):
    """Among hundreds of quiet keys ONE is made loud for the last row's query (its latent is the query's direction, scaled): the
    result must be that key's latent -- wherever it sits: position 0, the last slot of a page, the first of the next, far back,
    the row's own position -- and the key after the row's position must never show."""
    H, R, P, rot = shape
    rng = np.random.default_rng(7)
    T, block = 700, 16
    for loud in (0, 15, 16, 17, 255, 256, 640, T - 2, T - 1):
        q_lat = rounded(rng.standard_normal((T, H, R)) * 0.05, dtype)
        q_rot = np.zeros((T, H, P))
        rows = rounded(rng.standard_normal((T, R + P)) * 0.1, dtype)
        direction = rounded(rng.standard_normal(R), dtype)
        q_lat[T - 2] = direction * 0.5                                   # the row under test is T - 2; row T - 1 comes after it
        rows[loud, :R] = direction * 2.0
        cuts = [T - 2, 1, 1] if decoded else [T - 41, 41]
        got = attend(mops, q_lat, q_rot, rows, cuts, dtype, rot, 1.0, block=block, seed=loud)
        want = latent_oracle(q_lat[:T - 1], q_rot[:T - 1], rows[:T - 1], rot, 1.0, R, only=[T - 2])[T - 2]
        tol = 3e-5 if dtype == torch.float32 else 3e-2
        np.testing.assert_allclose(got[T - 2], want, rtol=tol, atol=tol, err_msg=str(loud))
        if loud <= T - 2:
            assert np.abs(got[T - 2, 0] - rows[loud, :R]).max() < 0.05 * np.abs(direction).max() + tol, loud
        else:
            assert np.abs(got[T - 2, 0]).max() < 0.5, loud                # the key after the row stays unseen


def test_rotation_depends_on_the_position_not_on_the_cut(mops):
    """Scores through the rotary part alone (the latent part of every query is zero): a portion that starts at position 37 must
    rotate its queries by 37 .. and not by 0 .. ."""
    H, R, P, rot = 2, 40, 12, dict(ROT_A, dims=12)
    rng = np.random.default_rng(3)
    T = 60
    q_lat, q_rot, rows = np.zeros((T, H, R)), rng.standard_normal((T, H, P)) * 2, rng.standard_normal((T, R + P))
    rows[:, R:] = O.rotate(rows[:, R:], np.arange(T), rot)                # what latent_prep would have stored
    want = latent_oracle(q_lat, q_rot, rows, rot, 0.8, R)
    for plain in (False, True):
        got = attend(mops, q_lat, q_rot, rows, [37, 2, 1, 20], torch.float32, rot, 0.8, plain=plain)
        np.testing.assert_allclose(got, want, rtol=3e-5, atol=3e-5)


def test_decoded_rows_split_long_key_ranges_in_unequal_batches(mops):
    """Matrix-core sizes, bfloat16: three decoded tokens with 1100, 515 and 3 keys beside each other (key ranges split over
    workgroups and merged), then a prompt portion beside a decoded token."""
    H, R, P, rot = 16, 128, 16, ROT_B
    dtype, block, scale = torch.bfloat16, 16, 0.2
    rng = np.random.default_rng(11)
    lens = [1100, 515, 3]
    r = rotary_of(rot)
    data = []
    for n in lens:
        data.append((rounded(rng.standard_normal((n, H, R)) * 0.3, dtype), rounded(rng.standard_normal((n, H, P)), dtype),
                     rounded(rng.standard_normal((n, R + P)), dtype)))
    pages = [list(range(a, a + (n + block - 1) // block)) for a, n in zip((0, 80, 120), lens)]
    cache = torch.full((130, block, R + P), float("nan"), dtype=dtype, device=DEV)
    for pg, (ql, qr, rw), n in zip(pages, data, lens):
        b = batch_of([(0, [0] * n)], [pg], [0], block)
        cache.view(-1, R + P)[b.slot_mapping] = dev(rw, dtype)
    for segs in ([(n - 1, [0]) for n in lens], [(lens[0] - 70, [0] * 70), (lens[1] - 1, [0])]):
        use = list(range(len(segs)))
        b = batch_of(segs, [pages[i] for i in use], use, block)
        ql = torch.cat([dev(data[i][0][c:c + len(t)], dtype) for i, (c, t) in zip(use, segs)])
        qr = torch.cat([dev(data[i][1][c:c + len(t)], dtype) for i, (c, t) in zip(use, segs)])
        o = torch.zeros(b.num_tokens, H, R, dtype=dtype, device=DEV)
        mops.latent_attention(o, ql, qr, cache, b.block_tables, b.q_start, b.q_len, b.ctx_len, b.seq_of_token,
                              (min(b.q_lens), max(b.q_lens)), r.inv_freq, r.mscale, P, scale, max_kv_len=max(lens))
        o = o.float().cpu().numpy()
        a = 0
        for i, (c, t) in zip(use, segs):
            n = len(t)
            # the oracle on the last rows only: softmax over the keys 0 .. position of each row
            q = np.concatenate([data[i][0], O.rotate(data[i][1], np.arange(lens[i]), rot)], -1)[c:c + n]
            for k in range(n):
                s = np.einsum("hd,jd->hj", q[k], data[i][2][:c + k + 1]) * scale
                w = np.exp(s - s.max(-1, keepdims=True))
                ref = (w / w.sum(-1, keepdims=True)) @ data[i][2][:c + k + 1, :R]
                np.testing.assert_allclose(o[a + k], ref, rtol=2.5e-2, atol=2.5e-2)
            a += n


# ---------------------------------------------------------------------------------------------------------------------
# router limited to groups, experts of the plain gated form
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("experts,groups,keep,top", [(6, 3, 2, 2), (18, 2, 1, 4), (8, 8, 3, 3), (12, 1, 1, 5), (130, 10, 4, 7), (64, 4, 4, 8)])
def test_router_keeps_the_best_groups_and_weights_by_the_score(mops, experts, groups, keep, top):
    rng = np.random.default_rng(experts)
    z = (rng.standard_normal((50, experts)) * 2).astype(np.float32)
    ids, w = mops.experts_route_grouped(dev(z), top, groups, keep, 1.75)
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    for t in range(50):
        chosen, weights = O.route(z[t].astype(np.float64), top, groups, keep, 1.75)
        assert ids[t].tolist() == chosen, t
        np.testing.assert_allclose(w[t], weights, rtol=1e-5)


def test_router_group_score_is_the_sum_of_the_two_largest(mops):
    """Group 0 holds the single largest score, group 1 the two next: with one group kept the choice must come from group 1."""
    z = np.full((1, 8), -4.0, np.float32)
    z[0, 2], z[0, 5], z[0, 6] = 3.0, 2.0, 1.9
    ids, _ = mops.experts_route_grouped(dev(z), 2, 2, 1, 1.0)
    assert sorted(ids[0].tolist()) == [5, 6]
    ids, _ = mops.experts_route_grouped(dev(z), 2, 2, 2, 1.0)
    assert sorted(ids[0].tolist()) == [2, 5]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(72, 88, 6, 3, 2, 2, 45), (96, 64, 12, 2, 1, 3, 300), (75, 40, 4, 4, 4, 1, 9)])
def test_experts_of_the_plain_gated_form_against_the_restatement_and_alone(mops, dtype, shape):
    from aphrodite_engine_amd.mixers import RoutedExperts
    width, ff, E, groups, keep, top, T = shape
    rng = np.random.default_rng(ff)
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top, "scale": 1.25, "groups": {"count": groups, "keep": keep}}}
    W = {"router": U.bf16_round(rng.standard_normal((E, width)) * 3 / np.sqrt(width)).astype(np.float64)}
    m = RoutedExperts(width, ff, E, top, 0, 0.0, dtype, alpha=1.0, score="sigmoid_grouped", groups=groups, keep=keep, route_scale=1.25).to(DEV)
    m.router.data.copy_(dev(W["router"]))
    for j in range(E):
        for n, shp in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff))):
            W[f"e{j}.{n}"] = U.bf16_round(rng.standard_normal(shp) * (2.0 if n != "down" else 1.0) / np.sqrt(shp[1])).astype(np.float64)
        m.w_gate_up.data[j, :ff], m.w_gate_up.data[j, ff:] = dev(W[f"e{j}.gate"], dtype), dev(W[f"e{j}.up"], dtype)
        m.w_down.data[j] = dev(W[f"e{j}.down"], dtype)
    h = rounded(rng.standard_normal((T, width)), dtype)
    want = O.moe_ff(h, W, "", mlp)
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
A = U.latent_layer
CONFIGS = {
    # layers that differ in everything; one without a feed-forward; dense and routed feed-forwards
    "mixed": lambda: U.make_config([A(), A(heads=2, dim=16, rot_dim=12, vdim=24, q_rank=40, kv_rank=36, scaling=None, base=300.0, mlp="moe"),
                                    A(heads=5, dim=8, rot_dim=4, vdim=8, q_rank=24, kv_rank=64, mlp=None, scaling=(8.0, 16, 4.0, 1.0)),
                                    A(mlp="moe", ff=40, experts=8, groups=2, keep=1, top=3, route_scale=0.6)]),
    # sizes of the matrix-core kernel (in bfloat16); no hashed pairs, one layer routed with every group kept, top 1
    "wide": lambda: U.make_config([A(heads=5, dim=24, rot_dim=32, vdim=40, q_rank=72, kv_rank=128, mlp="moe", ff=64, experts=4, groups=2,
                                     keep=2, top=1, route_scale=1.0),
                                   A(heads=16, dim=16, rot_dim=16, vdim=8, q_rank=64, kv_rank=128, scaling=None, mlp="dense", ff=96)],
                                  width=128, vocab=211, logit_scale=1.0, bigram=None),
    "pair": lambda: U.make_config([A(heads=1, dim=64, rot_dim=64, vdim=32, q_rank=32, kv_rank=32, mlp="dense", ff=96, limit=0.7),
                                   A(heads=4, dim=20, rot_dim=8, vdim=20, q_rank=48, kv_rank=48, mlp=None)], width=96, bigram=(1, 3, 2)),
}


def build(tmp_path, name, dtype, seed=0, **engine_args):
    from aphrodite_engine_amd.engine import LLMEngine
    cfg = CONFIGS[name]()
    W = U.make_weights(cfg, seed=seed)
    path = U.write_checkpoint(str(tmp_path / f"{name}-{seed}"), cfg, W)
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
        assert np.quantile(U.logit_errors(np.concatenate(got), whole), 0.9) < (2e-4 if dtype == torch.float32 else 0.03), rid


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
    cfg, W, eng = build(tmp_path, "pair", torch.float32, max_tokens=64, max_num_seqs=1)
    a, b = prompts(cfg, [60, 50], seed=3)
    eng.run_segments([("a", a, [])])
    with pytest.raises(Exception):
        eng.run_segments([("b", b, [])])             # neither pages nor a slot are left
    eng.requests.pop("b", None)
    eng.release("a")
    # the new request starts with single tokens in the slot the old one left: its first token must not pair with a's last one
    got = [eng.run_segments([("b", b[:1], [0])]), eng.run_segments([("b", b[1:3], [0, 1])]), eng.run_segments([("b", b[3:31], list(range(28)))]),
           eng.run_segments([("b", b[31:], list(range(19)))])]
    U.assert_logits(torch.cat(got).cpu().numpy(), O.forward(cfg, W, b), True)


def test_long_decoding(mops, tmp_path):
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
    cfg = U.make_config([A(heads=2, dim=48, rot_dim=16, vdim=80, q_rank=30, kv_rank=50, mlp="moe", ff=48, experts=9, groups=3, keep=1, top=3),
                         A(heads=7, dim=8, rot_dim=32, vdim=16, q_rank=64, kv_rank=256, mlp="dense", ff=100, scaling=(1.5, 32, 8.0, 0.5)),
                         A(heads=2, dim=48, rot_dim=2, vdim=80, q_rank=30, kv_rank=50, mlp=None)],
                        vocab=300, width=104, logit_scale=1.3, bigram=(97, 1, 0))
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
