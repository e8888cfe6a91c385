"""Torch-tensor front of libaphrodite_mi355x_mixers.so (include/aphrodite_mi355x_mixers.h), in the manner of
``_custom_ops``: every wrapper checks on the host what the kernel and its grid assume (shapes, strides, dtypes, devices)
before it launches, issues on the current stream, allocates only its result, and raises on CPU tensors -- there is no
fallback."""
from typing import Optional

import torch

from . import _lib
from ._lib import check_mixers as check

_DT = {torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}
ACT_SILU, ACT_GELU_TANH = 0, 1
MEMORY_DECAY, MEMORY_MLSTM = 0, 1


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise RuntimeError(f"mixer ops serve bfloat16 and float32 activations, not {t.dtype}")
    return _DT[t.dtype]


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _cuda(*ts) -> None:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("mixer ops run on the GPU only (no CPU fallback)")
        dev = dev or t.device
        _need(t.device == dev, "mixer ops: tensors on different devices")


def _rows(t: torch.Tensor, cols: int, what: str) -> int:
    """Row stride (elements) of a [T, cols] view whose rows are dense."""
    _need(t.dim() == 2 and t.shape[1] == cols and (t.stride(1) == 1 or cols == 1), f"{what}: expected dense rows of {cols}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), cols)


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() == n, f"{what}: int32 [{n}] expected")


def embed_scale(table: torch.Tensor, ids: torch.Tensor, scale: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 residual rows ``table[ids] * scale`` (into ``out`` fp32 [T, width] if given)."""
    _cuda(table, ids, out)
    _need(table.dim() == 2 and table.is_contiguous() and ids.dtype == torch.int64 and ids.dim() == 1 and ids.is_contiguous(),
          "embed_scale: table [vocab, width] contiguous, ids int64 [T]")
    if out is None:
        out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (ids.shape[0], table.shape[1]),
          "embed_scale: out fp32 [T, width], contiguous")
    check(_lib.mixers_lib().aphro_embed_scale_f32(out.data_ptr(), table.data_ptr(), ids.data_ptr(), ids.shape[0],
                                                  table.shape[1], table.shape[0], float(scale), _dt(table), _stream()),
          "embed_scale")
    return out


def residual_layer_norm(residual: torch.Tensor, y: Optional[torch.Tensor] = None, post=None,
                        y_bias: Optional[torch.Tensor] = None, add_vec: Optional[torch.Tensor] = None, pre=None,
                        eps: float = 1e-5, dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """``residual += layer_norm(y + y_bias; *post)``, ``residual += add_vec``, return ``layer_norm(residual; *pre)``; each
    step only if its operands are given.  ``post`` / ``pre`` are (weight, bias) pairs of the activation dtype."""
    T, W = residual.shape
    _need(residual.dtype == torch.float32 and residual.is_contiguous(), "residual_layer_norm: the residual is fp32, contiguous")
    some = y if y is not None else (pre[0] if pre is not None else add_vec)
    _need(some is not None, "residual_layer_norm: nothing to do")
    adt = dtype or some.dtype
    vecs = [add_vec] + list(post or ()) + list(pre or ())
    _cuda(residual, y, y_bias, *vecs)
    for v in vecs:
        _need(v is None or (v.dtype == adt and v.numel() == W and v.is_contiguous()), "residual_layer_norm: vectors are [width] of the activation dtype")
    _need(y_bias is None or (y_bias.dtype == torch.float32 and y_bias.numel() == W and y_bias.is_contiguous()),
          "residual_layer_norm: y_bias is fp32 [width]")
    ys = 0
    if y is not None:
        _need(post is not None and y.dtype == adt and y.shape[0] == T, "residual_layer_norm: y needs its norm and the batch's rows")
        ys = _rows(y, W, "residual_layer_norm y")
    out = torch.empty(T, W, dtype=adt, device=residual.device) if pre is not None else None
    if _dt_of(adt) is None:
        raise RuntimeError(f"residual_layer_norm: dtype {adt}")
    check(_lib.mixers_lib().aphro_residual_layer_norm(
        residual.data_ptr(), _p(y), ys, _p(y_bias), _p(post[0]) if post else None, _p(post[1]) if post else None,
        _p(add_vec), _p(pre[0]) if pre else None, _p(pre[1]) if pre else None, _p(out), T, W, float(eps), _DT[adt], _stream()),
        "residual_layer_norm")
    return out


def _dt_of(dtype):
    return _DT.get(dtype)


def act_and_mul(x: torch.Tensor, act: int) -> torch.Tensor:
    """[T, 2 d] -> [T, d]: act(x[:, :d]) * x[:, d:]."""
    _cuda(x)
    _need(x.dim() == 2 and x.shape[1] % 2 == 0, "act_and_mul: [T, 2 d]")
    d = x.shape[1] // 2
    out = torch.empty(x.shape[0], d, dtype=x.dtype, device=x.device)
    check(_lib.mixers_lib().aphro_act_and_mul(out.data_ptr(), x.data_ptr(), _rows(x, 2 * d, "act_and_mul"), x.shape[0], d,
                                              int(act), _dt(x), _stream()), "act_and_mul")
    return out


def gated_group_rms_norm(out: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor], gate: Optional[torch.Tensor],
                         group: int, eps: float, out_scale: float = 1.0) -> None:
    """out[:, :N] (a view with dense rows, any row stride) = out_scale * x / rms(x per group) * weight * sigmoid(gate)."""
    _cuda(out, x, weight, gate)
    T, N = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous(), "gated_group_rms_norm: x is fp32 contiguous")
    _need(out.shape == (T, N) and N % group == 0, "gated_group_rms_norm: out [T, N], N a multiple of the group")
    _need(weight is None or (weight.dtype == out.dtype and weight.numel() == N and weight.is_contiguous()), "gated_group_rms_norm: weight [N]")
    gs = 0
    if gate is not None:
        _need(gate.dtype == out.dtype and gate.shape == (T, N), "gated_group_rms_norm: gate [T, N] of the output dtype")
        gs = _rows(gate, N, "gated_group_rms_norm gate")
    check(_lib.mixers_lib().aphro_gated_group_rms_norm(out.data_ptr(), _rows(out, N, "gated_group_rms_norm out"), x.data_ptr(),
                                                       _p(weight), _p(gate), gs, T, N, int(group), float(eps),
                                                       float(out_scale), _dt(out), _stream()), "gated_group_rms_norm")


def paged_kv_write(k_cache: torch.Tensor, v_cache: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                   slot_mapping: torch.Tensor) -> None:
    """k_cache [blocks, block, G, d], v_cache [blocks, block, G, e]; k [T, G d], v [T, G e] (dense rows); slots int64 [T]."""
    _cuda(k_cache, v_cache, k, v, slot_mapping)
    nb, bs, G, d = k_cache.shape
    e = v_cache.shape[3]
    _need(v_cache.shape[:3] == (nb, bs, G) and k_cache.is_contiguous() and v_cache.is_contiguous(), "paged_kv_write: cache shapes")
    _need(k.dtype == k_cache.dtype == v.dtype == v_cache.dtype, "paged_kv_write: one dtype")
    T = k.shape[0]
    _need(v.shape[0] == T and slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous(),
          "paged_kv_write: slots int64 [T]")
    check(_lib.mixers_lib().aphro_paged_kv_write(k_cache.data_ptr(), v_cache.data_ptr(), k.data_ptr(), _rows(k, G * d, "k"),
                                                 v.data_ptr(), _rows(v, G * e, "v"), slot_mapping.data_ptr(), T, G, d, e,
                                                 nb * bs, _dt(k), _stream()), "paged_kv_write")


def distance_bias_attention(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor], k_cache: torch.Tensor,
                            v_cache: torch.Tensor, block_tables: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                            ctx_len: torch.Tensor, seq_of_token: torch.Tensor, q_len_range, heads: int, scale: float,
                            bias_lut: Optional[torch.Tensor], temp_coef: float = 0.0, temp_every: int = 1,
                            out_scale: float = 1.0, max_kv_len: int = 0) -> None:
    """Causal attention of a batch of segments over the paged cache, written into ``out`` [T, heads * e] (dense rows, any
    row stride).  q [T, heads * d]; gate [T, heads] raw (sigmoid inside) or None; bias_lut fp32 [heads, L] indexed by
    min(distance, L - 1) or None.  ``q_len_range``: (shortest, longest) segment of the batch, known on the host -- it
    chooses between the matrix-core kernel for prompt portions and the shared-key kernel for single tokens.
    ``max_kv_len``: the longest ctx_len + q_len of the batch (host); given, long key ranges of decoded rows are split over
    several workgroups through a scratch tensor."""
    _cuda(out, q, gate, k_cache, v_cache, block_tables, q_start, q_len, ctx_len, seq_of_token, bias_lut)
    lo, hi = int(q_len_range[0]), int(q_len_range[1])
    _need(0 < lo <= hi, "distance_bias_attention: q_len_range (shortest, longest)")
    nb, bs, G, d = k_cache.shape
    e = v_cache.shape[3]
    T = q.shape[0]
    S = q_start.numel()
    _need(v_cache.shape[:3] == (nb, bs, G) and k_cache.is_contiguous() and v_cache.is_contiguous(), "distance_bias_attention: cache shapes")
    _need(q.dtype == out.dtype == k_cache.dtype == v_cache.dtype, "distance_bias_attention: one dtype")
    _need(heads % G == 0 and out.shape == (T, heads * e), "distance_bias_attention: out [T, heads * vdim]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] == S and block_tables.is_contiguous(),
          "distance_bias_attention: block_tables int32 [S, max_blocks]")
    _i32(q_start, S, "q_start")
    _i32(q_len, S, "q_len")
    _i32(ctx_len, S, "ctx_len")
    _i32(seq_of_token, T, "seq_of_token")
    gs = 0
    if gate is not None:
        _need(gate.dtype == q.dtype and gate.shape[0] == T, "distance_bias_attention: gate [T, heads]")
        gs = _rows(gate, heads, "gate")
    L = 0
    if bias_lut is not None:
        _need(bias_lut.dtype == torch.float32 and bias_lut.dim() == 2 and bias_lut.shape[0] == heads and bias_lut.is_contiguous(),
              "distance_bias_attention: bias_lut fp32 [heads, L]")
        L = bias_lut.shape[1]
    ws, ws_n = None, 0
    if q.dtype == torch.bfloat16 and max_kv_len >= 512 and lo < 8:
        ws_n = T * heads * 8 * (2 + e)
        ws = torch.empty(ws_n, dtype=torch.float32, device=q.device)
    check(_lib.mixers_lib().aphro_distance_bias_attention(
        out.data_ptr(), _rows(out, heads * e, "out"), q.data_ptr(), _rows(q, heads * d, "q"), _p(gate), gs, k_cache.data_ptr(),
        v_cache.data_ptr(), block_tables.data_ptr(), block_tables.shape[1], nb, bs, q_start.data_ptr(), q_len.data_ptr(),
        ctx_len.data_ptr(), seq_of_token.data_ptr(), T, S, lo, hi, heads, G, d, e, float(scale), _p(bias_lut), L, float(temp_coef), int(temp_every),
        float(out_scale), int(max_kv_len), _p(ws), ws_n, _dt(q), _stream()), "distance_bias_attention")


def memory_state_shapes(slots: int, heads: int, dim: int, vdim: int, mode: int):
    """Shapes of the fp32 state tensors of ``outer_memory_scan`` for a pool of ``slots`` requests."""
    tiles = (vdim + 15) // 16
    s = (slots, heads, dim, vdim)
    return (s, ) if mode == MEMORY_DECAY else (s, (slots, heads, tiles, dim), (slots, heads, tiles))


def outer_memory_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state, slot_of_seq: torch.Tensor,
                      q_start: torch.Tensor, q_len: torch.Tensor, ctx_len: torch.Tensor, heads: int, mode: int,
                      decay: Optional[torch.Tensor] = None, gate_i: Optional[torch.Tensor] = None,
                      gate_f: Optional[torch.Tensor] = None, q_scale: float = 1.0, gate_cap: float = 1.0,
                      max_q_len: int = 1) -> torch.Tensor:
    """Scan every segment through its slot's state (updated in place); returns o fp32 [T, heads * vdim].  ``state`` is
    the tuple of tensors shaped by ``memory_state_shapes``.  q, k [T, heads * d], v [T, heads * e]; gates [T, heads] raw.
    ``max_q_len`` (host: the batch's longest segment) picks the work split: wide for prompt portions, narrow for tokens."""
    _cuda(q, k, v, slot_of_seq, q_start, q_len, ctx_len, decay, gate_i, gate_f, *state)
    T = q.shape[0]
    S = q_start.numel()
    slots, H, d, e = state[0].shape
    _need(H == heads and k.shape[0] == T and v.shape[0] == T and q.dtype == k.dtype == v.dtype, "outer_memory_scan: q, k, v rows / dtype")
    for st, shp in zip(state, memory_state_shapes(slots, heads, d, e, mode)):
        _need(st.dtype == torch.float32 and st.is_contiguous() and tuple(st.shape) == shp, "outer_memory_scan: state tensors")
    _need(len(state) == (1 if mode == MEMORY_DECAY else 3), "outer_memory_scan: state tuple")
    for t, nm in ((slot_of_seq, "slot_of_seq"), (q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    gs = 0
    if mode == MEMORY_DECAY:
        _need(decay is not None and decay.dtype == torch.float32 and decay.numel() == heads and decay.is_contiguous(),
              "outer_memory_scan: decay fp32 [heads]")
    else:
        _need(gate_i is not None and gate_f is not None and gate_i.dtype == q.dtype == gate_f.dtype
              and gate_i.shape[0] == T and gate_f.shape[0] == T, "outer_memory_scan: gates [T, heads]")
        gs = _rows(gate_i, heads, "gate_i")
        _need(_rows(gate_f, heads, "gate_f") == gs, "outer_memory_scan: the two gates share a row stride")
    out = torch.empty(T, heads * e, dtype=torch.float32, device=q.device)
    check(_lib.mixers_lib().aphro_outer_memory_scan(
        out.data_ptr(), q.data_ptr(), _rows(q, heads * d, "q"), k.data_ptr(), _rows(k, heads * d, "k"), v.data_ptr(),
        _rows(v, heads * e, "v"), _p(gate_i), _p(gate_f), gs, state[0].data_ptr(),
        state[1].data_ptr() if len(state) > 1 else None, state[2].data_ptr() if len(state) > 2 else None,
        slot_of_seq.data_ptr(), slots, q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(), S, T, heads, d, e, int(mode),
        _p(decay), float(q_scale), float(gate_cap), int(max_q_len), _dt(q), _stream()), "outer_memory_scan")
    return out


# ---- residual stream joined over depth, scalar-gain RMS norm, polynomial norm activation -------------------------------------
def depth_residual_rms_norm(x_in: torch.Tensor, x_out: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None,
                            history: Optional[torch.Tensor] = None, n_hist: int = 0, depth_w: Optional[torch.Tensor] = None,
                            gain: float = 1.0, weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
                            dtype: Optional[torch.dtype] = None, want_out: bool = True) -> Optional[torch.Tensor]:
    """r = x_in + y; with ``depth_w`` (fp32 [n_hist + 1]): history[n_hist] = r, r = sum_j depth_w[j] history[j];
    x_out = r; returns rms_norm(r) * gain * weight in ``dtype`` (``want_out`` False: nothing).  x_in / x_out fp32 [T, W]
    (may be the same tensor), history fp32 [entries, T, W]."""
    T, W = x_in.shape
    _cuda(x_in, x_out, y, history, depth_w, weight)
    _need(x_in.dtype == torch.float32 and x_in.is_contiguous(), "depth_residual_rms_norm: x_in is fp32, contiguous")
    _need(x_out is None or (x_out.dtype == torch.float32 and x_out.is_contiguous() and x_out.shape == x_in.shape),
          "depth_residual_rms_norm: x_out is fp32 [T, W], contiguous")
    adt = dtype or (y.dtype if y is not None else (weight.dtype if weight is not None else None))
    _need(adt in _DT, "depth_residual_rms_norm: the activation dtype is not given")
    ys = 0
    if y is not None:
        _need(y.dtype == adt and y.shape[0] == T, "depth_residual_rms_norm: y [T, W] of the activation dtype")
        ys = _rows(y, W, "depth_residual_rms_norm y")
    hs = 0
    if depth_w is not None:
        _need(history is not None and history.dtype == torch.float32 and history.dim() == 3 and history.is_contiguous()
              and tuple(history.shape[1:]) == (T, W) and 0 <= n_hist < history.shape[0],
              "depth_residual_rms_norm: history fp32 [entries > n_hist, T, W]")
        _need(depth_w.dtype == torch.float32 and depth_w.is_contiguous() and depth_w.numel() == n_hist + 1,
              "depth_residual_rms_norm: depth_w fp32 [n_hist + 1]")
        hs = history.stride(0)
    _need(weight is None or (weight.dtype == adt and weight.numel() == W and weight.is_contiguous()),
          "depth_residual_rms_norm: weight [W] of the activation dtype")
    out = torch.empty(T, W, dtype=adt, device=x_in.device) if want_out else None
    _need(out is not None or x_out is not None, "depth_residual_rms_norm: nothing to write")
    check(_lib.mixers_lib().aphro_depth_residual_rms_norm(
        x_in.data_ptr(), _p(x_out), _p(y), ys, _p(history) if depth_w is not None else None, hs, int(n_hist), _p(depth_w),
        float(gain), _p(weight), _p(out), T, W, float(eps), _DT[adt], _stream()), "depth_residual_rms_norm")
    return out


def poly_norm(z: torch.Tensor, coef, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e per row, N = division by the row's root mean square; coef = (a, b, c, e) floats."""
    _cuda(z)
    _need(z.dim() == 2 and len(coef) == 4, "poly_norm: z [T, n], four coefficients")
    T, n = z.shape
    out = torch.empty(T, n, dtype=z.dtype, device=z.device)
    check(_lib.mixers_lib().aphro_poly_norm(out.data_ptr(), z.data_ptr(), _rows(z, n, "poly_norm z"), T, n, float(coef[0]),
                                            float(coef[1]), float(coef[2]), float(coef[3]), float(eps), _dt(z), _stream()),
          "poly_norm")
    return out


def differential_norm_gate(out: torch.Tensor, a: torch.Tensor, gate: Optional[torch.Tensor], heads: int, maps: int, vdim: int,
                           lam: float, out_scale: float, eps: float) -> None:
    """out [T, heads * vdim] = out_scale * unit_rms_per_head(a_1 - lam a_2) * sigmoid(gate); a fp32 [T, heads * maps * vdim]."""
    _cuda(out, a, gate)
    T = a.shape[0]
    _need(a.dtype == torch.float32 and out.shape == (T, heads * vdim), "differential_norm_gate: a fp32, out [T, heads * vdim]")
    gs = 0
    if gate is not None:
        _need(gate.dtype == out.dtype and gate.shape == (T, heads * vdim), "differential_norm_gate: gate [T, heads * vdim]")
        gs = _rows(gate, heads * vdim, "differential_norm_gate gate")
    check(_lib.mixers_lib().aphro_differential_norm_gate(
        out.data_ptr(), _rows(out, heads * vdim, "differential_norm_gate out"), a.data_ptr(),
        _rows(a, heads * maps * vdim, "differential_norm_gate a"), _p(gate), gs, T, heads, maps, vdim, float(lam), float(out_scale),
        float(eps), _dt(out), _stream()), "differential_norm_gate")


def short_conv(u: torch.Tensor, w: torch.Tensor, state: Optional[torch.Tensor], state_slots: torch.Tensor, q_start: torch.Tensor,
               q_len: torch.Tensor, ctx_len: torch.Tensor, seq_of_token: torch.Tensor, cq: int, ck: int = 0, cv: int = 0,
               k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
               slot_mapping: Optional[torch.Tensor] = None, act: int = 0) -> Optional[torch.Tensor]:
    """Short causal convolution over time on the channels of u [T, cq + ck + cv] (dense rows, any row stride) with w
    [channels, taps]; returns the first cq channels [T, cq]; the ck and cv channels go into the paged caches
    (k_cache [blocks, block, ck], v_cache [blocks, block, cv] in any further split of the last axis) at ``slot_mapping``.
    state [slots, taps - 1, channels] holds every request's last inputs and is advanced.  ``act`` 1: silu on the result."""
    _cuda(u, w, state, state_slots, q_start, q_len, ctx_len, seq_of_token, k_cache, v_cache, slot_mapping)
    C = cq + ck + cv
    T, S = u.shape[0], q_start.numel()
    taps = w.shape[1]
    _need(w.dim() == 2 and w.shape[0] == C and w.is_contiguous() and w.dtype == u.dtype, "short_conv: w [channels, taps]")
    if taps > 1:
        _need(state is not None and state.dtype == u.dtype and state.dim() == 3 and state.is_contiguous()
              and tuple(state.shape[1:]) == (taps - 1, C), "short_conv: state [slots, taps - 1, channels]")
    for t, nm in ((state_slots, "state_slots"), (q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    _i32(seq_of_token, T, "seq_of_token")
    ncs = 0
    if ck + cv:
        _need(k_cache is not None and v_cache is not None and slot_mapping is not None and k_cache.is_contiguous()
              and v_cache.is_contiguous() and k_cache.dtype == u.dtype == v_cache.dtype, "short_conv: caches of the activation dtype")
        ncs = k_cache.shape[0] * k_cache.shape[1]
        _need(k_cache.numel() == ncs * ck and v_cache.numel() == ncs * cv, "short_conv: cache rows do not fit the channels")
        _need(slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous(),
              "short_conv: slots int64 [T]")
    q = torch.empty(T, cq, dtype=u.dtype, device=u.device) if cq else None
    check(_lib.mixers_lib().aphro_short_conv(
        _p(q), cq, _p(k_cache) if ck + cv else None, _p(v_cache) if ck + cv else None, _p(slot_mapping) if ck + cv else None, ncs,
        u.data_ptr(), _rows(u, C, "short_conv u"), w.data_ptr(), _p(state) if taps > 1 else None, state_slots.data_ptr(),
        q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(), seq_of_token.data_ptr(), T, S, cq, ck, cv, taps, int(act), _dt(u),
        _stream()), "short_conv")
    return q


def windowed_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                       q_start: torch.Tensor, q_len: torch.Tensor, ctx_len: torch.Tensor, seq_of_token: torch.Tensor, q_len_range,
                       heads: int, maps: int, scale: float, window: int, keep_first: int, max_kv_len: int = 0) -> torch.Tensor:
    """Every map's softmax attention under a sliding window that keeps the first tokens, fp32 [T, heads * maps * vdim].
    q [T, heads * maps * dim]; k_cache [blocks, block, kv_heads * maps, dim], v_cache [blocks, block, kv_heads, vdim]."""
    _cuda(q, k_cache, v_cache, block_tables, q_start, q_len, ctx_len, seq_of_token)
    lo, hi = int(q_len_range[0]), int(q_len_range[1])
    _need(0 < lo <= hi, "windowed_attention: q_len_range (shortest, longest)")
    nb, bs, GM, d = k_cache.shape
    G, e = v_cache.shape[2], v_cache.shape[3]
    T, S = q.shape[0], q_start.numel()
    _need(v_cache.shape[:2] == (nb, bs) and GM == G * maps and k_cache.is_contiguous() and v_cache.is_contiguous(),
          "windowed_attention: cache shapes")
    _need(q.dtype == k_cache.dtype == v_cache.dtype and heads % G == 0, "windowed_attention: one dtype, heads a multiple of kv heads")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] == S and block_tables.is_contiguous(),
          "windowed_attention: block_tables int32 [S, max_blocks]")
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    _i32(seq_of_token, T, "seq_of_token")
    out = torch.empty(T, heads * maps * e, dtype=torch.float32, device=q.device)
    ws, ws_n = None, 0
    check(_lib.mixers_lib().aphro_windowed_attention(
        out.data_ptr(), heads * maps * e, q.data_ptr(), _rows(q, heads * maps * d, "windowed_attention q"), k_cache.data_ptr(),
        v_cache.data_ptr(), block_tables.data_ptr(), block_tables.shape[1], nb, bs, q_start.data_ptr(), q_len.data_ptr(),
        ctx_len.data_ptr(), seq_of_token.data_ptr(), T, S, lo, hi, heads, G, maps, d, e, float(scale), int(window), int(keep_first),
        int(max_kv_len), _p(ws), ws_n, _dt(q), _stream()), "windowed_attention")
    return out


def differential_window_attention_supported(heads: int, kv_heads: int, dim: int, vdim: int, dtype: torch.dtype) -> bool:
    return dtype in _DT and bool(_lib.mixers_lib().aphro_differential_window_attention_supported(heads, kv_heads, dim, vdim, _DT[dtype]))


def differential_window_attention(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor], k_cache: torch.Tensor,
                                  v_cache: torch.Tensor, block_tables: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                                  ctx_len: torch.Tensor, seq_of_token: torch.Tensor, q_len_range, heads: int, scale: float,
                                  window: int, keep_first: int, lam: float, out_scale: float, eps: float,
                                  max_kv_len: int = 0) -> None:
    """The two maps of every head under the window, joined (a_1 - lam a_2), unit RMS per head, out_scale, sigmoid gate, in one
    launch: out [T, heads * vdim] (dense rows, any row stride).  Sizes as ``differential_window_attention_supported`` says.
    ``max_kv_len``: the longest ctx_len + q_len of the batch (host); given, decoded rows that see many keys split them over
    several workgroups through a scratch tensor."""
    _cuda(out, q, gate, k_cache, v_cache, block_tables, q_start, q_len, ctx_len, seq_of_token)
    lo, hi = int(q_len_range[0]), int(q_len_range[1])
    _need(0 < lo <= hi, "differential_window_attention: q_len_range (shortest, longest)")
    nb, bs, G2, d = k_cache.shape
    G, e = v_cache.shape[2], v_cache.shape[3]
    T, S = q.shape[0], q_start.numel()
    _need(v_cache.shape[:2] == (nb, bs) and G2 == 2 * G and k_cache.is_contiguous() and v_cache.is_contiguous(),
          "differential_window_attention: cache shapes")
    _need(q.dtype == k_cache.dtype == v_cache.dtype == out.dtype and heads % G == 0 and out.shape == (T, heads * e),
          "differential_window_attention: one dtype, out [T, heads * vdim]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] == S and block_tables.is_contiguous(),
          "differential_window_attention: block_tables int32 [S, max_blocks]")
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    _i32(seq_of_token, T, "seq_of_token")
    gs = 0
    if gate is not None:
        _need(gate.dtype == q.dtype and gate.shape == (T, heads * e), "differential_window_attention: gate [T, heads * vdim]")
        gs = _rows(gate, heads * e, "differential_window_attention gate")
    ws, ws_n = None, 0
    visible = min(max_kv_len, window + keep_first) if window > 0 else max_kv_len
    if visible >= 512 and lo < 8:
        ws_n = T * heads * 2 * 8 * (2 + e)
        ws = torch.empty(ws_n, dtype=torch.float32, device=q.device)
    check(_lib.mixers_lib().aphro_differential_window_attention(
        out.data_ptr(), _rows(out, heads * e, "differential_window_attention out"), q.data_ptr(),
        _rows(q, heads * 2 * d, "differential_window_attention q"), _p(gate), gs, k_cache.data_ptr(), v_cache.data_ptr(),
        block_tables.data_ptr(), block_tables.shape[1], nb, bs, q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(),
        seq_of_token.data_ptr(), T, S, lo, hi, heads, G, d, e, float(scale), int(window), int(keep_first), float(lam), float(out_scale),
        float(eps), int(max_kv_len), _p(ws), ws_n, _dt(q), _stream()), "differential_window_attention")


# ---- mixture of experts on unquantised weights ---------------------------------------------------------------------------------
def experts_route(router_out: torch.Tensor, correction: Optional[torch.Tensor], top: int):
    """router_out fp32 [T, outputs] -> (ids int32 [T, top], weights fp32 [T, top])."""
    _cuda(router_out, correction)
    T, R = router_out.shape
    _need(router_out.dtype == torch.float32 and router_out.is_contiguous(), "experts_route: router outputs fp32, contiguous")
    _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == R and correction.is_contiguous()),
          "experts_route: correction fp32 [outputs]")
    ids = torch.empty(T, top, dtype=torch.int32, device=router_out.device)
    w = torch.empty(T, top, dtype=torch.float32, device=router_out.device)
    check(_lib.mixers_lib().aphro_experts_route(ids.data_ptr(), w.data_ptr(), router_out.data_ptr(), _p(correction), T, R, int(top),
                                                _stream()), "experts_route")
    return ids, w


def experts_forward(h: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                    limit: float, alpha: float, shared: Optional[torch.Tensor] = None,
                    shared_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Weighted sum of every token's chosen experts.  h [T, W]; ids / weights [T, top]; w_gate_up [E, 2 ff, W] (gate rows, then
    up rows), w_down [E, W, ff]; ids >= E are identity experts (their output is h).  ``shared`` [T, W] is added, times
    sigmoid(shared_gate [T, 1])."""
    _cuda(h, ids, weights, w_gate_up, w_down, shared, shared_gate)
    T, W = h.shape
    E, ff2, _ = w_gate_up.shape
    ff, top = ff2 // 2, ids.shape[1]
    lib = _lib.mixers_lib()
    _need(w_gate_up.shape == (E, 2 * ff, W) and w_down.shape == (E, W, ff) and w_gate_up.is_contiguous() and w_down.is_contiguous()
          and w_gate_up.dtype == h.dtype == w_down.dtype, "experts_forward: w_gate_up [E, 2 ff, W], w_down [E, W, ff] of h's dtype")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and weights.dtype == torch.float32 and weights.is_contiguous()
          and weights.shape == ids.shape and ids.shape[0] == T, "experts_forward: ids int32 / weights fp32 [T, top]")
    hs = _rows(h, W, "experts_forward h")
    cap = int(lib.aphro_experts_align_capacity(T * top, E))
    dev = h.device
    sorted_slots = torch.empty(cap, dtype=torch.int32, device=dev)
    block_expert = torch.empty(cap // int(lib.aphro_experts_block_rows(T * top, E)), dtype=torch.int32, device=dev)
    num_blocks = torch.empty(1, dtype=torch.int32, device=dev)
    y = torch.empty(cap, ff, dtype=h.dtype, device=dev)
    eo = torch.empty(T * top, W, dtype=torch.float32, device=dev)
    out = torch.empty(T, W, dtype=h.dtype, device=dev)
    st = _stream()
    check(lib.aphro_experts_align(sorted_slots.data_ptr(), cap, block_expert.data_ptr(), num_blocks.data_ptr(), ids.data_ptr(),
                                  T * top, E, st), "experts_align")
    check(lib.aphro_experts_glu_gemm(y.data_ptr(), h.data_ptr(), hs, w_gate_up.data_ptr(), sorted_slots.data_ptr(),
                                     block_expert.data_ptr(), num_blocks.data_ptr(), cap, T * top, E, top, ff, W, float(limit),
                                     float(alpha), _dt(h), st), "experts_glu_gemm")
    check(lib.aphro_experts_down_gemm(eo.data_ptr(), y.data_ptr(), w_down.data_ptr(), sorted_slots.data_ptr(),
                                      block_expert.data_ptr(), num_blocks.data_ptr(), cap, T * top, E, top, W, ff, _dt(h), st),
          "experts_down_gemm")
    ss = sgs = 0
    if shared is not None:
        _need(shared.dtype == h.dtype and shared.shape == (T, W), "experts_forward: shared [T, W]")
        ss = _rows(shared, W, "experts_forward shared")
        if shared_gate is not None:
            _need(shared_gate.dtype == h.dtype and shared_gate.shape == (T, 1), "experts_forward: shared_gate [T, 1]")
            sgs = shared_gate.stride(0)
    check(lib.aphro_experts_combine(out.data_ptr(), eo.data_ptr(), ids.data_ptr(), weights.data_ptr(), h.data_ptr(), hs, _p(shared),
                                    ss, _p(shared_gate) if shared is not None else None, sgs, T, W, top, E, _dt(h), st),
          "experts_combine")
    return out


def clamped_glu(x: torch.Tensor, d: int, limit: float, alpha: float) -> torch.Tensor:
    """[T, >= 2 d] -> [T, d]: g = min(x[:, :d], limit), u = clamp(x[:, d:2d], +-limit), g * sigmoid(alpha g) * (u + 1)."""
    _cuda(x)
    _need(x.dim() == 2 and x.shape[1] >= 2 * d and x.stride(1) == 1, "clamped_glu: [T, >= 2 d] with dense rows")
    out = torch.empty(x.shape[0], d, dtype=x.dtype, device=x.device)
    check(_lib.mixers_lib().aphro_clamped_glu(out.data_ptr(), x.data_ptr(), x.stride(0) if x.shape[0] > 1 else max(x.stride(0), 2 * d),
                                              x.shape[0], d, float(limit), float(alpha), _dt(x), _stream()), "clamped_glu")
    return out


# ---- sublayers side by side, hashed token-pair embedding, attention through a low-rank latent ------------------------------------
def hashed_pair_embed(table: torch.Tensor, pair_table: torch.Tensor, ids: torch.Tensor, token_state: torch.Tensor,
                      state_slots: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, ctx_len: torch.Tensor,
                      seq_of_token: torch.Tensor, mul_prev: int, mul_cur: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 rows ``table[id] + pair_table[(previous * mul_prev + id * mul_cur) mod buckets]`` (row ``buckets`` for a sequence's
    first token; pair_table has buckets + 1 rows).  ``token_state`` int32 [slots] holds every live request's last token: it is
    read for a segment's first row and advanced to the segment's last token."""
    _cuda(table, pair_table, ids, token_state, state_slots, q_start, q_len, ctx_len, seq_of_token, out)
    T, S, W = ids.shape[0], q_start.numel(), table.shape[1]
    _need(table.dim() == 2 and table.is_contiguous() and pair_table.dim() == 2 and pair_table.is_contiguous()
          and pair_table.shape[1] == W and pair_table.shape[0] >= 2 and pair_table.dtype == table.dtype,
          "hashed_pair_embed: table [vocab, width], pair_table [buckets + 1, width], one dtype")
    _need(ids.dtype == torch.int64 and ids.dim() == 1 and ids.is_contiguous(), "hashed_pair_embed: ids int64 [T]")
    _need(token_state.dtype == torch.int32 and token_state.dim() == 1 and token_state.is_contiguous(),
          "hashed_pair_embed: token_state int32 [slots]")
    for t, nm in ((state_slots, "state_slots"), (q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    _i32(seq_of_token, T, "seq_of_token")
    if out is None:
        out = torch.empty(T, W, dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, W), "hashed_pair_embed: out fp32 [T, width]")
    lib, st = _lib.mixers_lib(), _stream()
    check(lib.aphro_hashed_pair_embed(out.data_ptr(), table.data_ptr(), pair_table.data_ptr(), ids.data_ptr(), token_state.data_ptr(),
                                      state_slots.data_ptr(), q_start.data_ptr(), ctx_len.data_ptr(), seq_of_token.data_ptr(), T, W,
                                      table.shape[0], pair_table.shape[0] - 1, int(mul_prev), int(mul_cur), _dt(table), st),
          "hashed_pair_embed")
    check(lib.aphro_token_state_write(token_state.data_ptr(), ids.data_ptr(), state_slots.data_ptr(), q_start.data_ptr(),
                                      q_len.data_ptr(), S, st), "token_state_write")
    return out


def residual_add2_rms_norm(x: torch.Tensor, ya: Optional[torch.Tensor] = None, yb: Optional[torch.Tensor] = None,
                           bias: Optional[torch.Tensor] = None, weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
                           dtype: Optional[torch.dtype] = None, want_out: bool = True) -> Optional[torch.Tensor]:
    """x += ya + yb + bias in place (fp32 [T, W]; each term optional), then returns rms_norm(x) * weight in the activation dtype
    (``want_out`` False: the add alone)."""
    T, W = x.shape
    _cuda(x, ya, yb, bias, weight)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "residual_add2_rms_norm: x is fp32, contiguous")
    some = next((t for t in (ya, yb, weight, bias) if t is not None), None)
    adt = dtype or (some.dtype if some is not None else None)
    _need(adt in _DT, "residual_add2_rms_norm: the activation dtype is not given")
    sa = sb = 0
    if ya is not None:
        _need(ya.dtype == adt and ya.shape[0] == T, "residual_add2_rms_norm: ya [T, W] of the activation dtype")
        sa = _rows(ya, W, "residual_add2_rms_norm ya")
    if yb is not None:
        _need(yb.dtype == adt and yb.shape[0] == T, "residual_add2_rms_norm: yb [T, W] of the activation dtype")
        sb = _rows(yb, W, "residual_add2_rms_norm yb")
    for v in (bias, weight):
        _need(v is None or (v.dtype == adt and v.numel() == W and v.is_contiguous()), "residual_add2_rms_norm: vectors [W] of the activation dtype")
    out = torch.empty(T, W, dtype=adt, device=x.device) if want_out else None
    check(_lib.mixers_lib().aphro_residual_add2_rms_norm(x.data_ptr(), _p(ya), sa, _p(yb), sb, _p(bias), _p(weight), _p(out), T, W,
                                                         float(eps), _DT[adt], _stream()), "residual_add2_rms_norm")
    return out


def latent_prep(proj: torch.Tensor, q_at: int, q_rank: int, kv_at: int, kv_rank: int, rot_dim: int, rot_dims: int,
                wq: Optional[torch.Tensor], wkv: torch.Tensor, cache: torch.Tensor, slot_mapping: torch.Tensor,
                q_start: torch.Tensor, ctx_len: torch.Tensor, seq_of_token: torch.Tensor, inv_freq: Optional[torch.Tensor],
                mscale: float, eps: float) -> Optional[torch.Tensor]:
    """From the rows of one input product: the normed query latent [T, q_rank] (returned), and the cache row of every token --
    its normed key/value latent and the shared key part rotated at the token's position -- written at ``slot_mapping``.
    cache [blocks, block, kv_rank + rot_dim]."""
    _cuda(proj, wq, wkv, cache, slot_mapping, q_start, ctx_len, seq_of_token, inv_freq)
    T, S = proj.shape[0], q_start.numel()
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= max(q_at + q_rank, kv_at + kv_rank + rot_dim),
          "latent_prep: proj rows hold the latents")
    _need(cache.dim() == 3 and cache.is_contiguous() and cache.shape[2] == kv_rank + rot_dim and cache.dtype == proj.dtype,
          "latent_prep: cache [blocks, block, kv_rank + rot_dim] of the activation dtype")
    _need(wkv.dtype == proj.dtype and wkv.numel() == kv_rank and wkv.is_contiguous(), "latent_prep: wkv [kv_rank]")
    _need(q_rank == 0 or (wq is not None and wq.dtype == proj.dtype and wq.numel() == q_rank and wq.is_contiguous()),
          "latent_prep: wq [q_rank]")
    _need(slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous(), "latent_prep: slots int64 [T]")
    _i32(q_start, S, "q_start")
    _i32(ctx_len, S, "ctx_len")
    _i32(seq_of_token, T, "seq_of_token")
    _need(rot_dims == 0 or (inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2
                            and inv_freq.is_contiguous()), "latent_prep: inv_freq fp32 [rot_dims / 2]")
    cq = torch.empty(T, q_rank, dtype=proj.dtype, device=proj.device) if q_rank else None
    stride = proj.stride(0) if T > 1 else max(proj.stride(0), proj.shape[1])
    check(_lib.mixers_lib().aphro_latent_prep(_p(cq), cache.data_ptr(), cache.shape[0] * cache.shape[1], proj.data_ptr(), stride,
                                              int(q_at), int(kv_at), _p(wq), wkv.data_ptr(), slot_mapping.data_ptr(),
                                              q_start.data_ptr(), ctx_len.data_ptr(), seq_of_token.data_ptr(), _p(inv_freq),
                                              float(mscale), T, int(q_rank), int(kv_rank), int(rot_dim), int(rot_dims), float(eps),
                                              _dt(proj), _stream()), "latent_prep")
    return cq


def _head_view(t: torch.Tensor, T: int, heads: int, n: int, what: str):
    """(token stride, head stride) of a [T, heads, n] view whose last axis is dense."""
    _need(t.dim() == 3 and tuple(t.shape) == (T, heads, n) and (t.stride(2) == 1 or n == 1), f"{what}: [T, heads, {n}] with a dense last axis")
    return t.stride(0), t.stride(1)


def latent_attention(out: torch.Tensor, q_lat: torch.Tensor, q_rot: Optional[torch.Tensor], cache: torch.Tensor,
                     block_tables: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor, ctx_len: torch.Tensor,
                     seq_of_token: torch.Tensor, q_len_range, inv_freq: Optional[torch.Tensor], mscale: float, rot_dims: int,
                     scale: float, max_kv_len: int = 0, plain: bool = False, window: int = 0,
                     sink: Optional[torch.Tensor] = None) -> None:
    """Causal softmax attention of a batch of segments over latent cache rows [c | k_r] that all heads share.  q_lat
    [T, heads, kv_rank] (every head's query carried into the latent), q_rot [T, heads, rot_dim] (raw: rotated here at the row's
    position), out [T, heads, kv_rank] = sum_j p_ij c_j -- any strides over tokens and heads.  ``q_len_range`` (shortest, longest
    segment) and ``max_kv_len`` (longest ctx_len + q_len), known on the host, choose the work split of the matrix-core kernel,
    which serves the sizes ``latent_attention_fast_supported`` names; ``plain`` forces the fp32-math kernel of any size.
    ``window`` > 0: a row sees only the last ``window`` keys up to its own; ``sink`` fp32 [heads]: exp(sink) joins every row's
    softmax denominator (unscaled, without a value)."""
    _cuda(out, q_lat, q_rot, cache, block_tables, q_start, q_len, ctx_len, seq_of_token, inv_freq, sink)
    _need(sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == q_lat.shape[1]),
          "latent_attention: sink fp32 [heads]")
    window = max(int(window), 0)
    T, H, R = q_lat.shape
    nb, bs, D = cache.shape
    P_ = D - R
    S = q_start.numel()
    _need(cache.is_contiguous() and cache.dtype == q_lat.dtype == out.dtype and P_ >= 0, "latent_attention: cache [blocks, block, rank + rot]")
    os_, ohs = _head_view(out, T, H, R, "latent_attention out")
    qs, qhs = _head_view(q_lat, T, H, R, "latent_attention q_lat")
    rs = rhs = 0
    if P_:
        _need(q_rot is not None and q_rot.dtype == q_lat.dtype, "latent_attention: q_rot of the activation dtype")
        rs, rhs = _head_view(q_rot, T, H, P_, "latent_attention q_rot")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] == S and block_tables.is_contiguous(),
          "latent_attention: block_tables int32 [S, max_blocks]")
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    _i32(seq_of_token, T, "seq_of_token")
    _need(rot_dims == 0 or (inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2
                            and inv_freq.is_contiguous()), "latent_attention: inv_freq fp32 [rot_dims / 2]")
    lib = _lib.mixers_lib()
    if plain:
        check(lib.aphro_latent_attention_plain(
            out.data_ptr(), os_, ohs, q_lat.data_ptr(), qs, qhs, _p(q_rot), rs, rhs, cache.data_ptr(), block_tables.data_ptr(),
            block_tables.shape[1], nb, bs, q_start.data_ptr(), ctx_len.data_ptr(), seq_of_token.data_ptr(), _p(inv_freq), float(mscale),
            T, H, R, P_, int(rot_dims), float(scale), window, _p(sink), _dt(q_lat), _stream()), "latent_attention")
        return
    lo, hi = int(q_len_range[0]), int(q_len_range[1])
    _need(0 < lo <= hi, "latent_attention: q_len_range (shortest, longest)")
    ws, ws_n = None, 0
    if lib.aphro_latent_attention_fast_supported(R, P_, int(rot_dims), _dt(q_lat)):
        if window > 0:                         # what a row can see, not how long its sequence is, decides the split
            max_kv_len = min(int(max_kv_len), window + hi)
        splits = int(lib.aphro_latent_attention_splits(T, S, hi, H, int(max_kv_len)))
        if splits > 1:
            ws_n = T * H * splits * (2 + R)
            ws = torch.empty(ws_n, dtype=torch.float32, device=q_lat.device)
    check(lib.aphro_latent_attention(
        out.data_ptr(), os_, ohs, q_lat.data_ptr(), qs, qhs, _p(q_rot), rs, rhs, cache.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], nb, bs, q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(), seq_of_token.data_ptr(), _p(inv_freq),
        float(mscale), T, S, hi, int(max_kv_len), H, R, P_, int(rot_dims), float(scale), window, _p(sink), _p(ws), ws_n, _dt(q_lat),
        _stream()), "latent_attention")


def latent_attention_fast_supported(kv_rank: int, rot_dim: int, rot_dims: int, dtype: torch.dtype) -> bool:
    return dtype in _DT and bool(_lib.mixers_lib().aphro_latent_attention_fast_supported(kv_rank, rot_dim, rot_dims, _DT[dtype]))


def sigmoid_gate_mul(x: torch.Tensor, gate: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x * sigmoid(gate), [T, n] with dense rows of any stride; into ``out`` (which may be x) if given."""
    _cuda(x, gate, out)
    T, n = x.shape
    _need(gate.shape == (T, n) and gate.dtype == x.dtype, "sigmoid_gate_mul: gate [T, n] of x's dtype")
    if out is None:
        out = torch.empty(T, n, dtype=x.dtype, device=x.device)
    _need(out.shape == (T, n) and out.dtype == x.dtype, "sigmoid_gate_mul: out [T, n]")
    check(_lib.mixers_lib().aphro_sigmoid_gate_mul(out.data_ptr(), _rows(out, n, "sigmoid_gate_mul out"), x.data_ptr(),
                                                   _rows(x, n, "sigmoid_gate_mul x"), gate.data_ptr(),
                                                   _rows(gate, n, "sigmoid_gate_mul gate"), T, n, _dt(x), _stream()), "sigmoid_gate_mul")
    return out


def experts_route_grouped(router_out: torch.Tensor, top: int, groups: int, keep: int, scale: float, group_top: int = 2):
    """router_out fp32 [T, experts] -> (ids int32 [T, top], weights fp32 [T, top]): sigmoid scores, choice limited to the ``keep``
    best of ``groups`` equal groups of neighbouring experts (a group's score: the sum of its ``group_top`` largest scores),
    weights = score * scale."""
    _cuda(router_out)
    T, E = router_out.shape
    _need(router_out.dtype == torch.float32 and router_out.is_contiguous(), "experts_route_grouped: router outputs fp32, contiguous")
    ids = torch.empty(T, top, dtype=torch.int32, device=router_out.device)
    w = torch.empty(T, top, dtype=torch.float32, device=router_out.device)
    check(_lib.mixers_lib().aphro_experts_route_grouped(ids.data_ptr(), w.data_ptr(), router_out.data_ptr(), T, E, int(top), int(groups),
                                                        int(keep), int(group_top), float(scale), _stream()), "experts_route_grouped")
    return ids, w


def experts_route_topk(router_out: torch.Tensor, bias: Optional[torch.Tensor], top: int):
    """router_out fp32 [T, experts] (+ bias fp32 [experts]) -> (ids int32 [T, top], weights fp32 [T, top]): the ``top`` largest
    logits are chosen (ties to the lower index), the weights are the softmax over the chosen logits only."""
    _cuda(router_out, bias)
    T, E = router_out.shape
    _need(router_out.dtype == torch.float32 and router_out.is_contiguous(), "experts_route_topk: router outputs fp32, contiguous")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == E and bias.is_contiguous()), "experts_route_topk: bias fp32 [experts]")
    ids = torch.empty(T, top, dtype=torch.int32, device=router_out.device)
    w = torch.empty(T, top, dtype=torch.float32, device=router_out.device)
    check(_lib.mixers_lib().aphro_experts_route_topk(ids.data_ptr(), w.data_ptr(), router_out.data_ptr(), _p(bias), T, E, int(top),
                                                     _stream()), "experts_route_topk")
    return ids, w


# ---- a residual in several streams, the gated delta rule, rotary attention's preparation ---------------------------------------
def _host_floats(values, n: int, what: str):
    """A ctypes float array (host memory) of n numbers, or None."""
    import ctypes
    if values is None:
        return None
    if isinstance(values, ctypes.Array):           # made once by the caller (host_floats)
        _need(len(values) == n, f"{what}: {n} numbers expected, {len(values)} given")
        return values
    vals = [float(v) for v in values]
    _need(len(vals) == n, f"{what}: {n} numbers expected, {len(vals)} given")
    return (ctypes.c_float * n)(*vals)


def host_floats(values):
    """A host array of floats for the coefficient arguments of ``hyper_residual_rms_norm`` (rows of a matrix are flattened), made once
    instead of at every call."""
    import ctypes
    vals = [float(c) for row in values for c in (row if isinstance(row, (list, tuple)) else [row])]
    return (ctypes.c_float * len(vals))(*vals)


def hyper_residual_rms_norm(x: torch.Tensor, y: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None, mix=None,
                            out_coef=None, mult: float = 1.0, in_coef=None, weight: Optional[torch.Tensor] = None,
                            eps: float = 1e-6, dtype: Optional[torch.dtype] = None, want_out: bool = True,
                            want_sum: bool = False):
    """x fp32 [T, streams, W] in place.  With ``y`` [T, W]: every stream t becomes sum_s mix[s][t] x_s + mult * out_coef[t] *
    (scale * y).  Then u = sum_s in_coef[s] x_s and the result is rms_norm(u) * weight in the activation dtype (``want_out``
    False: none); ``want_sum``: u itself (fp32 [T, W]) is returned as a second value.  mix (rows of [from][to]), out_coef and
    in_coef are host numbers (None: identity / ones); scale and weight are [W] tensors of the activation dtype (None: ones)."""
    import ctypes
    _cuda(x, y, scale, weight)
    _need(x.dim() == 3 and x.dtype == torch.float32 and x.is_contiguous(), "hyper_residual_rms_norm: x fp32 [T, streams, W], contiguous")
    T, n, W = x.shape
    some = next((t for t in (y, weight, scale) if t is not None), None)
    adt = dtype or (some.dtype if some is not None else None)
    _need(adt in _DT, "hyper_residual_rms_norm: the activation dtype is not given")
    ys = 0
    if y is not None:
        _need(y.dtype == adt and y.shape[0] == T, "hyper_residual_rms_norm: y [T, W] of the activation dtype")
        ys = _rows(y, W, "hyper_residual_rms_norm y")
    for v in (scale, weight):
        _need(v is None or (v.dtype == adt and v.numel() == W and v.is_contiguous()), "hyper_residual_rms_norm: vectors [W] of the activation dtype")
    import ctypes as _ct
    mixa = _host_floats(mix if mix is None or isinstance(mix, _ct.Array) else [c for row in mix for c in row], n * n,
                        "hyper_residual_rms_norm mix")
    outa = _host_floats(out_coef, n, "hyper_residual_rms_norm out_coef")
    ina = _host_floats(in_coef, n, "hyper_residual_rms_norm in_coef")
    out = torch.empty(T, W, dtype=adt, device=x.device) if want_out else None
    total = torch.empty(T, W, dtype=torch.float32, device=x.device) if want_sum else None
    ptr = lambda a: None if a is None else ctypes.cast(a, ctypes.c_void_p)
    check(_lib.mixers_lib().aphro_hyper_residual_rms_norm(x.data_ptr(), _p(y), ys, _p(scale), ptr(mixa), ptr(outa), float(mult), ptr(ina),
                                                          _p(weight), _p(out), _p(total), T, n, W, float(eps), _DT[adt], _stream()),
          "hyper_residual_rms_norm")
    return (out, total) if want_sum else out


def logit_softcap(z: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """fp32 ``cap * tanh(z * scale / cap)`` (``cap`` <= 0: ``z * scale``) of a contiguous tensor of the activation dtype."""
    _cuda(z)
    _need(z.is_contiguous(), "logit_softcap: contiguous input")
    out = torch.empty(z.shape, dtype=torch.float32, device=z.device)
    check(_lib.mixers_lib().aphro_logit_softcap(out.data_ptr(), z.data_ptr(), z.numel(), float(scale), float(cap), _dt(z), _stream()),
          "logit_softcap")
    return out


def gated_delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b: torch.Tensor, a: torch.Tensor, a_log: torch.Tensor,
                     dt_bias: torch.Tensor, state: torch.Tensor, slot_of_seq: torch.Tensor, q_start: torch.Tensor,
                     q_len: torch.Tensor, ctx_len: torch.Tensor, heads: int, kv_heads: int, q_scale: float, norm_eps: float = 1e-6,
                     max_q_len: int = 1) -> torch.Tensor:
    """Scan every segment through its slot's state S fp32 [slots, heads, dim, vdim] (updated in place) with the gated delta rule;
    returns o fp32 [T, heads * vdim].  q, k [T, kv_heads * dim] (made unit vectors per head inside), v [T, heads * vdim], b and a
    [T, heads] raw (beta = sigmoid(b), decay = exp(-exp(a_log) softplus(a + dt_bias))); a_log, dt_bias fp32 [heads]."""
    _cuda(q, k, v, b, a, a_log, dt_bias, state, slot_of_seq, q_start, q_len, ctx_len)
    T, S = q.shape[0], q_start.numel()
    _need(state.dim() == 4 and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] == heads,
          "gated_delta_scan: state fp32 [slots, heads, dim, vdim]")
    slots, _, d, e = state.shape
    _need(q.dtype == k.dtype == v.dtype == b.dtype == a.dtype and k.shape[0] == T and v.shape[0] == T and b.shape[0] == T
          and a.shape[0] == T, "gated_delta_scan: q, k, v, b, a rows / dtype")
    for t, nm in ((a_log, "a_log"), (dt_bias, "dt_bias")):
        _need(t.dtype == torch.float32 and t.numel() == heads and t.is_contiguous(), f"gated_delta_scan: {nm} fp32 [heads]")
    for t, nm in ((slot_of_seq, "slot_of_seq"), (q_start, "q_start"), (q_len, "q_len"), (ctx_len, "ctx_len")):
        _i32(t, S, nm)
    out = torch.empty(T, heads * e, dtype=torch.float32, device=q.device)
    check(_lib.mixers_lib().aphro_gated_delta_scan(
        out.data_ptr(), q.data_ptr(), _rows(q, kv_heads * d, "q"), k.data_ptr(), _rows(k, kv_heads * d, "k"), v.data_ptr(),
        _rows(v, heads * e, "v"), b.data_ptr(), _rows(b, heads, "b"), a.data_ptr(), _rows(a, heads, "a"), a_log.data_ptr(),
        dt_bias.data_ptr(), state.data_ptr(), slot_of_seq.data_ptr(), slots, q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(),
        S, T, heads, kv_heads, d, e, float(q_scale), float(norm_eps), int(max_q_len), _dt(q), _stream()), "gated_delta_scan")
    return out


GATE_SIGMOID, GATE_SILU = 0, 1


def gated_head_rms_norm(out: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor], gate: Optional[torch.Tensor],
                        heads: int, eps: float, act: int = GATE_SIGMOID) -> None:
    """out [T, heads * vdim] (dense rows, any row stride) = x / rms(x over each head) * weight[vdim] * act(gate); x fp32
    [T, heads * vdim] contiguous; weight is shared by the heads."""
    _cuda(out, x, weight, gate)
    T, N = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and N % heads == 0, "gated_head_rms_norm: x fp32 [T, heads * vdim], contiguous")
    e = N // heads
    _need(out.shape == (T, N), "gated_head_rms_norm: out [T, heads * vdim]")
    _need(weight is None or (weight.dtype == out.dtype and weight.numel() == e and weight.is_contiguous()), "gated_head_rms_norm: weight [vdim]")
    gs = 0
    if gate is not None:
        _need(gate.dtype == out.dtype and gate.shape == (T, N), "gated_head_rms_norm: gate [T, heads * vdim] of the output dtype")
        gs = _rows(gate, N, "gated_head_rms_norm gate")
    check(_lib.mixers_lib().aphro_gated_head_rms_norm(out.data_ptr(), _rows(out, N, "gated_head_rms_norm out"), x.data_ptr(), _p(weight),
                                                      _p(gate), gs, T, heads, e, float(eps), int(act), _dt(out), _stream()),
          "gated_head_rms_norm")


ROTARY_HALF, ROTARY_INTERLEAVED = 0, 1


def rotary_qk_norm_kv_write(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            slot_mapping: torch.Tensor, q_start: torch.Tensor, ctx_len: torch.Tensor, seq_of_token: torch.Tensor,
                            inv_freq: Optional[torch.Tensor], rot_dims: int, layout: int = ROTARY_HALF, qk_norm: bool = False,
                            eps: float = 1e-6, v_other: Optional[torch.Tensor] = None, lam: float = 0.0) -> torch.Tensor:
    """q [T, heads * dim], k [T, kv_heads * dim], v [T, kv_heads * vdim] (dense rows of one input product): rotates the first
    ``rot_dims`` numbers of every q and k head at the row's position, optionally brings every q and k head to unit RMS, blends v
    with ``v_other`` ((1 - lam) v + lam v_other), writes k and v into the paged caches k_cache [blocks, block, kv_heads, dim] /
    v_cache [.., vdim] at ``slot_mapping`` and returns the prepared queries [T, heads * dim]."""
    _cuda(q, k, v, k_cache, v_cache, slot_mapping, q_start, ctx_len, seq_of_token, inv_freq, v_other)
    nb, bs, G, d = k_cache.shape
    e = v_cache.shape[3]
    T, S = q.shape[0], q_start.numel()
    _need(v_cache.shape[:3] == (nb, bs, G) and k_cache.is_contiguous() and v_cache.is_contiguous(), "rotary_qk_norm_kv_write: cache shapes")
    _need(q.dim() == 2 and q.shape[1] % d == 0 and k.shape[0] == T and v.shape[0] == T, "rotary_qk_norm_kv_write: q [T, heads * dim]")
    H = q.shape[1] // d
    _need(q.dtype == k.dtype == v.dtype == k_cache.dtype == v_cache.dtype, "rotary_qk_norm_kv_write: one dtype")
    _need(slot_mapping.dtype == torch.int64 and slot_mapping.numel() == T and slot_mapping.is_contiguous(), "rotary_qk_norm_kv_write: slots int64 [T]")
    _i32(q_start, S, "q_start")
    _i32(ctx_len, S, "ctx_len")
    _i32(seq_of_token, T, "seq_of_token")
    _need(rot_dims == 0 or (inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2
                            and inv_freq.is_contiguous()), "rotary_qk_norm_kv_write: inv_freq fp32 [rot_dims / 2]")
    vos = 0
    if v_other is not None:
        _need(v_other.dtype == v.dtype and v_other.shape[0] == T, "rotary_qk_norm_kv_write: v_other [T, kv_heads * vdim]")
        vos = _rows(v_other, G * e, "v_other")
    q_out = torch.empty(T, H * d, dtype=q.dtype, device=q.device)
    check(_lib.mixers_lib().aphro_rotary_qk_norm_kv_write(
        q_out.data_ptr(), H * d, k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(), nb * bs, q.data_ptr(),
        _rows(q, H * d, "q"), k.data_ptr(), _rows(k, G * d, "k"), v.data_ptr(), _rows(v, G * e, "v"), _p(v_other), vos, float(lam),
        q_start.data_ptr(), ctx_len.data_ptr(), seq_of_token.data_ptr(), _p(inv_freq), T, H, G, d, e, int(rot_dims), int(layout),
        1 if qk_norm else 0, float(eps), _dt(q), _stream()), "rotary_qk_norm_kv_write")
    return q_out
