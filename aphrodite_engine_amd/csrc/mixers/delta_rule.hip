// Gated delta rule: per (request slot, head) a matrix state S [dim, vdim] that forgets, corrects what it holds under the key
// towards the new value, and is read AFTER the write:
//     S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
// with k and q made unit vectors per head (x / sqrt(sum x^2 + norm_eps); q times q_scale), beta_t = sigmoid(b_t) and
// g_t = exp(-exp(A_log) * softplus(a_t + dt_bias)) per head.  State, the unit norms, beta, g and every sum are fp32 whatever
// the activations' storage.  Query / key head of value head h: h / (heads / kv_heads).
//
// With r_k = S_old^T k and r_q = S_old^T q (ONE pass over the state, two dot products per column):
//     u = beta (v - g r_k),   S_new = g S_old + k u^T,   o = g r_q + (k . q) u
// so a token costs one read pass and one update pass over the registers that hold the state.
//
// Work split (that of the gated outer-product memories): a workgroup of 256 threads owns 64 -- for prompt portions 16 -- value
// columns of one (segment, head); thread = (column, slice of the key dimension); 16 tokens at a time are staged in LDS, sixteen
// lanes per token, which also make the token's unit norms, k . q, beta and g; the next 16 tokens' raw values are in flight in
// registers meanwhile.  The per-token partial dot products are folded over the slices with DPP moves.
//
// gated_head_rms_norm: out = o / rms(o over the head's vdim) * weight[vdim] * act(gate), one wave per (token, head).
#include "mixers_common.h"

namespace aphro {

constexpr int GDR_CH = 16;

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, int DPT, int SLOG>
__global__ __launch_bounds__(256) void gated_delta_scan_kernel(
    float* __restrict__ out, const typename T::storage* __restrict__ q, int64_t q_stride,
    const typename T::storage* __restrict__ k, int64_t k_stride, const typename T::storage* __restrict__ v, int64_t v_stride,
    const typename T::storage* __restrict__ b, int64_t b_stride, const typename T::storage* __restrict__ a, int64_t a_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ state,
    const int32_t* __restrict__ slot_of_seq, int num_slots, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len, int heads, int kv_heads, int dim, int vdim,
    float q_scale, float norm_eps) {
  constexpr int NS = 1 << SLOG;        // slices of the key dimension = lanes that share a column
  constexpr int TW = 256 >> SLOG;      // value columns per workgroup
  constexpr int DP = NS * DPT;         // key dimension, padded
  constexpr int NQ = (DP + 15) / 16;   // numbers of q (and of k) a staging lane holds: sixteen lanes per token
  constexpr int NV = (GDR_CH * TW + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs[GDR_CH][DP];
  __shared__ __attribute__((aligned(16))) float ks[GDR_CH][DP];
  __shared__ float vs[GDR_CH][TW];
  __shared__ float g_s[GDR_CH], b_s[GDR_CH], kq_s[GDR_CH];
  const int s = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * TW;
  const int hk = h / (heads / kv_heads);
  const int tid = threadIdx.x, c = tid >> SLOG, sl = tid & (NS - 1), col = c0 + c;
  const int n = q_len[s];
  const int slot = slot_of_seq[s];
  if (n <= 0 || slot < 0 || slot >= num_slots) return;
  const int64_t t0 = q_start[s];
  const bool fresh = ctx_len[s] == 0;
  float S[DPT];
  float* sbase = state + ((int64_t)slot * heads + h) * dim * (int64_t)vdim;
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int r = sl * DPT + i;
    S[i] = (!fresh && r < dim && col < vdim) ? sbase[(int64_t)r * vdim + col] : 0.f;
  }
  const float neg_rate = -expf(a_log[h]), dtb = dt_bias[h];
  const int stok = tid >> 4, sln = tid & 15;               // staging: token of the stage, lane within the token

  float rq[NQ], rk[NQ], rv[NV], rb = 0.f, ra = 0.f;
  auto fetch = [&](int base) {
    const int cnt = min(GDR_CH, n - base);
#pragma unroll
    for (int it = 0; it < NQ; ++it) {
      const int r = sln + 16 * it;
      rq[it] = rk[it] = 0.f;
      if (stok < cnt && r < dim) {
        rq[it] = T::to_f32(q[(t0 + base + stok) * q_stride + hk * dim + r]);
        rk[it] = T::to_f32(k[(t0 + base + stok) * k_stride + hk * dim + r]);
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + 256 * it, tt = idx / TW, cc = idx % TW;
      rv[it] = (tt < cnt && c0 + cc < vdim) ? T::to_f32(v[(t0 + base + tt) * v_stride + h * vdim + c0 + cc]) : 0.f;
    }
    if (sln == 0 && stok < cnt) {
      rb = T::to_f32(b[(t0 + base + stok) * b_stride + h]);
      ra = T::to_f32(a[(t0 + base + stok) * a_stride + h]);
    }
  };
  fetch(0);
  for (int base = 0; base < n; base += GDR_CH) {
    const int cnt = min(GDR_CH, n - base);
    __syncthreads();                                        // the previous stage is consumed
    {
      float sq = 0.f, sk = 0.f;
#pragma unroll
      for (int it = 0; it < NQ; ++it) {
        sq += rq[it] * rq[it];
        sk += rk[it] * rk[it];
      }
      sq = group_sum<4>(sq);
      sk = group_sum<4>(sk);
      const float fq = q_scale / sqrtf(sq + norm_eps), fk = 1.0f / sqrtf(sk + norm_eps);
      float kq = 0.f;
#pragma unroll
      for (int it = 0; it < NQ; ++it) {
        const int r = sln + 16 * it;
        const float qv = rq[it] * fq, kv = rk[it] * fk;
        kq += qv * kv;
        if (r < DP) {
          qs[stok][r] = qv;
          ks[stok][r] = kv;
        }
      }
      kq = group_sum<4>(kq);
      if (sln == 0) {
        kq_s[stok] = kq;
        b_s[stok] = sigmoid_f(rb);
        g_s[stok] = expf(neg_rate * softplus_f(ra + dtb));
      }
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int idx = tid + 256 * it;
      if (idx < GDR_CH * TW) vs[idx / TW][idx % TW] = rv[it];
    }
    __syncthreads();
    if (base + GDR_CH < n) fetch(base + GDR_CH);
#pragma unroll 2
    for (int tt = 0; tt < cnt; ++tt) {
      const float g = g_s[tt], beta = b_s[tt], kq = kq_s[tt];
      float pk[4] = {0.f, 0.f, 0.f, 0.f}, pq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < DPT; i4 += 4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(&ks[tt][sl * DPT + i4]);
        const f32x4 qq = *reinterpret_cast<const f32x4*>(&qs[tt][sl * DPT + i4]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pk[e] += S[i4 + e] * kk[e];
          pq[e] += S[i4 + e] * qq[e];
        }
      }
      const float rk_ = group_sum<SLOG>((pk[0] + pk[1]) + (pk[2] + pk[3]));
      const float rq_ = group_sum<SLOG>((pq[0] + pq[1]) + (pq[2] + pq[3]));
      const float u = beta * (vs[tt][c] - g * rk_);
#pragma unroll
      for (int i4 = 0; i4 < DPT; i4 += 4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(&ks[tt][sl * DPT + i4]);
#pragma unroll
        for (int e = 0; e < 4; ++e) S[i4 + e] = g * S[i4 + e] + kk[e] * u;
      }
      if (sl == 0 && col < vdim) out[(t0 + base + tt) * ((int64_t)heads * vdim) + h * vdim + col] = g * rq_ + kq * u;
    }
  }
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int r = sl * DPT + i;
    if (r < dim && col < vdim) sbase[(int64_t)r * vdim + col] = S[i];
  }
}

// act: 0 sigmoid(gate), 1 silu(gate); gate NULL: none.  weight [vdim] is shared by the heads (NULL: ones).
template <typename T>
__global__ __launch_bounds__(256) void gated_head_rms_norm_kernel(typename T::storage* __restrict__ out, int64_t out_stride,
                                                                  const float* __restrict__ x, const typename T::storage* __restrict__ weight,
                                                                  const typename T::storage* __restrict__ gate, int64_t gate_stride,
                                                                  int64_t num_tokens, int heads, int vdim, float eps, int act) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= num_tokens * heads) return;
  const int64_t t = unit / heads;
  const int h = (int)(unit - t * heads);
  const float* xr = x + (t * heads + h) * (int64_t)vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += 64) ss += xr[i] * xr[i];
  const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  for (int i = lane; i < vdim; i += 64) {
    float val = xr[i] * rstd;
    if (weight) val *= T::to_f32(weight[i]);
    if (gate) {
      const float gv = T::to_f32(gate[t * gate_stride + (int64_t)h * vdim + i]);
      val *= act == 1 ? silu_f(gv) : sigmoid_f(gv);
    }
    out[t * out_stride + (int64_t)h * vdim + i] = T::from_f32(val);
  }
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_gated_delta_scan(float* out, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                      int64_t v_stride, const void* b, int64_t b_stride, const void* a, int64_t a_stride,
                                      const float* a_log, const float* dt_bias, float* state, const int32_t* slot_of_seq,
                                      int num_slots, const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                                      int num_seqs, int64_t num_tokens, int heads, int kv_heads, int dim, int vdim, float q_scale,
                                      float norm_eps, int max_q_len, int dtype, void* stream) {
  if (num_tokens == 0 || num_seqs == 0) return APHRO_OK;
  APHRO_CHECK(out && q && k && v && b && a && a_log && dt_bias && state && slot_of_seq && q_start && q_len && ctx_len,
              "gated_delta_scan: null argument");
  APHRO_CHECK(heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 256 && vdim > 0 &&
                  vdim <= 16 * 65535 && num_slots > 0,
              "gated_delta_scan: heads %d over %d key heads, dim %d (<= 256), vdim %d", heads, kv_heads, dim, vdim);
  APHRO_CHECK(q_stride >= (int64_t)kv_heads * dim && k_stride >= (int64_t)kv_heads * dim && v_stride >= (int64_t)heads * vdim &&
                  b_stride >= heads && a_stride >= heads, "gated_delta_scan: row strides smaller than the rows");
  const bool wide = max_q_len >= 32;
  const int tw = wide ? 16 : 64;
  const dim3 grid((unsigned)num_seqs, (unsigned)heads, (unsigned)((vdim + tw - 1) / tw));
#define GDR_LAUNCH(DPT, SLOG)                                                                                                  \
  hipLaunchKernelGGL((gated_delta_scan_kernel<T, DPT, SLOG>), grid, dim3(256), 0, (hipStream_t)stream, out, (const S*)q, q_stride, \
                     (const S*)k, k_stride, (const S*)v, v_stride, (const S*)b, b_stride, (const S*)a, a_stride, a_log, dt_bias,  \
                     state, slot_of_seq, num_slots, q_start, q_len, ctx_len, heads, kv_heads, dim, vdim, q_scale, norm_eps)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (wide) {
      if (dim <= 64) GDR_LAUNCH(4, 4);
      else if (dim <= 128) GDR_LAUNCH(8, 4);
      else GDR_LAUNCH(16, 4);
    } else if (dim <= 32) GDR_LAUNCH(8, 2);
    else if (dim <= 64) GDR_LAUNCH(16, 2);
    else if (dim <= 128) GDR_LAUNCH(32, 2);
    else GDR_LAUNCH(64, 2);
  });
#undef GDR_LAUNCH
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_gated_head_rms_norm(void* out, int64_t out_stride, const float* x, const void* weight, const void* gate,
                                         int64_t gate_stride, int64_t num_tokens, int heads, int vdim, float eps, int act, int dtype,
                                         void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && x && heads > 0 && vdim > 0 && out_stride >= (int64_t)heads * vdim && (!gate || gate_stride >= (int64_t)heads * vdim) &&
                  (act == 0 || act == 1), "gated_head_rms_norm: bad arguments (%d heads of %d)", heads, vdim);
  const int64_t units = num_tokens * heads;
  APHRO_CHECK((units + 3) / 4 <= 0x7fffffff, "gated_head_rms_norm: too many rows");
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((gated_head_rms_norm_kernel<T>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, (hipStream_t)stream, (S*)out,
                       out_stride, x, (const S*)weight, (const S*)gate, gate_stride, num_tokens, heads, vdim, eps, act);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
