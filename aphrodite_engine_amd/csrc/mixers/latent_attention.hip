// Softmax attention through a low-rank latent: a token leaves ONE row in the paged cache, [c | k_r] -- its normed latent c
// (rank R) and one rotated key part k_r (P numbers) shared by all heads.  A head's key is [W_uk c | k_r] and its value W_uv c, so
//   score_ij = (q_n . W_uk c_j + q_r . k_r,j) * scale = ([W_uk^T q_n | q_r] . [c_j | k_r,j]) * scale
//   o_i      = W_uv sum_j p_ij c_j
// and the kernels here run in the latent: every head's query arrives as q_lat = W_uk^T q_n (rank R, a product the caller
// makes) beside its raw rotary part, all heads read the same cache rows, and the result is sum_j p_ij c_j per head (the
// caller applies W_uv).  Nothing per head is ever stored per token.
//
//   latent_prep        per token: RMS norm of the query latent -> [T, q_rank]; RMS norm of the key/value latent and the rotation
//                      of the shared key part at the token's position -> the cache row at its slot
//   latent_attention   any sizes, fp32 math: a workgroup of four waves per (row, head); lane = key for the scores, lane =
//                      column for P C; rotates the query's rotary part on load; optional sliding window (row i sees key j
//                      with 0 <= i - j < window) and per-head sink (exp(sink) joins the softmax denominator, unscaled)
//   sigmoid_gate_mul   out = x * sigmoid(gate), elementwise
// Rotation ("rotate half" over the first rot_dims numbers of the rotary part): the pair (u, v) = (x[i], x[i + rot_dims / 2])
// becomes (u cos a - v sin a, v cos a + u sin a) * mscale with a = position * inv_freq[i], all in fp32.
#include "mixers_common.h"

namespace aphro {

constexpr int LA_WAVES = 4;
constexpr int LA_MAX_DIM = 2048;        // R + P
constexpr int LA_MAX_EPL = 16;          // R <= 1024

template <typename T>
__global__ void latent_prep_kernel(typename T::storage* __restrict__ cq, typename T::storage* __restrict__ cache,
                                   const typename T::storage* __restrict__ proj, int64_t proj_stride, int q_at, int kv_at,
                                   const typename T::storage* __restrict__ wq, const typename T::storage* __restrict__ wkv,
                                   const int64_t* __restrict__ slot_mapping, int64_t num_cache_rows,
                                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
                                   const int32_t* __restrict__ seq_of_token, const float* __restrict__ inv_freq, float mscale,
                                   int q_rank, int kv_rank, int rot_dim, int rot_dims, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const typename T::storage* row = proj + t * proj_stride;
  float ssq = 0.f, ss = 0.f;                                  // both statistics are gathered before either is waited for
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = T::to_f32(row[q_at + i]);
    ssq += v * v;
  }
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = T::to_f32(row[kv_at + i]);
    ss += v * v;
  }
  if (q_rank > 0) {
    const float rstd = 1.0f / sqrtf(wg_sum(ssq, red) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
      cq[t * (int64_t)q_rank + i] = T::from_f32(T::to_f32(row[q_at + i]) * rstd * T::to_f32(wq[i]));
  }
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= num_cache_rows) return;             // a padded row
  typename T::storage* dst = cache + slot * (int64_t)(kv_rank + rot_dim);
  const float rstd = 1.0f / sqrtf(wg_sum(ss, red) / (float)kv_rank + eps);
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x)
    dst[i] = T::from_f32(T::to_f32(row[kv_at + i]) * rstd * T::to_f32(wkv[i]));
  const int s = seq_of_token[t];
  const float pos = (float)(ctx_len[s] + (int)(t - q_start[s]));
  const int half = rot_dims >> 1;
  const typename T::storage* kr = row + kv_at + kv_rank;
  for (int i = threadIdx.x; i < rot_dim; i += blockDim.x) {
    float v = T::to_f32(kr[i]);
    if (i < 2 * half) {
      const int f = i < half ? i : i - half;
      float c, sn;
      sincosf(pos * inv_freq[f], &sn, &c);
      c *= mscale;
      sn *= mscale;
      const float other = T::to_f32(kr[i < half ? i + half : i - half]);
      v = i < half ? v * c - other * sn : v * c + other * sn;
    }
    dst[kv_rank + i] = T::from_f32(v);
  }
}

template <typename T>
__device__ __forceinline__ float la_dot(const float* __restrict__ qsh, const typename T::storage* __restrict__ kr, int dim) {
  float d0 = 0.f, d1 = 0.f;
  if constexpr (sizeof(typename T::storage) == 2) {
    if ((dim & 7) == 0) {
      for (int i = 0; i < dim; i += 8) {
        const u16x8 kk = *reinterpret_cast<const u16x8*>(kr + i);
        const f32x4 qa = *reinterpret_cast<const f32x4*>(qsh + i), qb = *reinterpret_cast<const f32x4*>(qsh + i + 4);
        d0 += qa[0] * T::to_f32(kk[0]) + qa[1] * T::to_f32(kk[1]) + qa[2] * T::to_f32(kk[2]) + qa[3] * T::to_f32(kk[3]);
        d1 += qb[0] * T::to_f32(kk[4]) + qb[1] * T::to_f32(kk[5]) + qb[2] * T::to_f32(kk[6]) + qb[3] * T::to_f32(kk[7]);
      }
      return d0 + d1;
    }
  } else {
    if ((dim & 3) == 0) {
      for (int i = 0; i < dim; i += 4) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(kr + i);
        const f32x4 qa = *reinterpret_cast<const f32x4*>(qsh + i);
        d0 += qa[0] * kk[0] + qa[1] * kk[1];
        d1 += qa[2] * kk[2] + qa[3] * kk[3];
      }
      return d0 + d1;
    }
  }
  for (int i = 0; i < dim; ++i) d0 += qsh[i] * T::to_f32(kr[i]);
  return d0;
}

template <typename T, int EPL>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    typename T::storage* __restrict__ out, int64_t out_stride, int64_t out_head_stride,
    const typename T::storage* __restrict__ q_lat, int64_t ql_stride, int64_t ql_head_stride,
    const typename T::storage* __restrict__ q_rot, int64_t qr_stride, int64_t qr_head_stride,
    const typename T::storage* __restrict__ cache, const int32_t* __restrict__ block_tables, int max_blocks, int64_t num_blocks,
    int block_size, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ seq_of_token, const float* __restrict__ inv_freq, float mscale, int kv_rank, int rot_dim,
    int rot_dims, float scale, int window, const float* __restrict__ sink) {
  __shared__ __attribute__((aligned(16))) float qsh[LA_MAX_DIM];
  __shared__ float merge[LA_WAVES][2 + EPL * 64];
  const int t = blockIdx.x, h = blockIdx.y;
  const int s = seq_of_token[t];
  const int pos = ctx_len[s] + (t - q_start[s]);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int dim = kv_rank + rot_dim;
  const typename T::storage* ql = q_lat + (int64_t)t * ql_stride + (int64_t)h * ql_head_stride;
  const typename T::storage* qr = q_rot + (int64_t)t * qr_stride + (int64_t)h * qr_head_stride;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) qsh[i] = T::to_f32(ql[i]);
  const int half = rot_dims >> 1;
  for (int i = threadIdx.x; i < rot_dim; i += blockDim.x) {
    float v = T::to_f32(qr[i]);
    if (i < 2 * half) {
      const int f = i < half ? i : i - half;
      float c, sn;
      sincosf((float)pos * inv_freq[f], &sn, &c);
      c *= mscale;
      sn *= mscale;
      const float other = T::to_f32(qr[i < half ? i + half : i - half]);
      v = i < half ? v * c - other * sn : v * c + other * sn;
    }
    qsh[kv_rank + i] = v;
  }
  __syncthreads();
  const int32_t* bt = block_tables + (int64_t)s * max_blocks;
  float m = -INFINITY, l = 0.f, acc[EPL];
#pragma unroll
  for (int c = 0; c < EPL; ++c) acc[c] = 0.f;
  const int n = pos + 1;
  const int first = window > 0 ? max(0, n - window) : 0;     // the oldest key the row sees
  const int ntiles = (n + 63) >> 6;
  for (int tile = (first >> 6) + wave; tile < ntiles; tile += LA_WAVES) {
    const int j = tile * 64 + lane;
    float sc = -INFINITY;
    if (j < n && j >= first) {
      const int blk = bt[j / block_size];
      if (blk >= 0 && blk < num_blocks) sc = la_dot<T>(qsh, cache + ((int64_t)blk * block_size + j % block_size) * dim, dim) * scale;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    const float p = (sc == -INFINITY) ? 0.f : expf(sc - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < EPL; ++c) acc[c] *= alpha;
    const int cnt = min(64, n - tile * 64);
#pragma unroll 4
    for (int jj = max(0, first - tile * 64); jj < cnt; ++jj) {
      const float pj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), jj));
      const int j2 = tile * 64 + jj;
      int blk = bt[j2 / block_size];
      if (blk < 0 || blk >= num_blocks) blk = 0;           // its probability is 0
      const typename T::storage* vr = cache + ((int64_t)blk * block_size + j2 % block_size) * dim;
#pragma unroll
      for (int c = 0; c < EPL; ++c) {
        const int col = lane + 64 * c;
        if (col < kv_rank) acc[c] += pj * T::to_f32(vr[col]);
      }
    }
  }
  if (lane == 0) {
    merge[wave][0] = m;
    merge[wave][1] = l;
  }
#pragma unroll
  for (int c = 0; c < EPL; ++c) merge[wave][2 + lane + 64 * c] = acc[c];
  __syncthreads();
  if (wave != 0) return;
  float M = sink ? sink[h] : -INFINITY;                      // the sink: one more term of the denominator, no value
#pragma unroll
  for (int w = 0; w < LA_WAVES; ++w) M = fmaxf(M, merge[w][0]);
  float L = sink ? expf(sink[h] - M) : 0.f, f[LA_WAVES];
#pragma unroll
  for (int w = 0; w < LA_WAVES; ++w) {
    f[w] = (merge[w][0] == -INFINITY) ? 0.f : expf(merge[w][0] - M);
    L += merge[w][1] * f[w];
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int c = 0; c < EPL; ++c) {
    const int col = lane + 64 * c;
    if (col < kv_rank) {
      float o = 0.f;
#pragma unroll
      for (int w = 0; w < LA_WAVES; ++w) o += merge[w][2 + col] * f[w];
      out[(int64_t)t * out_stride + (int64_t)h * out_head_stride + col] = T::from_f32(o * inv);
    }
  }
}

template <typename T>
__global__ void sigmoid_gate_mul_kernel(typename T::storage* __restrict__ out, int64_t out_stride,
                                        const typename T::storage* __restrict__ x, int64_t x_stride,
                                        const typename T::storage* __restrict__ gate, int64_t gate_stride, int n) {
  const int64_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= n) return;
  out[t * out_stride + i] = T::from_f32(T::to_f32(x[t * x_stride + i]) * sigmoid_f(T::to_f32(gate[t * gate_stride + i])));
}

template <typename T>
__global__ void sigmoid_gate_mul_vec8_kernel(typename T::storage* __restrict__ out, int64_t out_stride,
                                             const typename T::storage* __restrict__ x, int64_t x_stride,
                                             const typename T::storage* __restrict__ gate, int64_t gate_stride, int n) {
  const int64_t t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= n) return;
  if constexpr (sizeof(typename T::storage) == 2) {
    const u16x8 xv = *reinterpret_cast<const u16x8*>(x + t * x_stride + i), gv = *reinterpret_cast<const u16x8*>(gate + t * gate_stride + i);
    u16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = T::from_f32(T::to_f32(xv[j]) * sigmoid_f(T::to_f32(gv[j])));
    *reinterpret_cast<u16x8*>(out + t * out_stride + i) = r;
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const f32x4 xv = *reinterpret_cast<const f32x4*>(x + t * x_stride + i + 4 * h);
      const f32x4 gv = *reinterpret_cast<const f32x4*>(gate + t * gate_stride + i + 4 * h);
      f32x4 r;
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = xv[j] * sigmoid_f(gv[j]);
      *reinterpret_cast<f32x4*>(out + t * out_stride + i + 4 * h) = r;
    }
  }
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_latent_prep(void* cq, void* cache, int64_t num_cache_rows, const void* proj, int64_t proj_stride, int q_at,
                                 int kv_at, const void* wq, const void* wkv, const int64_t* slot_mapping, const int32_t* q_start,
                                 const int32_t* ctx_len, const int32_t* seq_of_token, const float* inv_freq, float mscale,
                                 int64_t num_tokens, int q_rank, int kv_rank, int rot_dim, int rot_dims, float eps, int dtype,
                                 void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(cache && proj && wkv && slot_mapping && q_start && ctx_len && seq_of_token && (rot_dims == 0 || inv_freq),
              "latent_prep: null argument");
  APHRO_CHECK(q_rank >= 0 && (q_rank == 0 || (cq && wq)), "latent_prep: a query latent needs its output and weight");
  APHRO_CHECK(kv_rank > 0 && rot_dim >= 0 && rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0,
              "latent_prep: rank %d, rotary part %d of which %d rotate", kv_rank, rot_dim, rot_dims);
  APHRO_CHECK(q_at >= 0 && kv_at >= 0 && proj_stride >= q_at + q_rank && proj_stride >= kv_at + kv_rank + rot_dim,
              "latent_prep: the projection's rows do not hold the latents");
  const int widest = q_rank > kv_rank ? q_rank : kv_rank;
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((latent_prep_kernel<T>), dim3((unsigned)num_tokens), dim3(widest >= 1024 ? 256 : (widest > 256 ? 128 : 64)), 0,
                       (hipStream_t)stream, (S*)cq, (S*)cache, (const S*)proj, proj_stride, q_at, kv_at, (const S*)wq,
                       (const S*)wkv, slot_mapping, num_cache_rows, q_start, ctx_len, seq_of_token, inv_freq, mscale, q_rank, kv_rank,
                       rot_dim, rot_dims, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_latent_attention_plain(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_lat,
                                            int64_t ql_stride, int64_t ql_head_stride, const void* q_rot, int64_t qr_stride,
                                            int64_t qr_head_stride, const void* cache, const int32_t* block_tables, int max_blocks,
                                            int64_t num_blocks, int block_size, const int32_t* q_start, const int32_t* ctx_len,
                                            const int32_t* seq_of_token, const float* inv_freq, float mscale, int64_t num_tokens,
                                            int heads, int kv_rank, int rot_dim, int rot_dims, float scale, int window,
                                            const float* sink, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && q_lat && (q_rot || rot_dim == 0) && cache && block_tables && q_start && ctx_len && seq_of_token &&
                  (rot_dims == 0 || inv_freq), "latent_attention: null argument");
  APHRO_CHECK(heads > 0 && heads <= 65535 && kv_rank > 0 && kv_rank <= 64 * LA_MAX_EPL && rot_dim >= 0 &&
                  kv_rank + rot_dim <= LA_MAX_DIM && rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0,
              "latent_attention: %d heads, rank %d (<= %d), rotary part %d of which %d rotate", heads, kv_rank, 64 * LA_MAX_EPL,
              rot_dim, rot_dims);
  APHRO_CHECK(block_size > 0 && max_blocks > 0 && num_blocks > 0, "latent_attention: bad cache geometry");
  const dim3 grid((unsigned)num_tokens, (unsigned)heads);
  const int epl = (kv_rank + 63) / 64;
#define LA_LAUNCH(EPL)                                                                                                         \
  hipLaunchKernelGGL((latent_attention_kernel<T, EPL>), grid, dim3(256), 0, (hipStream_t)stream, (S*)out, out_stride,           \
                     out_head_stride, (const S*)q_lat, ql_stride, ql_head_stride, (const S*)q_rot, qr_stride, qr_head_stride,   \
                     (const S*)cache, block_tables, max_blocks, num_blocks, block_size, q_start, ctx_len, seq_of_token, inv_freq, \
                     mscale, kv_rank, rot_dim, rot_dims, scale, window, sink)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    switch (epl) {
      case 1: LA_LAUNCH(1); break;
      case 2: LA_LAUNCH(2); break;
      case 3: LA_LAUNCH(3); break;
      case 4: LA_LAUNCH(4); break;
      case 5: case 6: LA_LAUNCH(6); break;
      case 7: case 8: LA_LAUNCH(8); break;
      case 9: case 10: case 11: case 12: LA_LAUNCH(12); break;
      default: LA_LAUNCH(16); break;
    }
  });
#undef LA_LAUNCH
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_sigmoid_gate_mul(void* out, int64_t out_stride, const void* x, int64_t x_stride, const void* gate,
                                      int64_t gate_stride, int64_t num_tokens, int n, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && x && gate && n > 0 && out_stride >= n && x_stride >= n && gate_stride >= n && (n + 255) / 256 <= 65535,
              "sigmoid_gate_mul: bad arguments");
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool vec = n % 8 == 0 && out_stride % 8 == 0 && x_stride % 8 == 0 && gate_stride % 8 == 0 && al16(out) && al16(x) && al16(gate);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec)
      hipLaunchKernelGGL((sigmoid_gate_mul_vec8_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((n / 8 + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, (S*)out, out_stride, (const S*)x, x_stride, (const S*)gate, gate_stride, n);
    else
      hipLaunchKernelGGL((sigmoid_gate_mul_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((n + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, (S*)out, out_stride, (const S*)x, x_stride, (const S*)gate, gate_stride, n);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
