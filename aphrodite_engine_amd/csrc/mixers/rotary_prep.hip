// What happens between the input product [q | k | v] of a rotary grouped-query attention and its paged cache, in one launch:
//   * the first rot_dims numbers of every query and key head are turned by position * inv_freq[i] -- layout 0 pairs number i
//     with number i + rot_dims / 2 ("rotate half"), layout 1 pairs number 2 i with number 2 i + 1 (interleaved); the pair
//     (u, v) becomes (u cos a - v sin a, v cos a + u sin a); the rest of the head passes unchanged;
//   * optionally every query and key head is then divided by its root mean square over the head (a norm without a weight);
//   * optionally the values are blended with another tensor's values of the same tokens, v <- (1 - lambda) v + lambda v_other;
//   * queries go to a dense output, keys and values into the token-major paged caches at the rows' slots.
// Positions, angles, cos / sin, the statistics and the blend are fp32; one rounding to the storage type.
// One wave per (token, unit): units are the query heads, then the key heads, then the value heads.
#include "mixers_common.h"

namespace aphro {

template <typename T>
__global__ __launch_bounds__(256) void rotary_qk_norm_kv_write_kernel(
    typename T::storage* __restrict__ q_out, int64_t q_out_stride, typename T::storage* __restrict__ k_cache,
    typename T::storage* __restrict__ v_cache, const int64_t* __restrict__ slot_mapping, int64_t num_cache_rows,
    const typename T::storage* __restrict__ q, int64_t q_stride, const typename T::storage* __restrict__ k, int64_t k_stride,
    const typename T::storage* __restrict__ v, int64_t v_stride, const typename T::storage* __restrict__ v_other,
    int64_t v_other_stride, float lambda, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ seq_of_token, const float* __restrict__ inv_freq, int heads, int kv_heads, int dim, int vdim,
    int rot_dims, int layout, int qk_norm, float eps) {
  const int64_t t = blockIdx.x;
  const int unit = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= heads + 2 * kv_heads) return;
  const int64_t slot = slot_mapping[t];
  const bool cached = slot >= 0 && slot < num_cache_rows;
  if (unit >= heads + kv_heads) {                            // a value head
    if (!cached) return;
    const int g = unit - heads - kv_heads;
    const typename T::storage* src = v + t * v_stride + (int64_t)g * vdim;
    typename T::storage* dst = v_cache + (slot * kv_heads + g) * (int64_t)vdim;
    for (int i = lane; i < vdim; i += 64) {
      float x = T::to_f32(src[i]);
      if (v_other) x = (1.0f - lambda) * x + lambda * T::to_f32(v_other[t * v_other_stride + (int64_t)g * vdim + i]);
      dst[i] = T::from_f32(x);
    }
    return;
  }
  const bool is_q = unit < heads;
  if (!is_q && !cached) return;
  const int hd = is_q ? unit : unit - heads;
  const typename T::storage* src = is_q ? q + t * q_stride + (int64_t)hd * dim : k + t * k_stride + (int64_t)hd * dim;
  typename T::storage* dst = is_q ? q_out + t * q_out_stride + (int64_t)hd * dim : k_cache + (slot * kv_heads + hd) * (int64_t)dim;
  const int s = seq_of_token[t];
  const float pos = (float)(ctx_len[s] + (int)(t - q_start[s]));
  const int half = rot_dims >> 1;
  constexpr int MAXE = 8;                                    // dim <= 512
  float val[MAXE];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < MAXE; ++e) {
    const int i = lane + 64 * e;
    float x = 0.f;
    if (i < dim) {
      x = T::to_f32(src[i]);
      if (i < 2 * half) {
        int f, partner;
        bool first;
        if (layout == 0) {
          first = i < half;
          f = first ? i : i - half;
          partner = first ? i + half : i - half;
        } else {
          first = (i & 1) == 0;
          f = i >> 1;
          partner = i ^ 1;
        }
        float c, sn;
        sincosf(pos * inv_freq[f], &sn, &c);
        const float other = T::to_f32(src[partner]);
        x = first ? x * c - other * sn : x * c + other * sn;
      }
    }
    val[e] = x;
    ss += x * x;
  }
  float f = 1.0f;
  if (qk_norm) f = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
#pragma unroll
  for (int e = 0; e < MAXE; ++e) {
    const int i = lane + 64 * e;
    if (i < dim) dst[i] = T::from_f32(val[e] * f);
  }
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_rotary_qk_norm_kv_write(void* q_out, int64_t q_out_stride, void* k_cache, void* v_cache, const int64_t* slot_mapping,
                                             int64_t num_cache_rows, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                             const void* v, int64_t v_stride, const void* v_other, int64_t v_other_stride, float lambda,
                                             const int32_t* q_start, const int32_t* ctx_len, const int32_t* seq_of_token,
                                             const float* inv_freq, int64_t num_tokens, int heads, int kv_heads, int dim, int vdim,
                                             int rot_dims, int layout, int qk_norm, float eps, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(q_out && k_cache && v_cache && slot_mapping && q && k && v && q_start && ctx_len && seq_of_token && (rot_dims == 0 || inv_freq),
              "rotary_qk_norm_kv_write: null argument");
  APHRO_CHECK(heads > 0 && kv_heads > 0 && dim > 0 && dim <= 512 && vdim > 0 && rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 &&
                  (layout == 0 || layout == 1) && heads + 2 * kv_heads <= 4 * 65535,
              "rotary_qk_norm_kv_write: %d / %d heads of %d (<= 512) and %d, %d numbers rotate", heads, kv_heads, dim, vdim, rot_dims);
  APHRO_CHECK(q_stride >= (int64_t)heads * dim && q_out_stride >= (int64_t)heads * dim && k_stride >= (int64_t)kv_heads * dim &&
                  v_stride >= (int64_t)kv_heads * vdim && (!v_other || v_other_stride >= (int64_t)kv_heads * vdim) && num_cache_rows > 0,
              "rotary_qk_norm_kv_write: row strides smaller than the rows");
  const int units = heads + 2 * kv_heads;
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((rotary_qk_norm_kv_write_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((units + 3) / 4)), dim3(256), 0,
                       (hipStream_t)stream, (S*)q_out, q_out_stride, (S*)k_cache, (S*)v_cache, slot_mapping, num_cache_rows, (const S*)q,
                       q_stride, (const S*)k, k_stride, (const S*)v, v_stride, (const S*)v_other, v_other_stride, lambda, q_start,
                       ctx_len, seq_of_token, inv_freq, heads, kv_heads, dim, vdim, rot_dims, layout, qk_norm, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
