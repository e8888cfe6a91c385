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

template <typename T>
__device__ __forceinline__ void rp_load8(const typename T::storage* p, float* o) {
  if constexpr (sizeof(typename T::storage) == 2) {
    const u16x8 v = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = T::to_f32(v[j]);
  } else {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[j] = a[j];
      o[4 + j] = b[j];
    }
  }
}
template <typename T>
__device__ __forceinline__ void rp_store8(typename T::storage* p, const float* v) {
  if constexpr (sizeof(typename T::storage) == 2) {
    u16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = T::from_f32(v[j]);
    *reinterpret_cast<u16x8*>(p) = r;
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
}

// The same for head sizes that are multiples of 8 with 16-byte-aligned rows: a thread owns 8 neighbouring numbers of one unit,
// tph (a power of two, <= 64) threads share a unit, a wave holds 64 / tph units; the rotation partner of a chunk is the chunk
// half the rotated part away (layout 0: rot_dims / 2 is a multiple of 8) or lies within the chunk (layout 1).
template <typename T>
__global__ __launch_bounds__(256) void rotary_qk_norm_kv_write_vec8_kernel(
    typename T::storage* __restrict__ q_out, int64_t q_out_stride, typename T::storage* __restrict__ k_cache,
    typename T::storage* __restrict__ v_cache, const int64_t* __restrict__ slot_mapping, int64_t num_cache_rows,
    const typename T::storage* __restrict__ q, int64_t q_stride, const typename T::storage* __restrict__ k, int64_t k_stride,
    const typename T::storage* __restrict__ v, int64_t v_stride, const typename T::storage* __restrict__ v_other,
    int64_t v_other_stride, float lambda, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ seq_of_token, const float* __restrict__ inv_freq, int heads, int kv_heads, int dim, int vdim,
    int rot_dims, int layout, int qk_norm, float eps, int tph) {
  const int64_t t = blockIdx.x;
  const int per_block = 256 / tph;
  const int unit = blockIdx.y * per_block + threadIdx.x / tph, i0 = 8 * (threadIdx.x % tph);
  const bool live = unit < heads + 2 * kv_heads;          // every lane stays for the shuffles below
  const int64_t slot = slot_mapping[t];
  const bool cached = slot >= 0 && slot < num_cache_rows;
  if (live && unit >= heads + kv_heads) {                   // a value head
    const int g = unit - heads - kv_heads;
    if (cached && i0 < vdim) {
      float x[8];
      rp_load8<T>(v + t * v_stride + (int64_t)g * vdim + i0, x);
      if (v_other) {
        float o[8];
        rp_load8<T>(v_other + t * v_other_stride + (int64_t)g * vdim + i0, o);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (1.0f - lambda) * x[e] + lambda * o[e];
      }
      rp_store8<T>(v_cache + (slot * kv_heads + g) * (int64_t)vdim + i0, x);
    }
  }
  const bool qk = live && unit < heads + kv_heads;
  const bool is_q = unit < heads;
  const int hd = is_q ? unit : unit - heads;
  const bool work = qk && i0 < dim && (is_q || cached);
  float x[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = 0.f;
  if (work) {
    const typename T::storage* src = is_q ? q + t * q_stride + (int64_t)hd * dim : k + t * k_stride + (int64_t)hd * dim;
    rp_load8<T>(src + i0, x);
    if (i0 < rot_dims) {
      const int s = seq_of_token[t];
      const float pos = (float)(ctx_len[s] + (int)(t - q_start[s]));
      const int half = rot_dims >> 1;
      if (layout == 0) {
        const bool first = i0 < half;
        float o[8];
        rp_load8<T>(src + (first ? i0 + half : i0 - half), o);
        const int f0 = first ? i0 : i0 - half;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float c, sn;
          sincosf(pos * inv_freq[f0 + e], &sn, &c);
          x[e] = first ? x[e] * c - o[e] * sn : x[e] * c + o[e] * sn;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          float c, sn;
          sincosf(pos * inv_freq[(i0 + e) >> 1], &sn, &c);
          const float a = x[e], b = x[e + 1];
          x[e] = a * c - b * sn;
          x[e + 1] = b * c + a * sn;
        }
      }
    }
  }
  float f = 1.0f;
  if (qk_norm) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
    for (int o = tph >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    f = 1.0f / sqrtf(ss / (float)dim + eps);
  }
  if (work) {
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] *= f;
    typename T::storage* dst = is_q ? q_out + t * q_out_stride + (int64_t)hd * dim : k_cache + (slot * kv_heads + hd) * (int64_t)dim;
    rp_store8<T>(dst + i0, x);
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
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  int tph = 1;
  while (8 * tph < (dim > vdim ? dim : vdim)) tph *= 2;
  const bool vec = dim % 8 == 0 && vdim % 8 == 0 && tph <= 64 && (layout == 1 || (rot_dims / 2) % 8 == 0) && rot_dims % 8 == 0 &&
                   q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 && q_out_stride % 8 == 0 && v_other_stride % 8 == 0 &&
                   al16(q) && al16(k) && al16(v) && al16(v_other) && al16(q_out) && al16(k_cache) && al16(v_cache);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec) {
      const int per_block = 256 / tph;
      hipLaunchKernelGGL((rotary_qk_norm_kv_write_vec8_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((units + per_block - 1) / per_block)),
                         dim3(256), 0, (hipStream_t)stream, (S*)q_out, q_out_stride, (S*)k_cache, (S*)v_cache, slot_mapping, num_cache_rows,
                         (const S*)q, q_stride, (const S*)k, k_stride, (const S*)v, v_stride, (const S*)v_other, v_other_stride, lambda,
                         q_start, ctx_len, seq_of_token, inv_freq, heads, kv_heads, dim, vdim, rot_dims, layout, qk_norm, eps, tph);
    } else
    hipLaunchKernelGGL((rotary_qk_norm_kv_write_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((units + 3) / 4)), dim3(256), 0,
                       (hipStream_t)stream, (S*)q_out, q_out_stride, (S*)k_cache, (S*)v_cache, slot_mapping, num_cache_rows, (const S*)q,
                       q_stride, (const S*)k, k_stride, (const S*)v, v_stride, (const S*)v_other, v_other_stride, lambda, q_start,
                       ctx_len, seq_of_token, inv_freq, heads, kv_heads, dim, vdim, rot_dims, layout, qk_norm, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
