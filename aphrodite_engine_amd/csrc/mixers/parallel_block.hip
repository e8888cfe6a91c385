// Launches of a decoder whose sublayers run side by side on one normed input, around an fp32 residual stream:
//   * hashed_pair_embed: x = table[token] + pair_table[hash(previous token, token)] -- the pair row is
//     (previous * mul_prev + token * mul_cur) mod buckets, row `buckets` for a sequence's first token; the previous token of a
//     segment's first row comes from the request's state slot (token_state), which token_state_write advances afterwards;
//   * residual_add2_rms_norm: x += y_a + y_b + bias (the results of the sublayers that read the same normed input), then the
//     RMS norm with a per-channel weight that feeds the next layer -- one launch.
// fp32 math whatever the storage type.  Rows that are a multiple of 8 elements and 16-byte aligned are held in registers
// (8 elements per thread); any other width goes through an LDS row.
#include "mixers_common.h"

namespace aphro {

template <typename T>
__device__ __forceinline__ void pb_load8(const typename T::storage* p, float* o) {
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
__device__ __forceinline__ void pb_store8(typename T::storage* p, const float* v) {
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

// one workgroup per row
template <typename T>
__global__ void hashed_pair_embed_kernel(float* __restrict__ x, const typename T::storage* __restrict__ table,
                                         const typename T::storage* __restrict__ pair_table, const int64_t* __restrict__ ids,
                                         const int32_t* __restrict__ token_state, const int32_t* __restrict__ state_slots,
                                         const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
                                         const int32_t* __restrict__ seq_of_token, int width, int64_t vocab, int64_t buckets,
                                         int64_t mul_prev, int64_t mul_cur) {
  const int64_t t = blockIdx.x;
  const int s = seq_of_token[t];
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;
  int64_t row = buckets;
  const int64_t first = q_start[s];
  if (t > first) {
    row = -1 - ids[t - 1];                       // marks "previous token known": hashed below
  } else if (ctx_len[s] > 0) {
    row = -1 - (int64_t)token_state[state_slots[s]];
  }
  if (row < 0) {
    const int64_t prev = -1 - row;
    row = (prev * mul_prev + id * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const typename T::storage* a = table + id * (int64_t)width;
  const typename T::storage* b = pair_table + row * (int64_t)width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) x[t * (int64_t)width + i] = T::to_f32(a[i]) + T::to_f32(b[i]);
}

__global__ void token_state_write_kernel(int32_t* __restrict__ token_state, const int64_t* __restrict__ ids,
                                         const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start,
                                         const int32_t* __restrict__ q_len, int num_seqs) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s < num_seqs) token_state[state_slots[s]] = (int32_t)ids[q_start[s] + q_len[s] - 1];
}

template <typename T>
__global__ void residual_add2_rms_norm_kernel(float* __restrict__ x, const typename T::storage* __restrict__ ya, int64_t ya_stride,
                                              const typename T::storage* __restrict__ yb, int64_t yb_stride,
                                              const typename T::storage* __restrict__ bias,
                                              const typename T::storage* __restrict__ weight,
                                              typename T::storage* __restrict__ out, int width, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float y = 0.f;
    if (ya) y = T::to_f32(ya[t * ya_stride + i]);
    if (yb) y += T::to_f32(yb[t * yb_stride + i]);
    if (bias) y += T::to_f32(bias[i]);
    const float r = x[t * (int64_t)width + i] + y;
    if (ya || yb || bias) x[t * (int64_t)width + i] = r;
    row[i] = r;
    ss += r * r;
  }
  if (out == nullptr) return;
  const float rstd = 1.0f / sqrtf(wg_sum(ss, red) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    out[t * (int64_t)width + i] = T::from_f32(row[i] * rstd * (weight ? T::to_f32(weight[i]) : 1.0f));
}

template <typename T>
__global__ void residual_add2_rms_norm_vec8_kernel(float* __restrict__ x, const typename T::storage* __restrict__ ya,
                                                   int64_t ya_stride, const typename T::storage* __restrict__ yb,
                                                   int64_t yb_stride, const typename T::storage* __restrict__ bias,
                                                   const typename T::storage* __restrict__ weight,
                                                   typename T::storage* __restrict__ out, int width, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int i0 = threadIdx.x * 8;
  const bool act = i0 < width;
  const int ia = act ? i0 : 0;
  const int64_t at = t * (int64_t)width + ia;
  float r[8], a[8], b[8], c[8], w[8];
  pb_load8<Float>(x + at, r);
  if (ya) pb_load8<T>(ya + t * ya_stride + ia, a);
  if (yb) pb_load8<T>(yb + t * yb_stride + ia, b);
  if (bias) pb_load8<T>(bias + ia, c);
  if (out && weight) pb_load8<T>(weight + ia, w);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float y = 0.f;
    if (ya) y = a[j];
    if (yb) y += b[j];
    if (bias) y += c[j];
    r[j] += y;
  }
  if ((ya || yb || bias) && act) pb_store8<Float>(x + at, r);
  if (out == nullptr) return;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) ss += act ? r[j] * r[j] : 0.f;
  const float rstd = 1.0f / sqrtf(wg_sum(ss, red) / (float)width + eps);
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = r[j] * rstd * (weight ? w[j] : 1.0f);
  if (act) pb_store8<T>(out + at, r);
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_hashed_pair_embed(float* x, const void* table, const void* pair_table, const int64_t* ids,
                                       const int32_t* token_state, const int32_t* state_slots, const int32_t* q_start,
                                       const int32_t* ctx_len, const int32_t* seq_of_token, int64_t num_tokens, int width,
                                       int64_t vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(x && table && pair_table && ids && token_state && state_slots && q_start && ctx_len && seq_of_token,
              "hashed_pair_embed: null argument");
  APHRO_CHECK(width > 0 && vocab > 0 && buckets > 0, "hashed_pair_embed: width %d, vocab %lld, buckets %lld", width,
              (long long)vocab, (long long)buckets);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    hipLaunchKernelGGL((hashed_pair_embed_kernel<T>), dim3((unsigned)num_tokens), dim3(width >= 1024 ? 256 : 64), 0,
                       (hipStream_t)stream, x, (const S*)table, (const S*)pair_table, ids, token_state, state_slots, q_start, ctx_len,
                       seq_of_token, width, vocab, buckets, mul_prev, mul_cur);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_token_state_write(int32_t* token_state, const int64_t* ids, const int32_t* state_slots, const int32_t* q_start,
                                       const int32_t* q_len, int num_seqs, void* stream) {
  if (num_seqs == 0) return APHRO_OK;
  APHRO_CHECK(token_state && ids && state_slots && q_start && q_len && num_seqs > 0, "token_state_write: null argument");
  hipLaunchKernelGGL(token_state_write_kernel, dim3((unsigned)((num_seqs + 63) / 64)), dim3(64), 0, (hipStream_t)stream, token_state,
                     ids, state_slots, q_start, q_len, num_seqs);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_residual_add2_rms_norm(float* x, const void* ya, int64_t ya_stride, const void* yb, int64_t yb_stride,
                                            const void* bias, const void* weight, void* out, int64_t num_tokens, int width,
                                            float eps, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(x && num_tokens > 0 && width > 0 && width <= 16000, "residual_add2_rms_norm: bad sizes (width %d)", width);
  APHRO_CHECK((!ya || ya_stride >= width) && (!yb || yb_stride >= width), "residual_add2_rms_norm: a row stride is smaller than the row");
  APHRO_CHECK(ya || yb || bias || out, "residual_add2_rms_norm: nothing to do");
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool vec = (width & 7) == 0 && width <= 8192 && (ya_stride & 7) == 0 && (yb_stride & 7) == 0 && al16(x) && al16(ya) &&
                   al16(yb) && al16(bias) && al16(weight) && al16(out);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec)
      hipLaunchKernelGGL((residual_add2_rms_norm_vec8_kernel<T>), dim3((unsigned)num_tokens), dim3(((width / 8) + 63) / 64 * 64), 0,
                         (hipStream_t)stream, x, (const S*)ya, ya_stride, (const S*)yb, yb_stride, (const S*)bias, (const S*)weight,
                         (S*)out, width, eps);
    else
      hipLaunchKernelGGL((residual_add2_rms_norm_kernel<T>), dim3((unsigned)num_tokens), dim3(width >= 1024 ? 256 : (width > 256 ? 128 : 64)),
                         (size_t)width * sizeof(float), (hipStream_t)stream, x, (const S*)ya, ya_stride, (const S*)yb, yb_stride,
                         (const S*)bias, (const S*)weight, (S*)out, width, eps);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
