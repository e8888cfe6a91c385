// Short causal convolution over time on every channel of a projection's output, for a batch of segments:
//   y_t[c] = sum_j w[c, j] * u_(t - taps + 1 + j)[c],   zeros before the sequence's start.
// The taps - 1 inputs that precede a segment come from the request's state slot, which afterwards holds the last taps - 1
// inputs of the sequence.  A segment that starts a sequence never reads its slot, and no input older than the sequence's
// start is read from it either, so a slot taken over from another request needs no clearing.
//
// The channels are [q | k | v]: the q part goes to a dense output, the k and v parts straight into the token-major paged
// cache at the rows' slots (what attention reads is the convolved key and value).  Products and sums are fp32, one rounding
// to the storage type.  act 1: silu on the convolution's result (fp32, before the rounding).
#include "mixers_common.h"

namespace aphro {

constexpr int SC_MAX_TAPS = 16;

template <typename T>
__global__ void short_conv_kernel(typename T::storage* __restrict__ q_out, int64_t q_out_stride,
                                  typename T::storage* __restrict__ k_cache, typename T::storage* __restrict__ v_cache,
                                  const int64_t* __restrict__ cache_slots, int64_t num_cache_slots,
                                  const typename T::storage* __restrict__ u, int64_t u_stride,
                                  const typename T::storage* __restrict__ w, const typename T::storage* __restrict__ state,
                                  const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start,
                                  const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ seq_of_token, int cq, int ck,
                                  int cv, int taps, int act) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int C = cq + ck + cv;
  if (c >= C) return;
  const int s = seq_of_token[t];
  const int r = (int)t - q_start[s], ctx = ctx_len[s];
  const typename T::storage* st = state ? state + ((int64_t)state_slots[s] * (taps - 1)) * C + c : nullptr;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int i = r - taps + 1 + j;            // row of the segment, negative: before it
    float x = 0.f;
    if (i >= 0) x = T::to_f32(u[(t - r + i) * u_stride + c]);
    else if (ctx + i >= 0) x = T::to_f32(st[(int64_t)(taps - 1 + i) * C]);
    acc += T::to_f32(w[(int64_t)c * taps + j]) * x;
  }
  if (act) acc = silu_f(acc);
  const typename T::storage y = T::from_f32(acc);
  if (c < cq) {
    q_out[t * q_out_stride + c] = y;
  } else {
    const int64_t slot = cache_slots[t];
    if (slot < 0 || slot >= num_cache_slots) return;
    if (c < cq + ck) k_cache[slot * ck + (c - cq)] = y;
    else v_cache[slot * cv + (c - cq - ck)] = y;
  }
}

template <typename T>
__device__ __forceinline__ void sc_load8(const typename T::storage* p, float* o) {
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
__device__ __forceinline__ void sc_store8(typename T::storage* p, const float* v) {
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

// The same convolution for channel counts that are multiples of 8 and 16-byte-aligned rows: a thread owns 8 channels of TOK
// consecutive rows, reads the TOK + TAPS - 1 input rows they need once (16 bytes each) and its 8 x TAPS weights once.
template <typename T, int TAPS, int TOK>
__global__ __launch_bounds__(256) void short_conv_vec8_kernel(
    typename T::storage* __restrict__ q_out, int64_t q_out_stride, typename T::storage* __restrict__ k_cache,
    typename T::storage* __restrict__ v_cache, const int64_t* __restrict__ cache_slots, int64_t num_cache_slots,
    const typename T::storage* __restrict__ u, int64_t u_stride, const typename T::storage* __restrict__ w,
    const typename T::storage* __restrict__ state, const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ seq_of_token, int64_t num_tokens, int cq, int ck, int cv,
    int act) {
  const int c0 = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  const int C = cq + ck + cv;
  if (c0 >= C) return;
  const int64_t t0 = (int64_t)blockIdx.x * TOK;
  float wv[TAPS][8];                           // wv[j][i] = w[c0 + i, j]
  {
    float flat[8 * TAPS];
#pragma unroll
    for (int x = 0; x < TAPS; ++x) sc_load8<T>(w + (int64_t)c0 * TAPS + 8 * x, flat + 8 * x);
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < TAPS; ++j) wv[j][i] = flat[i * TAPS + j];
  }
  float rows[TOK + TAPS - 1][8];
#pragma unroll
  for (int x = 0; x < TOK + TAPS - 1; ++x) {
    const int64_t gr = t0 - (TAPS - 1) + x;
    if (gr >= 0 && gr < num_tokens) {
      sc_load8<T>(u + gr * u_stride + c0, rows[x]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) rows[x][i] = 0.f;
    }
  }
#pragma unroll
  for (int k = 0; k < TOK; ++k) {
    const int64_t t = t0 + k;
    if (t >= num_tokens) break;
    const int s = seq_of_token[t];
    const int r = (int)t - q_start[s], ctx = ctx_len[s];
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int i0 = r - TAPS + 1 + j;         // row of the segment, negative: before it
      float x[8];
      if (i0 >= 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = rows[k + j][i];
      } else if (ctx + i0 >= 0) {
        sc_load8<T>(state + ((int64_t)state_slots[s] * (TAPS - 1) + (TAPS - 1 + i0)) * C + c0, x);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += wv[j][i] * x[i];
    }
    if (act) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = silu_f(acc[i]);
    }
    if (c0 < cq) {
      sc_store8<T>(q_out + t * q_out_stride + c0, acc);
    } else {
      const int64_t slot = cache_slots[t];
      if (slot < 0 || slot >= num_cache_slots) continue;
      if (c0 < cq + ck) sc_store8<T>(k_cache + slot * ck + (c0 - cq), acc);
      else sc_store8<T>(v_cache + slot * cv + (c0 - cq - ck), acc);
    }
  }
}

// After the convolution: the slot takes the last taps - 1 inputs of the sequence (from the segment, or -- for a segment
// shorter than that -- from what the slot held, moved up).  One thread owns a channel of a segment and reads all it needs
// before it writes.
template <typename T>
__global__ void short_conv_state_kernel(typename T::storage* __restrict__ state, const typename T::storage* __restrict__ u,
                                        int64_t u_stride, const int32_t* __restrict__ state_slots,
                                        const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                        const int32_t* __restrict__ ctx_len, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int n = q_len[s], ctx = ctx_len[s], keep = taps - 1;
  typename T::storage* st = state + ((int64_t)state_slots[s] * keep) * C + c;
  typename T::storage val[SC_MAX_TAPS];
  for (int m = 0; m < keep; ++m) {
    const int p = ctx + n - keep + m;          // position in the sequence
    typename T::storage x = T::from_f32(0.f);
    if (p >= ctx) x = u[((int64_t)q_start[s] + (p - ctx)) * u_stride + c];
    else if (p >= 0) x = st[(int64_t)(p - ctx + keep) * C];
    val[m] = x;
  }
  for (int m = 0; m < keep; ++m) st[(int64_t)m * C] = val[m];
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_short_conv(void* q_out, int64_t q_out_stride, void* k_cache, void* v_cache, const int64_t* cache_slots,
                                int64_t num_cache_slots, const void* u, int64_t u_stride, const void* w, void* state,
                                const int32_t* state_slots, const int32_t* q_start, const int32_t* q_len,
                                const int32_t* ctx_len, const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int cq,
                                int ck, int cv, int taps, int act, int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  const int C = cq + ck + cv;
  APHRO_CHECK(u && w && q_start && q_len && ctx_len && seq_of_token && num_seqs > 0 && cq >= 0 && ck >= 0 && cv >= 0 && C > 0,
              "short_conv: bad arguments");
  APHRO_CHECK(taps >= 1 && taps <= SC_MAX_TAPS, "short_conv: %d taps (1 .. %d)", taps, SC_MAX_TAPS);
  APHRO_CHECK(act == 0 || act == 1, "short_conv: activation %d (0 none, 1 silu)", act);
  APHRO_CHECK(taps == 1 || (state && state_slots), "short_conv: more than one tap needs the state slots");
  APHRO_CHECK(u_stride >= C && (cq == 0 || (q_out && q_out_stride >= cq)), "short_conv: row strides smaller than the rows");
  APHRO_CHECK(ck + cv == 0 || (k_cache && v_cache && cache_slots && num_cache_slots > 0 && ck > 0 && cv > 0),
              "short_conv: key / value channels need the cache and the rows' slots");
  APHRO_CHECK(num_tokens <= 0x7fffffff && (C + 255) / 256 <= 65535, "short_conv: too large");
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool vec = taps >= 2 && taps <= 4 && (cq & 7) == 0 && (ck & 7) == 0 && (cv & 7) == 0 && (u_stride & 7) == 0 &&
                   (q_out_stride & 7) == 0 && al16(u) && al16(w) && al16(q_out) && al16(k_cache) && al16(v_cache) && al16(state);
  constexpr int TOK = 4;
#define SC_VEC(TAPS)                                                                                                           \
  hipLaunchKernelGGL((short_conv_vec8_kernel<T, TAPS, TOK>), dim3((unsigned)((num_tokens + TOK - 1) / TOK), (unsigned)((C / 8 + 255) / 256)), \
                     dim3(C / 8 >= 256 ? 256 : (C / 8 + 63) / 64 * 64), 0, (hipStream_t)stream, (S*)q_out, q_out_stride, (S*)k_cache,     \
                     (S*)v_cache, cache_slots, num_cache_slots, (const S*)u, u_stride, (const S*)w, (const S*)state, state_slots,        \
                     q_start, ctx_len, seq_of_token, num_tokens, cq, ck, cv, act)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec && taps == 2) SC_VEC(2);
    else if (vec && taps == 3) SC_VEC(3);
    else if (vec && taps == 4) SC_VEC(4);
    else
    hipLaunchKernelGGL((short_conv_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((C + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (S*)q_out, q_out_stride, (S*)k_cache, (S*)v_cache, cache_slots, num_cache_slots,
                       (const S*)u, u_stride, (const S*)w, (const S*)state, state_slots, q_start, ctx_len, seq_of_token, cq, ck,
                       cv, taps, act);
    if (taps > 1)
      hipLaunchKernelGGL((short_conv_state_kernel<T>), dim3((unsigned)num_seqs, (unsigned)((C + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, (S*)state, (const S*)u, u_stride, state_slots, q_start, q_len, ctx_len, C, taps);
  });
#undef SC_VEC
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
