// A residual carried as several streams (hyper-connections): x [T, n, W] fp32, n copies of the residual that sublayers read
// through a learned combination and write back through a learned mixing matrix:
//     u      = sum_s in[s] x_s                      the sublayer's input (before its norm)
//     x_t   <- sum_s mix[s, t] x_s + mult * out[t] * (scale (.) y)        all streams at once from the old ones
// One launch folds the WRITE of the sublayer that has just run (y, its per-channel layer scale, its mix / out) and the READ of
// the next one (its in, the RMS norm with a per-channel weight); either half can be left out.  n = 1 with mix = out = in = 1
// is the plain residual x += mult * scale (.) y followed by the norm.  Everything is fp32 except y, the scale, the weight and
// the normed output, which are of the activation dtype.
//
// Also here: the logits' scale and soft cap.
#include "mixers_common.h"

namespace aphro {

constexpr int HC_MAX_STREAMS = 16;

struct HCCoef {
  float mix[HC_MAX_STREAMS * HC_MAX_STREAMS];   // [from, to]
  float out[HC_MAX_STREAMS];                    // already times mult
  float in[HC_MAX_STREAMS];
};

// one workgroup per token; u is kept in LDS (W floats) between the statistics and the output
template <typename T, int NS>
__global__ void hyper_residual_rms_norm_kernel(float* __restrict__ x, const typename T::storage* __restrict__ y, int64_t y_stride,
                                               const typename T::storage* __restrict__ scale, HCCoef cf, int has_mix,
                                               const typename T::storage* __restrict__ weight, typename T::storage* __restrict__ out,
                                               float* __restrict__ sum_out, int n, int width, float eps) {
  extern __shared__ float u_lds[];
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float* xr = x + t * (int64_t)n * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float xs[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) xs[s] = s < n ? xr[(int64_t)s * width + i] : 0.f;
    if (y) {
      float yv = T::to_f32(y[t * y_stride + i]);
      if (scale) yv *= T::to_f32(scale[i]);
      float nx[NS];
#pragma unroll
      for (int to = 0; to < NS; ++to) {
        float a = cf.out[to] * yv;
        if (has_mix) {
#pragma unroll
          for (int s = 0; s < NS; ++s)
            if (s < n) a += cf.mix[s * HC_MAX_STREAMS + to] * xs[s];
        } else {
          a += xs[to];
        }
        nx[to] = a;
      }
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (s < n) {
          xs[s] = nx[s];
          xr[(int64_t)s * width + i] = nx[s];
        }
    }
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (s < n) u += cf.in[s] * xs[s];
    if (sum_out) sum_out[t * (int64_t)width + i] = u;
    u_lds[i] = u;
    ss += u * u;
  }
  if (!out) return;
  const float rstd = 1.0f / sqrtf(wg_sum(ss, red) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = u_lds[i] * rstd;
    if (weight) v *= T::to_f32(weight[i]);
    out[t * (int64_t)width + i] = T::from_f32(v);
  }
}

// the same with four neighbouring channels per thread (16-byte accesses to the streams): width a multiple of 4, aligned rows
template <typename T>
__device__ __forceinline__ f32x4 hc_load4(const typename T::storage* p) {
  if constexpr (sizeof(typename T::storage) == 2) {
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    return f32x4{T::to_f32(v[0]), T::to_f32(v[1]), T::to_f32(v[2]), T::to_f32(v[3])};
  } else {
    return *reinterpret_cast<const f32x4*>(p);
  }
}
template <typename T>
__device__ __forceinline__ void hc_store4(typename T::storage* p, f32x4 v) {
  if constexpr (sizeof(typename T::storage) == 2) {
    *reinterpret_cast<u16x4*>(p) = u16x4{T::from_f32(v[0]), T::from_f32(v[1]), T::from_f32(v[2]), T::from_f32(v[3])};
  } else {
    *reinterpret_cast<f32x4*>(p) = v;
  }
}

template <typename T, int NS>
__global__ void hyper_residual_rms_norm_vec4_kernel(float* __restrict__ x, const typename T::storage* __restrict__ y, int64_t y_stride,
                                                    const typename T::storage* __restrict__ scale, HCCoef cf, int has_mix,
                                                    const typename T::storage* __restrict__ weight, typename T::storage* __restrict__ out,
                                                    float* __restrict__ sum_out, int n, int width, float eps) {
  extern __shared__ float u_lds[];
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float* xr = x + t * (int64_t)n * width;
  float ss = 0.f;
  for (int i = 4 * threadIdx.x; i < width; i += 4 * blockDim.x) {
    f32x4 xs[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) xs[s] = s < n ? *reinterpret_cast<const f32x4*>(xr + (int64_t)s * width + i) : f32x4{0.f, 0.f, 0.f, 0.f};
    if (y) {
      f32x4 yv = hc_load4<T>(y + t * y_stride + i);
      if (scale) yv *= hc_load4<T>(scale + i);
      f32x4 nx[NS];
#pragma unroll
      for (int to = 0; to < NS; ++to) {
        f32x4 a = yv * cf.out[to];
        if (has_mix) {
#pragma unroll
          for (int s = 0; s < NS; ++s)
            if (s < n) a += xs[s] * cf.mix[s * HC_MAX_STREAMS + to];
        } else {
          a += xs[to];
        }
        nx[to] = a;
      }
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (s < n) {
          xs[s] = nx[s];
          *reinterpret_cast<f32x4*>(xr + (int64_t)s * width + i) = nx[s];
        }
    }
    f32x4 u = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (s < n) u += xs[s] * cf.in[s];
    if (sum_out) *reinterpret_cast<f32x4*>(sum_out + t * (int64_t)width + i) = u;
    *reinterpret_cast<f32x4*>(u_lds + i) = u;
    ss += (u[0] * u[0] + u[1] * u[1]) + (u[2] * u[2] + u[3] * u[3]);
  }
  if (!out) return;
  const float rstd = 1.0f / sqrtf(wg_sum(ss, red) / (float)width + eps);
  for (int i = 4 * threadIdx.x; i < width; i += 4 * blockDim.x) {
    f32x4 v = *reinterpret_cast<const f32x4*>(u_lds + i) * rstd;
    if (weight) v *= hc_load4<T>(weight + i);
    hc_store4<T>(out + t * (int64_t)width + i, v);
  }
}

template <typename T>
__global__ void logit_softcap_kernel(float* __restrict__ out, const typename T::storage* __restrict__ in, int64_t n, float scale,
                                     float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v = T::to_f32(in[i]) * scale;
  if (cap > 0.f) v = cap * tanhf(v / cap);
  out[i] = v;
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_hyper_residual_rms_norm(float* x, const void* y, int64_t y_stride, const void* scale, const float* mix,
                                             const float* out_coef, float mult, const float* in_coef, const void* weight, void* out,
                                             float* sum_out, int64_t num_tokens, int streams, int width, float eps, int dtype,
                                             void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(x && streams >= 1 && streams <= HC_MAX_STREAMS && width > 0 && width <= 16384,
              "hyper_residual_rms_norm: %d streams (1 .. %d) of width %d (<= 16384)", streams, HC_MAX_STREAMS, width);
  APHRO_CHECK(!y || y_stride >= width, "hyper_residual_rms_norm: y's row stride is smaller than its rows");
  APHRO_CHECK(y || out || sum_out, "hyper_residual_rms_norm: nothing to do");
  // the coefficients are host arrays: a few dozen numbers that travel as a kernel argument
  HCCoef cf;
  for (int s = 0; s < HC_MAX_STREAMS; ++s) {
    cf.out[s] = s < streams ? mult * (out_coef ? out_coef[s] : 1.0f) : 0.f;
    cf.in[s] = s < streams ? (in_coef ? in_coef[s] : 1.0f) : 0.f;
    for (int to = 0; to < HC_MAX_STREAMS; ++to)
      cf.mix[s * HC_MAX_STREAMS + to] = (mix && s < streams && to < streams) ? mix[s * streams + to] : (s == to ? 1.0f : 0.f);
  }
  const int block = width >= 1024 ? 256 : (width > 256 ? 128 : 64);
  const size_t lds = (size_t)width * sizeof(float);
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool vec = width % 4 == 0 && y_stride % 8 == 0 && width % 8 == 0 && al16(x) && al16(y) && al16(scale) && al16(weight) && al16(out) &&
                   al16(sum_out) && streams <= 8;
#define HC_LAUNCH(NS)                                                                                                           \
  do {                                                                                                                          \
    if (vec)                                                                                                                    \
      hipLaunchKernelGGL((hyper_residual_rms_norm_vec4_kernel<T, (NS > 8 ? 8 : NS)>), dim3((unsigned)num_tokens),                \
                         dim3(width >= 1024 ? 256 : (width > 256 ? 128 : 64)), lds, (hipStream_t)stream, x, (const S*)y, y_stride, \
                         (const S*)scale, cf, mix ? 1 : 0, (const S*)weight, (S*)out, sum_out, streams, width, eps);            \
    else                                                                                                                        \
      hipLaunchKernelGGL((hyper_residual_rms_norm_kernel<T, NS>), dim3((unsigned)num_tokens), dim3(block), lds, (hipStream_t)stream, x, \
                         (const S*)y, y_stride, (const S*)scale, cf, mix ? 1 : 0, (const S*)weight, (S*)out, sum_out, streams, width, eps); \
  } while (0)
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (streams == 1) HC_LAUNCH(1);
    else if (streams == 2) HC_LAUNCH(2);
    else if (streams <= 4) HC_LAUNCH(4);
    else if (streams <= 8) HC_LAUNCH(8);
    else HC_LAUNCH(16);
  });
#undef HC_LAUNCH
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_logit_softcap(float* out, const void* in, int64_t n, float scale, float cap, int dtype, void* stream) {
  if (n == 0) return APHRO_OK;
  APHRO_CHECK(out && in && n > 0, "logit_softcap: bad arguments");
  MIX_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((logit_softcap_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                                               (hipStream_t)stream, out, (const typename T::storage*)in, n, scale, cap));
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
