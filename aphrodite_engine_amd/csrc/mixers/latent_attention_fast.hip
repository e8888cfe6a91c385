// bf16 matrix-core path of the attention through a low-rank latent (same semantics as latent_attention.hip, which stays the
// fp32 path and the path of sizes this does not tile).
//
// Every head reads the SAME cache rows [c (R) | k_r (P)], as key (all R + P numbers) and as value (the first R), so the
// query rows of a segment are flattened: row = token * heads + head.  A workgroup of eight waves owns 64 consecutive rows: a
// PAIR of waves shares 16 rows -- with 16 heads that is one token's heads -- both compute the rows' scores, each accumulates
// one half of the R output columns (two waves per SIMD hide each other's LDS latency, and half the accumulators leave
// registers for fragments in flight).  The workgroup walks the visible keys 32 at a time:
// the tile's cache rows come in with 16-byte loads, go to LDS once row-major (chunk-swizzled: the key operand) and, their
// first R numbers, once transposed (the value operand; layouts both their stores and their reads pass without bank conflicts);
// tiles alternate between two homes in LDS and the tile after the next is on its way in registers.  S^T = K Q^T on v_mfma_f32_16x16x32_bf16, so that the probabilities come out in the B-operand layout
// of O^T = C^T P^T; mask and online softmax (base 2) are fp32 on the accumulators.  The query operand is [q_lat | rotate(q_r)]
// padded with zeros to a multiple of 32, built once per workgroup (the rotation in fp32 at the row's position).
//
// Rows that see many keys while the launch has few workgroups (decoded tokens) split their key range over grid z; the
// partial (max, sum, accumulator) triples go through a scratch tensor and la_merge_kernel joins them.
#include "mixers_common.h"

namespace aphro {

struct LAParams {
  uint16_t* out;
  const uint16_t* q_lat;
  const uint16_t* q_rot;
  const uint16_t* cache;
  const int32_t* block_tables;
  const int32_t* q_start;
  const int32_t* q_len;
  const int32_t* ctx_len;
  const float* inv_freq;
  const float* sink;  // fp32 [heads] or NULL
  int window;         // <= 0: none
  int64_t out_stride, out_head_stride, ql_stride, ql_head_stride, qr_stride, qr_head_stride, num_blocks;
  int max_blocks, block_size, bs_shift, heads, nsplit;
  float scale, mscale;
  float* ws;          // split partials [T * heads, nsplit, 2 + R]
};

__device__ __forceinline__ int la_slot(const LAParams& p, const int32_t* bt, int key) {
  int blk, off;
  if (p.bs_shift >= 0) {
    blk = bt[key >> p.bs_shift];
    off = key & (p.block_size - 1);
  } else {
    blk = bt[key / p.block_size];
    off = key % p.block_size;
  }
  if (blk < 0 || blk >= p.num_blocks) blk = 0;             // never read outside the pool
  return blk * p.block_size + off;
}

constexpr int LF_BM = 64, LF_BN = 32;
// A thread brings in 16-byte chunks cl, cl + 32, ... of ONE pair of neighbouring keys (pair = tid / 32, cl = tid % 32): 32 lanes
// fetch 512 contiguous bytes, and a tile costs a thread two block-table lookups.  A tile has TWO homes in LDS: while the waves
// multiply from one, the next tile is stored into the other -- one barrier per tile, and one wave's stores run beside
// another's products.
// The transposed copy of a tile: column col of the latent is a row of LF_VS dwords (32 keys and one dword of padding) at row
// number (col & 7) * JS + (col >> 3), LF_VS = 17 and JS = 4 mod 32.  What the counters say about the LDS (32 banks of 4 bytes): a
// 4-byte access is served 32 lanes at a time, a 16-byte one 8 lanes.  A transposed store writes one dword per lane for 32
// consecutive chunks of one key pair per pass -- bank 17 cl: all 32 distinct; a 4-byte value-operand read of two lane groups
// finds its 16 columns x 2 key groups in banks 4 (c & 7) + 17 (c >> 3) + 2 g: all 32 distinct.  (Layouts that broke these rules
// showed SQ_LDS_BANK_CONFLICT at 0.31 of the LDS cycles.)  The row-major copy XORs the chunk index with key & 7: the 8 keys of a
// 16-byte fragment read pass hit 8 different bank quads.
constexpr int LF_VS = 17, LF_THREADS = 512, LF_CL = 32;

template <int R, int P>
struct LFGeom {
  static constexpr int D = R + P, DP = (D + 31) / 32 * 32, NCH = DP / 8, NKS = DP / 32, NDT = R / 16;
  static constexpr int SWZ = ((NCH & -NCH) - 1) & 7;       // chunk index ^ (key & SWZ): fragment reads spread over the banks
  static constexpr int NI = (NCH + LF_CL - 1) / LF_CL, NDH = NDT / 2;
  static constexpr int JS = (R / 8 + 27) / 32 * 32 + 4;
  static constexpr int KBUF = LF_BN * DP, VBUF = 8 * JS * LF_VS;         // one home: elements of the row-major copy, dwords of the other
  static constexpr size_t LDS_BYTES = 2 * ((size_t)KBUF * sizeof(uint16_t) + (size_t)VBUF * sizeof(uint32_t));
};

template <int R, int P>
struct LFStage {
  u16x8 a[LFGeom<R, P>::NI], b[LFGeom<R, P>::NI];
};

template <int R, int P>
__device__ __forceinline__ void lf_load(LFStage<R, P>& st, const LAParams& p, const int32_t* bt, int t0, int t_end) {
  typedef LFGeom<R, P> G;
  const int tp = threadIdx.x / LF_CL, c8 = threadIdx.x % LF_CL;
  const int k0 = t0 + 2 * tp;
  const bool ina = k0 < t_end, inb = k0 + 1 < t_end;
  const uint16_t* ra = p.cache + (int64_t)la_slot(p, bt, ina ? k0 : t0) * G::D + 8 * c8;
  const uint16_t* rb = p.cache + (int64_t)la_slot(p, bt, inb ? k0 + 1 : t0) * G::D + 8 * c8;
#pragma unroll
  for (int it = 0; it < G::NI; ++it) {
    u16x8 va = u16x8{0, 0, 0, 0, 0, 0, 0, 0}, vb = va;
    if (8 * LF_CL * it + 8 * c8 < G::D) {
      if (ina) va = *reinterpret_cast<const u16x8*>(ra + 8 * LF_CL * it);
      if (inb) vb = *reinterpret_cast<const u16x8*>(rb + 8 * LF_CL * it);
    }
    st.a[it] = va;
    st.b[it] = vb;
  }
}

template <int R, int P>
__device__ __forceinline__ void lf_store(const LFStage<R, P>& st, uint16_t* k_lds, uint32_t* vt_lds) {
  typedef LFGeom<R, P> G;
  const int tp = threadIdx.x / LF_CL, c8 = threadIdx.x % LF_CL;
  const int ta = 2 * tp, tb = 2 * tp + 1;
  uint16_t* ka = k_lds + ta * G::DP + 8 * (c8 ^ (ta & G::SWZ));      // chunk c8 + 32 it: the swizzle stays within the low 3 bits
  uint16_t* kb = k_lds + tb * G::DP + 8 * (c8 ^ (tb & G::SWZ));
  uint32_t* vt = vt_lds + c8 * LF_VS + tp;
#pragma unroll
  for (int it = 0; it < G::NI; ++it) {
    if (LF_CL * it + c8 < G::NCH) {
      *reinterpret_cast<u16x8*>(ka + 8 * LF_CL * it) = st.a[it];
      *reinterpret_cast<u16x8*>(kb + 8 * LF_CL * it) = st.b[it];
    }
    if (8 * LF_CL * it + 8 * c8 < R) {
      const u32x4 wa = __builtin_bit_cast(u32x4, st.a[it]), wb = __builtin_bit_cast(u32x4, st.b[it]);
#pragma unroll
      for (int j2 = 0; j2 < 4; ++j2) {        // numbers 2 j2 and 2 j2 + 1 of both keys: low halves, then high halves
        vt[((2 * j2) * G::JS + LF_CL * it) * LF_VS] = __builtin_amdgcn_perm(wb[j2], wa[j2], 0x05040100);
        vt[((2 * j2 + 1) * G::JS + LF_CL * it) * LF_VS] = __builtin_amdgcn_perm(wb[j2], wa[j2], 0x07060302);
      }
    }
  }
}

template <int R, int P>
__global__ __launch_bounds__(LF_THREADS) void la_mfma_kernel(LAParams p) {
  typedef LFGeom<R, P> G;
  constexpr int NH = LF_BN / 16, NPK = LF_BN / 32;
  extern __shared__ __attribute__((aligned(16))) uint16_t la_lds[];
  uint16_t* k_lds = la_lds;                                                     // two homes of KBUF elements
  uint32_t* vt_lds = reinterpret_cast<uint32_t*>(la_lds + 2 * G::KBUF);          // two homes of VBUF dwords
  // waves 2 k and 2 k + 1 share row group k: a launch with one row group (decoded tokens of 16 heads) still uses two SIMDs
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 7, half = (threadIdx.x >> 6) & 1, g = lane >> 4, c = lane & 15;
  const int seq = blockIdx.y, z = blockIdx.z;
  const int len = p.q_len[seq];
  const int H = p.heads;
  const int nrows = len * H;
  const int r0 = blockIdx.x * LF_BM;
  if (r0 >= nrows) return;
  const int ctx = p.ctx_len[seq], s0 = p.q_start[seq];
  const int row = r0 + 16 * wave + c;
  const bool rvalid = row < nrows;
  const int rowc = rvalid ? row : nrows - 1;
  const int tok = rowc / H, head = rowc - tok * H;
  const int qpos = ctx + tok;
  // rows of this wave span these positions
  const int wrow_lo = min(r0 + 16 * wave, nrows - 1), wrow_hi = min(r0 + 16 * wave + 15, nrows - 1);
  const int wpos_lo = ctx + wrow_lo / H, wpos_hi = ctx + wrow_hi / H;
  const int nk = ctx + min(r0 + LF_BM - 1, nrows - 1) / H + 1;          // keys the workgroup's last row sees
  // this workgroup's share of the key tiles
  // under a window the walk starts at the tile of the oldest key the workgroup's first row sees
  const int k_first = p.window > 0 ? max(0, ctx + r0 / H - p.window + 1) / LF_BN * LF_BN : 0;
  const int tiles = (nk - k_first + LF_BN - 1) / LF_BN, per = (tiles + p.nsplit - 1) / p.nsplit;
  const int t_begin = k_first + z * per * LF_BN, t_end = min(nk, k_first + (z + 1) * per * LF_BN);
  constexpr float LOG2E = 1.4426950408889634f;
  const float qs = p.scale * LOG2E;

  const int32_t* bt = p.block_tables + (int64_t)seq * p.max_blocks;
  LFStage<R, P> st;                                         // the first tiles are on their way while the query operand is made
  if (t_begin < t_end) {
    lf_load<R, P>(st, p, bt, t_begin, t_end);
    lf_store<R, P>(st, k_lds, vt_lds);
    if (t_begin + LF_BN < t_end) lf_load<R, P>(st, p, bt, t_begin + LF_BN, t_end);
  }

  // the query operand: [q_lat | rotate(q_rot) | zeros]
  u32x4 qf[G::NKS];
  {
    const uint16_t* ql = p.q_lat + (int64_t)(s0 + tok) * p.ql_stride + (int64_t)head * p.ql_head_stride;
    const uint16_t* qr = P ? p.q_rot + (int64_t)(s0 + tok) * p.qr_stride + (int64_t)head * p.qr_head_stride : nullptr;
#pragma unroll
    for (int ks = 0; ks < G::NKS; ++ks) {
      const int at = 32 * ks + 8 * g;
      u32x4 v = u32x4{0, 0, 0, 0};
      if (at < R) {
        v = *reinterpret_cast<const u32x4*>(ql + at);
      } else if (at < G::D) {
        constexpr int HALF = P / 2;
        const int i0 = at - R;
        const bool low = i0 < HALF;
        const int f0 = low ? i0 : i0 - HALF;
        const u16x8 mine = *reinterpret_cast<const u16x8*>(qr + i0);
        const u16x8 other = *reinterpret_cast<const u16x8*>(qr + (low ? i0 + HALF : i0 - HALF));
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float cs, sn;
          sincosf((float)qpos * p.inv_freq[f0 + j], &sn, &cs);
          cs *= p.mscale;
          sn *= p.mscale;
          const float x = BFloat::to_f32(mine[j]), y = BFloat::to_f32(other[j]);
          o[j] = low ? x * cs - y * sn : x * cs + y * sn;
        }
        v = u32x4{pack2_16<true>(o[0], o[1]), pack2_16<true>(o[2], o[3]), pack2_16<true>(o[4], o[5]), pack2_16<true>(o[6], o[7])};
      }
      qf[ks] = v;
    }
  }
  f32x4 o[G::NDH];                                          // this wave's half of the output columns
#pragma unroll
  for (int i = 0; i < G::NDH; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -1e30f, l_run = 0.f;
  const int kmax = min(qpos, t_end - 1);                    // the last key this row takes from this workgroup's share
  const int kmin = p.window > 0 ? qpos - p.window + 1 : 0;  // the oldest key this row sees (may be negative)
  const int wmin_lo = p.window > 0 ? wpos_lo - p.window + 1 : 0, wmin_hi = p.window > 0 ? wpos_hi - p.window + 1 : 0;

  const uint16_t* krow[2] = {k_lds + c * G::DP + 8 * (g ^ (c & G::SWZ)), k_lds + c * G::DP + 8 * ((4 | g) ^ (c & G::SWZ))};
  const uint32_t* vrow = vt_lds + ((c & 7) * G::JS + (c >> 3) + 2 * G::NDH * half) * LF_VS + 2 * g;
  const bool idle = r0 + 16 * wave >= nrows;                // a wave without rows only helps to move the tiles

  int cur = 0;
  __syncthreads();
  for (int t0 = t_begin; t0 < t_end; t0 += LF_BN, cur ^= 1) {
   if (!(idle || t0 > wpos_hi || t0 + LF_BN <= wmin_lo)) {  // else: every key of the tile is ahead of the wave's rows or behind their windows
    const int kofs = cur * G::KBUF, vofs = cur * G::VBUF;
    f32x4 s[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      s[h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < G::NKS; ++ks) {
        // chunk (4 ks + g) ^ swz(key) = 8 (ks / 2) + (((ks & 1) * 4 + g) ^ swz(c)): two lane offsets, the rest is immediate
        const u32x4 kf = *reinterpret_cast<const u32x4*>(krow[ks & 1] + kofs + (16 * h) * G::DP + 64 * (ks >> 1));
        s[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf), __builtin_bit_cast(bf16x8, qf[ks]), s[h], 0, 0, 0);
      }
    }
    const bool edge = t0 + LF_BN - 1 > min(wpos_lo, t_end - 1) || t0 < wmin_hi;   // some key of the tile is not for some row of the wave
    float pv[NH][4];
    float mx = -1e30f;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float xv = s[h][r] * qs;
        if (edge) {
          const int key = t0 + 16 * h + 4 * g + r;
          xv = (key <= kmax && key >= kmin) ? xv : -1e30f;
        }
        pv[h][r] = xv;
        mx = fmaxf(mx, xv);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float lsum = 0.f;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float e = pv[h][r] > -1e29f ? __builtin_amdgcn_exp2f(pv[h][r] - m_new) : 0.f;
        pv[h][r] = e;
        lsum += e;
      }
    l_run = l_run * alpha + lsum;
#pragma unroll
    for (int dt = 0; dt < G::NDH; ++dt) o[dt] *= alpha;
    u32x4 pf[NPK];
#pragma unroll
    for (int pk = 0; pk < NPK; ++pk)
      pf[pk] = u32x4{pack2_16<true>(pv[2 * pk][0], pv[2 * pk][1]), pack2_16<true>(pv[2 * pk][2], pv[2 * pk][3]),
                     pack2_16<true>(pv[2 * pk + 1][0], pv[2 * pk + 1][1]), pack2_16<true>(pv[2 * pk + 1][2], pv[2 * pk + 1][3])};
#pragma unroll
    for (int pk = 0; pk < NPK; ++pk) {
#pragma unroll
      for (int dt = 0; dt < G::NDH; ++dt) {
        const uint32_t* vr = vrow + vofs + 2 * dt * LF_VS + 16 * pk;
        const u32x4 vf = {vr[0], vr[1], vr[8], vr[9]};
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf[pk]), o[dt], 0, 0, 0);
      }
    }
   }
    if (t0 + LF_BN < t_end) {                               // the next tile goes to the other home, the one after it is requested
      lf_store<R, P>(st, k_lds + (cur ^ 1) * G::KBUF, vt_lds + (cur ^ 1) * G::VBUF);
      if (t0 + 2 * LF_BN < t_end) lf_load<R, P>(st, p, bt, t0 + 2 * LF_BN, t_end);
    }
    __syncthreads();
  }
  float l = l_run;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!rvalid) return;
  if (p.nsplit == 1) {
    float f = l > 0.f ? 1.f / l : 0.f;
    if (p.sink) {                                           // one more term of the denominator: exp(sink), no value
      const float s2 = p.sink[head] * LOG2E, M = fmaxf(m_run, s2), fo = __builtin_amdgcn_exp2f(m_run - M);
      f = fo / (l * fo + __builtin_amdgcn_exp2f(s2 - M));
    }
    uint16_t* op = p.out + (int64_t)(s0 + tok) * p.out_stride + (int64_t)head * p.out_head_stride + 16 * G::NDH * half;
#pragma unroll
    for (int dt = 0; dt < G::NDH; ++dt)
      *reinterpret_cast<u32x2*>(op + 16 * dt + 4 * g) = u32x2{pack2_16<true>(o[dt][0] * f, o[dt][1] * f), pack2_16<true>(o[dt][2] * f, o[dt][3] * f)};
  } else {
    float* wp = p.ws + (((int64_t)(s0 + tok) * H + head) * p.nsplit + z) * (2 + R);
    if (g == 0 && half == 0) {
      wp[0] = m_run;
      wp[1] = l;
    }
#pragma unroll
    for (int dt = 0; dt < G::NDH; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) wp[2 + 16 * (G::NDH * half + dt) + 4 * g + r] = o[dt][r];
  }
}

// one workgroup per (token, head): joins the nsplit partial results; a thread owns two neighbouring columns and has every
// split's piece in flight before it adds them up
constexpr int LA_MAX_SPLIT = 16;
__global__ void la_merge_kernel(uint16_t* __restrict__ out, int64_t out_stride, int64_t out_head_stride, const float* __restrict__ ws,
                                int heads, int nsplit, int R, const float* __restrict__ sink) {
  const int64_t t = blockIdx.x;
  const int head = blockIdx.y;
  const float* wp = ws + ((t * heads + head) * nsplit) * (int64_t)(2 + R);
  const int col = 2 * threadIdx.x;
  f32x2 ml[LA_MAX_SPLIT], v[LA_MAX_SPLIT];
#pragma unroll
  for (int zz = 0; zz < LA_MAX_SPLIT; ++zz)
    if (zz < nsplit) {
      ml[zz] = *reinterpret_cast<const f32x2*>(wp + (int64_t)zz * (2 + R));
      v[zz] = col < R ? *reinterpret_cast<const f32x2*>(wp + (int64_t)zz * (2 + R) + 2 + col) : f32x2{0.f, 0.f};
    }
  const float s2 = sink ? sink[head] * 1.4426950408889634f : -1e30f;
  float M = s2;
#pragma unroll
  for (int zz = 0; zz < LA_MAX_SPLIT; ++zz)
    if (zz < nsplit) M = fmaxf(M, ml[zz][0]);
  float L = sink ? __builtin_amdgcn_exp2f(s2 - M) : 0.f, a0 = 0.f, a1 = 0.f;
#pragma unroll
  for (int zz = 0; zz < LA_MAX_SPLIT; ++zz)
    if (zz < nsplit && ml[zz][1] > 0.f) {
      const float f = __builtin_amdgcn_exp2f(ml[zz][0] - M);
      L += ml[zz][1] * f;
      a0 += v[zz][0] * f;
      a1 += v[zz][1] * f;
    }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  if (col < R)
    *reinterpret_cast<uint32_t*>(out + t * out_stride + (int64_t)head * out_head_stride + col) = pack2_16<true>(a0 * inv, a1 * inv);
}

template <int R, int P>
static int la_launch(const LAParams& p, int num_seqs, int max_q_len, int64_t num_tokens, hipStream_t stream) {
  typedef LFGeom<R, P> G;
  static bool configured = false;
  if (!configured) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(la_mfma_kernel<R, P>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)G::LDS_BYTES);
    if (e != hipSuccess) {
      set_error("latent_attention: %zu bytes of LDS refused: %s", G::LDS_BYTES, hipGetErrorString(e));
      return APHRO_ERR_INVALID;
    }
    configured = true;
  }
  const int64_t tiles = ((int64_t)max_q_len * p.heads + LF_BM - 1) / LF_BM;
  hipLaunchKernelGGL((la_mfma_kernel<R, P>), dim3((unsigned)tiles, (unsigned)num_seqs, (unsigned)p.nsplit), dim3(LF_THREADS), G::LDS_BYTES,
                     stream, p);
  if (p.nsplit > 1)
    hipLaunchKernelGGL(la_merge_kernel, dim3((unsigned)num_tokens, (unsigned)p.heads), dim3((R / 2 + 63) / 64 * 64), 0, stream, p.out,
                       p.out_stride, p.out_head_stride, p.ws, p.heads, p.nsplit, R, p.sink);
  return APHRO_OK;
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_latent_attention_plain(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_lat,
                                            int64_t ql_stride, int64_t ql_head_stride, const void* q_rot, int64_t qr_stride,
                                            int64_t qr_head_stride, const void* cache, const int32_t* block_tables, int max_blocks,
                                            int64_t num_blocks, int block_size, const int32_t* q_start, const int32_t* ctx_len,
                                            const int32_t* seq_of_token, const float* inv_freq, float mscale, int64_t num_tokens,
                                            int heads, int kv_rank, int rot_dim, int rot_dims, float scale, int window,
                                            const float* sink, int dtype, void* stream);

#define LA_FAST_SIZES(X) X(128, 16) X(128, 32) X(256, 32) X(256, 64) X(512, 64)

extern "C" int aphro_latent_attention_fast_supported(int kv_rank, int rot_dim, int rot_dims, int dtype) {
  if (dtype != APHRO_BF16 || rot_dims != rot_dim) return 0;
#define LA_IS(R_, P_) if (kv_rank == R_ && rot_dim == P_) return 1;
  LA_FAST_SIZES(LA_IS)
#undef LA_IS
  return 0;
}

/* The number of key-range splits the matrix-core kernel would use, and so the scratch it needs: floats = num_tokens * heads *
 * splits * (2 + kv_rank) when splits > 1. */
extern "C" int aphro_latent_attention_splits(int64_t num_tokens, int num_seqs, int max_q_len, int heads, int max_kv_len) {
  const int64_t tiles = ((int64_t)max_q_len * heads + LF_BM - 1) / LF_BM * num_seqs;
  if (tiles >= 128 || max_kv_len < 512) return 1;
  int s = max_kv_len / 128;                                // two tiles of keys per workgroup
  const int64_t room = 512 / (tiles > 0 ? tiles : 1);
  if (s > room) s = (int)room;
  if (s > LA_MAX_SPLIT) s = LA_MAX_SPLIT;
  return s < 1 ? 1 : s;
}

extern "C" int aphro_latent_attention(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_lat, int64_t ql_stride,
                                      int64_t ql_head_stride, const void* q_rot, int64_t qr_stride, int64_t qr_head_stride,
                                      const void* cache, const int32_t* block_tables, int max_blocks, int64_t num_blocks,
                                      int block_size, const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                                      const int32_t* seq_of_token, const float* inv_freq, float mscale, int64_t num_tokens,
                                      int num_seqs, int max_q_len, int max_kv_len, int heads, int kv_rank, int rot_dim, int rot_dims,
                                      float scale, int window, const float* sink, float* workspace, int64_t workspace_floats,
                                      int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  const auto al16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
  const bool fast = aphro_latent_attention_fast_supported(kv_rank, rot_dim, rot_dims, dtype) && q_len && num_seqs > 0 && max_q_len > 0 &&
                    al16(q_lat) && al16(q_rot) && al16(cache) && al16(out) && ql_stride % 8 == 0 && ql_head_stride % 8 == 0 &&
                    qr_stride % 8 == 0 && qr_head_stride % 8 == 0 && out_stride % 4 == 0 && out_head_stride % 4 == 0 &&
                    (int64_t)max_q_len * heads < (1 << 30);
  if (!fast)
    return aphro_latent_attention_plain(out, out_stride, out_head_stride, q_lat, ql_stride, ql_head_stride, q_rot, qr_stride,
                                        qr_head_stride, cache, block_tables, max_blocks, num_blocks, block_size, q_start, ctx_len,
                                        seq_of_token, inv_freq, mscale, num_tokens, heads, kv_rank, rot_dim, rot_dims, scale, window,
                                        sink, dtype, stream);
  APHRO_CHECK(out && q_lat && q_rot && cache && block_tables && q_start && ctx_len && inv_freq, "latent_attention: null argument");
  APHRO_CHECK(heads > 0 && heads <= 65535 && block_size > 0 && max_blocks > 0 && num_blocks > 0 && num_seqs <= 65535,
              "latent_attention: bad geometry");
  LAParams p;
  p.out = (uint16_t*)out;
  p.q_lat = (const uint16_t*)q_lat;
  p.q_rot = (const uint16_t*)q_rot;
  p.cache = (const uint16_t*)cache;
  p.block_tables = block_tables;
  p.q_start = q_start;
  p.q_len = q_len;
  p.ctx_len = ctx_len;
  p.inv_freq = inv_freq;
  p.sink = sink;
  p.window = window;
  p.out_stride = out_stride;
  p.out_head_stride = out_head_stride;
  p.ql_stride = ql_stride;
  p.ql_head_stride = ql_head_stride;
  p.qr_stride = qr_stride;
  p.qr_head_stride = qr_head_stride;
  p.num_blocks = num_blocks;
  p.max_blocks = max_blocks;
  p.block_size = block_size;
  p.bs_shift = (block_size & (block_size - 1)) == 0 ? __builtin_ctz(block_size) : -1;
  p.heads = heads;
  p.scale = scale;
  p.mscale = mscale;
  p.nsplit = 1;
  p.ws = nullptr;
  const int want = aphro_latent_attention_splits(num_tokens, num_seqs, max_q_len, heads, max_kv_len);
  if (want > 1 && workspace && workspace_floats >= num_tokens * (int64_t)heads * want * (2 + kv_rank)) {
    p.nsplit = want;
    p.ws = workspace;
  }
  int rc = APHRO_ERR_INVALID;
#define LA_GO(R_, P_) if (kv_rank == R_ && rot_dim == P_) rc = la_launch<R_, P_>(p, num_seqs, max_q_len, num_tokens, (hipStream_t)stream);
  LA_FAST_SIZES(LA_GO)
#undef LA_GO
  if (rc != APHRO_OK) return rc;
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
