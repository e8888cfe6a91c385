// Mixture of small feed-forward experts on unquantised weights (bf16 on the matrix cores, fp32 on the vector ALUs):
//   moe_route          softmax over the router's outputs, choice by score + correction, weight = the score itself
//   moe_align          the (token, choice) slots sorted by expert into blocks of 16 (64, 128 in prompt-sized steps) rows, one
//                      expert per block
//   moe_glu_gemm       per block: [gate | up] product of its expert with the clamped gated activation in the epilogue
//   moe_down_gemm      per block: the expert's down product, fp32 rows scattered back to their slots
//   moe_combine        per token: weighted sum over its choices (identity experts pass the input through), plus the
//                      sigmoid-gated shared expert
//   clamped_glu        the experts' activation alone (for the shared expert, whose products are plain dense ones)
// Nothing here depends on what else is in the batch: a slot's row is the same whichever block and row it lands in.
#include "mixers_common.h"

namespace aphro {

constexpr int MOE_BM = 16;

// limit > 0:  g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1)
// limit <= 0: the plain gated form gate * sigmoid(alpha gate) * up (alpha 1: silu)
__device__ __forceinline__ float clamped_glu_f(float gate, float up, float limit, float alpha) {
  if (limit <= 0.f) return gate * sigmoid_f(alpha * gate) * up;
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g * sigmoid_f(alpha * g) * (u + 1.0f);
}

// one wave per token; scores and choice values of the token in LDS
__global__ __launch_bounds__(256) void moe_route_kernel(int32_t* __restrict__ ids, float* __restrict__ weights,
                                                        const float* __restrict__ z, const float* __restrict__ correction,
                                                        int64_t num_tokens, int outputs, int top) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* s = lds + (size_t)wave * 2 * outputs;
  float* ch = s + outputs;
  const int64_t tt = (int64_t)blockIdx.x * 4 + wave;
  const bool live = tt < num_tokens;
  const int64_t t = live ? tt : num_tokens - 1;
  const float* zr = z + t * outputs;
  float mx = -INFINITY;
  for (int i = lane; i < outputs; i += 64) mx = fmaxf(mx, zr[i]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int i = lane; i < outputs; i += 64) {
    const float e = expf(zr[i] - mx);
    s[i] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  for (int i = lane; i < outputs; i += 64) {
    const float p = s[i] * inv;
    s[i] = p;
    ch[i] = p + (correction ? correction[i] : 0.f);
  }
  __syncthreads();
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < outputs; i += 64) {
      const float v = ch[i];
      if (v > bv) {
        bv = v;
        bi = i;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= outputs) bi = 0;                // every value was NaN: still a valid index
    if (lane == 0) {
      if (live) {
        ids[t * top + k] = bi;
        weights[t * top + k] = s[bi];
      }
      ch[bi] = -INFINITY;
    }
    __syncthreads();
  }
}

// Router whose weights are the softmax over the CHOSEN logits only: z + bias, the `top` largest are chosen (ties to the lower
// index), their weights are exp(z_k - max) / sum over the chosen.  One wave per token.
__global__ __launch_bounds__(256) void moe_route_topk_kernel(int32_t* __restrict__ ids, float* __restrict__ weights,
                                                             const float* __restrict__ z, const float* __restrict__ bias,
                                                             int64_t num_tokens, int outputs, int top) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* ch = lds + (size_t)wave * (outputs + top);
  float* we = ch + outputs;                     // the chosen logits' exponentials
  const int64_t tt = (int64_t)blockIdx.x * 4 + wave;
  const bool live = tt < num_tokens;
  const int64_t t = live ? tt : num_tokens - 1;
  const float* zr = z + t * outputs;
  for (int i = lane; i < outputs; i += 64) ch[i] = zr[i] + (bias ? bias[i] : 0.f);
  __syncthreads();
  float first = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < outputs; i += 64) {
      const float v = ch[i];
      if (v > bv) {
        bv = v;
        bi = i;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= outputs) bi = 0;                // every value was NaN: still a valid index
    if (k == 0) first = bv;                   // the first chosen is the largest
    const float e = expf(bv - first);
    sum += e;
    if (lane == 0) {
      if (live) ids[t * top + k] = bi;
      we[k] = e;
      ch[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (live)
    for (int k = lane; k < top; k += 64) weights[t * top + k] = we[k] / sum;
}

// Sigmoid router with a choice limited to the best groups of neighbouring experts; one wave per token.  s = sigmoid(z); a
// group's score is the sum of its `group_top` largest s; only experts of the `keep` best groups can be chosen; the `top`
// largest s among those are chosen and weighted by s * scale (not renormalised).  Ties go to the lower index.
__global__ __launch_bounds__(256) void moe_route_grouped_kernel(int32_t* __restrict__ ids, float* __restrict__ weights,
                                                                const float* __restrict__ z, int64_t num_tokens, int experts,
                                                                int top, int groups, int keep, int group_top, float scale) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* s = lds + (size_t)wave * (2 * experts + groups);
  float* ch = s + experts;
  float* gsc = ch + experts;
  const int64_t tt = (int64_t)blockIdx.x * 4 + wave;
  const bool live = tt < num_tokens;
  const int64_t t = live ? tt : num_tokens - 1;
  const float* zr = z + t * experts;
  const int gsz = experts / groups;
  for (int i = lane; i < experts; i += 64) {
    const float p = sigmoid_f(zr[i]);
    s[i] = p;
    ch[i] = -INFINITY;                        // not allowed until its group is kept
  }
  __syncthreads();
  for (int g = lane; g < groups; g += 64) {   // sum of the group's group_top largest, by repeated maximum
    float sum = 0.f;
    float last = INFINITY;
    int last_i = -1;
    for (int k = 0; k < group_top && k < gsz; ++k) {
      float bv = -INFINITY;
      int bi = -1;
      for (int i = 0; i < gsz; ++i) {
        const float v = s[g * gsz + i];
        const bool below = v < last || (v == last && i > last_i);      // after the previous pick in (value desc, index asc)
        if (below && v > bv) {
          bv = v;
          bi = i;
        }
      }
      if (bi < 0) break;
      sum += bv;
      last = bv;
      last_i = bi;
    }
    gsc[g] = sum;
  }
  __syncthreads();
  for (int k = 0; k < keep; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int g = lane; g < groups; g += 64) {
      const float v = gsc[g];
      if (v > bv) {
        bv = v;
        bi = g;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= groups) bi = 0;
    for (int i = lane; i < gsz; i += 64) ch[bi * gsz + i] = s[bi * gsz + i];
    if (lane == 0) gsc[bi] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < experts; i += 64) {
      const float v = ch[i];
      if (v > bv) {
        bv = v;
        bi = i;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (bi >= experts) bi = 0;
    if (lane == 0) {
      if (live) {
        ids[t * top + k] = bi;
        weights[t * top + k] = s[bi] * scale;
      }
      ch[bi] = -INFINITY;
    }
    __syncthreads();
  }
}

// one workgroup sorts every slot of the step
__global__ __launch_bounds__(1024) void moe_align_kernel(int32_t* __restrict__ sorted_slots, int32_t* __restrict__ block_expert,
                                                         int32_t* __restrict__ num_blocks, const int32_t* __restrict__ ids,
                                                         int64_t num_slots, int experts, int bm) {
  extern __shared__ int32_t li[];
  int32_t* count = li;
  int32_t* start = li + experts;
  __shared__ int32_t total;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < num_slots; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0;
    for (int e = 0; e < experts; ++e) {
      start[e] = off;
      off += (count[e] + bm - 1) / bm * bm;
    }
    total = off;
    num_blocks[0] = off / bm;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += blockDim.x) {
    const int nb = (count[e] + bm - 1) / bm;
    for (int j = 0; j < nb; ++j) block_expert[start[e] / bm + j] = e;
    count[e] = 0;                              // becomes the expert's cursor
  }
  for (int i = threadIdx.x; i < total; i += blockDim.x) sorted_slots[i] = -1;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < num_slots; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < experts) sorted_slots[start[e] + atomicAdd(&count[e], 1)] = (int32_t)i;
  }
}

// bf16 on v_mfma_f32_16x16x32_bf16: the weight rows are the A operand (16 output columns), the block's rows the B operand, so
// a lane ends with 4 consecutive output columns of one row.  A block is MT tiles of 16 rows; a wave owns all of them for 16
// output columns of the gated product (gate and up rows: 2 MT products per 32 of K from MT + 2 operand loads) or 32 columns of
// the down product, four waves per workgroup side by side along N.  Operands come straight from global memory in 16-byte
// pieces along K: with MT = 4 or 8 (prompt-sized steps, where an expert has hundreds of rows) every weight piece feeds MT
// products, with MT = 1 (decoded tokens: a handful of rows per expert) the weights are simply streamed once per block.
template <bool GLU, int MT>
__global__ __launch_bounds__(256) void moe_gemm_bf16_kernel(void* __restrict__ out, const uint16_t* __restrict__ a, int64_t a_stride,
                                                            const uint16_t* __restrict__ w, const int32_t* __restrict__ sorted_slots,
                                                            const int32_t* __restrict__ block_expert,
                                                            const int32_t* __restrict__ num_blocks, int top, int N, int K,
                                                            float limit, float alpha) {
  constexpr int BM = 16 * MT, NT = 2;                       // NT weight tiles per wave: (gate, up) of 16 columns, or 32 columns
  const int b = blockIdx.x;
  if (b >= num_blocks[0]) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  const int n0 = (blockIdx.y * 4 + wave) * (GLU ? 16 : 32);
  if (n0 >= N) return;
  const int e = block_expert[b];
  int slot[MT];
  const uint16_t* ar[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    slot[mt] = sorted_slots[b * BM + 16 * mt + c];
    if (GLU) ar[mt] = a + (int64_t)(slot[mt] >= 0 ? slot[mt] / top : 0) * a_stride + 8 * g;
    else ar[mt] = a + (int64_t)(b * BM + 16 * mt + c) * a_stride + 8 * g;
  }
  const bool second = GLU || n0 + 16 < N;                   // the down product's second tile may lie beyond N
  const uint16_t* w0 = w + ((int64_t)e * (GLU ? 2 : 1) * N + n0 + c) * K + 8 * g;
  const uint16_t* w1 = GLU ? w0 + (int64_t)N * K : (second ? w0 + (int64_t)16 * K : w0);
  f32x4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr int UNR = MT == 1 ? 8 : 2;                      // streaming weights: many pieces in flight per wave
#pragma unroll UNR
  for (int k0 = 0; k0 < K; k0 += 32) {
    const u32x4 wf0 = *reinterpret_cast<const u32x4*>(w0 + k0);
    const u32x4 wf1 = *reinterpret_cast<const u32x4*>(w1 + k0);
    u32x4 af[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) af[mt] = *reinterpret_cast<const u32x4*>(ar[mt] + k0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      acc[0][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf0), __builtin_bit_cast(bf16x8, af[mt]),
                                                           acc[0][mt], 0, 0, 0);
      acc[1][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf1), __builtin_bit_cast(bf16x8, af[mt]),
                                                           acc[1][mt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (GLU) {
      uint16_t* y = (uint16_t*)out + (int64_t)(b * BM + 16 * mt + c) * N + n0 + 4 * g;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = slot[mt] >= 0 ? clamped_glu_f(acc[0][mt][r], acc[1][mt][r], limit, alpha) : 0.f;
      *reinterpret_cast<u32x2*>(y) = u32x2{pack2_16<true>(v[0], v[1]), pack2_16<true>(v[2], v[3])};
    } else if (slot[mt] >= 0) {
      float* d = (float*)out + (int64_t)slot[mt] * N + n0 + 4 * g;
      *reinterpret_cast<f32x4*>(d) = acc[0][mt];
      if (second) *reinterpret_cast<f32x4*>(d + 16) = acc[1][mt];
    }
  }
}

// Prompt-sized steps, blocks of 128 rows: a workgroup owns the block's 128 rows x 128 weight rows (the gated product: 64 output
// columns, their gate rows and their up rows; the down product: 128 columns) and walks K in steps of 64: both tiles go through
// LDS (16-byte chunks XOR-swizzled by row so that the 16 rows of a fragment read hit different banks), the next step's pieces are
// in flight in registers while the current step's products run (fetching two steps ahead costs a third of the occupancy and
// measured 5-10 % slower).  Waves 2 x 2: 64 rows x 64 weight rows each, as 2 x 2 tiles of
// v_mfma_f32_32x32x16_bf16 (twice the multiply-adds per operand byte read from LDS of the 16 x 16 form, which measured 1.3 times
// slower here: LDS reads, not the matrix cores, were the limit).
constexpr int TG_BM = 128, TG_BN = 128, TG_BK = 64;
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_tiled_kernel(void* __restrict__ out, const uint16_t* __restrict__ a, int64_t a_stride,
                                                             const uint16_t* __restrict__ w, const int32_t* __restrict__ sorted_slots,
                                                             const int32_t* __restrict__ block_expert,
                                                             const int32_t* __restrict__ num_blocks, int top, int N, int K,
                                                             float limit, float alpha) {
  __shared__ __attribute__((aligned(16))) uint16_t a_lds[TG_BM * TG_BK];
  __shared__ __attribute__((aligned(16))) uint16_t w_lds[TG_BN * TG_BK];
  __shared__ int32_t slot_lds[TG_BM];
  // Workgroups go to the 8 XCDs round-robin by their linear index and each XCD has its own L2.  XCD x takes the column groups
  // x, x + 8, ... of every block, block after block: the few weight tiles of its column groups stay in its L2 over all blocks
  // of an expert, and a block's rows are fetched once per XCD by workgroups that run side by side.
  const int ncols = GLU ? TG_BN / 2 : TG_BN;               // output columns of the workgroup
  const int ny = (N + ncols - 1) / ncols, nyx = (ny + 7) / 8;
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int b = seq / nyx, y = (seq % nyx) * 8 + xcd;
  if (b >= num_blocks[0] || y >= ny) return;
  const int e = block_expert[b];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int n0 = y * ncols;
  if (threadIdx.x < TG_BM) slot_lds[threadIdx.x] = sorted_slots[b * TG_BM + threadIdx.x];
  // this thread's pieces of the two tiles: 4 + 4 chunks of 16 bytes per K step
  const uint16_t* ap[4];
  const uint16_t* wp[4];
  int lds_at[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = threadIdx.x + 256 * i, row = idx >> 3, ch = idx & 7;
    lds_at[i] = row * TG_BK + 8 * (ch ^ (row & 7));
    if (GLU) {
      const int slot = sorted_slots[b * TG_BM + row];
      ap[i] = a + (int64_t)(slot >= 0 ? slot / top : 0) * a_stride + 8 * ch;
      const int col = min(n0 + (row & 63), N - 1);          // weight rows 0..63: gate, 64..127: up, of the same columns
      wp[i] = w + ((int64_t)e * 2 * N + (row < 64 ? 0 : N) + col) * K + 8 * ch;
    } else {
      ap[i] = a + (int64_t)(b * TG_BM + row) * a_stride + 8 * ch;
      wp[i] = w + ((int64_t)e * N + min(n0 + row, N - 1)) * K + 8 * ch;
    }
  }
  f32x16 acc[2][2];                                         // [row tile of 32][weight tile of 32]
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;
  u32x4 ra[4], rw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ra[i] = *reinterpret_cast<const u32x4*>(ap[i]);
    rw[i] = *reinterpret_cast<const u32x4*>(wp[i]);
  }
  const int l31 = lane & 31, lh = lane >> 5;
  for (int k0 = 0; k0 < K; k0 += TG_BK) {
    __syncthreads();                                        // the previous step is consumed
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<u32x4*>(&a_lds[lds_at[i]]) = ra[i];
      *reinterpret_cast<u32x4*>(&w_lds[lds_at[i]]) = rw[i];
    }
    __syncthreads();
    if (k0 + TG_BK < K) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        ra[i] = *reinterpret_cast<const u32x4*>(ap[i] + k0 + TG_BK);
        rw[i] = *reinterpret_cast<const u32x4*>(wp[i] + k0 + TG_BK);
      }
    }
    // v_mfma_f32_32x32x16_bf16: a lane brings row (lane & 31), k = 8 (lane >> 5) .. + 7 of each operand
#pragma unroll
    for (int kk = 0; kk < TG_BK / 16; ++kk) {
      u32x4 af[2], wf[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int row = 64 * wm + 32 * mt + l31;
        af[mt] = *reinterpret_cast<const u32x4*>(&a_lds[row * TG_BK + 8 * ((2 * kk + lh) ^ (row & 7))]);
      }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        // the gated product: weight tile wn holds gate rows, tile 2 + wn the up rows of the same 32 columns
        const int row = 32 * (GLU ? 2 * nt + wn : 2 * wn + nt) + l31;
        wf[nt] = *reinterpret_cast<const u32x4*>(&w_lds[row * TG_BK + 8 * ((2 * kk + lh) ^ (row & 7))]);
      }
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wf[nt]), __builtin_bit_cast(bf16x8, af[mt]),
                                                                acc[mt][nt], 0, 0, 0);
    }
  }
  // a lane holds, per (row tile, weight tile) and quad q, the 4 consecutive weight rows 8 q + 4 (lane >> 5) .. + 3 of block row
  // 64 wm + 32 mt + (lane & 31)
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
    const int row = 64 * wm + 32 * mt + l31;
    const int slot = slot_lds[row];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (GLU) {
        const int col = n0 + 32 * wn + 8 * q + 4 * lh;
        if (col >= N) continue;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          v[r] = slot >= 0 ? clamped_glu_f(acc[mt][0][4 * q + r], acc[mt][1][4 * q + r], limit, alpha) : 0.f;
        *reinterpret_cast<u32x2*>((uint16_t*)out + (int64_t)(b * TG_BM + row) * N + col) =
            u32x2{pack2_16<true>(v[0], v[1]), pack2_16<true>(v[2], v[3])};
      } else if (slot >= 0) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          const int col = n0 + 64 * wn + 32 * nt + 8 * q + 4 * lh;
          if (col < N)
            *reinterpret_cast<f32x4*>((float*)out + (int64_t)slot * N + col) =
                f32x4{acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1], acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
        }
      }
    }
  }
}

// any storage type and size: thread = one output element of the block, fp32 multiply-adds along K
template <typename T, bool GLU>
__global__ __launch_bounds__(256) void moe_gemm_plain_kernel(void* __restrict__ out, const typename T::storage* __restrict__ a,
                                                             int64_t a_stride, const typename T::storage* __restrict__ w,
                                                             const int32_t* __restrict__ sorted_slots,
                                                             const int32_t* __restrict__ block_expert,
                                                             const int32_t* __restrict__ num_blocks, int top, int N, int K,
                                                             float limit, float alpha, int bm) {
  const int row = blockIdx.x * 16 + (threadIdx.x & 15);     // row of sorted_slots; a block of bm rows has one expert
  if (row >= num_blocks[0] * bm) return;
  const int n = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (n >= N) return;
  const int e = block_expert[row / bm];
  const int slot = sorted_slots[row];
  if (slot < 0) {
    if (GLU) ((typename T::storage*)out)[(int64_t)row * N + n] = T::from_f32(0.f);
    return;
  }
  const typename T::storage* ar = GLU ? a + (int64_t)(slot / top) * a_stride : a + (int64_t)row * a_stride;
  const typename T::storage* w0 = w + ((int64_t)e * (GLU ? 2 : 1) * N + n) * K;
  const typename T::storage* w1 = w0 + (int64_t)N * K;
  float acc0 = 0.f, acc1 = 0.f;
  for (int k = 0; k < K; ++k) {
    const float x = T::to_f32(ar[k]);
    acc0 += x * T::to_f32(w0[k]);
    if (GLU) acc1 += x * T::to_f32(w1[k]);
  }
  if (GLU) ((typename T::storage*)out)[(int64_t)row * N + n] = T::from_f32(clamped_glu_f(acc0, acc1, limit, alpha));
  else ((float*)out)[(int64_t)slot * N + n] = acc0;
}

constexpr int MOE_MAX_TOP = 64;

// one workgroup per token; its choices and weights are read once into LDS, the columns go 4 at a time where rows are 16-byte
// aligned (VEC), every choice's piece requested before the first is used
template <typename T, bool VEC>
__global__ void moe_combine_kernel(typename T::storage* __restrict__ out, const float* __restrict__ expert_out,
                                   const int32_t* __restrict__ ids, const float* __restrict__ weights,
                                   const typename T::storage* __restrict__ h, int64_t h_stride,
                                   const typename T::storage* __restrict__ shared, int64_t shared_stride,
                                   const typename T::storage* __restrict__ shared_gate, int64_t shared_gate_stride, int width,
                                   int top, int experts) {
  __shared__ int32_t sid[MOE_MAX_TOP];
  __shared__ float sw[MOE_MAX_TOP];
  const int64_t t = blockIdx.x;
  if ((int)threadIdx.x < top) {
    sid[threadIdx.x] = ids[t * top + threadIdx.x];
    sw[threadIdx.x] = weights[t * top + threadIdx.x];
  }
  const float sg = (shared && shared_gate) ? sigmoid_f(T::to_f32(shared_gate[t * shared_gate_stride])) : 1.0f;
  __syncthreads();
  const float* eo = expert_out + t * top * (int64_t)width;
  if constexpr (VEC) {
    for (int i = 4 * threadIdx.x; i < width; i += 4 * blockDim.x) {
      float hv[4], acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) hv[j] = T::to_f32(h[t * h_stride + i + j]);
#pragma unroll 4
      for (int k = 0; k < top; ++k) {
        const float wk = sw[k];
        if (sid[k] < experts) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(eo + (int64_t)k * width + i);
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] += wk * v[j];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] += wk * hv[j];
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (shared) acc[j] += sg * T::to_f32(shared[t * shared_stride + i + j]);
        out[t * (int64_t)width + i + j] = T::from_f32(acc[j]);
      }
    }
  } else {
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float hv = T::to_f32(h[t * h_stride + i]);
      float acc = 0.f;
      for (int k = 0; k < top; ++k) acc += sw[k] * (sid[k] < experts ? eo[(int64_t)k * width + i] : hv);
      if (shared) acc += sg * T::to_f32(shared[t * shared_stride + i]);
      out[t * (int64_t)width + i] = T::from_f32(acc);
    }
  }
}

template <typename T>
__global__ void clamped_glu_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ in,
                                   int64_t in_stride, int d, float limit, float alpha) {
  const int64_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= d) return;
  out[t * (int64_t)d + i] = T::from_f32(clamped_glu_f(T::to_f32(in[t * in_stride + i]), T::to_f32(in[t * in_stride + d + i]), limit, alpha));
}

// 8 neighbouring elements per thread where the rows allow 16-byte accesses
template <typename T>
__global__ void clamped_glu_vec8_kernel(typename T::storage* __restrict__ out, const typename T::storage* __restrict__ in,
                                        int64_t in_stride, int d, float limit, float alpha) {
  const int64_t t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= d) return;
  float g[8], u[8];
  if constexpr (sizeof(typename T::storage) == 2) {
    const u16x8 gv = *reinterpret_cast<const u16x8*>(in + t * in_stride + i), uv = *reinterpret_cast<const u16x8*>(in + t * in_stride + d + i);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      g[j] = T::to_f32(gv[j]);
      u[j] = T::to_f32(uv[j]);
    }
    u16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = T::from_f32(clamped_glu_f(g[j], u[j], limit, alpha));
    *reinterpret_cast<u16x8*>(out + t * (int64_t)d + i) = r;
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const f32x4 gv = *reinterpret_cast<const f32x4*>(in + t * in_stride + i + 4 * h);
      const f32x4 uv = *reinterpret_cast<const f32x4*>(in + t * in_stride + d + i + 4 * h);
      f32x4 r;
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = clamped_glu_f(gv[j], uv[j], limit, alpha);
      *reinterpret_cast<f32x4*>(out + t * (int64_t)d + i + 4 * h) = r;
    }
  }
}

}  // namespace aphro

using namespace aphro;

extern "C" int aphro_experts_route(int32_t* ids, float* weights, const float* router_out, const float* correction,
                               int64_t num_tokens, int outputs, int top, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(ids && weights && router_out && outputs > 0 && top > 0 && top <= outputs && outputs <= 2048,
              "moe_route: %d router outputs (<= 2048), top %d", outputs, top);
  hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)((num_tokens + 3) / 4)), dim3(256), (size_t)8 * outputs * sizeof(float),
                     (hipStream_t)stream, ids, weights, router_out, correction, num_tokens, outputs, top);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_experts_route_topk(int32_t* ids, float* weights, const float* router_out, const float* bias, int64_t num_tokens,
                                        int outputs, int top, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(ids && weights && router_out && outputs > 0 && top > 0 && top <= outputs && outputs <= 2048,
              "moe_route_topk: %d router outputs (<= 2048), top %d", outputs, top);
  hipLaunchKernelGGL(moe_route_topk_kernel, dim3((unsigned)((num_tokens + 3) / 4)), dim3(256), (size_t)4 * (outputs + top) * sizeof(float),
                     (hipStream_t)stream, ids, weights, router_out, bias, num_tokens, outputs, top);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_experts_route_grouped(int32_t* ids, float* weights, const float* router_out, int64_t num_tokens, int experts,
                                           int top, int groups, int keep, int group_top, float scale, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(ids && weights && router_out && experts > 0 && experts <= 2048 && groups > 0 && experts % groups == 0 && keep > 0 &&
                  keep <= groups && group_top > 0 && top > 0 && top <= keep * (experts / groups),
              "moe_route_grouped: %d experts (<= 2048) in %d groups of which %d are kept, top %d", experts, groups, keep, top);
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((unsigned)((num_tokens + 3) / 4)), dim3(256),
                     (size_t)4 * (2 * experts + groups) * sizeof(float), (hipStream_t)stream, ids, weights, router_out, num_tokens,
                     experts, top, groups, keep, group_top, scale);
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

// rows per block: 16 for a handful of rows per expert, 64 / 128 where an expert has hundreds (the prompt-sized products then
// reuse every weight piece 4 / 8 times)
extern "C" int aphro_experts_block_rows(int64_t num_slots, int experts) {
  const int64_t per = num_slots / (experts > 0 ? experts : 1);
  return per >= 512 ? 128 : (per >= 48 ? 64 : MOE_BM);
}

extern "C" int64_t aphro_experts_align_capacity(int64_t num_slots, int experts) {
  const int bm = aphro_experts_block_rows(num_slots, experts);
  return (num_slots + (int64_t)experts * (bm - 1) + bm - 1) / bm * bm;
}

extern "C" int aphro_experts_align(int32_t* sorted_slots, int64_t capacity, int32_t* block_expert, int32_t* num_blocks,
                                   const int32_t* ids, int64_t num_slots, int experts, void* stream) {
  APHRO_CHECK(sorted_slots && block_expert && num_blocks && ids && num_slots > 0 && experts > 0 && experts <= 4096,
              "experts_align: bad arguments (%d experts)", experts);
  APHRO_CHECK(capacity >= aphro_experts_align_capacity(num_slots, experts) && capacity < 0x7fffffff, "experts_align: capacity too small");
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)2 * experts * sizeof(int32_t), (hipStream_t)stream,
                     sorted_slots, block_expert, num_blocks, ids, num_slots, experts, aphro_experts_block_rows(num_slots, experts));
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

template <bool GLU>
static void moe_gemm_bf16_launch(int bm, dim3 grid, hipStream_t st, void* out, const uint16_t* a, int64_t a_stride, const uint16_t* w,
                                 const int32_t* sorted_slots, const int32_t* block_expert, const int32_t* num_blocks, int top, int N,
                                 int K, float limit, float alpha) {
  if (bm == 128)
    hipLaunchKernelGGL((moe_gemm_bf16_kernel<GLU, 8>), grid, dim3(256), 0, st, out, a, a_stride, w, sorted_slots, block_expert,
                       num_blocks, top, N, K, limit, alpha);
  else if (bm == 64)
    hipLaunchKernelGGL((moe_gemm_bf16_kernel<GLU, 4>), grid, dim3(256), 0, st, out, a, a_stride, w, sorted_slots, block_expert,
                       num_blocks, top, N, K, limit, alpha);
  else
    hipLaunchKernelGGL((moe_gemm_bf16_kernel<GLU, 1>), grid, dim3(256), 0, st, out, a, a_stride, w, sorted_slots, block_expert,
                       num_blocks, top, N, K, limit, alpha);
}

static int moe_gemm(bool glu, void* out, const void* a, int64_t a_stride, const void* w, const int32_t* sorted_slots,
                    const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int64_t num_slots, int experts, int top,
                    int N, int K, float limit, float alpha, int dtype, void* stream) {
  const int bm = aphro_experts_block_rows(num_slots, experts);
  APHRO_CHECK(out && a && w && sorted_slots && block_expert && num_blocks && capacity > 0 && capacity % bm == 0 && top > 0 &&
                  N > 0 && K > 0 && a_stride >= K && capacity == aphro_experts_align_capacity(num_slots, experts),
              "experts gemm: bad arguments");
  const bool mfma = dtype == APHRO_BF16 && N % 16 == 0 && K % 32 == 0 && a_stride % 8 == 0 && ((uintptr_t)a & 15) == 0 &&
                    ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0;
  if (mfma && bm == TG_BM && K % TG_BK == 0 && N % 4 == 0) {
    const int64_t ny = (N + (glu ? 63 : 127)) / (glu ? 64 : 128);
    const dim3 grid((unsigned)(8 * (capacity / bm) * ((ny + 7) / 8)));
    if (glu)
      hipLaunchKernelGGL((moe_gemm_tiled_kernel<true>), grid, dim3(256), 0, (hipStream_t)stream, out, (const uint16_t*)a, a_stride,
                         (const uint16_t*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha);
    else
      hipLaunchKernelGGL((moe_gemm_tiled_kernel<false>), grid, dim3(256), 0, (hipStream_t)stream, out, (const uint16_t*)a, a_stride,
                         (const uint16_t*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha);
  } else if (mfma) {
    const dim3 grid((unsigned)(capacity / bm), (unsigned)((N + (glu ? 63 : 127)) / (glu ? 64 : 128)));
    if (glu)
      moe_gemm_bf16_launch<true>(bm, grid, (hipStream_t)stream, out, (const uint16_t*)a, a_stride, (const uint16_t*)w, sorted_slots,
                                 block_expert, num_blocks, top, N, K, limit, alpha);
    else
      moe_gemm_bf16_launch<false>(bm, grid, (hipStream_t)stream, out, (const uint16_t*)a, a_stride, (const uint16_t*)w, sorted_slots,
                                  block_expert, num_blocks, top, N, K, limit, alpha);
  } else {
    const dim3 grid((unsigned)(capacity / 16), (unsigned)((N + 15) / 16));
    MIX_DISPATCH_DTYPE(dtype, {
      typedef typename T::storage S;
      if (glu)
        hipLaunchKernelGGL((moe_gemm_plain_kernel<T, true>), grid, dim3(256), 0, (hipStream_t)stream, out, (const S*)a, a_stride,
                           (const S*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha, bm);
      else
        hipLaunchKernelGGL((moe_gemm_plain_kernel<T, false>), grid, dim3(256), 0, (hipStream_t)stream, out, (const S*)a, a_stride,
                           (const S*)w, sorted_slots, block_expert, num_blocks, top, N, K, limit, alpha, bm);
    });
  }
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_experts_glu_gemm(void* y, const void* h, int64_t h_stride, const void* w_gate_up, const int32_t* sorted_slots,
                                  const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int64_t num_slots,
                                  int experts, int top, int ff, int width, float limit, float alpha, int dtype, void* stream) {
  return moe_gemm(true, y, h, h_stride, w_gate_up, sorted_slots, block_expert, num_blocks, capacity, num_slots, experts, top, ff,
                  width, limit, alpha, dtype, stream);
}

extern "C" int aphro_experts_down_gemm(float* expert_out, const void* y, const void* w_down, const int32_t* sorted_slots,
                                   const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int64_t num_slots,
                                   int experts, int top, int width, int ff, int dtype, void* stream) {
  return moe_gemm(false, expert_out, y, ff, w_down, sorted_slots, block_expert, num_blocks, capacity, num_slots, experts, top, width,
                  ff, 0.f, 0.f, dtype, stream);
}

extern "C" int aphro_experts_combine(void* out, const float* expert_out, const int32_t* ids, const float* weights, const void* h,
                                 int64_t h_stride, const void* shared, int64_t shared_stride, const void* shared_gate,
                                 int64_t shared_gate_stride, int64_t num_tokens, int width, int top, int experts, int dtype,
                                 void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && expert_out && ids && weights && h && width > 0 && top > 0 && experts >= 0 && h_stride >= width &&
                  (!shared || shared_stride >= width), "moe_combine: bad arguments");
  APHRO_CHECK(top <= MOE_MAX_TOP, "experts_combine: top %d (<= %d)", top, MOE_MAX_TOP);
  const bool vec = width % 4 == 0 && ((uintptr_t)expert_out & 15) == 0;
  const int threads = width >= 1024 ? 256 : (width >= 512 ? 128 : 64);
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec)
      hipLaunchKernelGGL((moe_combine_kernel<T, true>), dim3((unsigned)num_tokens), dim3(threads), 0, (hipStream_t)stream, (S*)out,
                         expert_out, ids, weights, (const S*)h, h_stride, (const S*)shared, shared_stride, (const S*)shared_gate,
                         shared_gate_stride, width, top, experts);
    else
      hipLaunchKernelGGL((moe_combine_kernel<T, false>), dim3((unsigned)num_tokens), dim3(threads), 0, (hipStream_t)stream, (S*)out,
                         expert_out, ids, weights, (const S*)h, h_stride, (const S*)shared, shared_stride, (const S*)shared_gate,
                         shared_gate_stride, width, top, experts);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}

extern "C" int aphro_clamped_glu(void* out, const void* in, int64_t in_stride, int64_t num_tokens, int d, float limit, float alpha,
                                 int dtype, void* stream) {
  if (num_tokens == 0) return APHRO_OK;
  APHRO_CHECK(out && in && d > 0 && in_stride >= 2 * (int64_t)d && num_tokens <= 0x7fffffff && (d + 255) / 256 <= 65535,
              "clamped_glu: bad arguments");
  const bool vec = d % 8 == 0 && in_stride % 8 == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0;
  MIX_DISPATCH_DTYPE(dtype, {
    typedef typename T::storage S;
    if (vec)
      hipLaunchKernelGGL((clamped_glu_vec8_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((d / 8 + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, (S*)out, (const S*)in, in_stride, d, limit, alpha);
    else
      hipLaunchKernelGGL((clamped_glu_kernel<T>), dim3((unsigned)num_tokens, (unsigned)((d + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, (S*)out, (const S*)in, in_stride, d, limit, alpha);
  });
  APHRO_LAUNCH_CHECK();
  return APHRO_OK;
}
