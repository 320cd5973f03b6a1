// Mixture of experts: softmax- or sigmoid-top-k router, the sort of (token, choice) pairs by expert that feeds the grouped GEMMs
// (stream32.hip gemm_any, `tiles` form), and the weighted combine with an optional gated shared expert.
#include "common.h"

namespace k8sllm {

// One wave per token.  mode 0: s = softmax(logits[t, :E]) in fp32, weights s_k / (sum of the chosen s + 1e-20) * scale;
// mode 1: s = sigmoid(logits), weights s_k * scale (not renormalised).  `top` rounds of arg-max (ties: the lowest index).
__global__ __launch_bounds__(64) void moe_route_kernel(int* __restrict__ idx, float* __restrict__ w,
                                                       const float* __restrict__ logits, int ld, int E, int top,
                                                       float scale, int mode) {
  extern __shared__ float sc[];   // [E] scores, then [top] chosen scores
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* z = logits + (size_t)t * ld;
  float sum = 1.f;
  if (mode == 1) {
    for (int e = lane; e < E; e += 64) sc[e] = 1.f / (1.f + expf(-z[e]));
  } else {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float v = expf(z[e] - mx);
      sc[e] = v;
      sum += v;
    }
    sum = wave_sum(sum);
  }
  __syncthreads();
  float chosen_sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -1.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > bv) {   // ascending e within a lane: the first maximum wins
        bv = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, WAVE);
      const int oi = __shfl_xor(bi, o, WAVE);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    const float s = bv / sum;
    chosen_sum += s;
    if (lane == 0) {
      idx[(size_t)t * top + k] = bi;
      sc[E + k] = s;
      sc[bi] = -2.f;
    }
    __syncthreads();
  }
  const float norm = mode == 1 ? 1.f : 1.f / (chosen_sum + 1e-20f);
  for (int k = lane; k < top; k += 64) w[(size_t)t * top + k] = sc[E + k] * norm * scale;
}

// One workgroup.  Pairs p = t * top + k are sorted by expert (any order inside an expert: rows are independent):
// sorted_tok[row] = token of the row, pos_of_pair[p] = row, seg[e] = first row of expert e, and the row tiles
// (expert, first row, rows <= BM) of every expert, padded with expert -1 up to ntiles.
__global__ __launch_bounds__(1024) void moe_align_kernel(int* __restrict__ sorted_tok, int* __restrict__ pos_of_pair,
                                                         int* __restrict__ seg, int* __restrict__ tiles, int ntiles,
                                                         const int* __restrict__ topk_idx, int P, int top, int E,
                                                         int BM) {
  extern __shared__ int sm[];   // cnt[E], off[E], used
  int* cnt = sm;
  int* off = sm + E;
  int* used = sm + 2 * E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    int e = topk_idx[p];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      seg[e] = run;
      off[e] = run;
      for (int r0 = 0; r0 < cnt[e] && nt < ntiles; r0 += BM, ++nt) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = run + r0;
        tiles[3 * nt + 2] = min(BM, cnt[e] - r0);
      }
      run += cnt[e];
    }
    seg[E] = run;
    *used = nt;
  }
  __syncthreads();
  for (int i = *used + threadIdx.x; i < ntiles; i += blockDim.x) {
    tiles[3 * i] = -1;
    tiles[3 * i + 1] = 0;
    tiles[3 * i + 2] = 0;
  }
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    int e = topk_idx[p];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    const int row = atomicAdd(&off[e], 1);
    sorted_tok[row] = p / top;
    pos_of_pair[p] = row;
  }
}

// z[t] = sum_k w[t, k] D[pos[t, k]] + gate_t * shared[t], gate_t = sigmoid(logits[t, sg_col]) (sg_col < 0: 1);
// w == null: plain sum (experts whose weight was applied to their input).
template <typename TA>
__global__ void moe_combine_kernel(TA* __restrict__ z, const TA* __restrict__ D, const int* __restrict__ pos,
                                   const float* __restrict__ w, const TA* __restrict__ shared,
                                   const float* __restrict__ logits, int ld, int sg_col, int W, int top) {
  const int t = blockIdx.x;
  float gate = 1.f;
  if (shared != nullptr && sg_col >= 0) gate = 1.f / (1.f + expf(-logits[(size_t)t * ld + sg_col]));
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float a = 0.f;
    for (int k = 0; k < top; ++k)
      a = fmaf(w != nullptr ? w[(size_t)t * top + k] : 1.f, ldf(D, (size_t)pos[(size_t)t * top + k] * W + i), a);
    if (shared != nullptr) a = fmaf(gate, ldf(shared, (size_t)t * W + i), a);
    stf(z, (size_t)t * W + i, a);
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_moe_route(int* idx, float* w, const float* logits, int ld, int T, int E, int top, float scale,
                             int mode, hipStream_t s) {
  if (T <= 0) return 0;
  if (E <= 0 || top <= 0 || top > E || E > 8192 || mode < 0 || mode > 1) return -1;
  moe_route_kernel<<<T, 64, (size_t)(E + top) * sizeof(float), s>>>(idx, w, logits, ld, E, top, scale, mode);
  return (int)hipGetLastError();
}

extern "C" int k8s_moe_align(int* sorted_tok, int* pos_of_pair, int* seg, int* tiles, int ntiles, const int* topk_idx,
                             int P, int top, int E, int BM, hipStream_t s) {
  if (P <= 0) return 0;
  if (E <= 0 || E > 4096 || BM <= 0 || ntiles < (P + BM - 1) / BM + E) return -1;
  moe_align_kernel<<<1, 1024, (size_t)(2 * E + 1) * sizeof(int), s>>>(sorted_tok, pos_of_pair, seg, tiles, ntiles,
                                                                     topk_idx, P, top, E, BM);
  return (int)hipGetLastError();
}

extern "C" int k8s_moe_combine(void* z, const void* D, const int* pos, const float* w, const void* shared,
                               const float* logits, int ld, int sg_col, int T, int W, int top, int f32,
                               hipStream_t s) {
  if (T <= 0) return 0;
  if (W <= 0 || top <= 0) return -1;
  if (f32)
    moe_combine_kernel<float><<<T, 256, 0, s>>>((float*)z, (const float*)D, pos, w, (const float*)shared, logits, ld,
                                                sg_col, W, top);
  else
    moe_combine_kernel<bf16_t><<<T, 256, 0, s>>>((bf16_t*)z, (const bf16_t*)D, pos, w, (const bf16_t*)shared, logits,
                                                 ld, sg_col, W, top);
  return (int)hipGetLastError();
}
