// Grouped-query sliding-window attention over a paged K / V cache, with pooled far context:
//   * the token at position p sees the cached tokens of positions max(0, p - window + 1) .. p and, beside them, one
//     key / value per block of P consecutive tokens that lies wholly before the window (block b = positions
//     b P .. b P + P - 1, seen when b P + P - 1 <= p - window): the mean of the block's cached keys / values;
//   * tokens and blocks share one softmax, optionally with a sink (a key of score 0 without a value: one more unit
//     in the denominator);
//   * queries and keys are prepared by one kernel per token: bias, interleaved-pair rotation of the first `dims`
//     dimensions, optional unit RMS per head, value mixing with another layer's values, paged cache write.
// Varlen batches as in mixers.hip: positions[t] < 0 marks an idle row that touches nothing.
#include "common.h"

namespace k8sllm {

// LDS written by some lanes of a wave is read by other lanes of the same wave: order the accesses.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One workgroup per token, one wave per head vector (H query heads, then G key heads; further passes when there are
// more vectors than waves).  x = proj + bias; (x[2i], x[2i + 1]) turns by the angle of cos_sin[pos] = [cos(dims / 2) |
// sin(dims / 2)]; then x / sqrt(mean(x^2) + eps) when `unit`.  Queries are written back in place, keys to
// kcache[slot][g][D].  Values: v = proj + bias, then (vfirst_in) v = (1 - lam) v + lam vfirst_in[t]; (vfirst_out)
// vfirst_out[t] = v in fp32; vcache[slot][g][V] = v.
template <typename TA>
__global__ __launch_bounds__(256) void window_kv_write_kernel(
    TA* __restrict__ kcache, TA* __restrict__ vcache, TA* __restrict__ qkv, long ld, int koff, int voff,
    const TA* __restrict__ qb, const TA* __restrict__ kb, const TA* __restrict__ vb, const float* __restrict__ cos_sin,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping, const float* __restrict__ vfirst_in,
    float* __restrict__ vfirst_out, float lam, int H, int G, int D, int V, int dims, float eps, int unit) {
  extern __shared__ float xs[];   // [waves][D]
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int slot = slot_mapping[t];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = blockDim.x >> 6;
  const int half = dims / 2;
  const float* cs = cos_sin + (size_t)pos * dims;
  TA* row = qkv + (size_t)t * ld;
  float* x = xs + (size_t)wave * D;
  for (int hv = wave; hv < H + G; hv += nw) {
    const bool isq = hv < H;
    const int hd = isq ? hv : hv - H;
    const TA* src = row + (isq ? 0 : koff) + (size_t)hd * D;
    const TA* bias = isq ? qb : kb;
    for (int d = lane; d < D; d += 64) x[d] = ldf(src, d) + (bias != nullptr ? ldf(bias, (size_t)hd * D + d) : 0.f);
    wave_lds_sync();
    float ss = 0.f;
    float y[8];   // D <= 512
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      const int d = lane + 64 * n;
      float v = 0.f;
      if (d < D) {
        v = x[d];
        if (d < dims) {
          const int i = d >> 1;
          const float c = cs[i], sn = cs[half + i];
          const float a = x[d & ~1], b = x[d | 1];
          v = (d & 1) ? b * c + a * sn : a * c - b * sn;
        }
      }
      y[n] = v;
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = unit ? 1.0f / sqrtf(ss / (float)D + eps) : 1.f;
    TA* dst = isq ? row + (size_t)hd * D : (slot >= 0 ? kcache + ((size_t)slot * G + hd) * D : nullptr);
    wave_lds_sync();   // every lane has read its partners before the query row (the source) is overwritten
    if (dst != nullptr) {
#pragma unroll
      for (int n = 0; n < 8; ++n) {
        const int d = lane + 64 * n;
        if (d < D) stf(dst, d, y[n] * inv);
      }
    }
  }
  for (int i = tid; i < G * V; i += blockDim.x) {
    float v = ldf(row + voff, i) + (vb != nullptr ? ldf(vb, i) : 0.f);
    if (vfirst_in != nullptr) v = (1.f - lam) * v + lam * vfirst_in[(size_t)t * G * V + i];
    if (vfirst_out != nullptr) vfirst_out[(size_t)t * G * V + i] = v;
    if (slot >= 0) stf(vcache, (size_t)slot * G * V + i, v);
  }
}

// Entry of pooled block b of a sequence: the block lives with the page that holds its first token.  A page of bs
// tokens holds the first token of at most ppb = ceil(bs / P) blocks.
__device__ __forceinline__ size_t pool_entry(const int* btr, int b, int P, int bs, int ppb) {
  const int page = (int)(((long)b * P) / bs);
  const int first = (int)(((long)page * bs + P - 1) / P);   // the first block that starts in this page
  return (size_t)btr[page] * ppb + (b - first);
}

// One workgroup per token; works only for tokens that end a block of P ((pos + 1) % P == 0): the mean, in fp32, of the
// P cached keys and values (as the cache holds them) -> kpool / vpool [pages * ppb][G][D or V] fp32.  Runs after the
// cache write of the same batch, so the block's earlier tokens are in the cache whether this batch or an earlier one
// brought them.
template <typename TA>
__global__ __launch_bounds__(256) void window_pool_kernel(float* __restrict__ kpool, float* __restrict__ vpool,
                                                          const TA* __restrict__ kcache, const TA* __restrict__ vcache,
                                                          const int* __restrict__ block_tables, int max_blocks,
                                                          const int* __restrict__ tok_seq,
                                                          const int* __restrict__ positions, int G, int D, int V, int P,
                                                          int bs, int ppb) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0 || (pos + 1) % P != 0) return;
  const int b = pos / P;
  const int* btr = block_tables + (size_t)tok_seq[t] * max_blocks;
  const size_t e = pool_entry(btr, b, P, bs, ppb);
  const float invp = 1.0f / (float)P;
  const int GD = G * D, GV = G * V;
  for (int i = threadIdx.x; i < GD + GV; i += blockDim.x) {
    float a = 0.f;
    for (int j = b * P; j < b * P + P; ++j) {
      const size_t slot = (size_t)btr[j / bs] * bs + (j % bs);
      a += i < GD ? ldf(kcache, slot * GD + i) : ldf(vcache, slot * GV + (i - GD));
    }
    if (i < GD) kpool[e * GD + i] = a * invp;
    else vpool[e * GV + (i - GD)] = a * invp;
  }
}

// One workgroup per (token, key / value head); one wave per query head of the group (further passes when the group has
// more heads than waves).  The visible keys are an ordered list: the nb pooled blocks, then the window's tokens.  They
// come in tiles of KB <= 64 rows staged in LDS as fp32 and shared by the group's heads; lane l scores row l
// (q . k * scale), the tile joins a running softmax, lane l accumulates value dimensions l, l + 64, ...
// A sink starts the running softmax at (max 0, sum 1).  out[t][head][V] = sum p v / sum, times sigmoid(gate) if given.
template <typename TA, int NACC>
__global__ void window_attention_kernel(TA* __restrict__ out, const TA* __restrict__ q, long ldq,
                                        const TA* __restrict__ gate, long ldg, const TA* __restrict__ kcache,
                                        const TA* __restrict__ vcache, const float* __restrict__ kpool,
                                        const float* __restrict__ vpool, const int* __restrict__ block_tables,
                                        int max_blocks, const int* __restrict__ tok_seq,
                                        const int* __restrict__ positions, int H, int G, int D, int V, int window,
                                        int P, float scale, int sink, int bs, int ppb, int KB) {
  extern __shared__ float smem[];
  const int t = blockIdx.x, g = blockIdx.y;
  const int R = H / G;
  const int p = positions[t];
  if (p < 0) {   // idle row: defined output, nothing read
    for (int i = threadIdx.x; i < R * V; i += blockDim.x) stf(out, (size_t)t * H * V + (size_t)g * R * V + i, 0.f);
    return;
  }
  const int DP = D + 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = blockDim.x >> 6;
  float* ktile = smem;                         // [KB][D + 1]
  float* vtile = ktile + (size_t)KB * DP;      // [KB][V]
  float* qs = vtile + (size_t)KB * V;          // [nw][D]
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int nb = (window > 0 && P > 0 && p - window + 1 >= P) ? (p - window + 1) / P : 0;
  const int nkeys = nb + (p + 1 - lo);
  const int* btr = block_tables + (size_t)tok_seq[t] * max_blocks;
  const int GD = G * D, GV = G * V;
  for (int h0 = 0; h0 < R; h0 += nw) {
    const int hd = g * R + h0 + wave;
    const bool hv = h0 + wave < R;
    float* qq = qs + (size_t)wave * D;
    if (hv)
      for (int d = lane; d < D; d += 64) qq[d] = ldf(q, (size_t)t * ldq + (size_t)hd * D + d);
    float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f, acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    for (int u0 = 0; u0 < nkeys; u0 += KB) {
      const int nk = min(KB, nkeys - u0);
      __syncthreads();
      for (int idx = tid; idx < nk * (D + V); idx += blockDim.x) {
        const int r = idx / (D + V), d = idx - r * (D + V), u = u0 + r;
        float val;
        if (u < nb) {
          const size_t e = pool_entry(btr, u, P, bs, ppb);
          val = d < D ? kpool[e * GD + (size_t)g * D + d] : vpool[e * GV + (size_t)g * V + (d - D)];
        } else {
          const int j = lo + (u - nb);
          const size_t slot = (size_t)btr[j / bs] * bs + (j % bs);
          val = d < D ? ldf(kcache, slot * GD + (size_t)g * D + d) : ldf(vcache, slot * GV + (size_t)g * V + (d - D));
        }
        if (d < D) ktile[r * DP + d] = val;
        else vtile[r * V + (d - D)] = val;
      }
      __syncthreads();
      if (hv) {
        float sc = -INFINITY;
        if (lane < nk) {
          const float* kr = ktile + lane * DP;
          float a = 0.f;
          for (int d = 0; d < D; ++d) a = fmaf(qq[d], kr[d], a);
          sc = a * scale;
        }
        const float mn = fmaxf(m, wave_max(sc));
        const float alpha = m == -INFINITY ? 0.f : expf(m - mn);
        const float pj = lane < nk ? expf(sc - mn) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = mn;
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[i] *= alpha;
        for (int jj = 0; jj < nk; ++jj) {
          const float pb = __shfl(pj, jj, WAVE);
#pragma unroll
          for (int i = 0; i < NACC; ++i) {
            const int d = lane + 64 * i;
            if (d < V) acc[i] = fmaf(pb, vtile[jj * V + d], acc[i]);
          }
        }
      }
    }
    if (hv) {
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < V) {
          float o = acc[i] / l;
          if (gate != nullptr) o *= 1.f / (1.f + expf(-ldf(gate, (size_t)t * ldg + (size_t)hd * V + d)));
          stf(out, (size_t)t * H * V + (size_t)hd * V + d, o);
        }
      }
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_window_kv_write(void* kcache, void* vcache, void* qkv, long ld, int koff, int voff, const void* qb,
                                   const void* kb, const void* vb, const float* cos_sin, const int* positions,
                                   const int* slot_mapping, const float* vfirst_in, float* vfirst_out, float lam, int T,
                                   int H, int G, int D, int V, int dims, float eps, int unit, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || D > 512 || V <= 0 || dims < 0 || dims > D || (dims & 1)) return -1;
  if (dims > 0 && cos_sin == nullptr) return -1;
  const size_t lds = (size_t)4 * D * sizeof(float);
#define K8S_WKW(TA)                                                                                                   \
  window_kv_write_kernel<TA><<<T, 256, lds, s>>>((TA*)kcache, (TA*)vcache, (TA*)qkv, ld, koff, voff, (const TA*)qb,    \
                                                 (const TA*)kb, (const TA*)vb, cos_sin, positions, slot_mapping,      \
                                                 vfirst_in, vfirst_out, lam, H, G, D, V, dims, eps, unit)
  if (f32) K8S_WKW(float);
  else K8S_WKW(bf16_t);
#undef K8S_WKW
  return (int)hipGetLastError();
}

extern "C" int k8s_window_pool(float* kpool, float* vpool, const void* kcache, const void* vcache,
                               const int* block_tables, int max_blocks, const int* tok_seq, const int* positions, int T,
                               int G, int D, int V, int P, int bs, int f32, hipStream_t s) {
  if (T <= 0 || P <= 0) return 0;
  if (G <= 0 || D <= 0 || V <= 0 || bs <= 0) return -1;
  const int ppb = (bs + P - 1) / P;
  if (f32)
    window_pool_kernel<float><<<T, 256, 0, s>>>(kpool, vpool, (const float*)kcache, (const float*)vcache, block_tables,
                                                max_blocks, tok_seq, positions, G, D, V, P, bs, ppb);
  else
    window_pool_kernel<bf16_t><<<T, 256, 0, s>>>(kpool, vpool, (const bf16_t*)kcache, (const bf16_t*)vcache,
                                                 block_tables, max_blocks, tok_seq, positions, G, D, V, P, bs, ppb);
  return (int)hipGetLastError();
}

extern "C" int k8s_window_attention(void* out, const void* q, long ldq, const void* gate, long ldg, const void* kcache,
                                    const void* vcache, const float* kpool, const float* vpool,
                                    const int* block_tables, int max_blocks, const int* tok_seq, const int* positions,
                                    int T, int H, int G, int D, int V, int window, int P, float scale, int sink, int bs,
                                    int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || V <= 0 || V > 256 || bs <= 0 || G > 65535) return -1;
  if (window > 0 && P > 0 && (kpool == nullptr || vpool == nullptr)) return -1;
  const int R = H / G;
  const int nw = R < 8 ? R : 8;
  // LDS floats: KB (D + 1 + V) tile + nw D queries, within 60 KB
  int KB = (15360 - nw * D) / (D + 1 + V);
  if (KB > 64) KB = 64;
  if (KB < 1) return -2;
  const size_t lds = ((size_t)KB * (D + 1 + V) + (size_t)nw * D) * sizeof(float);
  const int ppb = P > 0 ? (bs + P - 1) / P : 1;
  const int nacc = (V + 63) / 64;
#define K8S_WA(TA, NA)                                                                                                \
  window_attention_kernel<TA, NA><<<dim3(T, G), nw * 64, lds, s>>>(                                                   \
      (TA*)out, (const TA*)q, ldq, (const TA*)gate, ldg, (const TA*)kcache, (const TA*)vcache, kpool, vpool,          \
      block_tables, max_blocks, tok_seq, positions, H, G, D, V, window, P, scale, sink, bs, ppb, KB)
#define K8S_WA_T(TA)                   \
  do {                                 \
    if (nacc <= 1) K8S_WA(TA, 1);      \
    else if (nacc <= 2) K8S_WA(TA, 2); \
    else K8S_WA(TA, 4);                \
  } while (0)
  if (f32) K8S_WA_T(float);
  else K8S_WA_T(bf16_t);
#undef K8S_WA_T
#undef K8S_WA
  return (int)hipGetLastError();
}
