// Sequence mixers beside softmax attention over a full K/V cache:
//   * a recurrent mixer with a matrix state per head (token shift, data-dependent decay, current-token bonus,
//     per-head unit norm and output gate), its state carried per sequence slot in fp32;
//   * latent attention: one low-rank row per token (normed latent | rotated shared key) in a paged cache, queries
//     absorbed into the latent space, sliding window.
// Both run varlen batches: sequence s owns tokens cu_q[s] .. cu_q[s + 1] - 1, positions[t] is a token's position in
// its sequence (negative: the row is idle and touches nothing), seq_slots[s] the slot of its recurrent state.
#include "common.h"

namespace k8sllm {

// out[s, t, :] = h[t] + (prev[t] - h[t]) * mu[s], s < n.  prev: h[t - 1] inside a portion; at a portion's first token
// the slot's saved row, or zeros at position 0.
template <typename TA>
__global__ void token_shift_kernel(TA* __restrict__ out, const TA* __restrict__ h, const TA* __restrict__ mu,
                                   const TA* __restrict__ state, const int* __restrict__ cu_q,
                                   const int* __restrict__ tok_seq, const int* __restrict__ seq_slots,
                                   const int* __restrict__ positions, int n, int T, int W) {
  const int t = blockIdx.x;
  const int p = positions[t];
  const int s = tok_seq[t];
  const bool first = cu_q[s] == t;
  const TA* prev = nullptr;
  if (p > 0) prev = first ? state + (size_t)seq_slots[s] * W : h + (size_t)(t - 1) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float x = ldf(h, (size_t)t * W + i);
    const float d = (p > 0 ? ldf(prev, i) : 0.f) - x;
    for (int k = 0; k < n; ++k)
      stf(out, ((size_t)k * T + t) * W + i, p < 0 ? 0.f : x + d * ldf(mu, (size_t)k * W + i));
  }
}

// state[slot of s] = h[last token of s]
template <typename TA>
__global__ void shift_save_kernel(TA* __restrict__ state, const TA* __restrict__ h, const int* __restrict__ cu_q,
                                  const int* __restrict__ seq_slots, const int* __restrict__ positions, int W) {
  const int s = blockIdx.x;
  const int a = cu_q[s], b = cu_q[s + 1];
  if (b <= a || positions[a] < 0) return;
  const size_t dst = (size_t)seq_slots[s] * W, src = (size_t)(b - 1) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) state[dst + i] = h[src + i];
}

// One workgroup per (sequence, head), thread j owns column j of the head's state S[i][j] (i: key channel, j: value
// channel) in registers.  Per token:  o_j = sum_i r_i (S_ij + u_i k_i v_j);  S_ij = w_i S_ij + k_i v_j  with
// w = exp(-exp(z + w0)) in fp32; then the head's o / rms(o) * lnw * silu(g).
template <typename TA, int DMAX>
__global__ void wkv_scan_kernel(TA* __restrict__ out, const TA* __restrict__ r, const TA* __restrict__ k,
                                const TA* __restrict__ v, const TA* __restrict__ g, long ld,
                                const float* __restrict__ z, const TA* __restrict__ w0, const TA* __restrict__ u,
                                const TA* __restrict__ lnw, float* __restrict__ state, const int* __restrict__ cu_q,
                                const int* __restrict__ seq_slots, const int* __restrict__ positions, int H, int D,
                                float eps) {
  __shared__ float sr[DMAX], sk[DMAX], sw[DMAX], su[DMAX], red[16];
  const int s = blockIdx.x, hd = blockIdx.y;
  const int a = cu_q[s], b = cu_q[s + 1];
  if (b <= a) return;
  const int p0 = positions[a];
  if (p0 < 0) return;
  const int j = threadIdx.x;
  const bool on = j < D;
  const int HD = H * D;
  float* st = state + ((size_t)seq_slots[s] * H + hd) * D * D;
  float S[DMAX];
#pragma unroll
  for (int i = 0; i < DMAX; ++i) S[i] = (on && i < D && p0 > 0) ? st[(size_t)i * D + j] : 0.f;
  float w0j = 0.f, lnj = 0.f;
  if (on) {
    su[j] = ldf(u, (size_t)hd * D + j);
    w0j = ldf(w0, (size_t)hd * D + j);
    lnj = ldf(lnw, (size_t)hd * D + j);
  }
  for (int t = a; t < b; ++t) {
    const size_t base = (size_t)t * ld + (size_t)hd * D + j;
    float vj = 0.f, gj = 0.f;
    if (on) {
      sr[j] = ldf(r, base);
      sk[j] = ldf(k, base);
      sw[j] = expf(-expf(z[(size_t)t * HD + (size_t)hd * D + j] + w0j));
      vj = ldf(v, base);
      gj = ldf(g, base);
    }
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DMAX; ++i) {
      if (i < D) {
        const float kv = sk[i] * vj;
        o = fmaf(sr[i], fmaf(su[i], kv, S[i]), o);
        S[i] = fmaf(sw[i], S[i], kv);
      }
    }
    const float ss = block_sum(on ? o * o : 0.f, red);   // (its barriers also order the next token's LDS writes)
    if (on) {
      const float y = o / sqrtf(ss / (float)D + eps) * lnj * (gj / (1.f + expf(-gj)));
      stf(out, (size_t)t * HD + (size_t)hd * D + j, y);
    }
  }
  if (on) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < D) st[(size_t)i * D + j] = S[i];
  }
}

// One workgroup per token: cache[slot] = [rms(dkv[:C]) * normw | rope(dkv[C:])] and the rotated part of every
// head of q ([T, H, Dn + R], last R of a head) rotated in place.  Rotation pairs dimension i with i + dims / 2 over
// the first `dims` rotated dimensions; cos_sin[pos] = [cos(dims / 2) | sin(dims / 2)].
template <typename TA>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(TA* __restrict__ cache, const TA* __restrict__ dkv,
                                                              const TA* __restrict__ normw, TA* __restrict__ q,
                                                              const float* __restrict__ cos_sin,
                                                              const int* __restrict__ positions,
                                                              const int* __restrict__ slot_mapping, int C, int R, int H,
                                                              int Dn, int dims, float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int slot = slot_mapping[t];
  const int L = C + R, half = dims / 2;
  const TA* d = dkv + (size_t)t * L;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += blockDim.x) {
    const float x = ldf(d, i);
    ss += x * x;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)C + eps);
  const float* cs = cos_sin + (size_t)pos * dims;
  if (slot >= 0) {
    TA* row = cache + (size_t)slot * L;
    for (int i = threadIdx.x; i < C; i += blockDim.x) stf(row, i, ldf(d, i) * inv * ldf(normw, i));
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      const float a = ldf(d, C + i), b = ldf(d, C + half + i), c = cs[i], sn = cs[half + i];
      stf(row, C + i, a * c - b * sn);
      stf(row, C + half + i, b * c + a * sn);
    }
    for (int i = dims + threadIdx.x; i < R; i += blockDim.x) stf(row, C + i, ldf(d, C + i));
  }
  TA* qt = q + (size_t)t * H * (Dn + R);
  for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
    const int hh = idx / half, i = idx - hh * half;
    TA* qh = qt + (size_t)hh * (Dn + R) + Dn;
    const float a = ldf(qh, i), b = ldf(qh, half + i), c = cs[i], sn = cs[half + i];
    stf(qh, i, a * c - b * sn);
    stf(qh, half + i, b * c + a * sn);
  }
}

// One workgroup per token, one wave per head (heads beyond the wave count take further passes).  Keys come in blocks
// of KB <= 64 cached rows staged in LDS as fp32 and shared by the heads; lane l scores key l of the block
// ((q_abs . c + q_rot . k_rot) * scale), the block joins a running softmax, and lane l accumulates latent
// dimensions l, l + 64, ... of sum_j p_j c_j.  out [T, H, C] = that sum / the softmax denominator.
template <typename TA, int NACC>
__global__ void latent_attention_kernel(TA* __restrict__ out, const TA* __restrict__ q_abs, const TA* __restrict__ q,
                                        const TA* __restrict__ cache, const int* __restrict__ block_tables,
                                        int max_blocks, const int* __restrict__ tok_seq,
                                        const int* __restrict__ positions, int C, int R, int H, int Dn, int window,
                                        float scale, int bs, int KB) {
  extern __shared__ float smem[];
  const int t = blockIdx.x;
  const int p = positions[t];
  if (p < 0) return;
  const int L = C + R, LP = L + 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = blockDim.x >> 6;
  float* tile = smem;                     // [KB][LP]
  float* qs = tile + (size_t)KB * LP;     // [nw][L]
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int* btr = block_tables + (size_t)tok_seq[t] * max_blocks;
  for (int h0 = 0; h0 < H; h0 += nw) {
    const int hd = h0 + wave;
    const bool hv = hd < H;
    float* qq = qs + (size_t)wave * L;
    if (hv) {
      for (int d = lane; d < L; d += 64)
        qq[d] = d < C ? ldf(q_abs, ((size_t)t * H + hd) * C + d)
                      : ldf(q, ((size_t)t * H + hd) * (Dn + R) + Dn + (d - C));
    }
    float m = -INFINITY, l = 0.f, acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    for (int j0 = lo; j0 <= p; j0 += KB) {
      const int nk = min(KB, p + 1 - j0);
      __syncthreads();
      for (int idx = tid; idx < nk * L; idx += blockDim.x) {
        const int jj = idx / L, d = idx - jj * L, j = j0 + jj;
        const size_t slot = (size_t)btr[j / bs] * bs + (j % bs);
        tile[jj * LP + d] = ldf(cache, slot * L + d);
      }
      __syncthreads();
      if (hv) {
        float sc = -INFINITY;
        if (lane < nk) {
          const float* row = tile + lane * LP;
          float a = 0.f;
          for (int d = 0; d < L; ++d) a = fmaf(qq[d], row[d], a);
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
            if (d < C) acc[i] = fmaf(pb, tile[jj * LP + d], acc[i]);
          }
        }
      }
    }
    if (hv) {
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < C) stf(out, ((size_t)t * H + hd) * C + d, acc[i] / l);
      }
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_token_shift(void* out, const void* h, const void* mu, const void* state, const int* cu_q,
                               const int* tok_seq, const int* seq_slots, const int* positions, int n, int T, int W,
                               int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (n <= 0 || W <= 0) return -1;
  if (f32)
    token_shift_kernel<float><<<T, 256, 0, s>>>((float*)out, (const float*)h, (const float*)mu, (const float*)state,
                                                cu_q, tok_seq, seq_slots, positions, n, T, W);
  else
    token_shift_kernel<bf16_t><<<T, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)h, (const bf16_t*)mu,
                                                 (const bf16_t*)state, cu_q, tok_seq, seq_slots, positions, n, T, W);
  return (int)hipGetLastError();
}

extern "C" int k8s_shift_save(void* state, const void* h, const int* cu_q, const int* seq_slots, const int* positions,
                              int nseq, int W, int f32, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (f32) shift_save_kernel<float><<<nseq, 256, 0, s>>>((float*)state, (const float*)h, cu_q, seq_slots, positions, W);
  else shift_save_kernel<bf16_t><<<nseq, 256, 0, s>>>((bf16_t*)state, (const bf16_t*)h, cu_q, seq_slots, positions, W);
  return (int)hipGetLastError();
}

extern "C" int k8s_wkv_max_dim() { return 128; }

extern "C" int k8s_wkv_scan(void* out, const void* r, const void* k, const void* v, const void* g, long ld,
                            const float* z, const void* w0, const void* u, const void* lnw, float* state,
                            const int* cu_q, const int* seq_slots, const int* positions, int nseq, int H, int D,
                            float eps, int f32, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (H <= 0 || D <= 0 || D > 128 || H > 65535) return -1;
  const dim3 grid(nseq, H);
  const int threads = (D + 63) / 64 * 64;
#define K8S_WKV(TA, DM) \
  wkv_scan_kernel<TA, DM><<<grid, threads, 0, s>>>((TA*)out, (const TA*)r, (const TA*)k, (const TA*)v, (const TA*)g, \
                                                   ld, z, (const TA*)w0, (const TA*)u, (const TA*)lnw, state, cu_q, \
                                                   seq_slots, positions, H, D, eps)
  if (f32) {
    if (D <= 32) K8S_WKV(float, 32);
    else if (D <= 64) K8S_WKV(float, 64);
    else K8S_WKV(float, 128);
  } else {
    if (D <= 32) K8S_WKV(bf16_t, 32);
    else if (D <= 64) K8S_WKV(bf16_t, 64);
    else K8S_WKV(bf16_t, 128);
  }
#undef K8S_WKV
  return (int)hipGetLastError();
}

extern "C" int k8s_latent_kv_write(void* cache, const void* dkv, const void* normw, void* q, const float* cos_sin,
                                   const int* positions, const int* slot_mapping, int T, int C, int R, int H, int Dn,
                                   int dims, float eps, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (C <= 0 || R < 0 || dims < 0 || dims > R || (dims & 1) || H <= 0) return -1;
  if (f32)
    latent_kv_write_kernel<float><<<T, 256, 0, s>>>((float*)cache, (const float*)dkv, (const float*)normw, (float*)q,
                                                    cos_sin, positions, slot_mapping, C, R, H, Dn, dims, eps);
  else
    latent_kv_write_kernel<bf16_t><<<T, 256, 0, s>>>((bf16_t*)cache, (const bf16_t*)dkv, (const bf16_t*)normw,
                                                     (bf16_t*)q, cos_sin, positions, slot_mapping, C, R, H, Dn, dims,
                                                     eps);
  return (int)hipGetLastError();
}

extern "C" int k8s_latent_attention(void* out, const void* q_abs, const void* q, const void* cache,
                                    const int* block_tables, int max_blocks, const int* tok_seq, const int* positions,
                                    int T, int C, int R, int H, int Dn, int window, float scale, int bs, int f32,
                                    hipStream_t s) {
  if (T <= 0) return 0;
  if (C <= 0 || C > 512 || R < 0 || H <= 0 || bs <= 0) return -1;
  const int L = C + R;
  const int nw = H < 8 ? H : 8;
  // LDS floats: KB (L + 1) key tile + nw L queries, within 60 KB
  int KB = (15360 - nw * L) / (L + 1);
  if (KB > 64) KB = 64;
  if (KB < 1) return -2;
  const size_t lds = ((size_t)KB * (L + 1) + (size_t)nw * L) * sizeof(float);
  const int nacc = (C + 63) / 64;
#define K8S_LA(TA, NA) \
  latent_attention_kernel<TA, NA><<<T, nw * 64, lds, s>>>((TA*)out, (const TA*)q_abs, (const TA*)q, (const TA*)cache, \
                                                          block_tables, max_blocks, tok_seq, positions, C, R, H, Dn, \
                                                          window, scale, bs, KB)
#define K8S_LA_T(TA)                  \
  do {                                \
    if (nacc <= 1) K8S_LA(TA, 1);     \
    else if (nacc <= 2) K8S_LA(TA, 2); \
    else if (nacc <= 4) K8S_LA(TA, 4); \
    else K8S_LA(TA, 8);               \
  } while (0)
  if (f32) K8S_LA_T(float);
  else K8S_LA_T(bf16_t);
#undef K8S_LA_T
#undef K8S_LA
  return (int)hipGetLastError();
}
