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
  if (p < 0) {   // idle row: defined output, nothing read
    for (int i = threadIdx.x; i < H * C; i += blockDim.x) stf(out, (size_t)t * H * C + i, 0.f);
    return;
  }
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

// Latent attention on the matrix cores (bf16 cache, C % 16 == 0, every part a multiple of 8 elements).  All heads of a
// token attend the same cached rows, so a token's (up to 16) heads are the 16 columns of one MFMA tile:
//   S^T[key][head] = K Q^T      A = 16 cached rows (from the LDS tile), B = the heads' queries [q_abs | q_rot]
//   O[head][d]    += P C        A = the 32 keys' probabilities (registers, keys in the order the S^T tile left them),
//                               B = the tile's latent columns through the transposing LDS read
// one wave per (token, group of 16 heads, key split), 32 keys per step, scores / softmax / sums in fp32.  With
// splits > 1 (few tokens: decoding) every split writes (max, sum, unnormalised O) and latent_merge_kernel joins them.
typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;

template <int NDB>
__global__ __launch_bounds__(64) void latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, float* __restrict__ pacc, float* __restrict__ pml, const bf16_t* __restrict__ q_abs,
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int C, int R, int H, int Dn, int window,
    float scale, int bs, int nsplit) {
  extern __shared__ __attribute__((aligned(16))) char smem_b[];
  char* smem = smem_b;
  const int t = blockIdx.x, hg = blockIdx.y, split = blockIdx.z;
  const int lane = threadIdx.x, li = lane & 15, g = lane >> 4;
  const int L = C + R, rowb = (L + 8) * 2, ndb = C / 16, HP = gridDim.y * 16;
  const int p = positions[t];
  if (p < 0) {
    if (nsplit == 1)
      for (int i = lane; i < 16 * C; i += 64) {
        const int hd = hg * 16 + i / C;
        if (hd < H) out[((size_t)t * H + hd) * C + i % C] = 0;
      }
    return;
  }
  char* qlds = smem;                 // [16][L + 8] bf16
  char* klds = smem + 16 * rowb;     // [32][L + 8] bf16
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int ntiles = (p + 1 - lo + 31) / 32;
  const int tps = (ntiles + nsplit - 1) / nsplit;
  const int t0 = split * tps, t1 = min(ntiles, t0 + tps);
  const int* btr = block_tables + (size_t)tok_seq[t] * max_blocks;
  const int cpr = L / 8;             // 16-byte chunks per row
  const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
  for (int idx = lane; idx < 16 * cpr; idx += 64) {
    const int r = idx / cpr, c = idx - r * cpr, hd = hg * 16 + r;
    u32x4 v = zero;
    if (hd < H)
      v = 8 * c < C ? *reinterpret_cast<const u32x4*>(q_abs + ((size_t)t * H + hd) * C + 8 * c)
                    : *reinterpret_cast<const u32x4*>(q + ((size_t)t * H + hd) * (Dn + R) + Dn + (8 * c - C));
    *reinterpret_cast<u32x4*>(qlds + r * rowb + 16 * c) = v;
  }
  f32x4 o[NDB];
#pragma unroll
  for (int n = 0; n < NDB; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int nkk = (L + 31) / 32;
  const int qd = li >> 2, pd = li & 3;
  for (int tile = t0; tile < t1; ++tile) {
    const int j0 = lo + tile * 32;
    __syncthreads();
    for (int idx = lane; idx < 32 * cpr; idx += 64) {
      const int r = idx / cpr, c = idx - r * cpr, key = j0 + r;
      u32x4 v = zero;
      if (key <= p) {
        const size_t slot = (size_t)btr[key / bs] * bs + (key % bs);
        v = *reinterpret_cast<const u32x4*>(cache + slot * L + 8 * c);
      }
      *reinterpret_cast<u32x4*>(klds + r * rowb + 16 * c) = v;
    }
    __syncthreads();
    f32x4 sacc[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int kk = 0; kk < nkk; ++kk) {
        const int piece = 32 * kk + 8 * g;
        bf16x8 ka, qb;
        if (piece < L) {
          ka = *reinterpret_cast<const bf16x8*>(klds + (16 * m + li) * rowb + 2 * piece);
          qb = *reinterpret_cast<const bf16x8*>(qlds + li * rowb + 2 * piece);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) { ka[e] = (__bf16)0.f; qb[e] = (__bf16)0.f; }
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb, acc, 0, 0, 0);
      }
      sacc[m] = acc;   // S[key j0 + 16 m + 4 g + i][head li]
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = j0 + 16 * m + 4 * g + i;
        const float v = key <= p ? sacc[m][i] * scale : -INFINITY;
        sacc[m][i] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(m_run, tmax);       // finite: key j0 is always visible
    const float alpha = m_run == -INFINITY ? 0.f : expf(m_run - m_new);
    float rsum = 0.f;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = expf(sacc[m][i] - m_new);
        sacc[m][i] = pv;
        rsum += pv;
      }
    rsum += __shfl_xor(rsum, 16, WAVE);
    rsum += __shfl_xor(rsum, 32, WAVE);
    l_run = l_run * alpha + rsum;
    m_run = m_new;
    float a_i[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) a_i[i] = __shfl(alpha, g * 4 + i, WAVE);
    bf16x8 pa;       // slot j < 4: key 4 g + j; slot j >= 4: key 16 + 4 g + (j - 4)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pa[j] = (__bf16)sacc[0][j];
      pa[4 + j] = (__bf16)sacc[1][j];
    }
    const int r0 = 4 * g + qd, r1 = r0 + 16;
#pragma unroll
    for (int n = 0; n < NDB; ++n) {
      if (n < ndb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[n][i] *= a_i[i];
        const int col = 16 * n + 4 * pd;
        const bf16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(klds + r0 * rowb + 2 * col));
        const bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(klds + r1 * rowb + 2 * col));
        bf16x8 vb;
#pragma unroll
        for (int j = 0; j < 4; ++j) { vb[j] = v0[j]; vb[4 + j] = v1[j]; }
        o[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vb, o[n], 0, 0, 0);
      }
    }
  }
  // o[n][i] = O[head 4 g + i][d 16 n + li]; the head's (max, sum) live in the lanes with li == head
  float l_i[4], m_i[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    l_i[i] = __shfl(l_run, g * 4 + i, WAVE);
    m_i[i] = __shfl(m_run, g * 4 + i, WAVE);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int hd = hg * 16 + 4 * g + i;
    if (hd >= H) continue;
    if (nsplit == 1) {
      const float inv = 1.f / l_i[i];
#pragma unroll
      for (int n = 0; n < NDB; ++n)
        if (n < ndb) out[((size_t)t * H + hd) * C + 16 * n + li] = f2bf(o[n][i] * inv);
    } else {
      const size_t rec = ((size_t)t * HP + hg * 16 + 4 * g + i) * nsplit + split;
#pragma unroll
      for (int n = 0; n < NDB; ++n)
        if (n < ndb) pacc[rec * C + 16 * n + li] = o[n][i];
      if (li == 0) {
        pml[rec * 2] = m_i[i];      // -inf and 0 for a split without tiles
        pml[rec * 2 + 1] = l_i[i];
      }
    }
  }
}

// out[t][head] = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s over the key splits
__global__ void latent_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ pacc,
                                    const float* __restrict__ pml, const int* __restrict__ positions, int C, int H,
                                    int HP, int nsplit) {
  const int t = blockIdx.x, hd = blockIdx.y;
  if (positions[t] < 0) {
    for (int d = threadIdx.x; d < C; d += blockDim.x) out[((size_t)t * H + hd) * C + d] = 0;
    return;
  }
  const size_t rec0 = ((size_t)t * HP + hd) * nsplit;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, pml[(rec0 + s) * 2]);
  float den = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float ms = pml[(rec0 + s) * 2];
    if (ms != -INFINITY) den += expf(ms - M) * pml[(rec0 + s) * 2 + 1];
  }
  for (int d = threadIdx.x; d < C; d += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float ms = pml[(rec0 + s) * 2];
      if (ms != -INFINITY) a += expf(ms - M) * pacc[(rec0 + s) * C + d];
    }
    out[((size_t)t * H + hd) * C + d] = f2bf(a / den);
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

// Whether the MFMA kernel takes these sizes (else the caller uses k8s_latent_attention).
extern "C" int k8s_latent_mfma_ok(int C, int R, int Dn) {
  const int L = C + R;
  return C % 16 == 0 && R % 8 == 0 && Dn % 8 == 0 && C <= 512 && 48 * (L + 8) * 2 <= 64 * 1024;
}

extern "C" int k8s_latent_attention_mfma(void* out, float* pacc, float* pml, const void* q_abs, const void* q,
                                         const void* cache, const int* block_tables, int max_blocks,
                                         const int* tok_seq, const int* positions, int T, int C, int R, int H, int Dn,
                                         int window, float scale, int bs, int nsplit, hipStream_t s) {
  if (T <= 0) return 0;
  if (!k8s_latent_mfma_ok(C, R, Dn) || H <= 0 || bs <= 0 || nsplit < 1 || (nsplit > 1 && (!pacc || !pml))) return -1;
  const int L = C + R, HG = (H + 15) / 16;
  const size_t lds = (size_t)48 * (L + 8) * 2;
  const dim3 grid(T, HG, nsplit);
#define K8S_LM(NDB)   latent_attention_mfma_kernel<NDB><<<grid, 64, lds, s>>>((bf16_t*)out, pacc, pml, (const bf16_t*)q_abs,                                                           (const bf16_t*)q, (const bf16_t*)cache, block_tables,                                                           max_blocks, tok_seq, positions, C, R, H, Dn, window, scale,                                                           bs, nsplit)
  if (C <= 128) K8S_LM(8);
  else if (C <= 256) K8S_LM(16);
  else K8S_LM(32);
#undef K8S_LM
  if (nsplit > 1)
    latent_merge_kernel<<<dim3(T, H), 128, 0, s>>>((bf16_t*)out, pacc, pml, positions, C, H, HG * 16, nsplit);
  return (int)hipGetLastError();
}
