// Gated linear recurrences with a matrix state per head, S [D key channels][V value channels] in fp32, carried per
// sequence slot:
//   KIND 0 (HGRN2: the forget gate also sets what is written)
//       f = low + (1 - low) sigmoid(zf + bf)  per key channel;  S <- diag(f) S + (1 - f) v^T;  o = S^T silu(zq);
//       y = o / rms(o) * normw[V]
//   KIND 1 (mLSTM: exponential input gate under a running maximum m that starts at 0)
//       i = cap tanh((zi + bi) / cap), f = logsigmoid(cap tanh((zf + bf) / cap))  per head;
//       m' = max(f + m, i), a = exp(f + m - m'), b = exp(i - m');  S <- a S + b k v^T, n <- a n + b k;
//       o = S^T q / (max(|n . q|, exp(-m')) + 1e-6), q = zq / sqrt(D);  y = o / rms(o) * normw[H V] * sigmoid(zg)
// Everything that enters the recurrence (gates, decays, state, norms) is fp32: the kernels read the fused input
// projection as fp32 [T, ld] with the parts at column offsets, and write y in the activation type.
// Varlen batches: sequence s owns tokens cu_q[s] .. cu_q[s + 1] - 1 and the state record of slot seq_slots[s]; a portion
// that starts at position 0 starts from zero state (m = 0), so a reused slot needs no clearing.
#include "common.h"

namespace k8sllm {

struct ScanCols { int q, k, v, i, f, g; };   // column offsets of the parts inside a projected row

// One workgroup per (sequence, head).  Thread (x, c) owns value column x of the CH key channels [c CH, (c + 1) CH) of S;
// group c = 0 prepares each token's per-channel read / keep / write coefficients in LDS (and, KIND 1, owns n).  The
// partial outputs of the channel groups meet in LDS; group 0 normalises and stores.  The next token's inputs are
// loaded while the current one is computed; the barriers wait for LDS traffic only.
// blockDim = (DX, NS): DX = max(D, V) rounded up to 64, NS = ceil(D / CH).  State record: S [D][V] (, n [D], m).
template <typename TA, int CH, int KIND>
__global__ __launch_bounds__(1024) void gated_scan_kernel(TA* __restrict__ out, const float* __restrict__ proj, long ld,
                                                          ScanCols co, const TA* __restrict__ fbias,
                                                          const TA* __restrict__ ibias, const TA* __restrict__ lower,
                                                          const TA* __restrict__ normw, float* __restrict__ state,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ seq_slots,
                                                          const int* __restrict__ positions, int H, int D, int V,
                                                          float eps, float cap) {
  constexpr int DMAX = 128;
  __shared__ __attribute__((aligned(16))) float sq[DMAX], sa[DMAX], sb[DMAX];
  __shared__ float po[DMAX / CH][DMAX];
  __shared__ float red[2], rednq[2];
  const int s = blockIdx.x, hd = blockIdx.y;
  const int a0 = cu_q[s], b0 = cu_q[s + 1];
  if (b0 <= a0) return;
  const int p0 = positions[a0];
  if (p0 < 0) return;
  const bool from_zero = p0 == 0;
  const int x = threadIdx.x, c = threadIdx.y, NS = blockDim.y, DX = blockDim.x;
  const bool onv = x < V, ond = x < D;
  const int i0 = c * CH;
  const size_t rec = (size_t)D * V + (KIND == 1 ? D + 1 : 0);
  float* st = state + ((size_t)seq_slots[s] * H + hd) * rec;
  float S[CH];
#pragma unroll
  for (int e = 0; e < CH; ++e) S[e] = (onv && i0 + e < D && !from_zero) ? st[(size_t)(i0 + e) * V + x] : 0.f;
  float nx = 0.f, m = 0.f;
  if (KIND == 1 && !from_zero) {
    if (c == 0 && ond) nx = st[(size_t)D * V + x];
    m = st[(size_t)D * V + D];
  }
  if (c == 0)
    for (int e = x; e < DMAX; e += DX) sq[e] = sa[e] = sb[e] = 0.f;
  float lowx = 0.f, fbx = 0.f, nwx = 0.f, fbh = 0.f, ibh = 0.f;
  if (KIND == 0) {
    if (c == 0 && ond) {
      lowx = ldf(lower, (size_t)hd * D + x);
      fbx = fbias != nullptr ? ldf(fbias, (size_t)hd * D + x) : 0.f;
    }
    if (c == 0 && onv) nwx = ldf(normw, x);
  } else {
    fbh = fbias != nullptr ? ldf(fbias, hd) : 0.f;
    ibh = ibias != nullptr ? ldf(ibias, hd) : 0.f;
    if (c == 0 && onv) nwx = ldf(normw, (size_t)hd * V + x);
  }
  const float qscale = KIND == 1 ? 1.0f / sqrtf((float)D) : 1.f;
  lds_barrier();
  // inputs of the next token
  float nq = 0.f, nk = 0.f, nv = 0.f, nf = 0.f, ni = 0.f, ng = 0.f;
  auto fetch = [&](int t) {
    if (t >= b0) return;
    const float* r = proj + (size_t)t * ld;
    if (onv) nv = r[co.v + (size_t)hd * V + x];
    if (KIND == 1) {
      nf = r[co.f + hd];
      ni = r[co.i + hd];
      if (c == 0 && onv) ng = r[co.g + (size_t)hd * V + x];
    }
    if (c == 0 && ond) {
      nq = r[co.q + (size_t)hd * D + x];
      if (KIND == 0) nf = r[co.f + (size_t)hd * D + x];
      else nk = r[co.k + (size_t)hd * D + x];
    }
  };
  fetch(a0);
  for (int t = a0; t < b0; ++t) {
    const float cq = nq, ck = nk, cv = nv, cf = nf, ci = ni, cg = ng;
    fetch(t + 1);
    float ka = 1.f;   // KIND 1: the head's keep factor
    if (KIND == 0) {
      if (c == 0 && ond) {
        const float f = lowx + (1.f - lowx) / (1.f + expf(-(cf + fbx)));
        sq[x] = cq / (1.f + expf(-cq));
        sa[x] = f;
        sb[x] = 1.f - f;
      }
    } else {
      const float ig = cap * tanhf((ci + ibh) / cap);
      const float fr = cap * tanhf((cf + fbh) / cap);
      const float fg = fminf(fr, 0.f) - log1pf(expf(-fabsf(fr)));
      const float mn = fmaxf(fg + m, ig);
      ka = expf(fg + m - mn);
      const float kb = expf(ig - mn);
      m = mn;
      if (c == 0) {
        float nqp = 0.f;
        if (ond) {
          const float qv = cq * qscale;
          nx = ka * nx + kb * ck;
          nqp = nx * qv;
          sq[x] = qv;
          sb[x] = kb * ck;
        }
        nqp = wave_sum(nqp);
        if ((x & 63) == 0) rednq[x >> 6] = nqp;
      }
    }
    lds_barrier();
    float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e0 = 0; e0 < CH; e0 += 4) {
      const f32x4 q4 = *reinterpret_cast<const f32x4*>(&sq[i0 + e0]);
      const f32x4 b4 = *reinterpret_cast<const f32x4*>(&sb[i0 + e0]);
      f32x4 a4 = f32x4{ka, ka, ka, ka};
      if (KIND == 0) a4 = *reinterpret_cast<const f32x4*>(&sa[i0 + e0]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        S[e0 + e] = fmaf(a4[e], S[e0 + e], b4[e] * cv);
        o4[e] = fmaf(q4[e], S[e0 + e], o4[e]);
      }
    }
    if (onv) po[c][x] = (o4[0] + o4[1]) + (o4[2] + o4[3]);
    lds_barrier();
    float o = 0.f, ss = 0.f;
    if (c == 0) {
      if (onv)
        for (int g = 0; g < NS; ++g) o += po[g][x];
      if (KIND == 1) {
        const float nqs = rednq[0] + (D > 64 ? rednq[1] : 0.f);
        o /= fmaxf(fabsf(nqs), expf(-m)) + 1e-6f;
      }
      ss = wave_sum(onv ? o * o : 0.f);
      if (DX > 64 && (x & 63) == 0) red[x >> 6] = ss;
    }
    if (DX > 64) {                     // the channels span two waves: one more exchange (uniform branch)
      lds_barrier();
      ss = red[0] + red[1];
    }
    if (c == 0 && onv) {
      float y = o / sqrtf(ss / (float)V + eps) * nwx;
      if (KIND == 1) y *= 1.f / (1.f + expf(-cg));
      stf(out, (size_t)t * H * V + (size_t)hd * V + x, y);
    }
  }
  if (onv) {
#pragma unroll
    for (int e = 0; e < CH; ++e)
      if (i0 + e < D) st[(size_t)(i0 + e) * V + x] = S[e];
  }
  if (KIND == 1 && c == 0) {
    if (ond) st[(size_t)D * V + x] = nx;
    if (x == 0) st[(size_t)D * V + D] = m;
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_gated_scan_max_dim() { return 128; }

// floats of one (slot, head) state record
extern "C" long long k8s_gated_scan_record(int kind, int D, int V) {
  return (long long)D * V + (kind == 1 ? D + 1 : 0);
}

extern "C" int k8s_gated_scan(void* out, const float* proj, long ld, int kind, int cq, int ck, int cv, int ci, int cf,
                              int cg, const void* fbias, const void* ibias, const void* lower, const void* normw,
                              float* state, const int* cu_q, const int* seq_slots, const int* positions, int nseq, int H,
                              int D, int V, float eps, float cap, int f32, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (H <= 0 || H > 65535 || D <= 0 || D > 128 || V <= 0 || V > 128 || kind < 0 || kind > 1) return -1;
  if (kind == 0 && lower == nullptr) return -1;
  if (kind == 1 && !(cap > 0.f)) return -1;
  constexpr int CH = 16;
  const int m = D > V ? D : V;
  const dim3 block((m + 63) / 64 * 64, (D + CH - 1) / CH);
  const ScanCols co{cq, ck, cv, ci, cf, cg};
#define K8S_GS(TA, KIND)                                                                                            \
  gated_scan_kernel<TA, CH, KIND><<<dim3(nseq, H), block, 0, s>>>((TA*)out, proj, ld, co, (const TA*)fbias,          \
                                                                  (const TA*)ibias, (const TA*)lower,               \
                                                                  (const TA*)normw, state, cu_q, seq_slots,         \
                                                                  positions, H, D, V, eps, cap)
  if (kind == 0) {
    if (f32) K8S_GS(float, 0);
    else K8S_GS(bf16_t, 0);
  } else {
    if (f32) K8S_GS(float, 1);
    else K8S_GS(bf16_t, 1);
  }
#undef K8S_GS
  return (int)hipGetLastError();
}
