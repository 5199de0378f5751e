// Recurrent mixers fed by short causal convolutions, over varlen batches with per-slot fp32 state:
//   * short_conv: a causal convolution over time per channel (taps - 1 earlier inputs of a sequence come from the batch
//     or, before the portion, from the slot's saved inputs; zeros before position 0), bias, silu, and unit vectors over
//     groups of channels (the prepared queries / keys of the delta rule);
//   * delta_scan: the gated delta rule with a matrix state per head, S [D key channels][V value channels]:
//       S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;  y = o / rms(o) * normw * silu(gate)
//     with g = exp(neg_a softplus(a + dt_bias)) and beta = sigmoid(b) per head;
//   * rglru_scan: the real-gated linear recurrent unit per channel,
//       r, i = sigmoid(gate logits + bias);  a = exp(rate r);  S <- a S + sqrt(1 - a^2) i u;  out = S gelu_tanh(y + bias).
// Everything here is fp32 (inputs are fp32 projections); only the outputs take the activation type.  Sequence s owns
// tokens cu_q[s] .. cu_q[s + 1] - 1 and the records of slot seq_slots[s]; a portion that starts at position 0 starts
// from zero state, so a reused slot needs no clearing; positions[t] < 0 marks an idle row that touches nothing.
#include "common.h"

namespace k8sllm {

constexpr int CONV_MAX_TAPS = 16;

// Workgroups (token, slice of the channels).  The first unit_cols channels go one wave per group of unit_dim (<= 256)
// channels, the rest one thread per channel; the slices of a token share both lists.  `residual`: the token's own input
// is added to the result (y = x + conv(x), after bias and activation).  TO: the output's type (fp32, or bf16 for a
// convolution whose result feeds a bf16 projection).
template <typename TO>
__global__ __launch_bounds__(256) void short_conv_kernel(
    TO* __restrict__ out, const float* __restrict__ x, long ldx, const float* __restrict__ w,
    const float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ tok_seq,
    const int* __restrict__ seq_slots, const int* __restrict__ positions, const float* __restrict__ in_bias,
    const float* __restrict__ out_bias, int act, int C, int taps, int unit_cols, int unit_dim, int scale_cols,
    float scale, float unit_eps, int residual) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int seq = tok_seq[t];
  const int a0 = cu_q[seq];
  // state row r holds the input of position p0 - (taps - 1) + r, p0 the portion's first position
  const float* st = state + (size_t)seq_slots[seq] * (taps - 1) * C;
  auto value = [&](int ch) -> float {
    float acc = out_bias != nullptr ? out_bias[ch] : 0.f;
    const float ib = in_bias != nullptr ? in_bias[ch] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (pos - back < 0) continue;
      const int tt = t - back;
      const float xv = tt >= a0 ? x[(size_t)tt * ldx + ch] + ib : st[(size_t)(taps - 1 + (tt - a0)) * C + ch];
      acc = fmaf(w[(size_t)ch * taps + j], xv, acc);
    }
    if (act == 1) acc = acc / (1.f + expf(-acc));
    if (residual) acc += x[(size_t)t * ldx + ch] + ib;
    return acc;
  };
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = blockDim.x >> 6;
  TO* dst = out + (size_t)t * C;
  const int ngroups = unit_dim > 0 ? unit_cols / unit_dim : 0;
  for (int gv = blockIdx.y * nw + wave; gv < ngroups; gv += nw * gridDim.y) {
    float y[4], ss = 0.f;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int d = lane + 64 * n;
      y[n] = d < unit_dim ? value(gv * unit_dim + d) : 0.f;
      ss += y[n] * y[n];
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss + unit_eps);
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int d = lane + 64 * n, ch = gv * unit_dim + d;
      if (d < unit_dim) stf(dst, ch, y[n] * inv * (ch < scale_cols ? scale : 1.f));
    }
  }
  for (int ch = ngroups * unit_dim + blockIdx.y * blockDim.x + tid; ch < C; ch += blockDim.x * gridDim.y)
    stf(dst, ch, value(ch) * (ch < scale_cols ? scale : 1.f));
}

// state[slot of s] <- the last taps - 1 inputs of sequence s after this portion (a portion shorter than that keeps the
// newest of the old ones).  One thread per (sequence, channel); it reads everything it needs before it writes.
__global__ void conv_save_kernel(float* __restrict__ state, const float* __restrict__ x, long ldx,
                                 const int* __restrict__ cu_q, const int* __restrict__ seq_slots,
                                 const int* __restrict__ positions, const float* __restrict__ in_bias, int C, int taps) {
  const int s = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  const int a0 = cu_q[s], n = cu_q[s + 1] - a0;
  if (ch >= C || n <= 0) return;
  const int p0 = positions[a0];
  if (p0 < 0) return;
  float* st = state + (size_t)seq_slots[s] * (taps - 1) * C;
  const float ib = in_bias != nullptr ? in_bias[ch] : 0.f;
  float v[CONV_MAX_TAPS - 1];
#pragma unroll
  for (int r = 0; r < CONV_MAX_TAPS - 1; ++r) {
    v[r] = 0.f;
    if (r < taps - 1) {
      const int rel = n - (taps - 1) + r;      // token of the portion, or (negative) an input before it
      if (rel >= 0) v[r] = x[(size_t)(a0 + rel) * ldx + ch] + ib;
      else if (p0 + rel >= 0) v[r] = st[(size_t)(taps - 1 + rel) * C + ch];
    }
  }
#pragma unroll
  for (int r = 0; r < CONV_MAX_TAPS - 1; ++r)
    if (r < taps - 1) st[(size_t)r * C + ch] = v[r];
}

// One workgroup per (sequence or chunk, head).  Thread (x, c) owns value column x of the CH key channels
// [c CH, (c + 1) CH) of S.  Per token every thread forms its channels' part of S^T k and S^T q from the state before the
// update; the parts meet in LDS (one barrier), then every thread has u for its column and updates its channels, and
// group c = 0 finishes the output from o = g S_old^T q + (q . k) u, which equals S_new^T q.  The next token's inputs are
// loaded while the current one is computed; k and q rotate through three LDS rows and the partial sums through two, so
// one barrier per token orders everything (a second one when the value channels span several waves, for the output's
// norm).  blockDim = (DX, NS): DX = the columns rounded up to 64, NS = ceil(D / CH), CH (16, 32 or 64) the smallest
// that keeps DX NS within 1024 threads.  qkv rows: [q (G D) | k (G D) | v (H V)].
//
// MODE 0: a whole portion per workgroup, from the slot's state (zero at position 0) to the slot's state.
// Long portions run as three passes over chunks of Lc tokens, parallel over chunks.  A token maps S to
// g (I - beta k k^T) S + beta k v^T, so a chunk maps its start state to P S + L:
// MODE 1: a chunk run on D + V columns, the first V from zero with the tokens' values (-> L), the other D from the
//         identity with zero values (-> P, the same update applied to the identity's columns); no outputs; the record
//         [D][V + D] goes to cs_loc.  delta_prefix_kernel then walks a sequence's chunks, start[c + 1] = P_c start[c] + L_c.
// MODE 2: a chunk from its start state with outputs; a sequence's last chunk leaves the slot's state.
template <typename TA, int CH, int MODE>
__global__ __launch_bounds__(1024) void delta_scan_kernel(
    TA* __restrict__ out, const float* __restrict__ qkv, const float* __restrict__ proj, long ld, int cb, int ca, int cg,
    const float* __restrict__ neg_a, const float* __restrict__ dt_bias, const float* __restrict__ normw,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int H, int G, int D, int V, float eps, int nseq, int Lc,
    float* __restrict__ cs_loc, const float* __restrict__ cs_start) {
  constexpr int DMAX = 256;
  __shared__ __attribute__((aligned(16))) float sk[3][DMAX], sq[3][DMAX];
  __shared__ float pk[2][1024], pq[2][1024], pqk[2][16];
  __shared__ float red[8];
  const int hd = blockIdx.y;
  int s, a0, b0, p0;
  bool last = true;
  if (MODE == 0) {
    s = blockIdx.x;
    a0 = cu_q[s];
    b0 = cu_q[s + 1];
    if (b0 <= a0) return;
    p0 = positions[a0];
    if (p0 < 0) return;
  } else {
    const WkvChunk ck = wkv_find_chunk(blockIdx.x, cu_q, positions, nseq, Lc);
    if (ck.s < 0) return;
    s = ck.s;
    last = ck.c == ck.n - 1;
    if (MODE == 1 && last) return;          // nothing follows a sequence's last chunk
    a0 = cu_q[s] + ck.c * Lc;
    b0 = min(cu_q[s + 1], a0 + Lc);
    p0 = positions[a0];
  }
  const int x = threadIdx.x, c = threadIdx.y, NS = blockDim.y, DX = blockDim.x;
  const int VX = MODE == 1 ? V + D : V;     // columns of this pass
  const bool onv = x < VX, ond = x < D, isv = x < V;
  const int i0 = c * CH;
  const int gq = hd / (H / G);
  const long row = 2L * G * D + (long)H * V;
  float* st = state + ((size_t)seq_slots[s] * H + hd) * ((size_t)D * V);
  const size_t lrec = (size_t)D * (V + D), srec = (size_t)D * V;
  const size_t chunk = (size_t)blockIdx.x * H + hd;
  // MODE 2 never reads the slot's record, which the sequence's last chunk overwrites: the prefix pass left a copy
  const float* src = MODE == 2 ? cs_start + chunk * srec : st;
  float S[CH];
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    if (MODE == 1) S[e] = (onv && !isv && i0 + e == x - V) ? 1.f : 0.f;
    else S[e] = (onv && i0 + e < D && p0 != 0) ? src[(size_t)(i0 + e) * V + x] : 0.f;
  }
  if (c == 0)
    for (int e = x; e < 3 * DMAX; e += DX) (&sk[0][0])[e] = (&sq[0][0])[e] = 0.f;
  const float na = neg_a[hd], dtb = dt_bias[hd];
  const float nwx = (MODE != 1 && c == 0 && onv) ? normw[x] : 0.f;
  float nq = 0.f, nk = 0.f, nv = 0.f, nb = 0.f, nz = 0.f, ng = 0.f;
  auto fetch = [&](int t) {
    if (t >= b0) return;
    const float* r = qkv + (size_t)t * row;
    const float* pr = proj + (size_t)t * ld;
    if (isv) nv = r[2L * G * D + (long)hd * V + x];
    nb = pr[cb + hd];
    nz = pr[ca + hd];
    if (c == 0) {
      if (ond) {
        if (MODE != 1) nq = r[(long)gq * D + x];
        nk = r[(long)G * D + (long)gq * D + x];
      }
      if (MODE != 1 && onv) ng = pr[cg + (long)hd * V + x];
    }
  };
  fetch(a0);
  lds_barrier();                       // the rows are cleared
  if (c == 0 && ond) {
    sk[0][x] = nk;
    sq[0][x] = nq;
  }
  lds_barrier();
  for (int t = a0; t < b0; ++t) {
    const int i = t - a0, cur = i % 3, nxt = (i + 1) % 3, pb = i & 1;
    const float cv = nv, cbeta = nb, cz = nz, cgate = ng;
    fetch(t + 1);
    float ak[4] = {0.f, 0.f, 0.f, 0.f}, aq[4] = {0.f, 0.f, 0.f, 0.f}, aqk = 0.f;
#pragma unroll
    for (int e0 = 0; e0 < CH; e0 += 4) {
      const f32x4 k4 = *reinterpret_cast<const f32x4*>(&sk[cur][i0 + e0]);
      const f32x4 q4 = *reinterpret_cast<const f32x4*>(&sq[cur][i0 + e0]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ak[e] = fmaf(k4[e], S[e0 + e], ak[e]);
        if (MODE != 1) {
          aq[e] = fmaf(q4[e], S[e0 + e], aq[e]);
          aqk = fmaf(k4[e], q4[e], aqk);
        }
      }
    }
    pk[pb][c * DX + x] = (ak[0] + ak[1]) + (ak[2] + ak[3]);
    if (MODE != 1) {
      pq[pb][c * DX + x] = (aq[0] + aq[1]) + (aq[2] + aq[3]);
      if (x == 0) pqk[pb][c] = aqk;
    }
    if (c == 0 && ond && t + 1 < b0) {
      sk[nxt][x] = nk;
      sq[nxt][x] = nq;
    }
    lds_barrier();
    float kS = 0.f;
    for (int g = 0; g < NS; ++g) kS += pk[pb][g * DX + x];
    const float zz = cz + dtb;
    const float sp = zz > 20.f ? zz : log1pf(expf(zz));
    const float decay = expf(na * sp);
    const float beta = 1.f / (1.f + expf(-cbeta));
    const float u = beta * (cv - decay * kS);
#pragma unroll
    for (int e0 = 0; e0 < CH; e0 += 4) {
      const f32x4 k4 = *reinterpret_cast<const f32x4*>(&sk[cur][i0 + e0]);
#pragma unroll
      for (int e = 0; e < 4; ++e) S[e0 + e] = fmaf(k4[e], u, decay * S[e0 + e]);
    }
    if (MODE == 1) continue;
    float o = 0.f, ss = 0.f;
    if (c == 0) {
      float qS = 0.f, qk = 0.f;
      for (int g = 0; g < NS; ++g) {
        qS += pq[pb][g * DX + x];
        qk += pqk[pb][g];
      }
      o = onv ? fmaf(qk, u, decay * qS) : 0.f;
      ss = wave_sum(o * o);
      if (DX > 64 && (x & 63) == 0) red[x >> 6] = ss;
    }
    if (DX > 64) {                     // the value channels span several waves: one more exchange (uniform branch)
      lds_barrier();
      ss = red[0];
      for (int w = 1; w < DX / 64; ++w) ss += red[w];
    }
    if (c == 0 && onv) {
      const float y = o / sqrtf(ss / (float)V + eps) * nwx * (cgate / (1.f + expf(-cgate)));
      stf(out, (size_t)t * H * V + (size_t)hd * V + x, y);
    }
  }
  if (MODE == 2 && !last) return;
  if (onv) {
#pragma unroll
    for (int e = 0; e < CH; ++e) {
      if (i0 + e >= D) continue;
      if (MODE == 1) cs_loc[chunk * lrec + (size_t)(i0 + e) * (V + D) + x] = S[e];
      else st[(size_t)(i0 + e) * V + x] = S[e];
    }
  }
}

// Start states of a sequence's chunks from the slot's state (zero at position 0) and the chunks' records:
// start[c + 1] = P_c start[c] + L_c.  The value columns are independent, so a workgroup takes (sequence, head, XT value
// columns): thread (x, i) owns row i of its column; the running columns live in LDS (two buffers), P_c is staged in LDS
// and the next chunk's P is loaded into registers while the current product runs.  blockDim = (XT, D), XT D <= 1024;
// dynamic LDS: D (D + 1) + 2 D XT floats.  Chunk 0 starts from a copy of the slot's record.
template <int NP>
__global__ __launch_bounds__(1024) void delta_prefix_kernel(float* __restrict__ cs_start, const float* __restrict__ cs_loc,
                                                            const float* __restrict__ state,
                                                            const int* __restrict__ cu_q,
                                                            const int* __restrict__ seq_slots,
                                                            const int* __restrict__ positions, int H, int D, int V,
                                                            int Lc) {
  extern __shared__ float psm[];
  const int s = blockIdx.x, hd = blockIdx.y;
  int first = 0;
  for (int y = 0; y < s; ++y) {
    const int a = cu_q[y], len = cu_q[y + 1] - a;
    first += (len > 0 && positions[a] >= 0) ? (len + Lc - 1) / Lc : 0;
  }
  const int a = cu_q[s], len = cu_q[s + 1] - a;
  if (len <= 0 || positions[a] < 0) return;
  const int n = (len + Lc - 1) / Lc;
  const bool zero = positions[a] == 0;
  const int XT = blockDim.x, x = threadIdx.x, i = threadIdx.y;
  const int col = blockIdx.z * XT + x;
  const bool ok = col < V;
  const int DV = D * V, LW = V + D, DP = D + 1;
  const int tid = i * XT + x, nthr = XT * D;
  float* Psh = psm;                       // [D][D + 1]
  float* Ssh = psm + (size_t)D * DP;      // [2][D][XT]
  const float* st = state + ((size_t)seq_slots[s] * H + hd) * DV;
  float cur = (ok && !zero) ? st[(size_t)i * V + col] : 0.f;
  if (ok) cs_start[((size_t)first * H + hd) * DV + (size_t)i * V + col] = cur;
  Ssh[(size_t)i * XT + x] = cur;
  float pre[NP];
  auto load_p = [&](int c) {
    const float* loc = cs_loc + ((size_t)(first + c) * H + hd) * ((size_t)D * LW);
#pragma unroll
    for (int k = 0; k < NP; ++k) {
      const int e = tid + k * nthr;
      pre[k] = e < D * D ? loc[(size_t)(e / D) * LW + V + (e % D)] : 0.f;
    }
  };
  if (n > 1) load_p(0);
  for (int c = 0; c + 1 < n; ++c) {
    const int b = c & 1;
    __syncthreads();                     // the previous product has read Psh; Ssh[b] is complete
#pragma unroll
    for (int k = 0; k < NP; ++k) {
      const int e = tid + k * nthr;
      if (e < D * D) Psh[(size_t)(e / D) * DP + (e % D)] = pre[k];
    }
    const float* loc = cs_loc + ((size_t)(first + c) * H + hd) * ((size_t)D * LW);
    float acc = ok ? loc[(size_t)i * LW + col] : 0.f;
    __syncthreads();
    if (c + 2 < n) load_p(c + 1);
    const float* pr = Psh + (size_t)i * DP;
    const float* sc = Ssh + (size_t)b * D * XT + x;
#pragma unroll 8
    for (int j = 0; j < D; ++j) acc = fmaf(pr[j], sc[(size_t)j * XT], acc);
    Ssh[(size_t)(b ^ 1) * D * XT + (size_t)i * XT + x] = acc;
    if (ok) cs_start[((size_t)(first + c + 1) * H + hd) * DV + (size_t)i * V + col] = acc;
  }
}

// One workgroup per (sequence, 64 channels); blockDim = (64, NT).  A long portion is cut into NT time slices that run
// side by side: every slice first composes its own tokens into (A, B) with S_out = A S_in + B, the slices' start states
// follow from the slot's state by walking the earlier slices' pairs, then every slice runs again from its start state
// and writes outputs.  NT == 1 (decoding, short portions): one pass.
template <typename TA>
__global__ __launch_bounds__(1024) void rglru_scan_kernel(
    TA* __restrict__ out, const float* __restrict__ u, const float* __restrict__ gates,
    const float* __restrict__ gate_bias, const float* __restrict__ rate, const float* __restrict__ proj, long ld,
    int ycol, const float* __restrict__ ybias, float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ seq_slots, const int* __restrict__ positions, int C, int blocks) {
  __shared__ float sA[16][64], sB[16][64];
  const int s = blockIdx.x;
  const int a0 = cu_q[s], b0 = cu_q[s + 1];
  if (b0 <= a0) return;
  const int p0 = positions[a0];
  if (p0 < 0) return;
  const int x = threadIdx.x, j = threadIdx.y, NT = blockDim.y;
  const int ch = blockIdx.y * 64 + x;
  const bool ok = ch < C;
  const int n = b0 - a0, L = (n + NT - 1) / NT;
  const int t0 = min(b0, a0 + j * L), t1 = min(b0, t0 + L);
  const int bw = C / blocks;
  const int chc = ok ? ch : 0;
  const int gr = (chc / bw) * 2 * bw + (chc % bw);          // this channel's recurrence-gate logit; the input gate's is bw on
  const float br = gate_bias[gr], bi = gate_bias[gr + bw], rt = rate[chc];
  auto coef = [&](int t, float& a, float& b) {
    const float* gt = gates + (size_t)t * 2 * C;
    const float r = 1.f / (1.f + expf(-(gt[gr] + br)));
    const float ig = 1.f / (1.f + expf(-(gt[gr + bw] + bi)));
    const float la = rt * r;
    a = expf(la);
    b = sqrtf(-expm1f(2.f * la)) * ig * u[(size_t)t * C + chc];
  };
  if (NT > 1) {
    float A = 1.f, B = 0.f;
    if (ok) {
#pragma unroll 4
      for (int t = t0; t < t1; ++t) {
        float a, b;
        coef(t, a, b);
        B = fmaf(a, B, b);
        A *= a;
      }
    }
    sA[j][x] = A;
    sB[j][x] = B;
    __syncthreads();
  }
  float* st = state + (size_t)seq_slots[s] * C;
  float S = (ok && p0 != 0) ? st[chc] : 0.f;
  for (int jj = 0; jj < j; ++jj) S = fmaf(sA[jj][x], S, sB[jj][x]);
  if (!ok) return;
  const float yb = ybias[ch];
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    float a, b;
    coef(t, a, b);
    S = fmaf(a, S, b);
    const float g = proj[(size_t)t * ld + ycol + ch] + yb;
    const float y = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    stf(out, (size_t)t * C + ch, S * y);
  }
  if (j == NT - 1) st[ch] = S;
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_short_conv(void* out, const float* x, long ldx, const float* w, float* state, const int* cu_q,
                              const int* tok_seq, const int* seq_slots, const int* positions, const float* in_bias,
                              const float* out_bias, int act, int T, int C, int taps, int nseq, int unit_cols,
                              int unit_dim, int scale_cols, float scale, float unit_eps, int residual, int out_f32,
                              hipStream_t s) {
  if (T <= 0 || nseq <= 0) return 0;
  if (C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || act < 0 || act > 1) return -1;
  if (taps > 1 && state == nullptr) return -1;
  if (unit_cols < 0 || unit_cols > C || (unit_cols > 0 && (unit_dim <= 0 || unit_dim > 256 || unit_cols % unit_dim)))
    return -1;
  // few tokens (decoding): the channels of a token are spread over several workgroups
  const int ngroups = unit_cols > 0 ? unit_cols / unit_dim : 0;
  int ny = (ngroups + 3) / 4 > (C - unit_cols + 255) / 256 ? (ngroups + 3) / 4 : (C - unit_cols + 255) / 256;
  const int want = T >= 1024 ? 1 : (1024 + T - 1) / T;
  ny = ny < 1 ? 1 : (ny > want ? want : ny);
  if (out_f32)
    short_conv_kernel<float><<<dim3(T, ny), 256, 0, s>>>((float*)out, x, ldx, w, state, cu_q, tok_seq, seq_slots,
                                                         positions, in_bias, out_bias, act, C, taps, unit_cols, unit_dim,
                                                         scale_cols, scale, unit_eps, residual);
  else
    short_conv_kernel<bf16_t><<<dim3(T, ny), 256, 0, s>>>((bf16_t*)out, x, ldx, w, state, cu_q, tok_seq, seq_slots,
                                                          positions, in_bias, out_bias, act, C, taps, unit_cols,
                                                          unit_dim, scale_cols, scale, unit_eps, residual);
  if (taps > 1) {
    const dim3 grid(nseq, (C + 255) / 256);
    if (grid.y > 65535) return -2;
    conv_save_kernel<<<grid, 256, 0, s>>>(state, x, ldx, cu_q, seq_slots, positions, in_bias, C, taps);
  }
  return (int)hipGetLastError();
}

// Block shape for `cols` columns: DX x NS threads with CH key channels per thread; false when it exceeds 1024 threads.
static bool delta_shape(int D, int cols, int* dx, int* ch) {
  const int m = D > cols ? D : cols;
  *dx = (m + 63) / 64 * 64;
  *ch = 16;
  while (*ch < 64 && *dx * ((D + *ch - 1) / *ch) > 1024) *ch *= 2;
  return *dx * ((D + *ch - 1) / *ch) <= 1024;
}

// Whether portions of these head sizes can run as passes over chunks (the first pass carries D + V columns).
extern "C" int k8s_delta_scan_chunks_ok(int D, int V) {
  int dx, ch;
  // the prefix pass keeps a chunk's D x D transition in LDS (within 150 KB)
  return D > 0 && V > 0 && D <= 256 && V <= 256 && delta_shape(D, V + D, &dx, &ch) && (long)D * (D + 1) * 4 <= 150 * 1024;
}

// ws (chunked passes): floats for chunks x H records of D (V + D) and of D V, chunks = ceil(T / Lc) + nseq.
extern "C" long long k8s_delta_scan_workspace(int T, int nseq, int H, int D, int V, int Lc) {
  if (Lc <= 0) return 0;
  const long long chunks = (T + Lc - 1) / Lc + nseq;
  return chunks * H * ((long long)D * (V + D) + (long long)D * V);
}

extern "C" int k8s_delta_scan(void* out, const float* qkv, const float* proj, long ld, int cb, int ca, int cg,
                              const float* neg_a, const float* dt_bias, const float* normw, float* state,
                              const int* cu_q, const int* seq_slots, const int* positions, int nseq, int H, int G, int D,
                              int V, float eps, int f32, int T, int Lc, float* ws, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (H <= 0 || H > 65535 || G <= 0 || H % G || D <= 0 || D > 256 || V <= 0 || V > 256) return -1;
  int dx, ch;
  if (!delta_shape(D, V, &dx, &ch)) return -2;
  dim3 block(dx, (D + ch - 1) / ch);
  float* loc = nullptr;
  float* start = nullptr;
#define K8S_DS(TA, CH, MODE, GX)                                                                                      \
  delta_scan_kernel<TA, CH, MODE><<<dim3(GX, H), block, 0, s>>>((TA*)out, qkv, proj, ld, cb, ca, cg, neg_a, dt_bias,  \
                                                                normw, state, cu_q, seq_slots, positions, H, G, D, V, \
                                                                eps, nseq, Lc, loc, start)
#define K8S_DS_C(TA, MODE, GX)                 \
  do {                                         \
    if (ch == 16) K8S_DS(TA, 16, MODE, GX);    \
    else if (ch == 32) K8S_DS(TA, 32, MODE, GX); \
    else K8S_DS(TA, 64, MODE, GX);             \
  } while (0)
#define K8S_DS_T(MODE, GX)                     \
  do {                                         \
    if (f32) K8S_DS_C(float, MODE, GX);        \
    else K8S_DS_C(bf16_t, MODE, GX);           \
  } while (0)
  if (Lc <= 0 || ws == nullptr || !k8s_delta_scan_chunks_ok(D, V)) {
    K8S_DS_T(0, nseq);
    return (int)hipGetLastError();
  }
  const int chunks = (T + Lc - 1) / Lc + nseq;
  loc = ws;
  start = ws + (size_t)chunks * H * ((size_t)D * (V + D));
  const dim3 block2 = block;
  const int ch2 = ch;
  delta_shape(D, V + D, &dx, &ch);
  block = dim3(dx, (D + ch - 1) / ch);
  K8S_DS_T(1, chunks);
  {
    int xt = 16;
    while (xt > 1 && xt * D > 1024) xt /= 2;
    const dim3 pgrid(nseq, H, (V + xt - 1) / xt), pblock(xt, D);
    const size_t plds = ((size_t)D * (D + 1) + 2 * (size_t)D * xt) * sizeof(float);
    const int np = (D * D + xt * D - 1) / (xt * D);     // elements of P per thread: D / xt
#define K8S_DP(NP)                                                                                                     \
  do {                                                                                                                 \
    if (plds > 48 * 1024 &&                                                                                            \
        hipFuncSetAttribute((const void*)delta_prefix_kernel<NP>, hipFuncAttributeMaxDynamicSharedMemorySize,          \
                            (int)plds) != hipSuccess)                                                                  \
      return -3;                                                                                                       \
    delta_prefix_kernel<NP><<<pgrid, pblock, plds, s>>>(start, loc, state, cu_q, seq_slots, positions, H, D, V, Lc);   \
  } while (0)
    if (np <= 4) K8S_DP(4);
    else if (np <= 16) K8S_DP(16);
    else K8S_DP(64);
#undef K8S_DP
  }
  block = block2;
  ch = ch2;
  K8S_DS_T(2, chunks);
#undef K8S_DS_T
#undef K8S_DS_C
#undef K8S_DS
  return (int)hipGetLastError();
}

extern "C" int k8s_rglru_scan(void* out, const float* u, const float* gates, const float* gate_bias, const float* rate,
                              const float* proj, long ld, int ycol, const float* ybias, float* state, const int* cu_q,
                              const int* seq_slots, const int* positions, int nseq, int C, int blocks, int max_qlen,
                              int f32, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (C <= 0 || blocks <= 0 || C % blocks || (C + 63) / 64 > 65535) return -1;
  int nt = (max_qlen + 31) / 32;       // time slices of at least 32 tokens
  nt = nt < 1 ? 1 : (nt > 16 ? 16 : nt);
  const dim3 grid(nseq, (C + 63) / 64), block(64, nt);
  if (f32)
    rglru_scan_kernel<float><<<grid, block, 0, s>>>((float*)out, u, gates, gate_bias, rate, proj, ld, ycol, ybias, state,
                                                    cu_q, seq_slots, positions, C, blocks);
  else
    rglru_scan_kernel<bf16_t><<<grid, block, 0, s>>>((bf16_t*)out, u, gates, gate_bias, rate, proj, ld, ycol, ybias,
                                                     state, cu_q, seq_slots, positions, C, blocks);
  return (int)hipGetLastError();
}
