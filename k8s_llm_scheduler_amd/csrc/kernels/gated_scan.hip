// Gated linear recurrences with a matrix state per head, S [D key channels][V value channels] in fp32, carried per
// sequence slot:
//   KIND 0 (HGRN2: the forget gate also sets what is written)
//       f = low + (1 - low) sigmoid(zf + bf)  per key channel;  S <- diag(f) S + (1 - f) v^T;  o = S^T silu(zq);
//       y = o / rms(o) * normw[V]
//   KIND 1 (mLSTM: exponential input gate under a running maximum m that starts at 0)
//       i = cap tanh((zi + bi) / cap), f = logsigmoid(cap tanh((zf + bf) / cap))  per head;
//       m' = max(f + m, i), a = exp(f + m - m'), b = exp(i - m');  S <- a S + b k v^T, n <- a n + b k;
//       o = S^T q / (max(|n . q|, exp(-m')) + 1e-6), q = zq / sqrt(D);  y = o / rms(o) * normw[H V] * sigmoid(zg)
//   KIND 2 (state-space duality: one decay per head and token, set by a step size)
//       dt = softplus(zdt + dt_bias), a = exp(neg_a dt) with neg_a = -exp(A_log) per head;  S <- a S + dt B x^T;
//       y = (S^T C + skip x) * silu(zg);  B and C [D] are shared by the R heads of a group, x [V] is the head's own;
//       no norm here (it runs over groups of heads afterwards) and y is stored in fp32.  x, B and C come from `proj`
//       (the convolved branch), zdt and zg from `aux` (the input projection); neg_a, dt_bias and skip from `hpar`
//       ([3][H] fp32).
// Everything that enters the recurrence (gates, decays, state, norms) is fp32: the kernels read the fused input
// projection as fp32 [T, ld] with the parts at column offsets, and write y in the activation type.
// Varlen batches: sequence s owns tokens cu_q[s] .. cu_q[s + 1] - 1 and the state record of slot seq_slots[s]; a portion
// that starts at position 0 starts from zero state (m = 0), so a reused slot needs no clearing.
#include "common.h"

namespace k8sllm {

struct ScanCols { int q, k, v, i, f, g; };   // column offsets of the parts inside a projected row

// One workgroup per (sequence or chunk, head).  Thread (x, c) owns value column x of the CH key channels
// [c CH, (c + 1) CH) of S; group c = 0 prepares each token's per-channel read / keep / write coefficients in LDS (and,
// KIND 1, owns n).  The partial outputs of the channel groups meet in LDS; group 0 normalises and stores.  The next
// token's inputs are loaded while the current one is computed; the barriers wait for LDS traffic only.
// blockDim = (DX, NS): DX = max(D, V) (KIND 2: V) rounded up to 64, NS = ceil(D / CH), CH (16, 32 or 64) the smallest
// that keeps DX NS within 1024 threads.  State record: S [D][V] (, n [D], m).
//
// MODE 0: a whole portion per workgroup, from the slot's state (zero at position 0) to the slot's state.
// Long portions run as three passes over chunks of Lc tokens, so the recurrence is parallel over chunks; a chunk record
// is S [D][V], then D floats (KIND 0: the product of the chunk's decays per channel; KIND 1: n), then (KIND 1) m and
// the sum F of the chunk's log forget gates:
// MODE 1: a chunk from the empty state, no outputs -> its record in cs_loc (KIND 1: the running maximum starts at
//         minus infinity, so the record is the chunk's own contribution under its own maximum);
//         gated_prefix_kernel then walks a sequence's chunks:
//           KIND 0: start[c + 1] = dec[c] * start[c] + loc[c]
//           KIND 1: m' = max(F + m, m_loc); (S, n)[c + 1] = e^(F + m - m') (S, n)[c] + e^(m_loc - m') (S, n)_loc
// MODE 2: a chunk from its start state with outputs; a sequence's last chunk leaves the slot's state.
template <typename TA, int CH, int KIND, int MODE>
__global__ __launch_bounds__(1024) void gated_scan_kernel(TA* __restrict__ out, const float* __restrict__ proj, long ld,
                                                          ScanCols co, const TA* __restrict__ fbias,
                                                          const TA* __restrict__ ibias, const TA* __restrict__ lower,
                                                          const TA* __restrict__ normw, float* __restrict__ state,
                                                          const int* __restrict__ cu_q,
                                                          const int* __restrict__ seq_slots,
                                                          const int* __restrict__ positions, int H, int D, int V,
                                                          float eps, float cap, int nseq, int Lc,
                                                          float* __restrict__ cs_loc,
                                                          const float* __restrict__ cs_start,
                                                          const float* __restrict__ aux, long ldaux,
                                                          const float* __restrict__ hpar, int R) {
  constexpr int DMAX = 256;
  __shared__ __attribute__((aligned(16))) float sq[DMAX], sa[DMAX], sb[DMAX];
  __shared__ float po[DMAX / CH][DMAX];
  __shared__ float red[4], rednq[4];
  const int hd = blockIdx.y;
  int s, a0, b0, p0;
  bool from_zero, last = true;
  if (MODE == 0) {
    s = blockIdx.x;
    a0 = cu_q[s];
    b0 = cu_q[s + 1];
    if (b0 <= a0) return;
    p0 = positions[a0];
    if (p0 < 0) return;
    from_zero = p0 == 0;
  } else {
    const WkvChunk ck = wkv_find_chunk(blockIdx.x, cu_q, positions, nseq, Lc);
    if (ck.s < 0) return;
    s = ck.s;
    last = ck.c == ck.n - 1;
    if (MODE == 1 && last) return;          // nothing follows a sequence's last chunk
    a0 = cu_q[s] + ck.c * Lc;
    b0 = min(cu_q[s + 1], a0 + Lc);
    p0 = positions[a0];
    from_zero = MODE == 1 || p0 == 0;
  }
  const int x = threadIdx.x, c = threadIdx.y, NS = blockDim.y, DX = blockDim.x;
  const bool onv = x < V, ond = x < D;
  // KIND 2: the block is as wide as the value columns only, and the D shared inputs of a token (B, C) are loaded by the
  // first ceil(D / DX) thread groups, element c DX + x each
  const int le = c * DX + x;
  const bool ldr = KIND == 2 && le < D;
  const int i0 = c * CH;
  const size_t rec = (size_t)D * V + (KIND == 1 ? D + 1 : 0);       // slot record
  const size_t crec = (size_t)D * V + D + 2;                         // chunk record
  float* st = state + ((size_t)seq_slots[s] * H + hd) * rec;
  const size_t cbase = ((size_t)blockIdx.x * H + hd) * crec;         // this chunk's record in cs_loc / cs_start
  // MODE 2 never reads the slot's record, which the sequence's last chunk overwrites: the prefix pass left a copy
  const float* src = MODE == 2 ? cs_start + cbase : st;
  float S[CH], decp[CH];
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    S[e] = (onv && i0 + e < D && !from_zero) ? src[(size_t)(i0 + e) * V + x] : 0.f;
    decp[e] = 1.f;
  }
  float nx = 0.f, m = MODE == 1 ? -INFINITY : 0.f, fsum = 0.f;
  if (KIND == 1 && !from_zero) {
    if (c == 0 && ond) nx = src[(size_t)D * V + x];
    m = src[(size_t)D * V + D];
  }
  if (c == 0)
    for (int e = x; e < DMAX; e += DX) sq[e] = sa[e] = sb[e] = 0.f;
  float lowx = 0.f, fbx = 0.f, nwx = 0.f, fbh = 0.f, ibh = 0.f;
  float nega = 0.f, skip = 0.f;
  const int qk0 = KIND == 2 ? (hd / R) * D : hd * D;    // the head's (KIND 2: its group's) query / key columns
  if (KIND == 2) {
    nega = hpar[hd];
    fbh = hpar[H + hd];
    skip = hpar[2 * H + hd];
  } else if (KIND == 0) {
    if (c == 0 && ond) {
      lowx = ldf(lower, (size_t)hd * D + x);
      fbx = fbias != nullptr ? ldf(fbias, (size_t)hd * D + x) : 0.f;
    }
    if (MODE != 1 && c == 0 && onv) nwx = ldf(normw, x);
  } else {
    fbh = fbias != nullptr ? ldf(fbias, hd) : 0.f;
    ibh = ibias != nullptr ? ldf(ibias, hd) : 0.f;
    if (MODE != 1 && c == 0 && onv) nwx = ldf(normw, (size_t)hd * V + x);
  }
  const float qscale = KIND == 1 ? 1.0f / sqrtf((float)D) : 1.f;
  lds_barrier();
  // inputs of the next token
  float nq = 0.f, nk = 0.f, nv = 0.f, nf = 0.f, ni = 0.f, ng = 0.f;
  auto fetch = [&](int t) {
    if (t >= b0) return;
    const float* r = proj + (size_t)t * ld;
    if (onv) nv = r[co.v + (size_t)hd * V + x];
    if (KIND == 2) {
      const float* ar = aux + (size_t)t * ldaux;
      nf = ar[co.f + hd];
      if (MODE != 1 && c == 0 && onv) ng = ar[co.g + (size_t)hd * V + x];
      if (ldr) {
        if (MODE != 1) nq = r[co.q + qk0 + le];
        nk = r[co.k + qk0 + le];
      }
      return;
    }
    if (KIND == 1) {
      nf = r[co.f + hd];
      ni = r[co.i + hd];
      if (MODE != 1 && c == 0 && onv) ng = r[co.g + (size_t)hd * V + x];
    }
    if (c == 0 && ond) {
      if (MODE != 1) nq = r[co.q + (size_t)hd * D + x];
      if (KIND == 0) nf = r[co.f + (size_t)hd * D + x];
      else nk = r[co.k + (size_t)hd * D + x];
    }
  };
  fetch(a0);
  for (int t = a0; t < b0; ++t) {
    const float cq = nq, ck = nk, cv = nv, cf = nf, ci = ni, cg = ng;
    fetch(t + 1);
    float ka = 1.f;   // KIND 1, 2: the head's keep factor
    if (KIND == 2) {
      const float zd = cf + fbh;
      const float dt = fmaxf(zd, 0.f) + log1pf(expf(-fabsf(zd)));
      ka = expf(nega * dt);
      if (ldr) {
        sq[le] = cq;
        sb[le] = dt * ck;
      }
    } else if (KIND == 0) {
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
      ka = expf(fg + m - mn);           // 0 at the first token of a chunk from the empty state (m = -inf)
      const float kb = expf(ig - mn);
      m = mn;
      fsum += fg;
      if (c == 0) {
        float nqp = 0.f;
        if (ond) {
          const float qv = cq * qscale;
          nx = ka * nx + kb * ck;
          nqp = nx * qv;
          sq[x] = qv;
          sb[x] = kb * ck;
        }
        if (MODE != 1) {
          nqp = wave_sum(nqp);
          if ((x & 63) == 0) rednq[x >> 6] = nqp;
        }
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
        if (MODE != 1) o4[e] = fmaf(q4[e], S[e0 + e], o4[e]);
        if (MODE == 1 && KIND != 1) decp[e0 + e] *= a4[e];
      }
    }
    if (MODE == 1) {
      lds_barrier();                   // the LDS rows are free for the next token
      continue;
    }
    if (onv) po[c][x] = (o4[0] + o4[1]) + (o4[2] + o4[3]);
    lds_barrier();
    float o = 0.f, ss = 0.f;
    if (KIND == 2) {
      if (c == 0 && onv) {
        for (int g = 0; g < NS; ++g) o += po[g][x];
        o = fmaf(skip, cv, o);
        reinterpret_cast<float*>(out)[(size_t)t * H * V + (size_t)hd * V + x] = o * cg / (1.f + expf(-cg));
      }
      continue;      // po is next written after the next token's first barrier
    }
    if (c == 0) {
      if (onv)
        for (int g = 0; g < NS; ++g) o += po[g][x];
      if (KIND == 1) {
        float nqs = rednq[0];
        for (int w = 1; w < (D + 63) / 64; ++w) nqs += rednq[w];
        o /= fmaxf(fabsf(nqs), expf(-m)) + 1e-6f;
      }
      ss = wave_sum(onv ? o * o : 0.f);
      if (DX > 64 && (x & 63) == 0) red[x >> 6] = ss;
    }
    if (DX > 64) {                     // the channels span several waves: one more exchange (uniform branch)
      lds_barrier();
      ss = red[0];
      for (int w = 1; w < DX / 64; ++w) ss += red[w];
    }
    if (c == 0 && onv) {
      float y = o / sqrtf(ss / (float)V + eps) * nwx;
      if (KIND == 1) y *= 1.f / (1.f + expf(-cg));
      stf(out, (size_t)t * H * V + (size_t)hd * V + x, y);
    }
  }
  if (MODE == 2 && !last) return;
  float* dst = MODE == 1 ? cs_loc + cbase : st;
  if (onv) {
#pragma unroll
    for (int e = 0; e < CH; ++e)
      if (i0 + e < D) dst[(size_t)(i0 + e) * V + x] = S[e];
  }
  if (KIND == 1 && c == 0) {
    if (ond) dst[(size_t)D * V + x] = nx;
    if (x == 0) {
      dst[(size_t)D * V + D] = m;
      if (MODE == 1) dst[(size_t)D * V + D + 1] = fsum;
    }
  }
  if (KIND != 1 && MODE == 1 && x == 0) {
#pragma unroll
    for (int e = 0; e < CH; ++e)
      if (i0 + e < D) dst[(size_t)D * V + i0 + e] = decp[e];
  }
}

// Start states of a sequence's chunks from the slot's state (zero at position 0: chunk 0 has no record then) and the
// chunks' records.
// Workgroups (sequence, head, slice of the record's elements); every thread walks the chunks for its elements of (S, n).
template <int KIND>
__global__ void gated_prefix_kernel(float* __restrict__ cs_start, const float* __restrict__ cs_loc,
                                    const float* __restrict__ state, const int* __restrict__ cu_q,
                                    const int* __restrict__ seq_slots, const int* __restrict__ positions, int H, int D,
                                    int V, int Lc) {
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
  if (zero && n < 2) return;
  const int DV = D * V;
  const size_t rec = (size_t)DV + (KIND == 1 ? D + 1 : 0), crec = (size_t)DV + D + 2;
  const float* st = state + ((size_t)seq_slots[s] * H + hd) * rec;
  const int nel = KIND == 1 ? DV + D : DV;
  float* own = cs_start + ((size_t)first * H + hd) * crec;        // chunk 0 starts from a copy of the slot's record
  for (int e = blockIdx.z * blockDim.x + threadIdx.x; e < nel; e += blockDim.x * gridDim.z) {
    float X = zero ? 0.f : st[e];
    float m = (KIND == 1 && !zero) ? st[DV + D] : 0.f;
    if (!zero) {
      own[e] = X;
      if (KIND == 1 && e == 0) own[DV + D] = m;
    }
    for (int c = 0; c + 1 < n; ++c) {
      const float* loc = cs_loc + ((size_t)(first + c) * H + hd) * crec;
      float* nxt = cs_start + ((size_t)(first + c + 1) * H + hd) * crec;
      if (KIND == 0) {
        X = fmaf(loc[DV + e / V], X, loc[e]);
      } else {
        const float ml = loc[DV + D], F = loc[DV + D + 1];
        const float mn = fmaxf(F + m, ml);
        X = expf(F + m - mn) * X + expf(ml - mn) * loc[e];
        m = mn;
        if (e == 0) nxt[DV + D] = m;
      }
      nxt[e] = X;
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_gated_scan_max_dim() { return 256; }

// floats of one (slot, head) state record
extern "C" long long k8s_gated_scan_record(int kind, int D, int V) {
  return (long long)D * V + (kind == 1 ? D + 1 : 0);
}

// ws (chunked passes): floats for 2 x chunks x H chunk records, chunks = ceil(T / Lc) + nseq; Lc == 0 (or no
// workspace): one workgroup per sequence.
extern "C" long long k8s_gated_scan_workspace(int T, int nseq, int H, int D, int V, int Lc) {
  if (Lc <= 0) return 0;
  const long long chunks = (T + Lc - 1) / Lc + nseq;
  return 2 * chunks * H * ((long long)D * V + D + 2);
}

extern "C" int k8s_gated_scan(void* out, const float* proj, long ld, int kind, int cq, int ck, int cv, int ci, int cf,
                              int cg, const void* fbias, const void* ibias, const void* lower, const void* normw,
                              float* state, const int* cu_q, const int* seq_slots, const int* positions, int nseq, int H,
                              int D, int V, float eps, float cap, int f32, int T, int Lc, float* ws, const float* aux,
                              long ldaux, const float* hpar, int R, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (H <= 0 || H > 65535 || D <= 0 || D > 256 || V <= 0 || V > 256 || kind < 0 || kind > 2) return -1;
  if (kind == 2 && (aux == nullptr || hpar == nullptr || R <= 0 || H % R)) return -1;
  if (kind == 0 && lower == nullptr) return -1;
  if (kind == 1 && !(cap > 0.f)) return -1;
  const int m = (kind == 2 || V > D) ? V : D, DX = (m + 63) / 64 * 64;
  int ch = 16;
  while (ch < 64 && DX * ((D + ch - 1) / ch) > 1024) ch *= 2;
  if (DX * ((D + ch - 1) / ch) > 1024) return -2;
  const dim3 block(DX, (D + ch - 1) / ch);
  const ScanCols co{cq, ck, cv, ci, cf, cg};
#define K8S_GS(TA, CH, KIND, MODE, GX, LOC, START)                                                                  \
  gated_scan_kernel<TA, CH, KIND, MODE><<<dim3(GX, H), block, 0, s>>>(                                              \
      (TA*)out, proj, ld, co, (const TA*)fbias, (const TA*)ibias, (const TA*)lower, (const TA*)normw, state, cu_q,  \
      seq_slots, positions, H, D, V, eps, cap, nseq, Lc, LOC, START, aux, ldaux, hpar, R)
#define K8S_GS_C(TA, KIND, MODE, GX, LOC, START)                     \
  do {                                                               \
    if (ch == 16) K8S_GS(TA, 16, KIND, MODE, GX, LOC, START);        \
    else if (ch == 32) K8S_GS(TA, 32, KIND, MODE, GX, LOC, START);   \
    else K8S_GS(TA, 64, KIND, MODE, GX, LOC, START);                 \
  } while (0)
#define K8S_GS_K(TA, MODE, GX, LOC, START)                       \
  do {                                                           \
    if (kind == 0) K8S_GS_C(TA, 0, MODE, GX, LOC, START);        \
    else if (kind == 1) K8S_GS_C(TA, 1, MODE, GX, LOC, START);   \
    else K8S_GS_C(float, 2, MODE, GX, LOC, START);               \
  } while (0)
#define K8S_GS_T(MODE, GX, LOC, START)                      \
  do {                                                      \
    if (f32) K8S_GS_K(float, MODE, GX, LOC, START);         \
    else K8S_GS_K(bf16_t, MODE, GX, LOC, START);            \
  } while (0)
  if (Lc <= 0 || ws == nullptr) {
    K8S_GS_T(0, nseq, nullptr, nullptr);
    return (int)hipGetLastError();
  }
  const int chunks = (T + Lc - 1) / Lc + nseq;
  float* loc = ws;
  float* start = ws + (size_t)chunks * H * ((size_t)D * V + D + 2);
  K8S_GS_T(1, chunks, loc, nullptr);
  // a record's elements walk the chunks independently of each other: at most four per thread
  int pz = (D * V + D + 1023) / 1024;
  pz = pz < 1 ? 1 : (pz > 64 ? 64 : pz);
  const dim3 pgrid(nseq, H, pz);
  if (kind != 1)     // one decay per key channel (KIND 2: the head's, repeated)
    gated_prefix_kernel<0><<<pgrid, 256, 0, s>>>(start, loc, state, cu_q, seq_slots, positions, H, D, V, Lc);
  else
    gated_prefix_kernel<1><<<pgrid, 256, 0, s>>>(start, loc, state, cu_q, seq_slots, positions, H, D, V, Lc);
  K8S_GS_T(2, chunks, nullptr, start);
#undef K8S_GS_T
#undef K8S_GS_K
#undef K8S_GS_C
#undef K8S_GS
  return (int)hipGetLastError();
}
