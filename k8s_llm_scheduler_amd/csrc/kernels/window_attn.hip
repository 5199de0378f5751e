// Grouped-query sliding-window attention over a paged K / V cache, with pooled far context:
//   * the token at position p sees the cached tokens of positions max(0, p - window + 1) .. p and, beside them, one
//     key / value per block of P consecutive tokens that lies wholly before the window (block b = positions
//     b P .. b P + P - 1, seen when b P + P - 1 <= p - window): the mean of the block's cached keys / values;
//   * tokens and blocks share one softmax, optionally with a sink (a key of score 0 without a value: one more unit
//     in the denominator);
//   * instead of a window the mask can be chunked: positions are cut into chunks of `chunk` counted from 0 and a token
//     sees the tokens of its own chunk up to itself; scores can be soft-capped (cap tanh(s / cap)); the sink can be a
//     learned number per head (e^sink in the denominator); the output gate is per element or one number per head;
//   * queries and keys are prepared by one kernel per token: bias, optional RMS norm over the whole projection with a
//     weight, rotation of the first `dims` dimensions (interleaved pairs or the half layout), optional unit RMS per
//     head, value mixing with another layer's values, paged cache write (none for a layer that reads another's cache).
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
// more vectors than waves).  x = proj + bias; (qnw / knw) x = x / rms(whole q or k projection) * weight;
// (x[2i], x[2i + 1]) -- half layout: (x[i], x[i + dims / 2]) -- turns by the angle of cos_sin[pos] = [cos(dims / 2) |
// sin(dims / 2)]; then x / sqrt(mean(x^2) + eps) when `unit`.  (hqw / hkw [D]) before the rotation every head is
// divided by its own root mean square and multiplied by the weight, the same for all heads.  Queries are written back
// in place, keys to
// kcache[slot][g][D].  Values: v = proj + bias, then (vfirst_in) v = (1 - lam) v + lam vfirst_in[t]; (vfirst_out)
// vfirst_out[t] = v in fp32; vcache[slot][g][V] = v.
template <typename TA>
__global__ __launch_bounds__(256) void window_kv_write_kernel(
    TA* __restrict__ kcache, TA* __restrict__ vcache, TA* __restrict__ qkv, long ld, int koff, int voff,
    const TA* __restrict__ qb, const TA* __restrict__ kb, const TA* __restrict__ vb, const float* __restrict__ cos_sin,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping, const float* __restrict__ vfirst_in,
    float* __restrict__ vfirst_out, float lam, int H, int G, int D, int V, int dims, float eps, int unit,
    int half_layout, const TA* __restrict__ qnw, const TA* __restrict__ knw, const TA* __restrict__ hqw,
    const TA* __restrict__ hkw) {
  extern __shared__ float xs[];   // [waves][D]
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int slot = slot_mapping[t];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = blockDim.x >> 6;
  const int half = dims / 2;
  const float* cs = cos_sin + (size_t)pos * dims;
  TA* row = qkv + (size_t)t * ld;
  float* x = xs + (size_t)wave * D;
  float invq = 1.f, invk = 1.f;
  if (qnw != nullptr) {           // uniform branches: the norm runs over all heads of the projection at once
    float ss = 0.f;
    for (int i = tid; i < H * D; i += blockDim.x) {
      const float v = ldf(row, i) + (qb != nullptr ? ldf(qb, i) : 0.f);
      ss += v * v;
    }
    invq = 1.0f / sqrtf(block_sum(ss, red) / (float)(H * D) + eps);
  }
  if (knw != nullptr && G > 0) {
    float ss = 0.f;
    for (int i = tid; i < G * D; i += blockDim.x) {
      const float v = ldf(row + koff, i) + (kb != nullptr ? ldf(kb, i) : 0.f);
      ss += v * v;
    }
    invk = 1.0f / sqrtf(block_sum(ss, red) / (float)(G * D) + eps);
  }
  for (int hv = wave; hv < H + G; hv += nw) {
    const bool isq = hv < H;
    const int hd = isq ? hv : hv - H;
    const TA* src = row + (isq ? 0 : koff) + (size_t)hd * D;
    const TA* bias = isq ? qb : kb;
    const TA* nrm = isq ? qnw : knw;
    const TA* hnw = isq ? hqw : hkw;
    const float inv0 = isq ? invq : invk;
    float hs = 0.f;
    for (int d = lane; d < D; d += 64) {
      float v = ldf(src, d) + (bias != nullptr ? ldf(bias, (size_t)hd * D + d) : 0.f);
      if (nrm != nullptr) v *= inv0 * ldf(nrm, (size_t)hd * D + d);
      x[d] = v;
      hs += v * v;
    }
    if (hnw != nullptr) {            // uniform over the wave; every lane rescales the elements it wrote itself
      const float hinv = 1.0f / sqrtf(wave_sum(hs) / (float)D + eps);
      for (int d = lane; d < D; d += 64) x[d] *= hinv * ldf(hnw, d);
    }
    wave_lds_sync();
    float ss = 0.f;
    float y[8];   // D <= 512
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      const int d = lane + 64 * n;
      float v = 0.f;
      if (d < D) {
        v = x[d];
        if (d < dims && half_layout) {
          const bool first = d < half;
          const int i = first ? d : d - half;
          const float c = cs[i], sn = cs[half + i];
          const float a = x[i], b = x[i + half];
          v = first ? a * c - b * sn : b * c + a * sn;
        } else if (d < dims) {
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

// Workgroups (token, slice of the row); only tokens that end a block of P work ((pos + 1) % P == 0): the mean, in fp32, of the
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
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < GD + GV; i += gridDim.y * blockDim.x) {
    float a = 0.f;
#pragma unroll 4
    for (int j = b * P; j < b * P + P; ++j) {
      const size_t slot = (size_t)btr[j / bs] * bs + (j % bs);
      a += i < GD ? ldf(kcache, slot * GD + i) : ldf(vcache, slot * GV + (i - GD));
    }
    if (i < GD) kpool[e * GD + i] = a * invp;
    else vpool[e * GV + (i - GD)] = a * invp;
  }
}

// 8 consecutive elements of a cached row as fp32 (one or two 16-byte loads).
__device__ __forceinline__ void load8(const bf16_t* p, float* o) {
  const u32x4 v = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = lo_bf(v[i]);
    o[2 * i + 1] = hi_bf(v[i]);
  }
}
__device__ __forceinline__ void load8(const float* p, float* o) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[i] = a[i];
    o[4 + i] = b[i];
  }
}

// One workgroup per (token, key / value head, key split); one wave per query head of the group (further passes when
// the group has more heads than waves).  The visible keys are an ordered list: the nb pooled blocks, then the window's
// tokens.  They come in tiles of KB <= 64 rows staged in LDS as fp32 and shared by the group's heads (the rows' cache
// slots are resolved once per tile; VEC: rows move as 16-byte vectors, D and V multiples of 8); lane l scores row l
// (q . k * scale), the tile joins a running softmax, lane l accumulates value dimensions l, l + 64, ...
// A sink starts the running softmax at (max 0, sum 1).  One split: out[t][head][V] = sum p v / sum, times
// sigmoid(gate) if given.  Several splits (few tokens, many keys: decoding) each take a run of tiles and leave
// (max, sum, unnormalised sum p v) for window_merge_kernel; the sink belongs to split 0.
template <typename TA, int NACC, bool VEC>
__global__ void window_attention_kernel(TA* __restrict__ out, float* __restrict__ pacc, float* __restrict__ pml,
                                        const TA* __restrict__ q, long ldq, const TA* __restrict__ gate, long ldg,
                                        const TA* __restrict__ kcache, const TA* __restrict__ vcache,
                                        const float* __restrict__ kpool, const float* __restrict__ vpool,
                                        const int* __restrict__ block_tables, int max_blocks,
                                        const int* __restrict__ tok_seq, const int* __restrict__ positions, int H, int G,
                                        int D, int V, int window, int P, float scale, int sink, int bs, int ppb, int KB,
                                        int nsplit, int chunk, float softcap, const float* __restrict__ sinkv,
                                        int gate_ph) {
  extern __shared__ float smem[];
  const int t = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int R = H / G;
  const int p = positions[t];
  if (p < 0) {   // idle row: defined output, nothing read
    if (nsplit == 1)
      for (int i = threadIdx.x; i < R * V; i += blockDim.x) stf(out, (size_t)t * H * V + (size_t)g * R * V + i, 0.f);
    return;
  }
  const int DP = D + 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = blockDim.x >> 6;
  float* ktile = smem;                         // [KB][D + 1]
  float* vtile = ktile + (size_t)KB * DP;      // [KB][V]
  float* qs = vtile + (size_t)KB * V;          // [nw][D]
  size_t roff = (size_t)KB * (DP + V) + (size_t)nw * D;
  roff += roff & 1;                            // 8-byte aligned
  long long* rowoff = reinterpret_cast<long long*>(smem + roff);   // [KB] a tile row's cache slot, or -1 - pool entry
  const int lo = chunk > 0 ? p - p % chunk : (window > 0 ? max(0, p - window + 1) : 0);
  const int nb = (window > 0 && P > 0 && p - window + 1 >= P) ? (p - window + 1) / P : 0;
  const int nkeys = nb + (p + 1 - lo);
  const int ntiles = (nkeys + KB - 1) / KB;
  const int tps = (ntiles + nsplit - 1) / nsplit;
  const int tile0 = split * tps, tile1 = min(ntiles, tile0 + tps);
  const int* btr = block_tables + (size_t)tok_seq[t] * max_blocks;
  const int GD = G * D, GV = G * V;
  const bool with_sink = sink && split == 0;
  for (int h0 = 0; h0 < R; h0 += nw) {
    const int hd = g * R + h0 + wave;
    const bool hv = h0 + wave < R;
    float* qq = qs + (size_t)wave * D;
    if (hv)
      for (int d = lane; d < D; d += 64) qq[d] = ldf(q, (size_t)t * ldq + (size_t)hd * D + d);
    float m = with_sink ? ((sinkv != nullptr && hv) ? sinkv[hd] : 0.f) : -INFINITY, l = with_sink ? 1.f : 0.f, acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    for (int tile = tile0; tile < tile1; ++tile) {
      const int u0 = tile * KB;
      const int nk = min(KB, nkeys - u0);
      __syncthreads();
      for (int r = tid; r < nk; r += blockDim.x) {
        const int u = u0 + r;
        if (u < nb) {
          rowoff[r] = -1 - (long long)pool_entry(btr, u, P, bs, ppb);
        } else {
          const int j = lo + (u - nb);
          rowoff[r] = (long long)btr[j / bs] * bs + (j % bs);
        }
      }
      __syncthreads();
      if (VEC) {
        const int ckd = D >> 3, cpr = ckd + (V >> 3);
        for (int idx = tid; idx < nk * cpr; idx += blockDim.x) {
          const int r = idx / cpr, c = idx - r * cpr;
          const bool isk = c < ckd;
          const int e8 = 8 * (isk ? c : c - ckd);
          const long long ro = rowoff[r];
          float v8[8];
          if (ro < 0) load8(isk ? kpool + (size_t)(-1 - ro) * GD + (size_t)g * D + e8
                                : vpool + (size_t)(-1 - ro) * GV + (size_t)g * V + e8, v8);
          else load8(isk ? kcache + (size_t)ro * GD + (size_t)g * D + e8 : vcache + (size_t)ro * GV + (size_t)g * V + e8, v8);
          float* dst = isk ? ktile + r * DP + e8 : vtile + r * V + e8;
#pragma unroll
          for (int i = 0; i < 8; ++i) dst[i] = v8[i];
        }
      } else {
        for (int idx = tid; idx < nk * (D + V); idx += blockDim.x) {
          const int r = idx / (D + V), d = idx - r * (D + V);
          const long long ro = rowoff[r];
          float val;
          if (ro < 0) {
            const size_t e = (size_t)(-1 - ro);
            val = d < D ? kpool[e * GD + (size_t)g * D + d] : vpool[e * GV + (size_t)g * V + (d - D)];
          } else {
            val = d < D ? ldf(kcache, (size_t)ro * GD + (size_t)g * D + d)
                        : ldf(vcache, (size_t)ro * GV + (size_t)g * V + (d - D));
          }
          if (d < D) ktile[r * DP + d] = val;
          else vtile[r * V + (d - D)] = val;
        }
      }
      __syncthreads();
      if (hv) {
        float sc = -INFINITY;
        if (lane < nk) {
          const float* kr = ktile + lane * DP;
          float a = 0.f;
          for (int d = 0; d < D; ++d) a = fmaf(qq[d], kr[d], a);
          sc = a * scale;
          if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
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
    if (hv && nsplit == 1) {
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < V) {
          float o = acc[i] / l;
          if (gate != nullptr)
            o *= 1.f / (1.f + expf(-ldf(gate, (size_t)t * ldg + (gate_ph ? (size_t)hd : (size_t)hd * V + d))));
          stf(out, (size_t)t * H * V + (size_t)hd * V + d, o);
        }
      }
    } else if (hv) {
      const size_t rec = ((size_t)t * H + hd) * nsplit + split;
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < V) pacc[rec * V + d] = acc[i];
      }
      if (lane == 0) {
        pml[rec * 2] = m;           // -inf and 0 for a split without tiles and without the sink
        pml[rec * 2 + 1] = l;
      }
    }
  }
}

// out[t][head] = sum_s e^(m_s - M) acc_s / sum_s e^(m_s - M) l_s over the key splits, times sigmoid(gate) if given.
template <typename TA>
__global__ void window_merge_kernel(TA* __restrict__ out, const float* __restrict__ pacc, const float* __restrict__ pml,
                                    const TA* __restrict__ gate, long ldg, const int* __restrict__ positions, int H,
                                    int V, int nsplit, int gate_ph) {
  const int t = blockIdx.x, hd = blockIdx.y;
  if (positions[t] < 0) {
    for (int d = threadIdx.x; d < V; d += blockDim.x) stf(out, (size_t)t * H * V + (size_t)hd * V + d, 0.f);
    return;
  }
  const size_t rec0 = ((size_t)t * H + hd) * nsplit;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, pml[(rec0 + s) * 2]);
  float den = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float ms = pml[(rec0 + s) * 2];
    if (ms != -INFINITY) den += expf(ms - M) * pml[(rec0 + s) * 2 + 1];
  }
  for (int d = threadIdx.x; d < V; d += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float ms = pml[(rec0 + s) * 2];
      if (ms != -INFINITY) a += expf(ms - M) * pacc[(rec0 + s) * V + d];
    }
    float o = a / den;
    if (gate != nullptr)
      o *= 1.f / (1.f + expf(-ldf(gate, (size_t)t * ldg + (gate_ph ? (size_t)hd : (size_t)hd * V + d))));
    stf(out, (size_t)t * H * V + (size_t)hd * V + d, o);
  }
}

// The same attention on the matrix cores for prompts in bf16 (D % 8 == 0, V % 16 == 0, R = H / G a power of two <= 16).
// A workgroup of 4 waves takes TPB consecutive tokens of one sequence and one key / value head; a wave owns NCB blocks
// of 16 query columns, a column being one (token, query head of the group) pair, 16 / R tokens per block.  The keys of
// the workgroup are the ordered list [pooled blocks 0 .. nb(last token) | tokens lo(first token) .. last token]; 32 of
// them per step are staged in LDS as bf16 (pooled rows converted from fp32) and shared by the waves, each column masks
// what its own token does not see:
//   S^T[key][column] = K Q^T      A = 16 staged key rows, B = the columns' queries (registers)
//   O[column][d]    += P V        A = the 32 keys' probabilities (registers, keys in the order the S^T tiles left
//                                 them), B = the staged value columns through the transposing LDS read
// scores, softmax and sums in fp32, the weights applied as two bf16 terms; a sink starts every column at (max 0, sum 1).
typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;

template <int NKK, int NVB, int NCB, bool PF>
__global__ __launch_bounds__(256) void window_attention_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long ldq, const bf16_t* __restrict__ gate, long ldg,
    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache, const float* __restrict__ kpool,
    const float* __restrict__ vpool, const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ positions, int H, int G, int D, int V, int window, int P, float scale, int sink, int bs,
    int ppb, int R, int chunk, float softcap, const float* __restrict__ sinkv, int gate_ph) {
  extern __shared__ __attribute__((aligned(16))) char smem_w[];
  const int seq = blockIdx.z, g = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 15, g4 = lane >> 4;
  const int TPC = 16 / R, TPB = 4 * NCB * TPC;
  const int tq0 = cu_q[seq] + blockIdx.x * TPB, tend = cu_q[seq + 1];
  if (tq0 >= tend) return;
  const int p_first = positions[tq0];
  const int nval = min(TPB, tend - tq0);
  if (p_first < 0) {   // idle rows: defined output
    for (int i = tid; i < nval * R * V; i += 256) {
      const int tt = i / (R * V), r = i - tt * (R * V);
      out[(size_t)(tq0 + tt) * H * V + (size_t)g * R * V + r] = 0;
    }
    return;
  }
  const int p_last = p_first + nval - 1;
  const int rowk = (D + 8) * 2, rowv = (V + 8) * 2;      // LDS row bytes
  char* klds = smem_w;                                   // [32][D + 8] bf16
  char* vlds = smem_w + 32 * rowk;                       // [32][V + 8] bf16
  const bool win = window > 0;
  // the first position a token at p sees: its chunk's first, the window's first, or 0 (never decreasing in p)
  auto lo_of = [&](int p) { return chunk > 0 ? p - p % chunk : (win ? max(0, p - window + 1) : 0); };
  const int lo_min = lo_of(p_first);
  const int nb_max = (win && P > 0 && p_last - window + 1 >= P) ? (p_last - window + 1) / P : 0;
  const int nkeys = nb_max + (p_last + 1 - lo_min);
  const int nsteps = (nkeys + 31) / 32;
  const int* btr = block_tables + (size_t)seq * max_blocks;
  const int GD = G * D, GV = G * V;
  const int ckd = D / 8, ckv = V / 8, cpr = ckd + ckv;   // 16-byte chunks per staged row
  const int nkk = (D + 31) / 32, nvb = V / 16;
  const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
  // this lane's column in every block of the wave: token, position, first visible token, visible pooled blocks
  int c_tok[NCB], c_p[NCB], c_lo[NCB], c_nb[NCB];
  bf16x8 qf[NCB][NKK];
  int w_pmin = 0x7fffffff, w_pmax = -1;
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int toff = (wave * NCB + cb) * TPC + li / R;
    const bool ok = toff < nval;
    c_tok[cb] = tq0 + toff;
    c_p[cb] = ok ? p_first + toff : -1;
    c_lo[cb] = ok ? lo_of(c_p[cb]) : 0;
    c_nb[cb] = (ok && win && P > 0 && c_p[cb] - window + 1 >= P) ? (c_p[cb] - window + 1) / P : 0;
    const int hd = g * R + li % R;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      const int piece = 32 * kk + 8 * g4;
      u32x4 v = zero;
      if (ok && piece < D) v = *reinterpret_cast<const u32x4*>(q + (size_t)c_tok[cb] * ldq + (size_t)hd * D + piece);
      qf[cb][kk] = __builtin_bit_cast(bf16x8, v);
    }
    const int t_lo = (wave * NCB + cb) * TPC, t_hi = min(t_lo + TPC, nval) - 1;
    if (t_lo < nval) {
      w_pmin = min(w_pmin, p_first + t_lo);
      w_pmax = max(w_pmax, p_first + t_hi);
    }
  }
  const bool w_any = w_pmax >= 0;
  const int w_lo = w_any ? lo_of(w_pmin) : 0;
  const int w_nb = (w_any && win && P > 0 && w_pmax - window + 1 >= P) ? (w_pmax - window + 1) / P : 0;
  f32x4 o[NCB][NVB];
  float m_run[NCB], l_run[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    m_run[cb] = sink ? (sinkv != nullptr ? sinkv[g * R + li % R] : 0.f) : -INFINITY;
    l_run[cb] = sink ? 1.f : 0.f;
#pragma unroll
    for (int n = 0; n < NVB; ++n) o[cb][n] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int qd = li >> 2, pd = li & 3;
  // Staging: every thread moves NST 16-byte chunks of a step's 32 rows.  PF: the chunks of step s + 1 are loaded into
  // registers before step s is computed and written to LDS after it, so the cache reads run under the MFMAs -- for
  // grids of at most one workgroup per CU, where nothing else hides them; larger grids run the variant without the
  // held registers, at twice the waves per SIMD.
  constexpr int NST = (NKK * 4 + NVB * 2 + 7) / 8;
  u32x4 pre[NST];
  auto stage_load = [&](int u0) {
#pragma unroll
    for (int i = 0; i < NST; ++i) {
      const int idx = tid + 256 * i;
      u32x4 v = zero;
      if (idx < 32 * cpr) {
        const int r = idx / cpr, c = idx - r * cpr, u = u0 + r;
        const bool isk = c < ckd;
        const int e8 = 8 * (isk ? c : c - ckd);
        if (u < nb_max) {
          const size_t e = pool_entry(btr, u, P, bs, ppb);
          const float* src = isk ? kpool + e * GD + (size_t)g * D + e8 : vpool + e * GV + (size_t)g * V + e8;
          const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
          v = u32x4{pack_bf2(a[0], a[1]), pack_bf2(a[2], a[3]), pack_bf2(b[0], b[1]), pack_bf2(b[2], b[3])};
        } else if (u < nkeys) {
          const int j = lo_min + (u - nb_max);
          const size_t slot = (size_t)btr[j / bs] * bs + (j % bs);
          v = isk ? *reinterpret_cast<const u32x4*>(kcache + slot * GD + (size_t)g * D + e8)
                  : *reinterpret_cast<const u32x4*>(vcache + slot * GV + (size_t)g * V + e8);
        }
      }
      pre[i] = v;
    }
  };
  auto stage_store = [&]() {
#pragma unroll
    for (int i = 0; i < NST; ++i) {
      const int idx = tid + 256 * i;
      if (idx < 32 * cpr) {
        const int r = idx / cpr, c = idx - r * cpr;
        const bool isk = c < ckd;
        const int e8 = 8 * (isk ? c : c - ckd);
        *reinterpret_cast<u32x4*>((isk ? klds + r * rowk : vlds + r * rowv) + 2 * e8) = pre[i];
      }
    }
  };
  if (PF) stage_load(0);
  for (int step = 0; step < nsteps; ++step) {
    const int u0 = step * 32;
    __syncthreads();          // the previous step's fragments have been read
    if (PF) {
      stage_store();
    } else {                  // chunk by chunk: no registers held across the step
      for (int idx = tid; idx < 32 * cpr; idx += 256) {
        const int r = idx / cpr, c = idx - r * cpr, u = u0 + r;
        const bool isk = c < ckd;
        const int e8 = 8 * (isk ? c : c - ckd);
        u32x4 v = zero;
        if (u < nb_max) {
          const size_t e = pool_entry(btr, u, P, bs, ppb);
          const float* src = isk ? kpool + e * GD + (size_t)g * D + e8 : vpool + e * GV + (size_t)g * V + e8;
          const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
          v = u32x4{pack_bf2(a[0], a[1]), pack_bf2(a[2], a[3]), pack_bf2(b[0], b[1]), pack_bf2(b[2], b[3])};
        } else if (u < nkeys) {
          const int j = lo_min + (u - nb_max);
          const size_t slot = (size_t)btr[j / bs] * bs + (j % bs);
          v = isk ? *reinterpret_cast<const u32x4*>(kcache + slot * GD + (size_t)g * D + e8)
                  : *reinterpret_cast<const u32x4*>(vcache + slot * GV + (size_t)g * V + e8);
        }
        *reinterpret_cast<u32x4*>((isk ? klds + r * rowk : vlds + r * rowv) + 2 * e8) = v;
      }
    }
    __syncthreads();
    if (PF && step + 1 < nsteps) stage_load(u0 + 32);
    // keys of this step that any column of the wave can see: pooled blocks below w_nb, tokens w_lo .. w_pmax
    bool any = false;
    if (w_any) {
      if (u0 < nb_max) any = u0 < w_nb;
      const int j_first = lo_min + max(u0 - nb_max, 0), j_last = lo_min + (u0 + 31 - nb_max);
      if (u0 + 31 >= nb_max && j_first <= w_pmax && j_last >= w_lo) any = true;
    }
    if (!any) continue;
    // every staged key fragment is read once and serves all column blocks of the wave
    f32x4 sacc[NCB][2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) sacc[cb][m] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        if (kk < nkk) {
          const int piece = 32 * kk + 8 * g4;
          bf16x8 ka = __builtin_bit_cast(bf16x8, zero);
          if (piece < D) ka = *reinterpret_cast<const bf16x8*>(klds + (16 * m + li) * rowk + 2 * piece);
#pragma unroll
          for (int cb = 0; cb < NCB; ++cb)
            sacc[cb][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[cb][kk], sacc[cb][m], 0, 0, 0);
        }
      }
    }   // sacc[cb][m][i] = S[key u0 + 16 m + 4 g4 + i][column li of block cb]
    bf16x8 pa[NCB], pl[NCB];   // slot j < 4: key 4 g4 + j; slot j >= 4: key 16 + 4 g4 + (j - 4)
    float a_i[NCB][4];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      float tmax = -INFINITY;
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int u = u0 + 16 * m + 4 * g4 + i;
          bool vis;
          if (u < nb_max) vis = u < c_nb[cb];
          else {
            const int j = lo_min + (u - nb_max);
            vis = j <= c_p[cb] && j >= c_lo[cb];
          }
          float v = -INFINITY;
          if (vis) {
            v = sacc[cb][m][i] * scale;
            if (softcap > 0.f) v = softcap * tanhf(v / softcap);
          }
          sacc[cb][m][i] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
      const float m_new = fmaxf(m_run[cb], tmax);
      const float m_ref = m_new == -INFINITY ? 0.f : m_new;      // a column that has seen nothing yet
      const float alpha = m_run[cb] == -INFINITY ? 0.f : expf(m_run[cb] - m_ref);
      float rsum = 0.f;
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pv = expf(sacc[cb][m][i] - m_ref);
          sacc[cb][m][i] = pv;
          rsum += pv;
        }
      rsum += __shfl_xor(rsum, 16, WAVE);
      rsum += __shfl_xor(rsum, 32, WAVE);
      l_run[cb] = l_run[cb] * alpha + rsum;
      m_run[cb] = m_new;
#pragma unroll
      for (int i = 0; i < 4; ++i) a_i[cb][i] = __shfl(alpha, g4 * 4 + i, WAVE);
      // the fp32 weights enter the product as two bf16 terms (p = hi + lo, |lo| <= 2^-9 p): 16 bits of each weight
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pa[cb][j] = (__bf16)sacc[cb][0][j];
        pa[cb][4 + j] = (__bf16)sacc[cb][1][j];
        pl[cb][j] = (__bf16)(sacc[cb][0][j] - (float)pa[cb][j]);
        pl[cb][4 + j] = (__bf16)(sacc[cb][1][j] - (float)pa[cb][4 + j]);
      }
    }
    const int r0 = 4 * g4 + qd, r1 = r0 + 16;
#pragma unroll
    for (int n = 0; n < NVB; ++n) {
      if (n < nvb) {
        const int col = 16 * n + 4 * pd;
        const bf16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(vlds + r0 * rowv + 2 * col));
        const bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(vlds + r1 * rowv + 2 * col));
        bf16x8 vb;
#pragma unroll
        for (int j = 0; j < 4; ++j) { vb[j] = v0[j]; vb[4 + j] = v1[j]; }
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
#pragma unroll
          for (int i = 0; i < 4; ++i) o[cb][n][i] *= a_i[cb][i];
          o[cb][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa[cb], vb, o[cb][n], 0, 0, 0);
          o[cb][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl[cb], vb, o[cb][n], 0, 0, 0);
        }
      }
    }
  }
  // o[cb][n][i] = O[column 4 g4 + i][d 16 n + li]; a column's sum lives in the lanes with li == column
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    float l_i[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) l_i[i] = __shfl(l_run[cb], g4 * 4 + i, WAVE);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = 4 * g4 + i;
      const int toff = (wave * NCB + cb) * TPC + c / R;
      if (toff >= nval) continue;
      const int t = tq0 + toff, hd = g * R + c % R;
      const float inv = 1.f / l_i[i];
#pragma unroll
      for (int n = 0; n < NVB; ++n)
        if (n < nvb) {
          const int d = 16 * n + li;
          float y = o[cb][n][i] * inv;
          if (gate != nullptr)
            y *= 1.f / (1.f + expf(-bf2f(gate[(size_t)t * ldg + (gate_ph ? (size_t)hd : (size_t)hd * V + d)])));
          out[(size_t)t * H * V + (size_t)hd * V + d] = f2bf(y);
        }
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_window_kv_write(void* kcache, void* vcache, void* qkv, long ld, int koff, int voff, const void* qb,
                                   const void* kb, const void* vb, const float* cos_sin, const int* positions,
                                   const int* slot_mapping, const float* vfirst_in, float* vfirst_out, float lam, int T,
                                   int H, int G, int D, int V, int dims, float eps, int unit, int half_layout,
                                   const void* qnw, const void* knw, const void* hqw, const void* hkw, int f32,
                                   hipStream_t s) {
  if (T <= 0) return 0;
  // G == 0: a layer that attends another layer's cache prepares its queries only
  if (H <= 0 || G < 0 || (G > 0 && H % G) || D <= 0 || D > 512 || V <= 0 || dims < 0 || dims > D || (dims & 1)) return -1;
  if (G > 0 && (kcache == nullptr || vcache == nullptr)) return -1;
  if (dims > 0 && cos_sin == nullptr) return -1;
  const size_t lds = (size_t)4 * D * sizeof(float);
#define K8S_WKW(TA)                                                                                                   \
  window_kv_write_kernel<TA><<<T, 256, lds, s>>>((TA*)kcache, (TA*)vcache, (TA*)qkv, ld, koff, voff, (const TA*)qb,    \
                                                 (const TA*)kb, (const TA*)vb, cos_sin, positions, slot_mapping,      \
                                                 vfirst_in, vfirst_out, lam, H, G, D, V, dims, eps, unit, half_layout, \
                                                 (const TA*)qnw, (const TA*)knw, (const TA*)hqw, (const TA*)hkw)
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
  const int slices = (G * (D + V) + 255) / 256;
  const dim3 grid(T, slices < 16 ? slices : 16);
  if (f32)
    window_pool_kernel<float><<<grid, 256, 0, s>>>(kpool, vpool, (const float*)kcache, (const float*)vcache,
                                                   block_tables, max_blocks, tok_seq, positions, G, D, V, P, bs, ppb);
  else
    window_pool_kernel<bf16_t><<<grid, 256, 0, s>>>(kpool, vpool, (const bf16_t*)kcache, (const bf16_t*)vcache,
                                                    block_tables, max_blocks, tok_seq, positions, G, D, V, P, bs, ppb);
  return (int)hipGetLastError();
}

// Tile rows of the plain kernel for these sizes (0: they do not fit) -- the caller sizes the key splits with it.
extern "C" int k8s_window_tile_rows(int H, int G, int D, int V) {
  if (G <= 0 || H % G) return 0;
  const int R = H / G, nw = R < 8 ? R : 8;
  // LDS floats: KB (D + 1 + V) tile + nw D queries + KB row offsets (2 floats each), within 60 KB
  int KB = (15360 - nw * D - 2) / (D + 1 + V + 2);
  return KB > 64 ? 64 : (KB < 1 ? 0 : KB);
}

// nsplit > 1: pacc [T, H, nsplit, V] and pml [T, H, nsplit, 2] fp32 workspaces.
extern "C" int k8s_window_attention(void* out, float* pacc, float* pml, const void* q, long ldq, const void* gate,
                                    long ldg, const void* kcache, const void* vcache, const float* kpool,
                                    const float* vpool, const int* block_tables, int max_blocks, const int* tok_seq,
                                    const int* positions, int T, int H, int G, int D, int V, int window, int P,
                                    float scale, int sink, int bs, int nsplit, int chunk, float softcap,
                                    const float* sinkv, int gate_ph, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || V <= 0 || V > 256 || bs <= 0 || G > 65535) return -1;
  if (window > 0 && P > 0 && (kpool == nullptr || vpool == nullptr)) return -1;
  if (nsplit < 1 || nsplit > 65535 || (nsplit > 1 && (pacc == nullptr || pml == nullptr))) return -1;
  const int R = H / G;
  const int nw = R < 8 ? R : 8;
  const int KB = k8s_window_tile_rows(H, G, D, V);
  if (KB < 1) return -2;
  const size_t lds = ((size_t)KB * (D + 1 + V) + (size_t)nw * D + 2 + 2 * (size_t)KB) * sizeof(float);
  const int ppb = P > 0 ? (bs + P - 1) / P : 1;
  const int nacc = (V + 63) / 64;
  const bool vec = D % 8 == 0 && V % 8 == 0 && (f32 || ((long)G * D) % 8 == 0);
#define K8S_WA(TA, NA, VEC)                                                                                           \
  window_attention_kernel<TA, NA, VEC><<<dim3(T, G, nsplit), nw * 64, lds, s>>>(                                      \
      (TA*)out, pacc, pml, (const TA*)q, ldq, (const TA*)gate, ldg, (const TA*)kcache, (const TA*)vcache, kpool,      \
      vpool, block_tables, max_blocks, tok_seq, positions, H, G, D, V, window, P, scale, sink, bs, ppb, KB, nsplit,   \
      chunk, softcap, sinkv, gate_ph)
#define K8S_WA_V(TA, NA)            \
  do {                              \
    if (vec) K8S_WA(TA, NA, true);  \
    else K8S_WA(TA, NA, false);     \
  } while (0)
#define K8S_WA_T(TA)                     \
  do {                                   \
    if (nacc <= 1) K8S_WA_V(TA, 1);      \
    else if (nacc <= 2) K8S_WA_V(TA, 2); \
    else K8S_WA_V(TA, 4);                \
  } while (0)
  if (f32) K8S_WA_T(float);
  else K8S_WA_T(bf16_t);
#undef K8S_WA_T
#undef K8S_WA_V
#undef K8S_WA
  if (nsplit > 1) {
    if (f32)
      window_merge_kernel<float><<<dim3(T, H), 64, 0, s>>>((float*)out, pacc, pml, (const float*)gate, ldg, positions, H,
                                                           V, nsplit, gate_ph);
    else
      window_merge_kernel<bf16_t><<<dim3(T, H), 64, 0, s>>>((bf16_t*)out, pacc, pml, (const bf16_t*)gate, ldg,
                                                            positions, H, V, nsplit, gate_ph);
  }
  return (int)hipGetLastError();
}

// Whether the matrix-core kernel takes these sizes (else the caller uses k8s_window_attention).
extern "C" int k8s_window_mfma_ok(int H, int G, int D, int V) {
  if (G <= 0 || H % G) return 0;
  const int R = H / G;
  return (R == 1 || R == 2 || R == 4 || R == 8 || R == 16) && D % 8 == 0 && V % 16 == 0 && D <= 256 && V <= 256;
}

// Prompt portions in bf16: nseq sequences of at most max_qlen tokens, cu_q their query offsets.
extern "C" int k8s_window_attention_mfma(void* out, const void* q, long ldq, const void* gate, long ldg,
                                         const void* kcache, const void* vcache, const float* kpool, const float* vpool,
                                         const int* block_tables, int max_blocks, const int* cu_q, const int* positions,
                                         int nseq, int max_qlen, int H, int G, int D, int V, int window, int P,
                                         float scale, int sink, int bs, int chunk, float softcap,
                                         const float* sinkv, int gate_ph, hipStream_t s) {
  if (nseq <= 0 || max_qlen <= 0) return 0;
  if (!k8s_window_mfma_ok(H, G, D, V) || bs <= 0 || nseq > 65535 || G > 65535 || ldq % 8 || ((uintptr_t)q & 15)) return -1;
  if (window > 0 && P > 0 && (kpool == nullptr || vpool == nullptr)) return -1;
  const int R = H / G, ppb = P > 0 ? (bs + P - 1) / P : 1;
  const size_t lds = (size_t)32 * ((D + 8) + (V + 8)) * 2;
  constexpr int NCB = 2;
  const int TPB = 4 * NCB * (16 / R);
  const dim3 grid((max_qlen + TPB - 1) / TPB, G, nseq);
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  const bool pf = (long)grid.x * grid.y * grid.z <= cus;
#define K8S_WM_P(NKK, NVB, PF)                                                                                        \
  window_attention_mfma_kernel<NKK, NVB, NCB, PF><<<grid, 256, lds, s>>>(                                             \
      (bf16_t*)out, (const bf16_t*)q, ldq, (const bf16_t*)gate, ldg, (const bf16_t*)kcache, (const bf16_t*)vcache,    \
      kpool, vpool, block_tables, max_blocks, cu_q, positions, H, G, D, V, window, P, scale, sink, bs, ppb, R, chunk, \
      softcap, sinkv, gate_ph)
#define K8S_WM(NKK, NVB)               \
  do {                                 \
    if (pf) K8S_WM_P(NKK, NVB, true);  \
    else K8S_WM_P(NKK, NVB, false);    \
  } while (0)
  if (D <= 64 && V <= 64) K8S_WM(2, 4);
  else if (D <= 128 && V <= 128) K8S_WM(4, 8);
  else K8S_WM_P(8, 16, false);
#undef K8S_WM
#undef K8S_WM_P
  return (int)hipGetLastError();
}
