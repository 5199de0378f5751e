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

// One workgroup per (sequence or chunk, head).  The head's state S[i][j] (i: key channel, j: value channel) lives in
// registers: thread (j, c) owns column j of the CH key channels [c CH, (c + 1) CH), so the per-token chain of a wave is
// CH steps, not D.  Per token:  o_j = sum_i r_i (S_ij + u_i k_i v_j);  S_ij = w_i S_ij + k_i v_j  with
// w = exp(-exp(z + w0)) in fp32; the channel groups' partial o_j meet in LDS, then group 0 applies the head's
// o / rms(o) * lnw * silu(g).  The next token's inputs are loaded while the current one is computed, and the barriers
// wait for LDS traffic only.  blockDim = (DV, NS): DV = D rounded up to 64, NS = ceil(D / CH).
//
// MODE 0: a whole sequence per workgroup, from the slot's state (zero at position 0) to the slot's state.
// Long prompts run as three passes over chunks of Lc tokens, so the recurrence is parallel over chunks:
// MODE 1: a chunk from a zero state, no outputs: its state contribution and the product of its decays -> cs_loc, cs_dec;
//         wkv_prefix_kernel then walks a sequence's chunks: start[c + 1] = dec[c] * start[c] + loc[c];
// MODE 2: a chunk from its start state with outputs; a sequence's last chunk leaves the slot's state.
template <typename TA, int CH, int MODE>
__global__ __launch_bounds__(1024) void wkv_scan_kernel(TA* __restrict__ out, const TA* __restrict__ r,
                                                        const TA* __restrict__ k, const TA* __restrict__ v,
                                                        const TA* __restrict__ g, long ld, const float* __restrict__ z,
                                                        const TA* __restrict__ w0, const TA* __restrict__ u,
                                                        const TA* __restrict__ lnw, float* __restrict__ state,
                                                        const int* __restrict__ cu_q, const int* __restrict__ seq_slots,
                                                        const int* __restrict__ positions, int H, int D, float eps,
                                                        int nseq, int Lc, float* __restrict__ cs_loc,
                                                        float* __restrict__ cs_dec, const float* __restrict__ cs_start) {
  constexpr int DMAX = 128;
  __shared__ __attribute__((aligned(16))) float sr[DMAX], sk[DMAX], sw[DMAX], su[DMAX];
  __shared__ float po[DMAX / CH][DMAX];
  __shared__ float red[4];
  const int hd = blockIdx.y;
  int s, a, b, p0;
  bool from_zero, last = true;
  if (MODE == 0) {
    s = blockIdx.x;
    a = cu_q[s];
    b = cu_q[s + 1];
    if (b <= a) return;
    p0 = positions[a];
    if (p0 < 0) return;
    from_zero = p0 == 0;
  } else {
    const WkvChunk ck = wkv_find_chunk(blockIdx.x, cu_q, positions, nseq, Lc);
    if (ck.s < 0) return;
    s = ck.s;
    last = ck.c == ck.n - 1;
    if (MODE == 1 && last) return;          // nothing follows a sequence's last chunk
    a = cu_q[s] + ck.c * Lc;
    b = min(cu_q[s + 1], a + Lc);
    p0 = positions[a];
    from_zero = MODE == 1 || p0 == 0;
  }
  const int j = threadIdx.x, c = threadIdx.y, NS = blockDim.y, DV = blockDim.x;
  const bool on = j < D;
  const int HD = H * D, i0 = c * CH;
  float* st = state + ((size_t)seq_slots[s] * H + hd) * D * D;
  const size_t crec = ((size_t)blockIdx.x * H + hd) * D * D;     // this chunk's record in cs_loc / cs_start
  const float* src = (MODE == 2 && a != cu_q[s]) ? cs_start + crec : st;
  float S[CH], decp[CH];
#pragma unroll
  for (int e = 0; e < CH; ++e) {
    S[e] = (on && i0 + e < D && !from_zero) ? src[(size_t)(i0 + e) * D + j] : 0.f;
    decp[e] = 1.f;
  }
  float w0j = 0.f, lnj = 0.f;
  if (c == 0) {                       // group 0 stages the token's r, k, w (and u once); channels >= D stay zero
    for (int x = j; x < DMAX; x += DV) sr[x] = sk[x] = sw[x] = su[x] = 0.f;
  }
  lds_barrier();
  if (c == 0 && on) {
    su[j] = ldf(u, (size_t)hd * D + j);
    w0j = ldf(w0, (size_t)hd * D + j);
    lnj = ldf(lnw, (size_t)hd * D + j);
  }
  // inputs of the next token (group 0: r, k, z, g and v; the others: v only)
  float nr = 0.f, nk = 0.f, nv = 0.f, ng = 0.f, nz = 0.f;
  auto fetch = [&](int t) {
    if (on && t < b) {
      const size_t base = (size_t)t * ld + (size_t)hd * D + j;
      nv = ldf(v, base);
      if (c == 0) {
        if (MODE != 1) {
          nr = ldf(r, base);
          ng = ldf(g, base);
        }
        nk = ldf(k, base);
        nz = z[(size_t)t * HD + (size_t)hd * D + j];
      }
    }
  };
  fetch(a);
  for (int t = a; t < b; ++t) {
    const float cr = nr, ck = nk, cv = nv, cg = ng, cz = nz;
    fetch(t + 1);
    if (c == 0 && on) {
      sr[j] = cr;
      sk[j] = ck;
      sw[j] = expf(-expf(cz + w0j));
    }
    lds_barrier();
    float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e0 = 0; e0 < CH; e0 += 4) {
      const f32x4 r4 = *reinterpret_cast<const f32x4*>(&sr[i0 + e0]);
      const f32x4 k4 = *reinterpret_cast<const f32x4*>(&sk[i0 + e0]);
      const f32x4 w4 = *reinterpret_cast<const f32x4*>(&sw[i0 + e0]);
      const f32x4 u4 = *reinterpret_cast<const f32x4*>(&su[i0 + e0]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float kv = k4[e] * cv;
        if (MODE != 1) o4[e] = fmaf(r4[e], fmaf(u4[e], kv, S[e0 + e]), o4[e]);
        S[e0 + e] = fmaf(w4[e], S[e0 + e], kv);
        if (MODE == 1) decp[e0 + e] *= w4[e];
      }
    }
    if (MODE == 1) {
      lds_barrier();                   // the LDS rows are free for the next token
      continue;
    }
    if (on) po[c][j] = (o4[0] + o4[1]) + (o4[2] + o4[3]);
    lds_barrier();
    float o = 0.f, ss = 0.f;
    if (c == 0) {
      if (on)
        for (int x = 0; x < NS; ++x) o += po[x][j];
      ss = wave_sum(on ? o * o : 0.f);
      if (DV > 64 && (j & 63) == 0) red[j >> 6] = ss;
    }
    if (DV > 64) {                     // the head's value channels span two waves: one more exchange (uniform branch)
      lds_barrier();
      ss = red[0] + red[1];
    }
    if (c == 0 && on) {
      const float y = o / sqrtf(ss / (float)D + eps) * lnj * (cg / (1.f + expf(-cg)));
      stf(out, (size_t)t * HD + (size_t)hd * D + j, y);
    }
  }
  if (on) {
    float* dst = MODE == 1 ? cs_loc + crec : st;
    if (MODE != 2 || last) {
#pragma unroll
      for (int e = 0; e < CH; ++e)
        if (i0 + e < D) dst[(size_t)(i0 + e) * D + j] = S[e];
    }
    if (MODE == 1 && j == 0) {
#pragma unroll
      for (int e = 0; e < CH; ++e)
        if (i0 + e < D) cs_dec[((size_t)blockIdx.x * H + hd) * D + i0 + e] = decp[e];
    }
  }
}

// start[first chunk + c + 1] = dec[c] * start[c] + loc[c] along a sequence's chunks; start of chunk 0 is the slot's state
// (or zero at position 0) and is read by the MODE 2 pass directly.  One workgroup per (sequence, head).
__global__ void wkv_prefix_kernel(float* __restrict__ cs_start, const float* __restrict__ cs_loc,
                                  const float* __restrict__ cs_dec, const float* __restrict__ state,
                                  const int* __restrict__ cu_q, const int* __restrict__ seq_slots,
                                  const int* __restrict__ positions, int H, int D, int Lc) {
  const int s = blockIdx.x, hd = blockIdx.y;
  int first = 0;
  for (int x = 0; x < s; ++x) {
    const int a = cu_q[x], len = cu_q[x + 1] - a;
    first += (len > 0 && positions[a] >= 0) ? (len + Lc - 1) / Lc : 0;
  }
  const int a = cu_q[s], len = cu_q[s + 1] - a;
  if (len <= 0 || positions[a] < 0) return;
  const int n = (len + Lc - 1) / Lc;
  if (n < 2) return;
  const bool zero = positions[a] == 0;
  const float* st = state + ((size_t)seq_slots[s] * H + hd) * D * D;
  for (int e = threadIdx.x; e < D * D; e += blockDim.x) {
    const int i = e / D;
    float S = zero ? 0.f : st[e];
    for (int c = 0; c + 1 < n; ++c) {
      const size_t rec = (size_t)(first + c) * H + hd;
      S = fmaf(cs_dec[rec * D + i], S, cs_loc[rec * D * D + e]);
      cs_start[(rec + H) * D * D + e] = S;      // chunk first + c + 1
    }
  }
}

// One workgroup per token: cache[slot] = [rms(dkv[:C]) * normw | rope(dkv[C:])] and the rotated part of every
// head of q ([T, H, Dn + R], last R of a head) rotated in place.  Rotation pairs dimension i with i + dims / 2 over
// the first `dims` rotated dimensions (`interleaved`: dimension 2i with 2i + 1); cos_sin[pos] = [cos(dims / 2) |
// sin(dims / 2)].  `ldd`: the row stride of dkv (a view into a wider projection).
template <typename TA>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(TA* __restrict__ cache, const TA* __restrict__ dkv,
                                                              const TA* __restrict__ normw, TA* __restrict__ q,
                                                              const float* __restrict__ cos_sin,
                                                              const int* __restrict__ positions,
                                                              const int* __restrict__ slot_mapping, int C, int R, int H,
                                                              int Dn, int dims, float eps, long ldd, int interleaved) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int slot = slot_mapping[t];
  const int L = C + R, half = dims / 2;
  const TA* d = dkv + (size_t)t * ldd;
  const int ia = interleaved ? 2 : 1, ib = interleaved ? 1 : half;   // pair i = elements (ia i, ia i + ib)
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
      const int e0 = C + ia * i, e1 = e0 + ib;
      const float a = ldf(d, e0), b = ldf(d, e1), c = cs[i], sn = cs[half + i];
      stf(row, e0, a * c - b * sn);
      stf(row, e1, b * c + a * sn);
    }
    for (int i = dims + threadIdx.x; i < R; i += blockDim.x) stf(row, C + i, ldf(d, C + i));
  }
  TA* qt = q + (size_t)t * H * (Dn + R);
  for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
    const int hh = idx / half, i = idx - hh * half;
    TA* qh = qt + (size_t)hh * (Dn + R) + Dn;
    const int e0 = ia * i, e1 = e0 + ib;
    const float a = ldf(qh, e0), b = ldf(qh, e1), c = cs[i], sn = cs[half + i];
    stf(qh, e0, a * c - b * sn);
    stf(qh, e1, b * c + a * sn);
  }
}

// One workgroup per token, one wave per head (heads beyond the wave count take further passes).  Keys come in blocks
// of KB <= 64 cached rows staged in LDS as fp32 and shared by the heads; lane l scores key l of the block
// ((q_abs . c + q_rot . k_rot) * scale), the block joins a running softmax, and lane l accumulates latent
// dimensions l, l + 64, ... of sum_j p_j c_j.  out [T, H, C] = that sum / the softmax denominator.  `sinks` [H] fp32
// (optional): the denominator of head h holds one more term e^sinks[h], which has no key and no value.
template <typename TA, int NACC>
__global__ void latent_attention_kernel(TA* __restrict__ out, const TA* __restrict__ q_abs, const TA* __restrict__ q,
                                        const TA* __restrict__ cache, const int* __restrict__ block_tables,
                                        int max_blocks, const int* __restrict__ tok_seq,
                                        const int* __restrict__ positions, int C, int R, int H, int Dn, int window,
                                        float scale, int bs, int KB, const float* __restrict__ sinks) {
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
      float inv = 1.f / l;
      if (sinks != nullptr) {          // join the sink under a common maximum
        const float sk = sinks[hd], mx = fmaxf(m, sk), am = expf(m - mx);
        inv = am / (l * am + expf(sk - mx));
      }
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < C) stf(out, ((size_t)t * H + hd) * C + d, acc[i] * inv);
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

// NWV = 1: one wave per (token, head group, key split) -- decoding, where every token is another sequence.
// NWV = 4: one workgroup per (4 consecutive tokens of a sequence, head group); the waves share every staged key step
// (the union of their windows) and mask their own range, so a prompt reads each cached row once per 4 queries.
// The queries stay in registers (NKK 32-wide pieces of [q_abs | q_rot] per lane).
// EX: the sizes fill the template's bounds exactly (C == 16 NDB, C + R == 32 NKK), so the unrolled loops hold no
// branches and the LDS reads of a step are issued ahead of the MFMAs that consume them.
template <int NDB, int NKK, int NWV, bool EX>
__global__ __launch_bounds__(64 * NWV) void latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, float* __restrict__ pacc, float* __restrict__ pml, const bf16_t* __restrict__ q_abs,
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, const int* __restrict__ cu_q, int C, int R,
    int H, int Dn, int window, float scale, int bs, int nsplit, const float* __restrict__ sinks, int bt_lds) {
  extern __shared__ __attribute__((aligned(16))) char smem_b[];
  char* klds = smem_b;               // [32][L + 8] bf16; then (bt_lds) the block-table entries of the keys this block reads
  const int hg = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 15, g = lane >> 4;
  const int L = C + R, rowb = (L + 8) * 2, ndb = EX ? NDB : C / 16, HP = gridDim.y * 16;
  int t, split, seq, p_first, p_last;
  bool valid;
  if (NWV == 1) {
    t = blockIdx.x;
    split = blockIdx.z;
    seq = tok_seq[t];
    p_first = p_last = positions[t];
    valid = true;
  } else {
    seq = blockIdx.z;
    split = 0;
    const int tq0 = cu_q[seq] + blockIdx.x * NWV, tend = cu_q[seq + 1];
    if (tq0 >= tend) return;
    const int nval = min(NWV, tend - tq0);
    t = tq0 + wave;
    valid = wave < nval;
    p_first = positions[tq0];
    p_last = p_first + nval - 1;
  }
  const int p = valid ? p_first + (NWV == 1 ? 0 : wave) : -1;
  if (p_first < 0) {                 // idle rows: defined output
    if (nsplit == 1 && valid)
      for (int i = lane; i < 16 * C; i += 64) {
        const int hd = hg * 16 + i / C;
        if (hd < H) out[((size_t)t * H + hd) * C + i % C] = 0;
      }
    return;
  }
  const int lo_min = window > 0 ? max(0, p_first - window + 1) : 0;
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int ntiles = (p_last + 1 - lo_min + 31) / 32;
  const int tps = (ntiles + nsplit - 1) / nsplit;
  const int t0 = split * tps, t1 = min(ntiles, t0 + tps);
  const int* btr = block_tables + (size_t)seq * max_blocks;
  const int cpr = EX ? 4 * NKK : L / 8;   // 16-byte chunks per row
  const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
  const int nkk = EX ? NKK : (L + 31) / 32;
  // NWV = 4: the block-table entries go to LDS once, so a step's row addresses do not wait for a global load each
  int* bts = reinterpret_cast<int*>(smem_b + 32 * rowb);
  const int b0 = lo_min / bs;
  const bool bt_staged = NWV == 4 && bt_lds != 0;
  if (bt_staged) {
    for (int i = tid; i <= p_last / bs - b0; i += 64 * NWV) bts[i] = btr[b0 + i];
    __syncthreads();
  }
  // B operand of S^T = K Q^T: lane (li = head, g) holds q[head][32 kk + 8 g .. + 7]
  bf16x8 qf[NKK];
  {
    const int hd = hg * 16 + li;
    const bool qok = valid && hd < H;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      const int piece = 32 * kk + 8 * g;
      u32x4 v = zero;
      if (qok && piece < L)
        v = piece < C ? *reinterpret_cast<const u32x4*>(q_abs + ((size_t)t * H + hd) * C + piece)
                      : *reinterpret_cast<const u32x4*>(q + ((size_t)t * H + hd) * (Dn + R) + Dn + (piece - C));
      qf[kk] = __builtin_bit_cast(bf16x8, v);
    }
  }
  f32x4 o[NDB];
#pragma unroll
  for (int n = 0; n < NDB; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int qd = li >> 2, pd = li & 3;
  // NWV = 4: the cache rows of the next step are loaded into registers under the MFMAs of the current one (PF 16-byte
  // pieces per thread cover 32 rows of up to 32 NKK elements); the LDS tile is written from them at the next step's start.
  constexpr int PF = NWV == 4 ? (NKK + 1) / 2 : 0;
  u32x4 pf[PF > 0 ? PF : 1];
  auto fetch = [&](int tile) {
    const int j0 = lo_min + tile * 32;
#pragma unroll
    for (int k = 0; k < PF; ++k) {
      const int idx = tid + k * 64 * NWV;
      u32x4 v = zero;
      if (idx < 32 * cpr) {
        const int r = idx / cpr, c = idx - r * cpr, key = j0 + r;
        if (key <= p_last) {
          const int kb = key / bs;
          const size_t slot = (size_t)(bt_staged ? bts[kb - b0] : btr[kb]) * bs + (key - kb * bs);
          v = *reinterpret_cast<const u32x4*>(cache + slot * L + 8 * c);
        }
      }
      pf[k] = v;
    }
  };
  if (PF > 0 && t0 < t1) fetch(t0);
  for (int tile = t0; tile < t1; ++tile) {
    const int j0 = lo_min + tile * 32;
    __syncthreads();
    if (PF > 0) {
#pragma unroll
      for (int k = 0; k < PF; ++k) {
        const int idx = tid + k * 64 * NWV;
        if (idx < 32 * cpr) {
          const int r = idx / cpr, c = idx - r * cpr;
          *reinterpret_cast<u32x4*>(klds + r * rowb + 16 * c) = pf[k];
        }
      }
    } else {
      for (int idx = tid; idx < 32 * cpr; idx += 64 * NWV) {
        const int r = idx / cpr, c = idx - r * cpr, key = j0 + r;
        u32x4 v = zero;
        if (key <= p_last) {
          const size_t slot = (size_t)btr[key / bs] * bs + (key % bs);
          v = *reinterpret_cast<const u32x4*>(cache + slot * L + 8 * c);
        }
        *reinterpret_cast<u32x4*>(klds + r * rowb + 16 * c) = v;
      }
    }
    __syncthreads();
    if (PF > 0 && tile + 1 < t1) fetch(tile + 1);
    if (!valid || j0 > p || j0 + 31 < lo) continue;     // no key of this step is visible to this wave's token
    f32x4 sacc[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        if (kk < nkk) {
          const int piece = 32 * kk + 8 * g;
          bf16x8 ka = __builtin_bit_cast(bf16x8, zero);
          if (EX || piece < L) ka = *reinterpret_cast<const bf16x8*>(klds + (16 * m + li) * rowb + 2 * piece);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[kk], acc, 0, 0, 0);
        }
      }
      sacc[m] = acc;   // S[key j0 + 16 m + 4 g + i][head li]
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = j0 + 16 * m + 4 * g + i;
        const float v = (key <= p && key >= lo) ? sacc[m][i] * scale : -INFINITY;
        sacc[m][i] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(m_run, tmax);       // finite: the step holds a visible key
    const float alpha = m_run == -INFINITY ? 0.f : __expf(m_run - m_new);
    float rsum = 0.f;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = __expf(sacc[m][i] - m_new);     // the weights are rounded to bf16 for the product
        sacc[m][i] = pv;
        rsum += pv;
      }
    rsum += __shfl_xor(rsum, 16, WAVE);
    rsum += __shfl_xor(rsum, 32, WAVE);
    l_run = l_run * alpha + rsum;
    m_run = m_new;
    // the running maxima settle after the first steps: the accumulators are rescaled only when some head's moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
      float a_i[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a_i[i] = __shfl(alpha, g * 4 + i, WAVE);
#pragma unroll
      for (int n = 0; n < NDB; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[n][i] *= a_i[i];
    }
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
  if (!valid) return;
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
      float inv = 1.f / l_i[i];
      if (sinks != nullptr) {
        const float sk = sinks[hd], mx = fmaxf(m_i[i], sk), am = expf(m_i[i] - mx);
        inv = am / (l_i[i] * am + expf(sk - mx));
      }
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

// out[t][head] = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s over the key splits; workgroups (token, head, slice of
// the latent columns)
__global__ void latent_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ pacc,
                                    const float* __restrict__ pml, const int* __restrict__ positions, int C, int H,
                                    int HP, int nsplit, const float* __restrict__ sinks) {
  const int t = blockIdx.x, hd = blockIdx.y;
  const int d0 = blockIdx.z * blockDim.x + threadIdx.x, dstep = blockDim.x * gridDim.z;
  if (positions[t] < 0) {
    for (int d = d0; d < C; d += dstep) out[((size_t)t * H + hd) * C + d] = 0;
    return;
  }
  const size_t rec0 = ((size_t)t * HP + hd) * nsplit;
  float M = sinks != nullptr ? sinks[hd] : -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, pml[(rec0 + s) * 2]);
  float den = sinks != nullptr ? expf(sinks[hd] - M) : 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float ms = pml[(rec0 + s) * 2];
    if (ms != -INFINITY) den += expf(ms - M) * pml[(rec0 + s) * 2 + 1];
  }
  for (int d = d0; d < C; d += dstep) {
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

// ws (MODE 1 / 2 passes): floats for 2 x chunks x H x D x D states + chunks x H x D decay products, chunks =
// ceil(T / Lc) + nseq; Lc == 0 (or no workspace): one workgroup per sequence.
extern "C" long long k8s_wkv_workspace(int T, int nseq, int H, int D, int Lc) {
  if (Lc <= 0) return 0;
  const long long chunks = (T + Lc - 1) / Lc + nseq;
  return chunks * H * ((long long)2 * D * D + D);
}

extern "C" int k8s_wkv_scan(void* out, const void* r, const void* k, const void* v, const void* g, long ld,
                            const float* z, const void* w0, const void* u, const void* lnw, float* state,
                            const int* cu_q, const int* seq_slots, const int* positions, int nseq, int H, int D,
                            float eps, int f32, int T, int Lc, float* ws, hipStream_t s) {
  if (nseq <= 0) return 0;
  if (H <= 0 || D <= 0 || D > 128 || H > 65535) return -1;
  constexpr int CH = 16;
  const dim3 block((D + 63) / 64 * 64, (D + CH - 1) / CH);
#define K8S_WKV(TA, MODE, GX, LOC, DEC, START)                                                                        \
  wkv_scan_kernel<TA, CH, MODE><<<dim3(GX, H), block, 0, s>>>((TA*)out, (const TA*)r, (const TA*)k, (const TA*)v,      \
                                                              (const TA*)g, ld, z, (const TA*)w0, (const TA*)u,        \
                                                              (const TA*)lnw, state, cu_q, seq_slots, positions, H, D, \
                                                              eps, nseq, Lc, LOC, DEC, START)
  if (Lc <= 0 || ws == nullptr) {
    if (f32) K8S_WKV(float, 0, nseq, nullptr, nullptr, nullptr);
    else K8S_WKV(bf16_t, 0, nseq, nullptr, nullptr, nullptr);
    return (int)hipGetLastError();
  }
  const int chunks = (T + Lc - 1) / Lc + nseq;
  float* loc = ws;
  float* start = ws + (size_t)chunks * H * D * D;
  float* dec = start + (size_t)chunks * H * D * D;
  if (f32) K8S_WKV(float, 1, chunks, loc, dec, nullptr);
  else K8S_WKV(bf16_t, 1, chunks, loc, dec, nullptr);
  wkv_prefix_kernel<<<dim3(nseq, H), 256, 0, s>>>(start, loc, dec, state, cu_q, seq_slots, positions, H, D, Lc);
  if (f32) K8S_WKV(float, 2, chunks, nullptr, nullptr, start);
  else K8S_WKV(bf16_t, 2, chunks, nullptr, nullptr, start);
#undef K8S_WKV
  return (int)hipGetLastError();
}

extern "C" int k8s_latent_kv_write(void* cache, const void* dkv, const void* normw, void* q, const float* cos_sin,
                                   const int* positions, const int* slot_mapping, int T, int C, int R, int H, int Dn,
                                   int dims, float eps, int f32, long ldd, int interleaved, hipStream_t s) {
  if (T <= 0) return 0;
  if (C <= 0 || R < 0 || dims < 0 || dims > R || (dims & 1) || H <= 0 || ldd < C + R) return -1;
  if (f32)
    latent_kv_write_kernel<float><<<T, 256, 0, s>>>((float*)cache, (const float*)dkv, (const float*)normw, (float*)q,
                                                    cos_sin, positions, slot_mapping, C, R, H, Dn, dims, eps, ldd,
                                                    interleaved);
  else
    latent_kv_write_kernel<bf16_t><<<T, 256, 0, s>>>((bf16_t*)cache, (const bf16_t*)dkv, (const bf16_t*)normw,
                                                     (bf16_t*)q, cos_sin, positions, slot_mapping, C, R, H, Dn, dims,
                                                     eps, ldd, interleaved);
  return (int)hipGetLastError();
}

extern "C" int k8s_latent_attention(void* out, const void* q_abs, const void* q, const void* cache,
                                    const int* block_tables, int max_blocks, const int* tok_seq, const int* positions,
                                    int T, int C, int R, int H, int Dn, int window, float scale, int bs, int f32,
                                    const float* sinks, hipStream_t s) {
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
                                                          window, scale, bs, KB, sinks)
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
  return C % 16 == 0 && R % 8 == 0 && Dn % 8 == 0 && C <= 512 && L <= 640;
}

// nsplit == 1 and cu_q given (nseq sequences of at most max_qlen tokens): 4 consecutive tokens of a sequence per
// workgroup; else one wave per (token, head group, key split).
extern "C" int k8s_latent_attention_mfma(void* out, float* pacc, float* pml, const void* q_abs, const void* q,
                                         const void* cache, const int* block_tables, int max_blocks,
                                         const int* tok_seq, const int* positions, int T, int C, int R, int H, int Dn,
                                         int window, float scale, int bs, int nsplit, const int* cu_q, int nseq,
                                         int max_qlen, const float* sinks, hipStream_t s) {
  if (T <= 0) return 0;
  if (!k8s_latent_mfma_ok(C, R, Dn) || H <= 0 || bs <= 0 || nsplit < 1 || (nsplit > 1 && (!pacc || !pml))) return -1;
  const int L = C + R, HG = (H + 15) / 16;
  const size_t lds = (size_t)32 * (L + 8) * 2;
  // the block table of one sequence beside the key tile, within the 64 KB a launch gets without asking for more
  const int bt_lds = lds + (size_t)max_blocks * sizeof(int) <= 65536;
  const size_t bt_bytes = bt_lds ? (size_t)max_blocks * sizeof(int) : 0;
  const bool tiles = nsplit == 1 && cu_q != nullptr && nseq > 0 && max_qlen > 1;
  if (tiles && nseq > 65535) return -2;
  const dim3 grid = tiles ? dim3((max_qlen + 3) / 4, HG, nseq) : dim3(T, HG, nsplit);
#define K8S_LM(NDB, NKK, EX)                                                                                            \
  do {                                                                                                                \
    if (tiles)                                                                                                        \
      latent_attention_mfma_kernel<NDB, NKK, 4, EX><<<grid, 256, lds + bt_bytes, s>>>(                                             \
          (bf16_t*)out, pacc, pml, (const bf16_t*)q_abs, (const bf16_t*)q, (const bf16_t*)cache, block_tables,        \
          max_blocks, tok_seq, positions, cu_q, C, R, H, Dn, window, scale, bs, nsplit, sinks, bt_lds);               \
    else                                                                                                              \
      latent_attention_mfma_kernel<NDB, NKK, 1, EX><<<grid, 64, lds, s>>>(                                             \
          (bf16_t*)out, pacc, pml, (const bf16_t*)q_abs, (const bf16_t*)q, (const bf16_t*)cache, block_tables,        \
          max_blocks, tok_seq, positions, cu_q, C, R, H, Dn, window, scale, bs, nsplit, sinks, 0);                    \
  } while (0)
  if (C == 512 && L == 576) K8S_LM(32, 18, true);        // sizes that fill an instantiation exactly
  else if (C == 256 && L == 320) K8S_LM(16, 10, true);
  else if (C == 128 && L == 192) K8S_LM(8, 6, true);
  else if (C == 128 && L == 160) K8S_LM(8, 5, true);
  else if (C == 64 && L == 96) K8S_LM(4, 3, true);
  else if (C <= 128 && L <= 256) K8S_LM(8, 8, false);
  else if (C <= 256 && L <= 256) K8S_LM(16, 8, false);
  else if (C <= 256) K8S_LM(16, 20, false);
  else K8S_LM(32, 20, false);
#undef K8S_LM
  if (nsplit > 1)
    latent_merge_kernel<<<dim3(T, H, (C + 127) / 128), 128, 0, s>>>((bf16_t*)out, pacc, pml, positions, C, H, HG * 16,
                                                                    nsplit, sinks);
  return (int)hipGetLastError();
}
