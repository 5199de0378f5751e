// fp32 residual stream: embedding rows, fused residual-add + RMS norm, gated activations, and a GEMM for any shape.
//
// Models whose residual sum lives in fp32 keep x as [T, W] floats; every branch output (bf16, or fp32 in the all-fp32
// mode) is added in fp32 by the norm that follows it, so the add costs no extra pass.  All kernels take the
// activation / weight element type as a template parameter: bf16 storage or true fp32.
#include "common.h"

namespace k8sllm {

// out[t, :] = float(table[ids[t], :]) * scale
template <typename TA>
__global__ void embed_rows_kernel(float* __restrict__ out, const int* __restrict__ ids, const TA* __restrict__ table,
                                  int W, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int i = threadIdx.x; i < W; i += blockDim.x) out[(size_t)t * W + i] = ldf(table, (size_t)id * W + i) * scale;
}

// x[t] += mult * (branch[t] + branch2[t]) + rowvec (each optional), stored back in fp32; then (w != null)
// out[t] = x[t] / sqrt(mean(x[t]^2) + eps) * (offset + w), the mean taken over each of `groups` equal consecutive parts
// of the row by itself.  One workgroup per row; groups > 1: one wave per part.
template <typename TA>
__global__ __launch_bounds__(256) void resnorm_kernel(float* __restrict__ x, const TA* __restrict__ branch,
                                                      const TA* __restrict__ branch2, float mult,
                                                      const TA* __restrict__ rowvec, const TA* __restrict__ w,
                                                      float offset, float eps, TA* __restrict__ out, int W, int groups) {
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * W;
  float ss = 0.f;
  const bool upd = branch != nullptr || rowvec != nullptr;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = x[base + i];
    if (branch != nullptr) v += mult * (ldf(branch, base + i) + (branch2 != nullptr ? ldf(branch2, base + i) : 0.f));
    if (rowvec != nullptr) v += ldf(rowvec, i);
    if (upd) x[base + i] = v;
    ss += v * v;
  }
  if (w == nullptr) return;
  if (groups <= 1) {
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x)
      stf(out, base + i, x[base + i] * inv * (offset + ldf(w, i)));
    return;
  }
  __syncthreads();   // the updated row is read back by other threads
  const int Wg = W / groups, wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  for (int g = wave; g < groups; g += nw) {
    const size_t b = base + (size_t)g * Wg;
    float sg = 0.f;
    for (int i = lane; i < Wg; i += 64) {
      const float v = x[b + i];
      sg += v * v;
    }
    sg = wave_sum(sg);
    const float inv = 1.0f / sqrtf(sg / (float)Wg + eps);
    for (int i = lane; i < Wg; i += 64) stf(out, b + i, x[b + i] * inv * (offset + ldf(w, (size_t)g * Wg + i)));
  }
}

// Norm after the sum: x[t] <- (alpha x[t] + c1 branch[t] + c2 branch2[t]) / sqrt(mean(.^2) + eps) * gain, stored back
// in fp32 (the stream stays normed); `out` (optional) receives the same row in the activation type, for the sublayer
// that reads it next.  `gain` is one number for the whole row.  One workgroup per row; the row is held in registers
// (W <= 256 * 16) or re-formed from its inputs on the second pass.
template <typename TA>
__global__ __launch_bounds__(256) void postnorm_kernel(float* __restrict__ x, const TA* __restrict__ branch,
                                                       const TA* __restrict__ branch2, float alpha, float c1, float c2,
                                                       float gain, float eps, TA* __restrict__ out, int W) {
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * W;
  auto value = [&](int i) -> float {
    float v = alpha * x[base + i];
    if (branch != nullptr) v = fmaf(c1, ldf(branch, base + i), v);
    if (branch2 != nullptr) v = fmaf(c2, ldf(branch2, base + i), v);
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = value(i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float m = gain / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float y = value(i) * m;      // element i is read and written by this thread only
    x[base + i] = y;
    if (out != nullptr) stf(out, base + i, y);
  }
}

// out[t, c] = y[t, c] * f(gate[t, c]) with f = sigmoid (kind 0) or silu (kind 1); y and gate are row-strided views.
template <typename TY, typename TA>
__global__ void gate_mul_kernel(TA* __restrict__ out, const TY* __restrict__ y, long ldy, const TA* __restrict__ gate,
                                long ldg, int T, int F, int kind) {
  const size_t n = (size_t)T * F;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / F, c = i - t * F;
    const float g = ldf(gate, t * ldg + c);
    const float s = 1.f / (1.f + expf(-g));
    stf(out, i, ldf(y, t * ldy + c) * (kind == 1 ? g * s : s));
  }
}

// kinds: 0 gelu_tanh(g) * u, 1 g' * sigmoid(alpha g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, +-limit)
// (limit <= 0: no clamp), 5 relu(g) * u -- these read [T, 2F] = [gate | up]; 2 tanh, 3 silu, 4 erf-gelu,
// 6 limit * tanh(x / limit): elementwise on [T, F].
// Elementwise kinds take a factor per row: logical row i is row row_map[i] (or i) and its input is multiplied by
// row_scale[i] before the function (experts whose router weight scales their input).
template <typename TA>
__global__ void act_kernel(TA* __restrict__ out, const TA* __restrict__ x, int T, int F, int kind, float limit,
                           float alpha, const float* __restrict__ row_scale, const int* __restrict__ row_map) {
  const size_t n = (size_t)T * F;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / F, c = i - t * F;
    float y;
    size_t o = i;
    if (kind >= 2 && kind != 5) {
      if (row_map != nullptr) o = (size_t)row_map[t] * F + c;
      float v = ldf(x, o);
      if (row_scale != nullptr) v *= row_scale[t];
      y = kind == 2   ? tanhf(v)
          : kind == 3 ? v / (1.f + expf(-v))
          : kind == 4 ? 0.5f * v * (1.f + erff(v * 0.7071067811865476f))
                      : limit * tanhf(v / limit);
    } else {
      float g = ldf(x, t * 2 * F + c), u = ldf(x, t * 2 * F + F + c);
      if (kind == 0) {
        y = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
      } else if (kind == 5) {
        y = fmaxf(g, 0.f) * u;
      } else {
        if (limit > 0.f) {
          g = fminf(g, limit);
          u = fminf(fmaxf(u, -limit), limit);
        }
        y = g / (1.f + expf(-alpha * g)) * (u + 1.f);
      }
    }
    stf(out, o, y);
  }
}

// out[t] = ca * a[t] / rms(a[t]) * wa + cb * b[t] / rms(b[t]) * wb (b optional): the outputs of two mixers that run side
// by side, each normed over the row in fp32, joined.  One workgroup per row.  `lda`: the row stride of a (a view into a
// wider projection).  groups > 1 (a alone): every one of that many equal consecutive parts of the row is divided by its
// own root mean square, one wave per part.
template <typename TA, typename TO>
__global__ __launch_bounds__(256) void norm_mix_kernel(TO* __restrict__ out, const TA* __restrict__ a, long lda,
                                                       const TA* __restrict__ wa, const TA* __restrict__ b,
                                                       const TA* __restrict__ wb, float eps, float ca, float cb, int W,
                                                       int groups) {
  __shared__ float red[16];
  const size_t base = (size_t)blockIdx.x * W;
  const TA* ar = a + (size_t)blockIdx.x * lda;
  if (groups > 1) {
    const int Wg = W / groups, wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    for (int g = wave; g < groups; g += nw) {
      const size_t o = (size_t)g * Wg;
      float sg = 0.f;
      for (int i = lane; i < Wg; i += 64) {
        const float v = ldf(ar, o + i);
        sg += v * v;
      }
      sg = wave_sum(sg);
      const float inv = ca / sqrtf(sg / (float)Wg + eps);
      for (int i = lane; i < Wg; i += 64) stf(out, base + o + i, ldf(ar, o + i) * inv * ldf(wa, o + i));
    }
    return;
  }
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float va = ldf(ar, i);
    sa += va * va;
    if (b != nullptr) {
      const float vb = ldf(b, base + i);
      sb += vb * vb;
    }
  }
  sa = block_sum(sa, red);
  const float ia = ca / sqrtf(sa / (float)W + eps);
  float ib = 0.f;
  if (b != nullptr) {   // uniform branch
    sb = block_sum(sb, red);
    ib = cb / sqrtf(sb / (float)W + eps);
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float y = ldf(ar, i) * ia * ldf(wa, i);
    if (b != nullptr) y += ldf(b, base + i) * ib * ldf(wb, i);
    stf(out, base + i, y);
  }
}

// C = A W^T for any M, N, K and any row strides: 64 x 64 output tile per workgroup, 16-deep k steps staged through LDS
// as fp32, 4 x 4 outputs per thread, fp32 FMA accumulation in k order (a row's result does not depend on which rows
// share its tile).  Three forms:
//   plain / strided-batched: blockIdx.z = batch g, operands offset by g * (sA, sW, sC);
//   row gather: A row r is A[a_rows[r]];
//   grouped: tiles[y] = (group, first row, rows) lists the row tiles of variable-size groups over one compact row
//   space (a mixture-of-experts' sorted tokens); group g uses W + g * sW; tiles with group < 0 are padding.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_any_kernel(TO* __restrict__ C, const TI* __restrict__ A,
                                                       const TI* __restrict__ Wt, int M, int N, int K, long lda,
                                                       long ldw, long ldc, long sA, long sW, long sC,
                                                       const int* __restrict__ a_rows, const int* __restrict__ tiles) {
  constexpr int BM = 64, BN = 64, BK = 16, LD = BM + 4;
  __shared__ __attribute__((aligned(16))) float As[BK][LD];
  __shared__ __attribute__((aligned(16))) float Ws[BK][LD];
  int row0, rows;
  if (tiles != nullptr) {
    const int g = tiles[3 * blockIdx.y];
    if (g < 0) return;
    row0 = tiles[3 * blockIdx.y + 1];
    rows = tiles[3 * blockIdx.y + 2];
    Wt += (size_t)g * sW;
  } else {
    row0 = blockIdx.y * BM;
    rows = min(BM, M - row0);
    A += (size_t)blockIdx.z * sA;
    Wt += (size_t)blockIdx.z * sW;
    C += (size_t)blockIdx.z * sC;
  }
  const int col0 = blockIdx.x * BN;
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int kk = tid & 15, r_l = tid >> 4;          // loader: k index, first of 4 rows (r_l + 16 i)
  size_t a_off[4], w_off[4];
  bool a_ok[4], w_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r_l + 16 * i;
    a_ok[i] = r < rows;
    const int gr = a_ok[i] ? (a_rows != nullptr ? a_rows[row0 + r] : row0 + r) : 0;
    a_off[i] = (size_t)gr * lda;
    w_ok[i] = col0 + r < N;
    w_off[i] = (size_t)(w_ok[i] ? col0 + r : 0) * ldw;
  }
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    const bool kin = k0 + kk < K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[kk][r_l + 16 * i] = (kin && a_ok[i]) ? ldf(A, a_off[i] + k0 + kk) : 0.f;
      Ws[kk][r_l + 16 * i] = (kin && w_ok[i]) ? ldf(Wt, w_off[i] + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(&As[k][ty * 4]);
      const f32x4 b = *reinterpret_cast<const f32x4*>(&Ws[k][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < N) stf(C, (size_t)(row0 + r) * ldc + c, acc[i][j]);
    }
  }
}

// The same product for bf16 operands whose rows are 16-byte aligned (k and every stride a multiple of 8 elements) on
// the matrix cores: 64 x 64 or (many rows and columns) 64 x 128 output tile, 32-deep k steps, 4 waves of 32 x 32 or
// 32 x 64 (2 x NF v_mfma_f32_16x16x32_bf16) in the swapped orientation C^T = W A^T, so a lane ends with 4 consecutive
// columns of one row; an output's accumulation is the same in both tile shapes.  The next k step's global
// loads are in flight during the current step's MFMAs.  Same three forms (batched, row gather, grouped tiles); the
// accumulation order of an output does not depend on M or on the rows that share its tile.
template <typename TO, int NF>   // NF 16-column fragments per wave: output tile 64 x (32 NF)
__global__ __launch_bounds__(256) void gemm_mfma_kernel(TO* __restrict__ C, const bf16_t* __restrict__ A,
                                                        const bf16_t* __restrict__ Wt, int M, int N, int K, long lda,
                                                        long ldw, long ldc, long sA, long sW, long sC,
                                                        const int* __restrict__ a_rows, const int* __restrict__ tiles) {
  constexpr int BM = 64, BN = 32 * NF, BK = 32, LDK = BK + 8;   // rows of 80 bytes: 16-byte aligned fragments
  constexpr int WL = BN / 64;                                    // W rows per loader thread
  __shared__ __attribute__((aligned(16))) bf16_t As[BM][LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[BN][LDK];
  int row0, rows;
  if (tiles != nullptr) {
    const int g = tiles[3 * blockIdx.y];
    if (g < 0) return;
    row0 = tiles[3 * blockIdx.y + 1];
    rows = tiles[3 * blockIdx.y + 2];
    Wt += (size_t)g * sW;
  } else {
    row0 = blockIdx.y * BM;
    rows = min(BM, M - row0);
    A += (size_t)blockIdx.z * sA;
    Wt += (size_t)blockIdx.z * sW;
    C += (size_t)blockIdx.z * sC;
  }
  const int col0 = blockIdx.x * BN;
  const int tid = threadIdx.x;
  // loader: thread -> (row tid / 4 (+ 64 c for W), 8-element chunk tid % 4)
  const int lr = tid >> 2, lc = tid & 3;
  const bool a_ok = lr < rows;
  const int gr = a_ok ? (a_rows != nullptr ? a_rows[row0 + lr] : row0 + lr) : 0;
  const bf16_t* ap = A + (size_t)gr * lda + lc * 8;
  const bf16_t* wp[WL];
  bool w_ok[WL];
#pragma unroll
  for (int c = 0; c < WL; ++c) {
    w_ok[c] = col0 + lr + 64 * c < N;
    wp[c] = Wt + (size_t)(w_ok[c] ? col0 + lr + 64 * c : 0) * ldw + lc * 8;
  }
  const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
  u32x4 ra, rw[WL];
  auto fetch = [&](int k0) {
    const bool kin = k0 + lc * 8 < K;
    ra = (kin && a_ok) ? *reinterpret_cast<const u32x4*>(ap + k0) : zero;
#pragma unroll
    for (int c = 0; c < WL; ++c) rw[c] = (kin && w_ok[c]) ? *reinterpret_cast<const u32x4*>(wp[c] + k0) : zero;
  };
  const int lane = tid & 63, wave = tid >> 6, li = lane & 15, g = lane >> 4;
  const int m0 = (wave & 1) * 32, n0 = (wave >> 1) * (16 * NF);
  f32x4 acc[NF][2];
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[f][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();
    *reinterpret_cast<u32x4*>(&As[lr][lc * 8]) = ra;
#pragma unroll
    for (int c = 0; c < WL; ++c) *reinterpret_cast<u32x4*>(&Ws[lr + 64 * c][lc * 8]) = rw[c];
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
    bf16x8 wf[NF], af[2];
#pragma unroll
    for (int f = 0; f < NF; ++f) wf[f] = *reinterpret_cast<const bf16x8*>(&Ws[n0 + 16 * f + li][8 * g]);
#pragma unroll
    for (int j = 0; j < 2; ++j) af[j] = *reinterpret_cast<const bf16x8*>(&As[m0 + 16 * j + li][8 * g]);
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[f][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[f], af[j], acc[f][j], 0, 0, 0);
  }
  // acc[f][j][i] = C[row m0 + 16 j + li][col n0 + 16 f + 4 g + i]
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int r = m0 + 16 * j + li;
    if (r >= rows) continue;
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = col0 + n0 + 16 * f + 4 * g + i;
        if (c < N) stf(C, (size_t)(row0 + r) * ldc + c, acc[f][j][i]);
      }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" int k8s_embed_rows(float* out, const int* ids, const void* table, int T, int W, int vocab, float scale,
                              int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (W <= 0 || vocab <= 0) return -1;
  if (f32) embed_rows_kernel<float><<<T, 256, 0, s>>>(out, ids, (const float*)table, W, vocab, scale);
  else embed_rows_kernel<bf16_t><<<T, 256, 0, s>>>(out, ids, (const bf16_t*)table, W, vocab, scale);
  return (int)hipGetLastError();
}

extern "C" int k8s_resnorm(float* x, const void* branch, const void* branch2, float mult, const void* rowvec,
                           const void* w, float offset, float eps, void* out, int T, int W, int groups, int f32,
                           hipStream_t s) {
  if (T <= 0) return 0;
  if (W <= 0 || (w != nullptr && out == nullptr) || groups < 1 || W % groups || (branch2 != nullptr && branch == nullptr))
    return -1;
  if (f32)
    resnorm_kernel<float><<<T, 256, 0, s>>>(x, (const float*)branch, (const float*)branch2, mult, (const float*)rowvec,
                                            (const float*)w, offset, eps, (float*)out, W, groups);
  else
    resnorm_kernel<bf16_t><<<T, 256, 0, s>>>(x, (const bf16_t*)branch, (const bf16_t*)branch2, mult,
                                             (const bf16_t*)rowvec, (const bf16_t*)w, offset, eps, (bf16_t*)out, W,
                                             groups);
  return (int)hipGetLastError();
}

extern "C" int k8s_norm_mix(void* out, const void* a, long lda, const void* wa, const void* b, const void* wb,
                            float eps, float ca, float cb, int T, int W, int groups, int in_f32, int out_f32,
                            hipStream_t s) {
  if (T <= 0) return 0;
  if (W <= 0 || a == nullptr || wa == nullptr || (b != nullptr && wb == nullptr) || lda < W) return -1;
  if (groups < 1 || W % groups || (groups > 1 && b != nullptr)) return -1;
#define K8S_NM(TA, TO)                                                                                             \
  norm_mix_kernel<TA, TO><<<T, 256, 0, s>>>((TO*)out, (const TA*)a, lda, (const TA*)wa, (const TA*)b, (const TA*)wb, \
                                            eps, ca, cb, W, groups)
  if (in_f32 && out_f32) K8S_NM(float, float);
  else if (in_f32) K8S_NM(float, bf16_t);
  else if (out_f32) K8S_NM(bf16_t, float);
  else K8S_NM(bf16_t, bf16_t);
#undef K8S_NM
  return (int)hipGetLastError();
}

extern "C" int k8s_postnorm(float* x, const void* branch, const void* branch2, float alpha, float c1, float c2,
                            float gain, float eps, void* out, int T, int W, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (W <= 0 || x == nullptr || (branch2 != nullptr && branch == nullptr)) return -1;
  if (f32)
    postnorm_kernel<float><<<T, 256, 0, s>>>(x, (const float*)branch, (const float*)branch2, alpha, c1, c2, gain, eps,
                                             (float*)out, W);
  else
    postnorm_kernel<bf16_t><<<T, 256, 0, s>>>(x, (const bf16_t*)branch, (const bf16_t*)branch2, alpha, c1, c2, gain,
                                              eps, (bf16_t*)out, W);
  return (int)hipGetLastError();
}

// y_f32: y is fp32 whatever the activation type (an fp32 intermediate gated into the activation type)
extern "C" int k8s_gate_mul(void* out, const void* y, long ldy, const void* gate, long ldg, int T, int F, int kind,
                            int y_f32, int f32, hipStream_t s) {
  if (T <= 0 || F <= 0) return 0;
  if (kind < 0 || kind > 1 || ldy < F || ldg < F || (f32 && !y_f32)) return -1;
  const size_t n = (size_t)T * F;
  const int blocks = (int)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
  if (f32)
    gate_mul_kernel<float, float><<<blocks, 256, 0, s>>>((float*)out, (const float*)y, ldy, (const float*)gate, ldg, T,
                                                         F, kind);
  else if (y_f32)
    gate_mul_kernel<float, bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)out, (const float*)y, ldy, (const bf16_t*)gate, ldg,
                                                          T, F, kind);
  else
    gate_mul_kernel<bf16_t, bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)y, ldy, (const bf16_t*)gate,
                                                           ldg, T, F, kind);
  return (int)hipGetLastError();
}

extern "C" int k8s_act(void* out, const void* x, int T, int F, int kind, float limit, float alpha,
                       const float* row_scale, const int* row_map, int f32, hipStream_t s) {
  if (T <= 0 || F <= 0) return 0;
  const bool gated = kind < 2 || kind == 5;
  if (kind < 0 || kind > 6 || (gated && (row_scale != nullptr || row_map != nullptr)) || (kind == 6 && !(limit > 0.f)))
    return -1;
  const size_t n = (size_t)T * F;
  const int blocks = (int)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
  if (f32) act_kernel<float><<<blocks, 256, 0, s>>>((float*)out, (const float*)x, T, F, kind, limit, alpha,
                                                    row_scale, row_map);
  else act_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)out, (const bf16_t*)x, T, F, kind, limit, alpha,
                                                row_scale, row_map);
  return (int)hipGetLastError();
}

extern "C" int k8s_gemm_any(void* C, const void* A, const void* W, int M, int N, int K, long lda, long ldw, long ldc,
                            int batch, long sA, long sW, long sC, const int* a_rows, const int* tiles, int ntiles,
                            int in_f32, int out_f32, hipStream_t s) {
  if (N <= 0 || K <= 0 || batch <= 0) return -1;
  int gy;
  if (tiles != nullptr) {
    if (ntiles <= 0) return 0;
    gy = ntiles;
    batch = 1;
  } else {
    if (M <= 0) return 0;
    gy = (M + 63) / 64;
  }
  if (gy > 65535 || batch > 65535) return -2;
  // bf16 rows that can be moved as 16-byte vectors: the MFMA kernel; anything else (fp32, odd strides): plain FMAs
  const bool vec = !in_f32 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && sA % 8 == 0 && sW % 8 == 0 &&
                   ((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0;
  if (vec) {
    const bool wide = N >= 512 && (long)gy * ((N + 127) / 128) * batch >= 256;   // enough 64 x 128 tiles for the chip
    const dim3 g2((N + (wide ? 127 : 63)) / (wide ? 128 : 64), gy, batch);
#define K8S_GM(TO, NF) \
  gemm_mfma_kernel<TO, NF><<<g2, 256, 0, s>>>((TO*)C, (const bf16_t*)A, (const bf16_t*)W, M, N, K, lda, ldw, ldc, sA, \
                                              sW, sC, a_rows, tiles)
    if (out_f32) { if (wide) K8S_GM(float, 4); else K8S_GM(float, 2); }
    else { if (wide) K8S_GM(bf16_t, 4); else K8S_GM(bf16_t, 2); }
#undef K8S_GM
    return (int)hipGetLastError();
  }
  const dim3 grid((N + 63) / 64, gy, batch);
#define K8S_GA(TI, TO) \
  gemm_any_kernel<TI, TO><<<grid, 256, 0, s>>>((TO*)C, (const TI*)A, (const TI*)W, M, N, K, lda, ldw, ldc, sA, sW, sC, \
                                               a_rows, tiles)
  if (in_f32 && out_f32) K8S_GA(float, float);
  else if (in_f32) K8S_GA(float, bf16_t);
  else if (out_f32) K8S_GA(bf16_t, float);
  else K8S_GA(bf16_t, bf16_t);
#undef K8S_GA
  return (int)hipGetLastError();
}
