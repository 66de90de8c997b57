// minGRU scan over a flat varlen batch (fp32 state per slot), the fp32
// top-k routers (softmax over the chosen logits; softmax over every output
// with a choice correction and scaled, unnormalised weights; or plain sigmoid
// scores), and the
// mixture-of-experts feed-forward as two grouped GEMMs over expert-sorted
// rows (bf16: MFMA 16x16x32 tiles; fp32: plain FMA; SiLU-gated or clamped
// GLU experts) followed by a fixed-order weighted combine, which also adds
// the identity experts' share of the input. The routing weight multiplies an
// expert's output (in the combine) or, for designs that scale the expert's
// input, its gate and up products before the activation.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16v8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {

// ------------------------------------------------------------- minGRU
// One thread per (sequence row, channel); tokens of the row in order.
// zxg row = [z | x | g] pre-activations, bias still to add.
template <typename T>
__global__ __launch_bounds__(256) void mingru_scan_kernel(
    const T* __restrict__ zxg, const float* __restrict__ bias,
    float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slots, int n, T* __restrict__ out) {
  const int b = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= n) return;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 == t0) return;
  const int64_t slot = slots[b];
  const float bz = bias[ch], bx = bias[n + ch], bg = bias[2 * n + ch];
  float S = state[slot * n + ch];
  for (int t = t0; t < t1; ++t) {
    const T* row = zxg + (int64_t)t * 3 * n;
    const float z = sm_sigmoid(to_f(row[ch]) + bz);
    const float u = to_f(row[n + ch]) + bx;
    const float cand = (u >= 0.f) ? u + 0.5f : sm_sigmoid(u);
    S = (1.0f - z) * S + z * cand;
    const float g = to_f(row[2 * n + ch]) + bg;
    out[(int64_t)t * n + ch] = from_f<T>(S * (g * sm_sigmoid(g)));
  }
  state[slot * n + ch] = S;
}

// Chunked form for long rows: a row's tokens are cut into chunks that run
// in parallel. S_t = a_t S_(t-1) + b_t composes, so a chunk is summarised
// by (P, Q) with S_end = P S_start + Q (pass 1), the chunk starts follow
// from a short serial walk over the row's chunks (pass 2), and pass 3
// redoes each chunk from its true start and writes the outputs.
template <typename T>
SM_INLINE void mingru_gates(const T* row, int n, int ch, float bz, float bx,
                            float* z, float* cand) {
  *z = sm_sigmoid(to_f(row[ch]) + bz);
  const float u = to_f(row[n + ch]) + bx;
  *cand = (u >= 0.f) ? u + 0.5f : sm_sigmoid(u);
}

template <typename T>
__global__ __launch_bounds__(256) void mingru_chunk_reduce_kernel(
    const T* __restrict__ zxg, const float* __restrict__ bias,
    const int* __restrict__ chunks, int n, float* __restrict__ P,
    float* __restrict__ Q) {
  const int c = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= n) return;
  const int t0 = chunks[3 * c + 1], cnt = chunks[3 * c + 2];
  const float bz = bias[ch], bx = bias[n + ch];
  float p = 1.f, q = 0.f;
  for (int t = t0; t < t0 + cnt; ++t) {
    float z, cand;
    mingru_gates(zxg + (int64_t)t * 3 * n, n, ch, bz, bx, &z, &cand);
    q = (1.0f - z) * q + z * cand;
    p *= (1.0f - z);
  }
  P[(int64_t)c * n + ch] = p;
  Q[(int64_t)c * n + ch] = q;
}

__global__ __launch_bounds__(256) void mingru_chunk_carry_kernel(
    const float* __restrict__ P, const float* __restrict__ Q,
    float* __restrict__ state, const int* __restrict__ chunk_cu,
    const int* __restrict__ slots, int n, float* __restrict__ Sstart) {
  const int b = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= n) return;
  const int c0 = chunk_cu[b], c1 = chunk_cu[b + 1];
  if (c1 == c0) return;
  const int64_t slot = slots[b];
  float S = state[slot * n + ch];
  for (int c = c0; c < c1; ++c) {
    Sstart[(int64_t)c * n + ch] = S;
    S = P[(int64_t)c * n + ch] * S + Q[(int64_t)c * n + ch];
  }
  state[slot * n + ch] = S;
}

template <typename T>
__global__ __launch_bounds__(256) void mingru_chunk_apply_kernel(
    const T* __restrict__ zxg, const float* __restrict__ bias,
    const int* __restrict__ chunks, const float* __restrict__ Sstart, int n,
    T* __restrict__ out) {
  const int c = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= n) return;
  const int t0 = chunks[3 * c + 1], cnt = chunks[3 * c + 2];
  const float bz = bias[ch], bx = bias[n + ch], bg = bias[2 * n + ch];
  float S = Sstart[(int64_t)c * n + ch];
  for (int t = t0; t < t0 + cnt; ++t) {
    const T* row = zxg + (int64_t)t * 3 * n;
    float z, cand;
    mingru_gates(row, n, ch, bz, bx, &z, &cand);
    S = (1.0f - z) * S + z * cand;
    const float g = to_f(row[2 * n + ch]) + bg;
    out[(int64_t)t * n + ch] = from_f<T>(S * (g * sm_sigmoid(g)));
  }
}

// ------------------------------------------------------------- router
// One workgroup per token: the waves share the experts' fp32 logits, then
// one lane picks the top-k by repeated arg-max (ties: the lowest index) and
// takes the softmax over the chosen logits.
// ALL: scores s = softmax over all E outputs (no bias); the top-k of
// s + corr are chosen; weights = s[chosen] * wscale, not renormalised.
// sig (not ALL): weights = sigmoid of the chosen logits, not renormalised.
#define SM_MAX_EXPERTS 256
template <typename T, bool ALL>
__global__ __launch_bounds__(256) void moe_route_kernel(
    const T* __restrict__ h, const float* __restrict__ w,
    const float* __restrict__ bias, int D, int E, int top,
    int* __restrict__ idx, float* __restrict__ wts,
    const float* __restrict__ corr, float wscale, bool sig) {
  __shared__ float z[SM_MAX_EXPERTS];
  __shared__ float sc[SM_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = wave; e < E; e += 4) {
    const float* we = w + (int64_t)e * D;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int d = lane;
    for (; d + 192 < D; d += 256) {
      a0 = fmaf(to_f(h[t * D + d]), we[d], a0);
      a1 = fmaf(to_f(h[t * D + d + 64]), we[d + 64], a1);
      a2 = fmaf(to_f(h[t * D + d + 128]), we[d + 128], a2);
      a3 = fmaf(to_f(h[t * D + d + 192]), we[d + 192], a3);
    }
    for (; d < D; d += 64) a0 = fmaf(to_f(h[t * D + d]), we[d], a0);
    const float acc = sm_wave_sum((a0 + a1) + (a2 + a3));
    if (lane == 0) z[e] = acc + (bias != nullptr ? bias[e] : 0.f);
  }
  __syncthreads();
  if (ALL) {
    if (threadIdx.x == 0) {
      float vmax = -INFINITY, sum = 0.f;
      for (int e = 0; e < E; ++e) vmax = fmaxf(vmax, z[e]);
      for (int e = 0; e < E; ++e) {
        sc[e] = expf(z[e] - vmax);
        sum += sc[e];
      }
      for (int e = 0; e < E; ++e) {
        sc[e] /= sum;
        z[e] = sc[e] + (corr != nullptr ? corr[e] : 0.f);
      }
      for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = -INFINITY;
        for (int e = 0; e < E; ++e)
          if (z[e] > bv) { bv = z[e]; best = e; }
        if (best < 0) best = 0;
        idx[t * top + k] = best;
        wts[t * top + k] = sc[best] * wscale;
        z[best] = -INFINITY;
      }
    }
    return;
  }
  if (threadIdx.x == 0) {
    float vmax = 0.f, sum = 0.f;
    for (int k = 0; k < top; ++k) {
      int best = -1;
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e)
        if (z[e] > bv) { bv = z[e]; best = e; }
      if (best < 0) best = 0;             // all NaN/-inf: keep the write in range
      if (k == 0) vmax = bv;
      const float p = sig ? sm_sigmoid(bv) : expf(bv - vmax);
      idx[t * top + k] = best;
      wts[t * top + k] = p;
      sum += p;
      z[best] = -INFINITY;
    }
    if (!sig)
      for (int k = 0; k < top; ++k) wts[t * top + k] /= sum;
  }
}

// Group the (token, choice) pairs by expert in one workgroup: off[e] = first
// sorted row of expert e, src[row] = token of that row, inv[pair] = its row.
// The order inside an expert is arbitrary; every row's result is independent
// of it and the combine reads rows back through inv. Called with E = weight
// sets + 1: indices at or above the weight sets (identity experts) share the
// last bin, whose rows no GEMM touches. With rw: rw[row] = the pair's routing
// weight (for experts whose input is scaled).
__global__ __launch_bounds__(1024) void moe_group_kernel(
    const int* __restrict__ idx, int M, int top, int E, int* __restrict__ off,
    int* __restrict__ src, int* __restrict__ inv, const float* __restrict__ wts,
    float* __restrict__ rw) {
  __shared__ int cnt[SM_MAX_EXPERTS + 1];
  __shared__ int start[SM_MAX_EXPERTS + 2];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < M; i += blockDim.x)
    atomicAdd(&cnt[min(max(idx[i], 0), E - 1)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = s;
      off[e] = s;
      s += cnt[e];
      cnt[e] = 0;
    }
    start[E] = s;
    off[E] = s;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < M; i += blockDim.x) {
    const int e = min(max(idx[i], 0), E - 1);
    const int row = start[e] + atomicAdd(&cnt[e], 1);
    src[row] = i / top;
    inv[i] = row;
    if (rw != nullptr) rw[row] = wts[i];
  }
}

// ------------------------------------------------- grouped GEMM, bf16
// Rows are sorted by expert: expert e owns rows off[e]..off[e+1]. A
// workgroup (4 waves) computes a 64-row x 64-column tile of one expert;
// wave w owns columns w*16..w*16+15 for the four 16-row m-tiles.
// MODE 0: out[i, f] = act(a_i . Wg[f], a_i . Wu[f]), a_i = A[src[i]],
//         act(g, u) = silu(g) u (limit 0) or the clamped GLU (limit > 0);
//         with rw both products are scaled by rw[i] first (W (w a) = w (W a));
//         W[e] = [gate (N rows); up (N rows)] x K;   out bf16 [M, N]
// MODE 1: out[i, n] = a_i . W[e][n], a_i = A[i];     out fp32 [M, N]
// MFMA 16x16x32 bf16 fragments: A lane l -> row l&15, k (l>>4)*8..+7;
// B lane l -> column l&15, same k; D lane l reg r -> row (l>>4)*4+r, col l&15.
SM_INLINE float moe_act(float g, float u, float limit) {
  return (limit > 0.f) ? sm_capped_glu(g, u, limit) : g * sm_sigmoid(g) * u;
}
SM_INLINE bf16v8 load8(const bf16_t* p, int valid, bool vec) {
  bf16v8 v;
  if (vec && valid >= 8) {
    v = *reinterpret_cast<const bf16v8*>(p);
  } else {
    #pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = (j < valid) ? (__bf16)__bfloat162float(p[j]) : (__bf16)0.0f;
  }
  return v;
}

#define GG_BK 64
#define GG_LD 72   // padded LDS row (bf16 elements)
// MT 16-row m-tiles per workgroup (rows BM = 16 MT) and NWV waves, each wave
// owning 16 columns: <4, 4> is the 64x64 prompt tile; <1, 1> gives decode
// batches (a few rows per expert) one wave per 16 columns, so that enough
// workgroups stream the expert weights.
template <int MODE, int MT, int NWV>
__global__ __launch_bounds__(64 * NWV) void moe_gemm_bf16_kernel(
    const bf16_t* __restrict__ A, const int* __restrict__ src,
    const bf16_t* __restrict__ W, const int* __restrict__ off, int E, int N,
    int K, void* __restrict__ outp, float limit, const float* __restrict__ rw) {
  constexpr int BM = 16 * MT;
  __shared__ __attribute__((aligned(16))) bf16_t a_lds[BM * GG_LD];
  // which expert / row range is this tile?
  int e = -1, row0 = 0, rows = 0, tiles = 0;
  for (int i = 0; i < E; ++i) {
    const int cnt = off[i + 1] - off[i];
    const int nt = SM_CDIV(cnt, BM);
    if ((int)blockIdx.x < tiles + nt) {
      e = i;
      row0 = off[i] + ((int)blockIdx.x - tiles) * BM;
      rows = min(BM, off[i + 1] - row0);
      break;
    }
    tiles += nt;
  }
  if (e < 0) return;                       // uniform over the workgroup
  const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63;
  const int lrow = l & 15, lk = l >> 4;
  const bool vec = (K % 8) == 0;
  const int n = blockIdx.y * (16 * NWV) + wave * 16 + lrow;     // this lane's B column
  const int Nw = (MODE == 0) ? 2 * N : N;
  const bf16_t* Wg = W + ((int64_t)e * Nw + (n < N ? n : 0)) * K;
  const bf16_t* Wu = Wg + (int64_t)N * K;
  f32x4 acc[MT], acc2[MT];
  #pragma unroll
  for (int i = 0; i < MT; ++i) {
    acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc2[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  for (int k0 = 0; k0 < K; k0 += GG_BK) {
    __syncthreads();
    for (int v = tid; v < BM * 8; v += 64 * NWV) {
      const int r = v >> 3, kc = (v & 7) * 8;
      bf16v8 val;
      if (r < rows) {
        const int64_t arow = (MODE == 0) ? src[row0 + r] : (row0 + r);
        val = load8(A + arow * K + k0 + kc, K - (k0 + kc), vec);
      } else {
        #pragma unroll
        for (int j = 0; j < 8; ++j) val[j] = (__bf16)0.0f;
      }
      *reinterpret_cast<bf16v8*>(a_lds + r * GG_LD + kc) = val;
    }
    __syncthreads();
    #pragma unroll
    for (int ks = 0; ks < GG_BK / 32; ++ks) {
      const int kk = k0 + ks * 32 + lk * 8;
      if (k0 + ks * 32 >= K) break;
      bf16v8 bg, bu;
      const int valid = (n < N) ? K - kk : 0;
      bg = load8(Wg + kk, valid, vec);
      if (MODE == 0) bu = load8(Wu + kk, valid, vec);
      #pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16v8 a = *reinterpret_cast<const bf16v8*>(
            a_lds + (mt * 16 + lrow) * GG_LD + ks * 32 + lk * 8);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bg, acc[mt], 0, 0, 0);
        if (MODE == 0)
          acc2[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bu, acc2[mt], 0, 0, 0);
      }
    }
  }
  if (n >= N) return;
  #pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int r = mt * 16 + lk * 4 + rr;
      if (r < rows) {
        const int64_t o = (int64_t)(row0 + r) * N + n;
        if (MODE == 0) {
          const float w = (rw != nullptr) ? rw[row0 + r] : 1.0f;
          reinterpret_cast<bf16_t*>(outp)[o] =
              __float2bfloat16(moe_act(w * acc[mt][rr], w * acc2[mt][rr], limit));
        } else {
          reinterpret_cast<float*>(outp)[o] = acc[mt][rr];
        }
      }
    }
  }
}

// Decode batches (a few rows per expert): one 16-row x 16-column tile per
// workgroup, the K axis dealt out to the four waves in 32-wide steps (every
// lane reads its A and B fragments straight from memory: no LDS, no barrier
// in the loop, four times the loads in flight), partial tiles summed
// through LDS in a fixed order.
template <int MODE>
__global__ __launch_bounds__(256) void moe_gemm_bf16_splitk_kernel(
    const bf16_t* __restrict__ A, const int* __restrict__ src,
    const bf16_t* __restrict__ W, const int* __restrict__ off, int E, int N,
    int K, void* __restrict__ outp, float limit, const float* __restrict__ rw) {
  __shared__ float red[3][64][8];
  int e = -1, row0 = 0, rows = 0, tiles = 0;
  for (int i = 0; i < E; ++i) {
    const int cnt = off[i + 1] - off[i];
    const int nt = SM_CDIV(cnt, 16);
    if ((int)blockIdx.x < tiles + nt) {
      e = i;
      row0 = off[i] + ((int)blockIdx.x - tiles) * 16;
      rows = min(16, off[i + 1] - row0);
      break;
    }
    tiles += nt;
  }
  if (e < 0) return;                       // uniform over the workgroup
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  const int lrow = l & 15, lk = l >> 4;
  const bool vec = (K % 8) == 0;
  const int n = blockIdx.y * 16 + lrow;
  const int Nw = (MODE == 0) ? 2 * N : N;
  const bf16_t* Wg = W + ((int64_t)e * Nw + (n < N ? n : 0)) * K;
  const bf16_t* Wu = Wg + (int64_t)N * K;
  const int64_t arow = (lrow < rows) ? ((MODE == 0) ? src[row0 + lrow] : (row0 + lrow)) : -1;
  const bf16_t* ap = A + (arow < 0 ? 0 : arow) * K;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
  #pragma unroll 4
  for (int k0 = wave * 32; k0 < K; k0 += 128) {      // uniform within a wave
    const int kk = k0 + lk * 8;
    const bf16v8 a = load8(ap + kk, arow < 0 ? 0 : K - kk, vec);
    const int valid = (n < N) ? K - kk : 0;
    const bf16v8 bg = load8(Wg + kk, valid, vec);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bg, acc, 0, 0, 0);
    if (MODE == 0) {
      const bf16v8 bu = load8(Wu + kk, valid, vec);
      acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bu, acc2, 0, 0, 0);
    }
  }
  if (wave > 0) {
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      red[wave - 1][l][rr] = acc[rr];
      red[wave - 1][l][4 + rr] = acc2[rr];
    }
  }
  __syncthreads();
  if (wave > 0 || n >= N) return;
  #pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    float g = acc[rr], u = acc2[rr];
    #pragma unroll
    for (int w = 0; w < 3; ++w) {
      g += red[w][l][rr];
      u += red[w][l][4 + rr];
    }
    const int r = lk * 4 + rr;
    if (r < rows) {
      const int64_t o = (int64_t)(row0 + r) * N + n;
      if (MODE == 0) {
        const float w = (rw != nullptr) ? rw[row0 + r] : 1.0f;
        reinterpret_cast<bf16_t*>(outp)[o] = __float2bfloat16(moe_act(w * g, w * u, limit));
      } else
        reinterpret_cast<float*>(outp)[o] = g;
    }
  }
}

// ------------------------------------------------- grouped GEMM, fp32
// One thread per output element; the expert of a row by scanning off[].
template <int MODE>
__global__ __launch_bounds__(256) void moe_gemm_f32_kernel(
    const float* __restrict__ A, const int* __restrict__ src,
    const float* __restrict__ W, const int* __restrict__ off, int E, int M,
    int N, int K, float* __restrict__ out, float limit, const float* __restrict__ rw) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= (int64_t)M * N) return;
  const int i = id / N, n = id % N;
  if (i >= off[E]) return;                 // rows of identity experts
  int e = 0;
  while (e + 1 < E && i >= off[e + 1]) ++e;
  const int Nw = (MODE == 0) ? 2 * N : N;
  const float* a = A + (int64_t)((MODE == 0) ? src[i] : i) * K;
  const float* wg = W + ((int64_t)e * Nw + n) * K;
  float g = 0.f, u = 0.f;
  for (int k = 0; k < K; ++k) {
    g = fmaf(a[k], wg[k], g);
    if (MODE == 0) u = fmaf(a[k], wg[(int64_t)N * K + k], u);
  }
  if (MODE == 0 && rw != nullptr) { g *= rw[i]; u *= rw[i]; }
  out[id] = (MODE == 0) ? moe_act(g, u, limit) : g;
}

// out[t, d] = sum_k wts[t, k] * y[inv[t * top + k], d]   (k in order; wts
// null: every weight is 1); a choice at or above E is an identity expert: its
// output is the input row.
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    const float* __restrict__ y, const int* __restrict__ inv,
    const float* __restrict__ wts, const int* __restrict__ idx,
    const T* __restrict__ h, int E, int top, int D, float* __restrict__ out) {
  const int64_t t = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const float v = (idx[t * top + k] >= E) ? to_f(h[t * D + d])
                                              : y[(int64_t)inv[t * top + k] * D + d];
      acc += (wts != nullptr ? wts[t * top + k] : 1.0f) * v;
    }
    out[t * D + d] = acc;
  }
}

}  // namespace

torch::Tensor mingru_scan(torch::Tensor zxg, torch::Tensor bias, torch::Tensor state,
                          torch::Tensor cu, torch::Tensor slots,
                          c10::optional<torch::Tensor> chunks,
                          c10::optional<torch::Tensor> chunk_cu) {
  SM_CHECK_CUDA(zxg); SM_CHECK_CUDA(bias); SM_CHECK_F32(bias);
  SM_CHECK_CUDA(state); SM_CHECK_F32(state);
  SM_CHECK_CUDA(cu); SM_CHECK_I32(cu); SM_CHECK_CUDA(slots); SM_CHECK_I32(slots);
  const int64_t T = zxg.size(0);
  const int n = zxg.size(1) / 3;
  const int B = slots.numel();
  TORCH_CHECK(zxg.size(1) == 3 * n && bias.numel() == 3 * n, "mingru_scan: widths");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == n && cu.numel() == B + 1, "mingru_scan: state/batch layout");
  auto out = torch::empty({T, n}, zxg.options());
  if (T == 0 || B == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (chunks.has_value() && chunks->size(0) > 0) {
    TORCH_CHECK(chunk_cu.has_value(), "mingru_scan: chunk_cu missing");
    SM_CHECK_CUDA(*chunks); SM_CHECK_I32(*chunks); SM_CHECK_CUDA(*chunk_cu); SM_CHECK_I32(*chunk_cu);
    TORCH_CHECK(chunks->dim() == 2 && chunks->size(1) == 3 && chunk_cu->numel() == B + 1,
                "mingru_scan: chunk layout");
    const int nc = chunks->size(0);
    auto f32 = zxg.options().dtype(at::kFloat);
    auto P = torch::empty({nc, n}, f32), Q = torch::empty({nc, n}, f32), S0 = torch::empty({nc, n}, f32);
    dim3 gc(nc, SM_CDIV(n, 256)), gb(B, SM_CDIV(n, 256));
    if (zxg.scalar_type() == at::kBFloat16)
      mingru_chunk_reduce_kernel<bf16_t><<<gc, 256, 0, stream>>>(
          reinterpret_cast<const bf16_t*>(zxg.data_ptr()), bias.data_ptr<float>(),
          chunks->data_ptr<int>(), n, P.data_ptr<float>(), Q.data_ptr<float>());
    else {
      SM_CHECK_F32(zxg);
      mingru_chunk_reduce_kernel<float><<<gc, 256, 0, stream>>>(
          zxg.data_ptr<float>(), bias.data_ptr<float>(), chunks->data_ptr<int>(), n,
          P.data_ptr<float>(), Q.data_ptr<float>());
    }
    SM_CHECK_LAUNCH();
    mingru_chunk_carry_kernel<<<gb, 256, 0, stream>>>(
        P.data_ptr<float>(), Q.data_ptr<float>(), state.data_ptr<float>(),
        chunk_cu->data_ptr<int>(), slots.data_ptr<int>(), n, S0.data_ptr<float>());
    SM_CHECK_LAUNCH();
    if (zxg.scalar_type() == at::kBFloat16)
      mingru_chunk_apply_kernel<bf16_t><<<gc, 256, 0, stream>>>(
          reinterpret_cast<const bf16_t*>(zxg.data_ptr()), bias.data_ptr<float>(),
          chunks->data_ptr<int>(), S0.data_ptr<float>(), n, reinterpret_cast<bf16_t*>(out.data_ptr()));
    else
      mingru_chunk_apply_kernel<float><<<gc, 256, 0, stream>>>(
          zxg.data_ptr<float>(), bias.data_ptr<float>(), chunks->data_ptr<int>(),
          S0.data_ptr<float>(), n, out.data_ptr<float>());
    SM_CHECK_LAUNCH();
    return out;
  }
  dim3 grid(B, SM_CDIV(n, 256));
  if (zxg.scalar_type() == at::kBFloat16)
    mingru_scan_kernel<bf16_t><<<grid, 256, 0, stream>>>(
        reinterpret_cast<const bf16_t*>(zxg.data_ptr()), bias.data_ptr<float>(),
        state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(), n,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else {
    SM_CHECK_F32(zxg);
    mingru_scan_kernel<float><<<grid, 256, 0, stream>>>(
        zxg.data_ptr<float>(), bias.data_ptr<float>(), state.data_ptr<float>(),
        cu.data_ptr<int>(), slots.data_ptr<int>(), n, out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}

static std::vector<torch::Tensor> moe_route_impl(
    torch::Tensor h, torch::Tensor router_w, c10::optional<torch::Tensor> router_b,
    int64_t top, bool all, c10::optional<torch::Tensor> corr, double wscale,
    bool sig = false) {
  SM_CHECK_CUDA(h); SM_CHECK_CUDA(router_w); SM_CHECK_F32(router_w);
  const int64_t T = h.size(0);
  const int D = h.size(1);
  const int E = router_w.size(0);
  TORCH_CHECK(router_w.size(1) == D, "moe_route: shapes");
  TORCH_CHECK(E <= SM_MAX_EXPERTS && top >= 1 && top <= E, "moe_route: experts/top");
  const float* bp = nullptr;
  const float* cp = nullptr;
  if (router_b.has_value()) {
    SM_CHECK_CUDA(*router_b); SM_CHECK_F32(*router_b);
    TORCH_CHECK(router_b->numel() == E, "moe_route: bias shape");
    bp = router_b->data_ptr<float>();
  }
  if (corr.has_value()) {
    SM_CHECK_CUDA(*corr); SM_CHECK_F32(*corr);
    TORCH_CHECK(corr->numel() == E, "moe_route: correction shape");
    cp = corr->data_ptr<float>();
  }
  auto idx = torch::empty({T, top}, h.options().dtype(at::kInt));
  auto wts = torch::empty({T, top}, h.options().dtype(at::kFloat));
  if (T == 0) return {idx, wts};
  auto stream = at::cuda::getCurrentCUDAStream();
  const bool bf16 = h.scalar_type() == at::kBFloat16;
  if (!bf16) SM_CHECK_F32(h);
#define ROUTE(TY, ALLV)                                                                    \
  moe_route_kernel<TY, ALLV><<<T, 256, 0, stream>>>(                                       \
      reinterpret_cast<const TY*>(h.data_ptr()), router_w.data_ptr<float>(), bp, D, E,     \
      (int)top, idx.data_ptr<int>(), wts.data_ptr<float>(), cp, (float)wscale, sig)
  if (bf16) { if (all) ROUTE(bf16_t, true); else ROUTE(bf16_t, false); }
  else { if (all) ROUTE(float, true); else ROUTE(float, false); }
#undef ROUTE
  SM_CHECK_LAUNCH();
  return {idx, wts};
}

std::vector<torch::Tensor> moe_route(torch::Tensor h, torch::Tensor router_w,
                                     torch::Tensor router_b, int64_t top) {
  return moe_route_impl(h, router_w, router_b, top, false, c10::nullopt, 1.0);
}

std::vector<torch::Tensor> moe_route_all(torch::Tensor h, torch::Tensor router_w,
                                         c10::optional<torch::Tensor> correction,
                                         int64_t top, double scale) {
  return moe_route_impl(h, router_w, c10::nullopt, top, true, correction, scale);
}

std::vector<torch::Tensor> moe_route_sigmoid(torch::Tensor h, torch::Tensor router_w,
                                             int64_t top) {
  return moe_route_impl(h, router_w, c10::nullopt, top, false, c10::nullopt, 1.0, true);
}

static torch::Tensor moe_experts_impl(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                                      torch::Tensor exp_gu, torch::Tensor exp_down, float limit,
                                      bool scale_input = false) {
  SM_CHECK_CUDA(h); SM_CHECK_CUDA(idx); SM_CHECK_I32(idx); SM_CHECK_CUDA(wts); SM_CHECK_F32(wts);
  SM_CHECK_CUDA(exp_gu); SM_CHECK_CUDA(exp_down);
  const int64_t T = h.size(0);
  const int D = h.size(1);
  const int top = idx.size(1);
  const int E = exp_gu.size(0);
  const int ff = exp_gu.size(1) / 2;
  TORCH_CHECK(exp_gu.dim() == 3 && exp_gu.size(1) == 2 * ff && exp_gu.size(2) == D, "moe_experts: gate/up shape");
  TORCH_CHECK(exp_down.dim() == 3 && exp_down.size(0) == E && exp_down.size(1) == D &&
              exp_down.size(2) == ff, "moe_experts: down shape");
  TORCH_CHECK(idx.size(0) == T && wts.size(0) == T && wts.size(1) == top, "moe_experts: routing shape");
  TORCH_CHECK(E <= SM_MAX_EXPERTS, "moe_experts: too many experts");
  TORCH_CHECK(exp_gu.scalar_type() == h.scalar_type() && exp_down.scalar_type() == h.scalar_type(),
              "moe_experts: dtypes");
  auto out = torch::empty({T, D}, h.options().dtype(at::kFloat));
  if (T == 0) return out;
  const int64_t M = T * top;
  // group the (token, choice) pairs by expert on the device (no host sync)
  auto iopt = h.options().dtype(at::kInt);
  auto off = torch::empty({E + 2}, iopt);    // E weight sets + the identity bin
  auto src = torch::empty({M}, iopt);
  auto inv = torch::empty({M}, iopt);
  auto stream = at::cuda::getCurrentCUDAStream();
  torch::Tensor row_w;
  const float* rw = nullptr;
  if (scale_input) {
    row_w = torch::empty({M}, wts.options());
    rw = row_w.data_ptr<float>();
  }
  moe_group_kernel<<<1, 1024, 0, stream>>>(idx.data_ptr<int>(), (int)M, top, E + 1,
                                           off.data_ptr<int>(), src.data_ptr<int>(),
                                           inv.data_ptr<int>(), wts.data_ptr<float>(),
                                           scale_input ? row_w.data_ptr<float>() : nullptr);
  SM_CHECK_LAUNCH();
  auto y = torch::empty({M, D}, out.options());
  if (h.scalar_type() == at::kBFloat16) {
    auto act = torch::empty({M, ff}, h.options());
    const bf16_t* hp = reinterpret_cast<const bf16_t*>(h.data_ptr());
    const bf16_t* gup = reinterpret_cast<const bf16_t*>(exp_gu.data_ptr());
    const bf16_t* dnp = reinterpret_cast<const bf16_t*>(exp_down.data_ptr());
    if (M <= 16 * E) {
      // a few rows per expert (decoding): 16x16 tiles, K split over four waves
      const int row_tiles = SM_CDIV(M, 16) + E;
      moe_gemm_bf16_splitk_kernel<0><<<dim3(row_tiles, SM_CDIV(ff, 16)), 256, 0, stream>>>(
          hp, src.data_ptr<int>(), gup, off.data_ptr<int>(), E, ff, D, act.data_ptr(), limit, rw);
      SM_CHECK_LAUNCH();
      moe_gemm_bf16_splitk_kernel<1><<<dim3(row_tiles, SM_CDIV(D, 16)), 256, 0, stream>>>(
          reinterpret_cast<const bf16_t*>(act.data_ptr()), nullptr, dnp, off.data_ptr<int>(), E,
          D, ff, y.data_ptr(), 0.f, nullptr);
      SM_CHECK_LAUNCH();
    } else {
      const int row_tiles = SM_CDIV(M, 64) + E;
      moe_gemm_bf16_kernel<0, 4, 4><<<dim3(row_tiles, SM_CDIV(ff, 64)), 256, 0, stream>>>(
          hp, src.data_ptr<int>(), gup, off.data_ptr<int>(), E, ff, D, act.data_ptr(), limit, rw);
      SM_CHECK_LAUNCH();
      moe_gemm_bf16_kernel<1, 4, 4><<<dim3(row_tiles, SM_CDIV(D, 64)), 256, 0, stream>>>(
          reinterpret_cast<const bf16_t*>(act.data_ptr()), nullptr, dnp, off.data_ptr<int>(), E,
          D, ff, y.data_ptr(), 0.f, nullptr);
      SM_CHECK_LAUNCH();
    }
  } else {
    SM_CHECK_F32(h);
    auto act = torch::empty({M, ff}, h.options());
    moe_gemm_f32_kernel<0><<<SM_CDIV(M * ff, 256), 256, 0, stream>>>(
        h.data_ptr<float>(), src.data_ptr<int>(), exp_gu.data_ptr<float>(),
        off.data_ptr<int>(), E, (int)M, ff, D, act.data_ptr<float>(), limit, rw);
    SM_CHECK_LAUNCH();
    moe_gemm_f32_kernel<1><<<SM_CDIV(M * D, 256), 256, 0, stream>>>(
        act.data_ptr<float>(), nullptr, exp_down.data_ptr<float>(), off.data_ptr<int>(), E,
        (int)M, D, ff, y.data_ptr<float>(), 0.f, nullptr);
    SM_CHECK_LAUNCH();
  }
  if (h.scalar_type() == at::kBFloat16)
    moe_combine_kernel<bf16_t><<<T, 256, 0, stream>>>(
        y.data_ptr<float>(), inv.data_ptr<int>(), scale_input ? nullptr : wts.data_ptr<float>(),
        idx.data_ptr<int>(), reinterpret_cast<const bf16_t*>(h.data_ptr()), E, top, D,
        out.data_ptr<float>());
  else
    moe_combine_kernel<float><<<T, 256, 0, stream>>>(
        y.data_ptr<float>(), inv.data_ptr<int>(), scale_input ? nullptr : wts.data_ptr<float>(),
        idx.data_ptr<int>(), h.data_ptr<float>(), E, top, D, out.data_ptr<float>());
  SM_CHECK_LAUNCH();
  return out;
}

torch::Tensor moe_experts(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                          torch::Tensor exp_gu, torch::Tensor exp_down) {
  return moe_experts_impl(h, idx, wts, exp_gu, exp_down, 0.f);
}

torch::Tensor moe_experts_glu(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                              torch::Tensor exp_gu, torch::Tensor exp_down, double limit) {
  TORCH_CHECK(limit > 0, "moe_experts_glu: the clamp limit must be positive");
  return moe_experts_impl(h, idx, wts, exp_gu, exp_down, (float)limit);
}

torch::Tensor moe_experts_scaled_input(torch::Tensor h, torch::Tensor idx, torch::Tensor wts,
                                       torch::Tensor exp_gu, torch::Tensor exp_down) {
  return moe_experts_impl(h, idx, wts, exp_gu, exp_down, 0.f, true);
}
