// Windowed grouped-query softmax attention over paged [k | v] rows, with the
// extras of the pre-norm designs: RMS-normed q/k heads, half-layout rotary
// from a frequency table, scores mixed across heads before the softmax, a
// logarithmic distance bias, a window that keeps the first tokens and a
// per-head sigmoid output gate.
//
// Score mixing without the H x T x T scores: the mixed score of head h is
//   sum_g M[h, g] (q_g . k_c(g)) = sum_c (sum_{g in c} M[h, g] q_g) . k_c,
// one dot product of a folded query q'_h (kv_heads * dim entries, the sum of
// head h's row of M over the heads of each kv head) with the WHOLE key row of
// the cache. The prepare kernel folds the queries; the attention kernels only
// differ in which columns of the key row a head meets (its kv head's, or all).
//   qk_prepare_kv_write     per token: q/k norm, rotation, fold, page write
//   window_attention_group  one workgroup per (token, kv head, share of the
//                           keys) serves every query head of the kv head
//   window_attention        one wave per (token, head): any shape
// (the tiled MFMA kernel for bf16 prompt portions is in
// window_attention_mfma.hip)
// A query at position p sees the keys [0, min(keep, lo)) and [lo, p] with
// lo = max(0, p - window + 1); the kernels walk the two ranges as one list.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

namespace {

// Two neighbouring outputs as one store (the caller checks evenness).
SM_INLINE void wa_store2(float* p, float a, float b) {
  *reinterpret_cast<float2*>(p) = make_float2(a, b);
}
SM_INLINE void wa_store2(bf16_t* p, float a, float b) {
  const unsigned int lo = __bfloat16_as_ushort(__float2bfloat16(a));
  const unsigned int hi = __bfloat16_as_ushort(__float2bfloat16(b));
  *reinterpret_cast<unsigned int*>(p) = lo | (hi << 16);
}

// One workgroup per token. proj row = [q (H dk) | k (G dk) | v (G vd) | ...],
// rows ldp apart. The H + G heads pass through LDS as fp32: the whole row is
// fetched at once, then a wave per head norms it and rotates entries
// (i, i + half) by p * freqs[i] with cos and sin times mag (one sincos per
// pair and token, shared by the heads); then k -> cache row, v -> cache row,
// and q -> q_out [H, dk], or with mix (fp32 [H, H]) the folded queries
// [H, G dk]. PAIR: dk and vd are even and rows start on 4-byte borders, so
// outputs go out two at a time.
template <typename T, bool PAIR>
__global__ __launch_bounds__(256) void qk_prepare_kv_write_kernel(
    const T* __restrict__ proj, int64_t ldp, int H, int G, int dk, int vd,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const int* __restrict__ positions, const float* __restrict__ freqs, int half, float mag,
    const float* __restrict__ mix, const int* __restrict__ page_slot, T* __restrict__ cache,
    T* __restrict__ q_out) {
  extern __shared__ float hb[];                      // [(H + G) dk] | cos, sin [2 half] | mix [H H]
  const int nqk = (H + G) * dk;
  float* cs = hb + nqk;
  float* mx = cs + 2 * half;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = proj + t * ldp;
  for (int i = threadIdx.x; i < nqk; i += blockDim.x) hb[i] = to_f(row[i]);
  if ((int)threadIdx.x < half) {
    float s, c;
    sincosf((float)positions[t] * freqs[threadIdx.x], &s, &c);
    cs[threadIdx.x] = c * mag;
    cs[half + threadIdx.x] = s * mag;
  }
  if (mix != nullptr)
    for (int i = threadIdx.x; i < H * H; i += blockDim.x) mx[i] = mix[i];
  __syncthreads();
  if (qw != nullptr || half > 0) {
    for (int job = wave; job < H + G; job += 4) {    // q heads, then k heads
      float* e = hb + job * dk;
      if (qw != nullptr) {
        float ss = 0.f;
        for (int k = lane; k < dk; k += 64) ss += e[k] * e[k];
        ss = sm_wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)dk + eps);
        const float* w = (job >= H) ? kw : qw;
        for (int k = lane; k < dk; k += 64) e[k] = e[k] * inv * w[k];
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);          // the wave's LDS writes have landed
      }
      for (int pi = lane; pi < half; pi += 64) {
        const float c = cs[pi], sn = cs[half + pi];
        const float a = e[pi], b = e[pi + half];
        e[pi] = a * c - b * sn;
        e[pi + half] = b * c + a * sn;
      }
    }
    __syncthreads();
  }
  const int nk = G * dk, nv = G * vd;
  T* dst = cache + (int64_t)page_slot[t] * (nk + nv);
  const T* v = row + nqk;
  const int rep = H / G;
  if (PAIR) {
    for (int i = 2 * threadIdx.x; i < nk; i += 2 * blockDim.x)
      wa_store2(dst + i, hb[H * dk + i], hb[H * dk + i + 1]);
    for (int i = 2 * threadIdx.x; i < nv; i += 2 * blockDim.x)
      wa_store2(dst + nk + i, to_f(v[i]), to_f(v[i + 1]));
    if (mix == nullptr) {
      for (int i = 2 * threadIdx.x; i < H * dk; i += 2 * blockDim.x)
        wa_store2(q_out + t * H * dk + i, hb[i], hb[i + 1]);
      return;
    }
    for (int hc = wave; hc < H * G; hc += 4) {       // (output head, kv head) per wave
      const int h = hc / G, c = hc % G;
      const float* m = mx + h * H + c * rep;
      const float* src = hb + c * rep * dk;
      T* o = q_out + (t * H + h) * nk + c * dk;
      for (int k = 2 * lane; k < dk; k += 128) {
        float a0 = 0.f, a1 = 0.f;
        for (int r = 0; r < rep; ++r) {
          a0 = fmaf(m[r], src[r * dk + k], a0);
          a1 = fmaf(m[r], src[r * dk + k + 1], a1);
        }
        wa_store2(o + k, a0, a1);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < nk; i += blockDim.x) dst[i] = from_f<T>(hb[H * dk + i]);
  for (int i = threadIdx.x; i < nv; i += blockDim.x) dst[nk + i] = v[i];
  if (mix == nullptr) {
    for (int i = threadIdx.x; i < H * dk; i += blockDim.x) q_out[t * H * dk + i] = from_f<T>(hb[i]);
    return;
  }
  for (int hc = wave; hc < H * G; hc += 4) {
    const int h = hc / G, c = hc % G;
    for (int k = lane; k < dk; k += 64) {
      float a = 0.f;
      for (int r = 0; r < rep; ++r) a = fmaf(mx[h * H + c * rep + r], hb[(c * rep + r) * dk + k], a);
      q_out[(t * H + h) * nk + c * dk + k] = from_f<T>(a);
    }
  }
}

SM_INLINE float wa_bias(float r1, float r2, int dist) { return r1 * log1pf(r2 * (float)dist); }

// One wave per (token, head). The visible keys are taken 64 at a time: lane l
// scores key l over the KD query entries (the kv head's key columns, or the
// whole key row for folded queries), an online softmax carries max and sum,
// then the lanes switch to the value axis.
#define WA_REGS 8   // value entries per lane: vdim <= 512
template <typename T>
__global__ __launch_bounds__(64) void window_attention_kernel(
    const T* __restrict__ q, int KD,  // [Tn, H, KD]
    const T* __restrict__ cache,      // [rows, G dk + G vd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int H, int G,
    int dk, int vd, int whole_key, float scale, int window, int keep,
    const float* __restrict__ r1, const float* __restrict__ r2,
    const T* __restrict__ gate, int64_t ldg, T* __restrict__ out) {   // [Tn, H vd]
  extern __shared__ float lds[];
  float* qs = lds;                                   // KD
  float* pw = lds + KD;                              // 64 weights
  int* krow = reinterpret_cast<int*>(pw + 64);       // 64 cache rows
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const int g = hd / (H / G);
  const int64_t W = (int64_t)G * (dk + vd);
  const int koff = whole_key ? 0 : g * dk;
  for (int k = lane; k < KD; k += 64) qs[k] = to_f(q[((int64_t)t * H + hd) * KD + k]);
  const int b = tok_seq[t], p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int nfirst = (window > 0) ? min(keep, lo) : 0;
  const int n = nfirst + (p - lo + 1);
  const int* bt = block_tables + (int64_t)b * max_nb;
  const float a1 = (r1 != nullptr) ? r1[hd] : 0.f, a2 = (r1 != nullptr) ? r2[hd] : 0.f;
  float m = -INFINITY, l = 0.f;
  float acc[WA_REGS];
  #pragma unroll
  for (int i = 0; i < WA_REGS; ++i) acc[i] = 0.f;
  __syncthreads();
  for (int i0 = 0; i0 < n; i0 += 64) {
    const int i = i0 + lane;
    float s = -INFINITY;
    int row = 0;
    if (i < n) {
      const int j = (i < nfirst) ? i : lo + (i - nfirst);
      row = bt[j / block_size] * block_size + j % block_size;
      const T* kp = cache + (int64_t)row * W + koff;
      float dot = 0.f;
      for (int k = 0; k < KD; ++k) dot = fmaf(qs[k], to_f(kp[k]), dot);
      s = dot * scale;
      if (r1 != nullptr) s -= wa_bias(a1, a2, p - j);
    }
    const float m_new = fmaxf(m, sm_wave_max(s));      // finite: the list is never empty
    const float pj = (i < n) ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);                // first chunk: exp(-inf) = 0
    l = l * corr + sm_wave_sum(pj);
    m = m_new;
    __syncthreads();
    pw[lane] = pj;
    krow[lane] = row;
    __syncthreads();
    const int nkeys = min(64, n - i0);
    #pragma unroll
    for (int r = 0; r < WA_REGS; ++r) {
      const int d = lane + 64 * r;
      if (d < vd) {
        float a = acc[r] * corr;
        for (int jj = 0; jj < nkeys; ++jj)
          a = fmaf(pw[jj], to_f(cache[(int64_t)krow[jj] * W + G * dk + g * vd + d]), a);
        acc[r] = a;
      }
    }
  }
  float f = 1.0f / l;
  if (gate != nullptr) f *= sm_sigmoid(to_f(gate[(int64_t)t * ldg + hd]));
  #pragma unroll
  for (int r = 0; r < WA_REGS; ++r) {
    const int d = lane + 64 * r;
    if (d < vd) out[((int64_t)t * H + hd) * vd + d] = from_f<T>(acc[r] * f);
  }
}

// ---- steps of few tokens per row. One workgroup (4 waves) per (token, kv
// head g, key share z). The REP query heads of g sit in LDS as fp32 (KD
// entries each); the visible keys are cut into blocks of 64, share z takes a
// contiguous run of blocks and its waves take them in turn. Per block: lane =
// key, the key columns are read once in 16-byte pieces (four in flight) and
// dotted with all REP queries; every wave keeps its own running max and sum per head; the REP x 64
// weights go through a wave-private LDS tile; then lane = pair of value
// columns, and every V row is read once for all REP heads. The waves' states
// are merged in LDS; with ksplit > 1 the workgroup leaves (max, sum, weighted
// values) per head and window_attention_merge closes the softmax.
#define WAG_CP 2     // value column pairs per lane: vdim <= 256
template <typename T> struct wa_vec;
template <> struct wa_vec<bf16_t> {
  static constexpr int N = 8;
  SM_INLINE static void load(const bf16_t* p, float* o) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const unsigned int w[4] = {raw.x, raw.y, raw.z, raw.w};
    #pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  SM_INLINE static float2 load2(const bf16_t* p) {
    const unsigned int w = *reinterpret_cast<const unsigned int*>(p);
    return make_float2(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
  }
};
template <> struct wa_vec<float> {
  static constexpr int N = 4;
  SM_INLINE static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
  SM_INLINE static float2 load2(const float* p) { return *reinterpret_cast<const float2*>(p); }
};

template <typename T, int REP>
__global__ __launch_bounds__(256) void window_attention_group_kernel(
    const T* __restrict__ q, int KD,  // [Tn, H, KD]
    const T* __restrict__ cache,      // [rows, G dk + G vd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int H, int G,
    int dk, int vd, int whole_key, float scale, int window, int keep,
    const float* __restrict__ r1, const float* __restrict__ r2,
    const T* __restrict__ gate, int64_t ldg, int ksplit,
    float* __restrict__ part,         // [ksplit, Tn, H, vd] when ksplit > 1
    float* __restrict__ part_ml,      // [ksplit, Tn, H, 2] = (max, sum)
    T* __restrict__ out) {            // [Tn, H vd]
  extern __shared__ __attribute__((aligned(16))) float wgl[];
  constexpr int VN = wa_vec<T>::N;
  float* qs = wgl;                                   // [REP][KD]
  float* pw_all = qs + REP * KD;                     // [4][REP][64]
  int* krow_all = reinterpret_cast<int*>(pw_all + 4 * REP * 64);   // [4][64]
  float* red = reinterpret_cast<float*>(krow_all + 4 * 64);        // [4][REP][vd + 2]
  const int t = blockIdx.x, g = blockIdx.y, z = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t W = (int64_t)G * (dk + vd);
  const int koff = whole_key ? 0 : g * dk;
  const int h0 = g * REP;
  for (int i = tid; i < REP * KD; i += 256)
    qs[i] = to_f(q[((int64_t)t * H + h0 + i / KD) * KD + i % KD]);
  const int b = tok_seq[t], p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int nfirst = (window > 0) ? min(keep, lo) : 0;
  const int n = nfirst + (p - lo + 1);
  const int nblk = (n + 63) / 64;
  const int kb_lo = (int)(((int64_t)nblk * z) / ksplit);
  const int kb_hi = (int)(((int64_t)nblk * (z + 1)) / ksplit);
  const int* bt = block_tables + (int64_t)b * max_nb;
  float* pw = pw_all + wave * REP * 64;
  int* krow = krow_all + wave * 64;
  float a1[REP], a2[REP], m[REP], l[REP];
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh) {
    a1[hh] = (r1 != nullptr) ? r1[h0 + hh] : 0.f;
    a2[hh] = (r1 != nullptr) ? r2[h0 + hh] : 0.f;
    m[hh] = -INFINITY;
    l[hh] = 0.f;
  }
  float acc[REP][WAG_CP][2];
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh)
    #pragma unroll
    for (int c = 0; c < WAG_CP; ++c) acc[hh][c][0] = acc[hh][c][1] = 0.f;
  __syncthreads();
  for (int kb = kb_lo + wave; kb < kb_hi; kb += 4) {
    const int i = kb * 64 + lane;
    float s[REP];
    #pragma unroll
    for (int hh = 0; hh < REP; ++hh) s[hh] = 0.f;
    int row = 0, j = 0;
    if (i < n) {
      j = (i < nfirst) ? i : lo + (i - nfirst);
      row = bt[j / block_size] * block_size + j % block_size;
      const T* kp = cache + (int64_t)row * W + koff;
      // four 16-byte pieces of the key row in flight before their products
      for (int k = 0; k < KD; k += 4 * VN) {
        float kv[4][VN];
        #pragma unroll
        for (int u = 0; u < 4; ++u)
          wa_vec<T>::load(kp + min(k + u * VN, KD - VN), kv[u]);   // past the end: unused
        #pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int ku = k + u * VN;
          if (ku < KD) {
            #pragma unroll
            for (int hh = 0; hh < REP; ++hh)
              #pragma unroll
              for (int e = 0; e < VN; ++e) s[hh] = fmaf(qs[hh * KD + ku + e], kv[u][e], s[hh]);
          }
        }
      }
    }
    float corr[REP];
    #pragma unroll
    for (int hh = 0; hh < REP; ++hh) {
      float x = -INFINITY;
      if (i < n) {
        x = s[hh] * scale;
        if (r1 != nullptr) x -= wa_bias(a1[hh], a2[hh], p - j);
      }
      const float mn = fmaxf(m[hh], sm_wave_max(x));   // finite: the block holds a key
      const float pj = (i < n) ? expf(x - mn) : 0.f;
      corr[hh] = expf(m[hh] - mn);
      l[hh] = l[hh] * corr[hh] + sm_wave_sum(pj);
      m[hh] = mn;
      pw[hh * 64 + lane] = pj;
    }
    krow[lane] = row;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);              // the wave's LDS writes have landed
    #pragma unroll
    for (int hh = 0; hh < REP; ++hh)
      #pragma unroll
      for (int c = 0; c < WAG_CP; ++c) {
        acc[hh][c][0] *= corr[hh];
        acc[hh][c][1] *= corr[hh];
      }
    const int nkeys = min(64, n - kb * 64);
    // eight V rows in flight before their products
    for (int jj0 = 0; jj0 < nkeys; jj0 += 8) {
      float2 v[8][WAG_CP];
      #pragma unroll
      for (int u = 0; u < 8; ++u) {
        const T* vp = cache + (int64_t)krow[min(jj0 + u, nkeys - 1)] * W + G * dk + g * vd;
        #pragma unroll
        for (int c = 0; c < WAG_CP; ++c) {
          const int d = 2 * lane + 128 * c;
          v[u][c] = (d < vd) ? wa_vec<T>::load2(vp + d) : make_float2(0.f, 0.f);
        }
      }
      #pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (jj0 + u < nkeys) {
          #pragma unroll
          for (int c = 0; c < WAG_CP; ++c) {
            #pragma unroll
            for (int hh = 0; hh < REP; ++hh) {
              const float w = pw[hh * 64 + jj0 + u];
              acc[hh][c][0] = fmaf(w, v[u][c].x, acc[hh][c][0]);
              acc[hh][c][1] = fmaf(w, v[u][c].y, acc[hh][c][1]);
            }
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();                 // pw and krow are rewritten for the next block
  }
  // every wave leaves (max, sum, weighted values) per head; wave 0 merges them
  // in order. A wave (or a whole share) without a block has max = -inf.
  const int RS = vd + 2;
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh) {
    float* r = red + (wave * REP + hh) * RS;
    if (lane == 0) { r[vd] = m[hh]; r[vd + 1] = l[hh]; }
    #pragma unroll
    for (int c = 0; c < WAG_CP; ++c) {
      const int d = 2 * lane + 128 * c;
      if (d < vd) { r[d] = acc[hh][c][0]; r[d + 1] = acc[hh][c][1]; }
    }
  }
  __syncthreads();
  if (wave > 0) return;
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh) {
    float M = -INFINITY;
    for (int w = 0; w < 4; ++w) M = fmaxf(M, red[(w * REP + hh) * RS + vd]);
    float L = 0.f, e[4];
    for (int w = 0; w < 4; ++w) {
      const float mw = red[(w * REP + hh) * RS + vd];
      e[w] = (mw == -INFINITY) ? 0.f : expf(mw - M);
      L += red[(w * REP + hh) * RS + vd + 1] * e[w];
    }
    float f = 1.0f;
    if (ksplit == 1) {
      f = 1.0f / L;
      if (gate != nullptr) f *= sm_sigmoid(to_f(gate[(int64_t)t * ldg + h0 + hh]));
    } else if (lane == 0) {
      float* ml = part_ml + (((int64_t)z * gridDim.x + t) * H + h0 + hh) * 2;
      ml[0] = M;
      ml[1] = L;
    }
    #pragma unroll
    for (int c = 0; c < WAG_CP; ++c) {
      const int d = 2 * lane + 128 * c;
      if (d < vd) {
        float v0 = 0.f, v1 = 0.f;
        for (int w = 0; w < 4; ++w) {
          v0 += red[(w * REP + hh) * RS + d] * e[w];
          v1 += red[(w * REP + hh) * RS + d + 1] * e[w];
        }
        if (ksplit > 1) {
          float* dst = part + (((int64_t)z * gridDim.x + t) * H + h0 + hh) * vd + d;
          dst[0] = v0; dst[1] = v1;
        } else {
          T* dst = out + ((int64_t)t * H + h0 + hh) * vd + d;
          dst[0] = from_f<T>(v0 * f); dst[1] = from_f<T>(v1 * f);
        }
      }
    }
  }
}

// Close the softmax over the key shares of one (token, head), in order:
// M = max_s m_s, L = sum_s l_s e^(m_s - M), out = sum_s acc_s e^(m_s - M) / L,
// times the sigmoid of the head's gate.
template <typename T>
__global__ __launch_bounds__(64) void window_attention_merge_kernel(
    const float* __restrict__ part, const float* __restrict__ part_ml, int Tn, int H, int vd,
    int ksplit, const T* __restrict__ gate, int64_t ldg, T* __restrict__ out) {
  const int t = blockIdx.x, h = blockIdx.y;
  const int64_t th = (int64_t)t * H + h, stride = (int64_t)Tn * H;
  float M = -INFINITY;
  for (int s = 0; s < ksplit; ++s) M = fmaxf(M, part_ml[(s * stride + th) * 2]);
  float L = 0.f;
  for (int s = 0; s < ksplit; ++s) {
    const float ms = part_ml[(s * stride + th) * 2];
    if (ms != -INFINITY) L += part_ml[(s * stride + th) * 2 + 1] * expf(ms - M);
  }
  float f = 1.0f / L;
  if (gate != nullptr) f *= sm_sigmoid(to_f(gate[(int64_t)t * ldg + h]));
  for (int d = threadIdx.x; d < vd; d += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < ksplit; ++s) {
      const float ms = part_ml[(s * stride + th) * 2];
      if (ms != -INFINITY) a += part[(s * stride + th) * vd + d] * expf(ms - M);
    }
    out[th * vd + d] = from_f<T>(a * f);
  }
}

template <typename T>
bool launch_group(int rep, dim3 grid, size_t lds, hipStream_t stream, const T* q, int KD,
                  const T* cache, const int* bt, int max_nb, int bs, const int* tok_seq,
                  const int* pos, int H, int G, int dk, int vd, int whole, float scale, int window,
                  int keep, const float* r1, const float* r2, const T* gate, int64_t ldg,
                  int ksplit, float* part, float* part_ml, T* out) {
#define WAG_CASE(R)                                                                          \
  if (rep == R) {                                                                            \
    auto kern = window_attention_group_kernel<T, R>;                                         \
    static int raised = 0;                                                                   \
    if (lds > 64 * 1024 && (int)lds > raised) {                                              \
      TORCH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                   \
                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,   \
                  "window attention: cannot raise the LDS limit");                           \
      raised = (int)lds;                                                                     \
    }                                                                                        \
    kern<<<grid, 256, lds, stream>>>(q, KD, cache, bt, max_nb, bs, tok_seq, pos, H, G, dk,   \
                                     vd, whole, scale, window, keep, r1, r2, gate, ldg,      \
                                     ksplit, part, part_ml, out);                            \
    return true;                                                                             \
  }
  WAG_CASE(1) WAG_CASE(2) WAG_CASE(3) WAG_CASE(4) WAG_CASE(6) WAG_CASE(8)
#undef WAG_CASE
  return false;
}

template <typename T>
void run_plain(torch::Tensor& q, int KD, torch::Tensor& cache, torch::Tensor& block_tables,
               int block_size, torch::Tensor& tok_seq, torch::Tensor& positions, int H, int G,
               int dk, int vd, int whole, float scale, int window, int keep, const float* r1,
               const float* r2, const void* gate, int64_t ldg, int rep, bool grouped,
               torch::Tensor& out, hipStream_t stream) {
  const int64_t Tn = q.size(0);
  const T* qp = reinterpret_cast<const T*>(q.data_ptr());
  const T* cp = reinterpret_cast<const T*>(cache.data_ptr());
  const T* gp = reinterpret_cast<const T*>(gate);
  T* op = reinterpret_cast<T*>(out.data_ptr());
  const int max_nb = (int)block_tables.size(1);
  if (grouped) {
    const size_t lds = (size_t)(rep * KD + 4 * rep * 64 + 4 * 64 + 4 * rep * (vd + 2)) * 4;
    // enough key shares to fill the chip, at least four 64-key blocks each;
    // from host-side sizes only, so a captured step keeps its grid
    const int64_t longest = (window > 0) ? window + keep : (int64_t)max_nb * block_size;
    int ksplit = (int)std::min<int64_t>(std::max<int64_t>(1, 512 / std::max<int64_t>(1, Tn * G)),
                                        std::max<int64_t>(1, longest / 256));
    ksplit = std::min(ksplit, 16);
    torch::Tensor part, part_ml;
    float* pp = nullptr;
    float* pm = nullptr;
    if (ksplit > 1) {
      part = torch::empty({ksplit, Tn, (int64_t)H * vd}, q.options().dtype(at::kFloat));
      part_ml = torch::empty({ksplit, Tn, (int64_t)H * 2}, q.options().dtype(at::kFloat));
      pp = part.data_ptr<float>();
      pm = part_ml.data_ptr<float>();
    }
    const bool ran = launch_group<T>(rep, dim3(Tn, G, ksplit), lds, stream, qp, KD, cp,
                                     block_tables.data_ptr<int>(), max_nb, block_size,
                                     tok_seq.data_ptr<int>(), positions.data_ptr<int>(), H, G, dk,
                                     vd, whole, scale, window, keep, r1, r2, gp, ldg, ksplit, pp,
                                     pm, op);
    TORCH_CHECK(ran, "window_attention: no grouped kernel for this head ratio");
    SM_CHECK_LAUNCH();
    if (ksplit > 1) {
      window_attention_merge_kernel<T><<<dim3(Tn, H), 64, 0, stream>>>(pp, pm, (int)Tn, H, vd,
                                                                       ksplit, gp, ldg, op);
      SM_CHECK_LAUNCH();
    }
    return;
  }
  const size_t lds = (size_t)(KD + 64) * sizeof(float) + 64 * sizeof(int);
  window_attention_kernel<T><<<dim3(Tn, H), 64, lds, stream>>>(
      qp, KD, cp, block_tables.data_ptr<int>(), max_nb, block_size, tok_seq.data_ptr<int>(),
      positions.data_ptr<int>(), H, G, dk, vd, whole, scale, window, keep, r1, r2, gp, ldg, op);
  SM_CHECK_LAUNCH();
}

}  // namespace

torch::Tensor qk_prepare_kv_write(torch::Tensor proj, int64_t heads, int64_t kv_heads, int64_t dim,
                                  int64_t vdim, c10::optional<torch::Tensor> q_norm_w,
                                  c10::optional<torch::Tensor> k_norm_w, double eps,
                                  torch::Tensor positions, c10::optional<torch::Tensor> freqs,
                                  double mag, c10::optional<torch::Tensor> mix,
                                  torch::Tensor page_slot, torch::Tensor cache) {
  SM_CHECK_CUDA(positions); SM_CHECK_I32(positions); SM_CHECK_CUDA(page_slot); SM_CHECK_I32(page_slot);
  SM_CHECK_CUDA(cache);
  const int64_t T = proj.size(0);
  const int H = heads, G = kv_heads, dk = dim, vd = vdim;
  const int64_t need = (int64_t)(H + G) * dk + (int64_t)G * vd;
  TORCH_CHECK(G >= 1 && H % G == 0, "qk_prepare_kv_write: heads must be a multiple of kv_heads");
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1 && proj.size(1) >= need,
              "qk_prepare_kv_write: rows are [q | k | v | ...]");
  TORCH_CHECK(positions.numel() == T && page_slot.numel() == T, "qk_prepare_kv_write: batch layout");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == (int64_t)G * (dk + vd) &&
              cache.scalar_type() == proj.scalar_type(), "qk_prepare_kv_write: cache shape/dtype");
  TORCH_CHECK(q_norm_w.has_value() == k_norm_w.has_value(), "qk_prepare_kv_write: both norms or none");
  const float* qw = nullptr;
  const float* kw = nullptr;
  if (q_norm_w.has_value()) {
    SM_CHECK_CUDA(*q_norm_w); SM_CHECK_F32(*q_norm_w); SM_CHECK_CUDA(*k_norm_w); SM_CHECK_F32(*k_norm_w);
    TORCH_CHECK(q_norm_w->numel() == dk && k_norm_w->numel() == dk, "qk_prepare_kv_write: norm weights");
    qw = q_norm_w->data_ptr<float>();
    kw = k_norm_w->data_ptr<float>();
  }
  const float* fp = nullptr;
  int half = 0;
  if (freqs.has_value() && freqs->numel() > 0) {
    SM_CHECK_CUDA(*freqs); SM_CHECK_F32(*freqs);
    half = (int)freqs->numel();
    TORCH_CHECK(2 * half <= dk, "qk_prepare_kv_write: more rotated entries than the head has");
    fp = freqs->data_ptr<float>();
  }
  const float* mp = nullptr;
  if (mix.has_value()) {
    SM_CHECK_CUDA(*mix); SM_CHECK_F32(*mix);
    TORCH_CHECK(mix->dim() == 2 && mix->size(0) == H && mix->size(1) == H,
                "qk_prepare_kv_write: the mixing matrix is [H, H]");
    mp = mix->data_ptr<float>();
  }
  auto q = torch::empty({T, H, mp != nullptr ? (int64_t)G * dk : (int64_t)dk}, proj.options());
  if (T == 0) return q;
  const size_t lds = ((size_t)(H + G) * dk + 2 * half + (mp != nullptr ? H * H : 0)) * sizeof(float);
  TORCH_CHECK(lds <= 150 * 1024, "qk_prepare_kv_write: heads * dim too large");
  TORCH_CHECK(half <= 256, "qk_prepare_kv_write: more than 512 rotated entries");
  auto stream = at::cuda::getCurrentCUDAStream();
  const bool is_bf16 = proj.scalar_type() == at::kBFloat16;
  if (!is_bf16) SM_CHECK_F32(proj);
  // outputs two at a time: even sizes, rows that start on 4-byte (bf16) or
  // 8-byte (fp32) borders
  const int64_t esz = is_bf16 ? 2 : 4;
  const bool pair = dk % 2 == 0 && vd % 2 == 0 && proj.stride(0) % 2 == 0 &&
                    reinterpret_cast<uintptr_t>(proj.data_ptr()) % (2 * esz) == 0;
#define QKP_LAUNCH(TY, PAIRV)                                                                  \
  do {                                                                                         \
    auto kern = qk_prepare_kv_write_kernel<TY, PAIRV>;                                         \
    static int raised = 0;     /* per variant; not repeated under graph capture */             \
    if (lds > 64 * 1024 && (int)lds > raised) {                                                \
      TORCH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                     \
                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,     \
                  "qk_prepare_kv_write: cannot raise the LDS limit");                          \
      raised = (int)lds;                                                                       \
    }                                                                                          \
    kern<<<T, 256, lds, stream>>>(                                                             \
        reinterpret_cast<const TY*>(proj.data_ptr()), proj.stride(0), H, G, dk, vd, qw, kw,    \
        (float)eps, positions.data_ptr<int>(), fp, half, (float)mag, mp,                       \
        page_slot.data_ptr<int>(), reinterpret_cast<TY*>(cache.data_ptr()),                    \
        reinterpret_cast<TY*>(q.data_ptr()));                                                  \
  } while (0)
  if (is_bf16) { if (pair) QKP_LAUNCH(bf16_t, true); else QKP_LAUNCH(bf16_t, false); }
  else { if (pair) QKP_LAUNCH(float, true); else QKP_LAUNCH(float, false); }
#undef QKP_LAUNCH
  SM_CHECK_LAUNCH();
  return q;
}

// defined in window_attention_mfma.hip
bool window_attention_mfma_fits(int KD, int vd);
void window_attention_mfma(torch::Tensor q, int KD, torch::Tensor cache, int H, int G, int dk, int vd,
                           int whole_key, torch::Tensor block_tables, int block_size,
                           torch::Tensor positions, float scale, int window, int keep,
                           const float* r1, const float* r2, const void* gate, int64_t ldg,
                           torch::Tensor tiles, torch::Tensor out);

torch::Tensor window_attention(torch::Tensor q, torch::Tensor cache, int64_t heads,
                               int64_t kv_heads, int64_t dim, int64_t vdim, bool whole_key,
                               torch::Tensor block_tables, int64_t block_size,
                               torch::Tensor tok_seq, torch::Tensor positions, double scale,
                               int64_t window, int64_t keep_first,
                               c10::optional<torch::Tensor> r1, c10::optional<torch::Tensor> r2,
                               c10::optional<torch::Tensor> gate,
                               c10::optional<torch::Tensor> tiles, int64_t max_tile_queries) {
  SM_CHECK_CUDA(q); SM_CHECK_CUDA(cache); SM_CHECK_CUDA(block_tables); SM_CHECK_I32(block_tables);
  SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq); SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  const int H = heads, G = kv_heads, dk = dim, vd = vdim;
  const int64_t T = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0, "window_attention: heads must be a multiple of kv_heads");
  const int KD = whole_key ? G * dk : dk;
  TORCH_CHECK(q.dim() == 3 && q.size(1) == H && q.size(2) == KD,
              "window_attention: q is [T, H, dim], or [T, H, kv_heads * dim] for folded queries");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == (int64_t)G * (dk + vd) &&
              cache.scalar_type() == q.scalar_type(), "window_attention: cache shape/dtype");
  TORCH_CHECK(block_tables.dim() == 2 && tok_seq.numel() == T && positions.numel() == T &&
              block_size > 0, "window_attention: batch layout");
  TORCH_CHECK(vd <= 64 * WA_REGS, "window_attention: value size above 512");
  TORCH_CHECK(window >= 0 && keep_first >= 0, "window_attention: window");
  TORCH_CHECK(r1.has_value() == r2.has_value(), "window_attention: both distance factors or none");
  const float* r1p = nullptr;
  const float* r2p = nullptr;
  if (r1.has_value()) {
    SM_CHECK_CUDA(*r1); SM_CHECK_F32(*r1); SM_CHECK_CUDA(*r2); SM_CHECK_F32(*r2);
    TORCH_CHECK(r1->numel() == H && r2->numel() == H, "window_attention: per-head tensors");
    r1p = r1->data_ptr<float>();
    r2p = r2->data_ptr<float>();
  }
  const void* gp = nullptr;
  int64_t ldg = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->is_cuda() && gate->dim() == 2 && gate->stride(1) == 1 && gate->size(0) == T &&
                gate->size(1) == H && gate->scalar_type() == q.scalar_type(),
                "window_attention: gate is [T, H] in the queries' dtype");
    gp = gate->data_ptr();
    ldg = gate->stride(0);
  }
  auto out = torch::empty({T, (int64_t)H * vd}, q.options());
  if (T == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  const bool is_bf16 = q.scalar_type() == at::kBFloat16;
  if (!is_bf16) SM_CHECK_F32(q);
  if (is_bf16 && tiles.has_value() && max_tile_queries > 4 &&
      window_attention_mfma_fits(KD, vd)) {
    SM_CHECK_CUDA(*tiles); SM_CHECK_I32(*tiles);
    TORCH_CHECK(tiles->dim() == 2 && tiles->size(1) == 3 && max_tile_queries <= 64,
                "window_attention: tiles");
    window_attention_mfma(q, KD, cache, H, G, dk, vd, whole_key ? 1 : 0, block_tables,
                          (int)block_size, positions, (float)scale, (int)window, (int)keep_first,
                          r1p, r2p, gp, ldg, *tiles, out);
    return out;
  }
  const int rep = H / G, vn = is_bf16 ? 8 : 4;
  const bool rep_ok = rep <= 4 || rep == 6 || rep == 8;
  // the grouped kernel needs 16-byte pieces of the key columns and column
  // pairs of V
  const bool grouped =
      rep_ok && dk % vn == 0 && vd % 2 == 0 && ((int64_t)G * (dk + vd)) % vn == 0 &&
      vd <= 128 * WAG_CP &&
      (size_t)(rep * KD + 4 * rep * 64 + 4 * 64 + 4 * rep * (vd + 2)) * 4 <= 150 * 1024;
  if (is_bf16)
    run_plain<bf16_t>(q, KD, cache, block_tables, (int)block_size, tok_seq, positions, H, G, dk, vd,
                      whole_key ? 1 : 0, (float)scale, (int)window, (int)keep_first, r1p, r2p, gp,
                      ldg, rep, grouped, out, stream);
  else
    run_plain<float>(q, KD, cache, block_tables, (int)block_size, tok_seq, positions, H, G, dk, vd,
                     whole_key ? 1 : 0, (float)scale, (int)window, (int)keep_first, r1p, r2p, gp,
                     ldg, rep, grouped, out, stream);
  return out;
}
