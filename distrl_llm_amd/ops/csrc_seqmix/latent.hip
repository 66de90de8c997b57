// Latent attention: cache write (latent RMS norm + rotated shared key part),
// query rotation, and windowed softmax attention in latent space over the
// paged cache. Prompt portions and single decode tokens run in the same
// step. Three attention kernels, chosen on the host:
//   latent_attention_coop    bf16 default: four waves per tile of <= 16 rows
//                            (queries of one head, or heads of one decoded
//                            token), key blocks staged in LDS, scores and
//                            weighted sum on MFMA
//   latent_attention_tiled   bf16 fallback (tile too wide for LDS, tiny
//                            portions): MFMA scores, fp32 FMA weighted sum
//   latent_attention         one wave per (token, head): fp32 models, any size
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

namespace {

// angle of pair i at position p: p * base^(-2 i / dims), or p * freqs[i] with
// cos and sin scaled by mag when a frequency table is given; all fp32
SM_INLINE void rot_cs(int p, int i, float base, int dims, const float* freqs, float mag,
                      float* c, float* s) {
  const float f = freqs != nullptr ? freqs[i] : powf(base, -2.0f * (float)i / (float)dims);
  sincosf((float)p * f, s, c);
  if (freqs != nullptr) { *c *= mag; *s *= mag; }
}

// Entry k of a rotated vector v (first dims entries rotated): pairs
// (i, i + dims/2), or (2i, 2i+1) with PAIRS.
template <typename T>
SM_INLINE float rot_entry(const T* v, int k, int p, float base, int dims, const float* freqs,
                          float mag, bool pairs) {
  if (k >= dims) return to_f(v[k]);
  const int half = dims / 2;
  int pi, ia, ib;
  bool first;
  if (pairs) { pi = k >> 1; ia = 2 * pi; ib = ia + 1; first = (k & 1) == 0; }
  else { pi = (k < half) ? k : k - half; ia = pi; ib = pi + half; first = k < half; }
  float c, s;
  rot_cs(p, pi, base, dims, freqs, mag, &c, &s);
  const float a = to_f(v[ia]), b = to_f(v[ib]);
  return first ? a * c - b * s : b * c + a * s;
}

// One workgroup per token. q row = H * (dn + rd) query entries, d row (when
// the layer owns a cache) = [latent (r) | shared key part (rd)]; rows are
// ldq / ldd apart.
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ q, int64_t ldq, const T* __restrict__ dkv, int64_t ldd, int H,
    int dn, int rd, int r, const float* __restrict__ norm_w, float eps,
    const int* __restrict__ positions, float base, int dims, const float* __restrict__ freqs,
    float mag, int pairs, const int* __restrict__ page_slot, T* __restrict__ cache,
    float* __restrict__ q_rot) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const T* row = q + t * ldq;
  const int p = positions[t];
  // rotated query part of every head
  for (int i = threadIdx.x; i < H * rd; i += blockDim.x) {
    const int hd = i / rd, k = i % rd;
    q_rot[(t * H + hd) * rd + k] =
        rot_entry(row + hd * (dn + rd) + dn, k, p, base, dims, freqs, mag, pairs != 0);
  }
  if (dkv == nullptr) return;
  const T* d = dkv + t * ldd;
  float ss = 0.f;
  for (int k = threadIdx.x; k < r; k += blockDim.x) {
    const float v = to_f(d[k]);
    ss += v * v;
  }
  ss = sm_block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)r + eps);
  T* dst = cache + (int64_t)page_slot[t] * (r + rd);
  for (int k = threadIdx.x; k < r; k += blockDim.x)
    dst[k] = from_f<T>(to_f(d[k]) * inv * norm_w[k]);
  for (int k = threadIdx.x; k < rd; k += blockDim.x)
    dst[r + k] = from_f<T>(rot_entry(d + r, k, p, base, dims, freqs, mag, pairs != 0));
}

// Closing factor of one (token, head): 1 / (sum + e^(sink - max)) when the
// head has a sink term in its softmax denominator, times sigmoid(gate) when
// the head's result is gated.
template <typename T>
SM_INLINE float lat_close(float M, float L, const float* sink, const T* gate, int64_t ldg,
                          int64_t t, int hd) {
  float f = 1.0f / L;
  if (sink != nullptr) {
    const float M2 = fmaxf(M, sink[hd]), e = expf(M - M2);
    f = e / (L * e + expf(sink[hd] - M2));
  }
  if (gate != nullptr) f *= sm_sigmoid(to_f(gate[t * ldg + hd]));
  return f;
}

// One wave per (token, head). Keys lo..p of the token's sequence are taken
// 64 at a time: lane l scores key l (dot over the whole cache row), an
// online softmax carries max and sum across chunks, then the lanes switch
// to the latent axis and accumulate sum_j p_j c_j.
#define SM_LAT_REGS 16   // latent dims per lane: kv_rank <= 64 * 16
template <typename T>
__global__ __launch_bounds__(64) void latent_attention_kernel(
    const T* __restrict__ q_lat,      // [H, Tn, r]
    const float* __restrict__ q_rot,  // [Tn, H, rd]
    const T* __restrict__ cache,      // [rows, r + rd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions,
    int Tn, int H, int r, int rd, int window, float scale,
    const float* __restrict__ sink, const T* __restrict__ gate, int64_t ldg,
    T* __restrict__ out) {            // [H, Tn, r]
  extern __shared__ float lds[];
  float* q = lds;                       // r + rd
  float* pw = lds + r + rd;             // 64 weights
  int* krow = reinterpret_cast<int*>(pw + 64);   // 64 cache rows
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const int W = r + rd;
  for (int k = lane; k < r; k += 64) q[k] = to_f(q_lat[((int64_t)hd * Tn + t) * r + k]);
  for (int k = lane; k < rd; k += 64) q[r + k] = q_rot[((int64_t)t * H + hd) * rd + k];
  const int b = tok_seq[t], p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* bt = block_tables + (int64_t)b * max_nb;
  float m = -INFINITY, l = 0.f;
  float acc[SM_LAT_REGS];
  #pragma unroll
  for (int i = 0; i < SM_LAT_REGS; ++i) acc[i] = 0.f;
  __syncthreads();
  for (int j0 = lo; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    int row = 0;
    if (j <= p) {
      row = bt[j / block_size] * block_size + j % block_size;
      const T* kv = cache + (int64_t)row * W;
      float dot = 0.f;
      for (int k = 0; k < W; ++k) dot += q[k] * to_f(kv[k]);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, sm_wave_max(s));
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);          // first chunk: exp(-inf) = 0
    l = l * corr + sm_wave_sum(pj);
    m = m_new;
    __syncthreads();
    pw[lane] = pj;
    krow[lane] = row;
    __syncthreads();
    const int nk = min(64, p - j0 + 1);
    #pragma unroll
    for (int i = 0; i < SM_LAT_REGS; ++i) {
      const int k = lane + 64 * i;
      if (k < r) {
        float a = acc[i] * corr;
        for (int jj = 0; jj < nk; ++jj)
          a += pw[jj] * to_f(cache[(int64_t)krow[jj] * W + k]);
        acc[i] = a;
      }
    }
  }
  const float invl = lat_close(m, l, sink, gate, ldg, t, hd);
  #pragma unroll
  for (int i = 0; i < SM_LAT_REGS; ++i) {
    const int k = lane + 64 * i;
    if (k < r) out[((int64_t)hd * Tn + t) * r + k] = from_f<T>(acc[i] * invl);
  }
}


// ---- tiled kernel (bf16): up to 16 consecutive queries of one sequence and
// one head per workgroup; NW waves split the key range and are combined at
// the end. Scores come from MFMA 16x16x32 (bf16 in, fp32 accumulate) on 32
// keys at a time; the softmax weights stay fp32 and the weighted latent sum
// is an fp32 FMA loop with the lanes on the latent axis, so every cache row
// is read once for all queries of the tile.
// MFMA fragments: A lane l -> row l&15, k (l>>4)*8..+7; B lane l -> column
// l&15, same k; D lane l reg r -> row (l>>4)*4+r, column l&15.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16v8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

SM_INLINE bf16v8_t lat_load8(const bf16_t* p, int valid, bool vec) {
  bf16v8_t v;
  if (vec && valid >= 8) {
    v = *reinterpret_cast<const bf16v8_t*>(p);
  } else {
    #pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = (j < valid) ? (__bf16)__bfloat162float(p[j]) : (__bf16)0.0f;
  }
  return v;
}

#define LT_TQ 16
#define LT_KB 32
// latent entry of accumulator i in lane l: lanes own adjacent pairs
#define LT_FEAT(l, i) (2 * (l) + 128 * ((i) >> 1) + ((i) & 1))
// HEADS: the tile's rows are up to 16 heads of ONE token (decoding: the
// keys of a sequence are read once for all its heads) instead of up to 16
// consecutive tokens of one head.
template <int RPL, bool HEADS>
__global__ __launch_bounds__(256) void latent_attention_tiled_kernel(
    const bf16_t* __restrict__ q_lat,   // [H, Tn, r]
    const float* __restrict__ q_rot,    // [Tn, H, rd]
    const bf16_t* __restrict__ cache,   // [rows, r + rd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tiles,      // [ntiles, 3] = (batch row, first token, queries)
    const int* __restrict__ positions, int Tn, int H, int r, int rd, int window,
    float scale, int nq_cap, bf16_t* __restrict__ out,
    int ksplit, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const float* __restrict__ sink, const bf16_t* __restrict__ gate, int64_t ldg) {
  // ksplit > 1 (HEADS only): blockIdx.z takes a contiguous share of the key
  // blocks and leaves (max, sum, unnormalised latent sum) for the combine
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int W = r + rd;
  const int Wp = ((W + 31) / 32) * 32 + 8;          // padded query row (bf16)
  const int NW = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  const int lrow = l & 15, lk = l >> 4;
  bf16_t* q_lds = reinterpret_cast<bf16_t*>(smem);                      // [16][Wp]
  float* wbase = reinterpret_cast<float*>(smem + (size_t)LT_TQ * Wp * 2);
  float* p_lds = wbase + wave * (LT_TQ * LT_KB + LT_KB + LT_TQ);        // [16][32]
  int* krow = reinterpret_cast<int*>(p_lds + LT_TQ * LT_KB);            // [32]
  float* corr_lds = p_lds + LT_TQ * LT_KB + LT_KB;                      // [16]
  float* comb = wbase + NW * (LT_TQ * LT_KB + LT_KB + LT_TQ);           // combine area

  const int tile = blockIdx.x;
  const int hd = HEADS ? blockIdx.y * LT_TQ : blockIdx.y;     // first / only head
  const int b = tiles[3 * tile], t0 = tiles[3 * tile + 1];
  const int nq = HEADS ? min(LT_TQ, H - hd) : tiles[3 * tile + 2];
  const int p0 = positions[t0], plast = HEADS ? p0 : p0 + nq - 1;
  const int lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
  const int nkeys = plast - lo + 1;
  const int nblk = (nkeys + LT_KB - 1) / LT_KB;
  const int* bt = block_tables + (int64_t)b * max_nb;
  const bool vec = (W % 8) == 0;
  const bool pair = (W % 2) == 0 && (r % 2) == 0;   // 4-byte aligned entry pairs

  // stage the query tile: [latent part | rotated part], zero padded
  if ((r % 8) == 0) {
    // latent part in 16-byte pieces, the rest entry by entry
    const int r8 = r / 8, w8 = (Wp - r);
    for (int i = threadIdx.x; i < LT_TQ * r8; i += blockDim.x) {
      const int q = i / r8, k = (i % r8) * 8;
      bf16v8_t v;
      #pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (__bf16)0.0f;
      if (q < nq) {
        const int tq = HEADS ? t0 : t0 + q, hq = HEADS ? hd + q : hd;
        v = *reinterpret_cast<const bf16v8_t*>(q_lat + ((int64_t)hq * Tn + tq) * r + k);
      }
      *reinterpret_cast<bf16v8_t*>(q_lds + q * Wp + k) = v;
    }
    for (int i = threadIdx.x; i < LT_TQ * w8; i += blockDim.x) {
      const int q = i / w8, k = r + i % w8;
      float v = 0.f;
      if (q < nq && k < W) {
        const int tq = HEADS ? t0 : t0 + q, hq = HEADS ? hd + q : hd;
        v = q_rot[((int64_t)tq * H + hq) * rd + (k - r)];
      }
      q_lds[q * Wp + k] = __float2bfloat16(v);
    }
  } else {
    for (int i = threadIdx.x; i < LT_TQ * Wp; i += blockDim.x) {
      const int q = i / Wp, k = i % Wp;
      float v = 0.f;
      if (q < nq) {
        const int tq = HEADS ? t0 : t0 + q, hq = HEADS ? hd + q : hd;
        if (k < r) v = to_f(q_lat[((int64_t)hq * Tn + tq) * r + k]);
        else if (k < W) v = q_rot[((int64_t)tq * H + hq) * rd + (k - r)];
      }
      q_lds[i] = __float2bfloat16(v);
    }
  }
  __syncthreads();

  float m[4], lsum[4];
  #pragma unroll
  for (int rr = 0; rr < 4; ++rr) { m[rr] = -INFINITY; lsum[rr] = 0.f; }
  float acc[LT_TQ][RPL];
  #pragma unroll
  for (int q = 0; q < LT_TQ; ++q)
    #pragma unroll
    for (int i = 0; i < RPL; ++i) acc[q][i] = 0.f;
  const int KS = (W + 31) / 32;

  const int kb_lo = (int)(((int64_t)nblk * blockIdx.z) / ksplit);
  const int kb_hi = (int)(((int64_t)nblk * (blockIdx.z + 1)) / ksplit);
  for (int kb = kb_lo + wave; kb < kb_hi; kb += NW) {
    const int j0 = lo + kb * LT_KB;
    // cache rows of this block's keys (lanes 0..31), clamped to the last key
    if (l < LT_KB) {
      const int j = min(j0 + l, plast);
      krow[l] = bt[j / block_size] * block_size + j % block_size;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): LDS writes visible to the wave
    const bf16_t* k0p = cache + (int64_t)krow[lrow] * W;
    const bf16_t* k1p = cache + (int64_t)krow[16 + lrow] * W;
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    #pragma unroll 4
    for (int ks = 0; ks < KS; ++ks) {
      const int f0 = ks * 32 + lk * 8;
      const bf16v8_t a = *reinterpret_cast<const bf16v8_t*>(q_lds + lrow * Wp + f0);
      const bf16v8_t b0 = lat_load8(k0p + f0, W - f0, vec);
      const bf16v8_t b1 = lat_load8(k1p + f0, W - f0, vec);
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b0, s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b1, s1, 0, 0, 0);
    }
    // mask, online softmax per query row (rows lk*4 + rr; 16 lanes share a row)
    float pv0[4], pv1[4], cr[4];
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int q = lk * 4 + rr;
      const int pq = HEADS ? p0 : p0 + q;
      const int ja = j0 + lrow, jb = j0 + 16 + lrow;
      const bool oka = q < nq && ja <= pq && (window <= 0 || pq - ja < window);
      const bool okb = q < nq && jb <= pq && (window <= 0 || pq - jb < window);
      const float sa = oka ? s0[rr] * scale : -INFINITY;
      const float sb = okb ? s1[rr] * scale : -INFINITY;
      float bm = fmaxf(sa, sb);
      #pragma unroll
      for (int off = 8; off > 0; off >>= 1) bm = fmaxf(bm, __shfl_xor(bm, off, SM_WAVE));
      const float mn = fmaxf(m[rr], bm);
      const float c = (mn == -INFINITY) ? 1.0f : expf(m[rr] - mn);
      const float pa = oka ? expf(sa - mn) : 0.f;
      const float pb = okb ? expf(sb - mn) : 0.f;
      float ps = pa + pb;
      #pragma unroll
      for (int off = 8; off > 0; off >>= 1) ps += __shfl_xor(ps, off, SM_WAVE);
      lsum[rr] = lsum[rr] * c + ps;
      m[rr] = mn;
      pv0[rr] = pa; pv1[rr] = pb; cr[rr] = c;
    }
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int q = lk * 4 + rr;
      p_lds[q * LT_KB + lrow] = pv0[rr];
      p_lds[q * LT_KB + 16 + lrow] = pv1[rr];
      if (lrow == 0) corr_lds[q] = cr[rr];
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
    // weighted latent sum: lanes on the latent axis
    const int nk = min(LT_KB, nkeys - kb * LT_KB);
    #pragma unroll
    for (int q = 0; q < LT_TQ; ++q) {
      if (q < nq) {
        const float c = corr_lds[q];
        #pragma unroll
        for (int i = 0; i < RPL; ++i) acc[q][i] *= c;
      }
    }
    #pragma unroll 8
    for (int kk = 0; kk < nk; ++kk) {
      const bf16_t* crow = cache + (int64_t)krow[kk] * W;
      float cv[RPL];
      if (pair) {                       // two adjacent entries per 4-byte load
        #pragma unroll
        for (int i = 0; i < RPL; i += 2) {
          const int f = LT_FEAT(l, i);
          uint32_t w2 = 0;
          if (f < r) w2 = *reinterpret_cast<const uint32_t*>(crow + f);
          cv[i] = __uint_as_float(w2 << 16);
          cv[i + 1] = __uint_as_float(w2 & 0xffff0000u);
        }
      } else {
        #pragma unroll
        for (int i = 0; i < RPL; ++i) {
          const int f = LT_FEAT(l, i);
          cv[i] = (f < r) ? to_f(crow[f]) : 0.f;
        }
      }
      #pragma unroll
      for (int q = 0; q < LT_TQ; ++q) {
        if (q < nq) {
          const float pw = p_lds[q * LT_KB + kk];
          #pragma unroll
          for (int i = 0; i < RPL; ++i) acc[q][i] = fmaf(pw, cv[i], acc[q][i]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // per-row max and sum to LDS (one lane of each 16-lane group writes)
  float* ml = comb;                                  // [NW][16][2]
  float* cacc = comb + NW * LT_TQ * 2;               // [NW - 1][nq_cap][r]: waves 1..
  #pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    if (lrow == 0) {
      ml[(wave * LT_TQ + lk * 4 + rr) * 2] = m[rr];
      ml[(wave * LT_TQ + lk * 4 + rr) * 2 + 1] = lsum[rr];
    }
  }
  if (wave > 0) {
    #pragma unroll
    for (int q = 0; q < LT_TQ; ++q) {
      if (q < nq) {
        #pragma unroll
        for (int i = 0; i < RPL; ++i) {
          const int f = LT_FEAT(l, i);
          if (f < r) cacc[((int64_t)(wave - 1) * nq_cap + q) * r + f] = acc[q][i];
        }
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  #pragma unroll
  for (int q = 0; q < LT_TQ; ++q) {
    if (q < nq) {
      float M = -INFINITY;
      for (int w = 0; w < NW; ++w) M = fmaxf(M, ml[(w * LT_TQ + q) * 2]);
      float L = 0.f;
      for (int w = 0; w < NW; ++w) {
        const float mw = ml[(w * LT_TQ + q) * 2];
        if (mw != -INFINITY) L += ml[(w * LT_TQ + q) * 2 + 1] * expf(mw - M);
      }
      const int tq_ = HEADS ? t0 : t0 + q, hq_ = HEADS ? hd + q : hd;
      const float invL = lat_close(M, L, sink, gate, ldg, tq_, hq_);
      if (ksplit > 1 && l == 0) {
        part_ml[(((int64_t)tq_ * H + hq_) * ksplit + blockIdx.z) * 2] = M;
        part_ml[(((int64_t)tq_ * H + hq_) * ksplit + blockIdx.z) * 2 + 1] = L;
      }
      #pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const int f = LT_FEAT(l, i);
        if (f < r) {
          const float m0 = ml[q * 2];
          float a = (m0 != -INFINITY) ? acc[q][i] * expf(m0 - M) : 0.f;
          for (int w = 1; w < NW; ++w) {
            const float mw = ml[(w * LT_TQ + q) * 2];
            if (mw != -INFINITY)
              a += cacc[((int64_t)(w - 1) * nq_cap + q) * r + f] * expf(mw - M);
          }
          if (ksplit > 1)
            part_acc[(((int64_t)tq_ * H + hq_) * ksplit + blockIdx.z) * r + f] = a;
          else
            out[((int64_t)hq_ * Tn + tq_) * r + f] = __float2bfloat16(a * invL);
        }
      }
    }
  }
}


// ---- prompt tiles, all on MFMA: four waves share one tile of up to 16
// queries of one head. Each 32-key block of the cache is staged in LDS once;
// the waves share the block's score MFMAs (a 16-key tile and half of the
// feature steps each, summed through LDS), every wave keeps the same fp32
// softmax state, then takes every fourth 16-wide slice of the latent axis of
// the weighted sum: O[q, f] += sum_k P[q, k] C[k, f] as MFMA with the weights
// split into two bf16 terms (p = hi + lo, |p - hi - lo| <= 2^-17 p), so the
// fp32 weights keep 16+ bits against the bf16 latents; accumulation is fp32.
#define LC_NT 8      // latent slices per wave: kv_rank <= 4 * 8 * 16
// LDS row length (bf16) of the staged queries / key block: a multiple of 8
// (16-byte pieces) that is 16 mod 64, so that neighbouring rows start 8
// banks apart and the four lane groups of a weighted-sum gather do not collide
#define LC_ROW(W) ((((W) + 31) / 32) * 32 + ((((W) + 31) / 32) % 2 ? 48 : 16))
// HEADS: rows are up to 16 heads of one token (decoding); blockIdx.z then
// takes a share of the key blocks and leaves (max, sum, unnormalised sum)
// for latent_combine when ksplit > 1.
template <bool HEADS>
__global__ __launch_bounds__(256) void latent_attention_coop_kernel(
    const bf16_t* __restrict__ q_lat, const float* __restrict__ q_rot,
    const bf16_t* __restrict__ cache, const int* __restrict__ block_tables,
    int max_nb, int block_size, const int* __restrict__ tiles,
    const int* __restrict__ positions, int Tn, int H, int r, int rd, int window,
    float scale, bf16_t* __restrict__ out, int ksplit,
    float* __restrict__ part_acc, float* __restrict__ part_ml,
    const float* __restrict__ sink, const bf16_t* __restrict__ gate, int64_t ldg) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int W = r + rd;
  const int Wp = LC_ROW(W);
  const int wave = threadIdx.x >> 6, l = threadIdx.x & 63;
  const int lrow = l & 15, lk = l >> 4;
  bf16_t* q_lds = reinterpret_cast<bf16_t*>(smem);                 // [16][Wp]
  bf16_t* c_lds = q_lds + LT_TQ * Wp;                               // [32][Wp]
  float* s_lds = reinterpret_cast<float*>(c_lds + LT_KB * Wp);     // [2][16][32] score halves
  float* p_lds = s_lds + 2 * LT_TQ * LT_KB + wave * (LT_TQ * LT_KB);

  const int tile = blockIdx.x;
  const int hd = HEADS ? blockIdx.y * LT_TQ : blockIdx.y;
  const int b = tiles[3 * tile], t0 = tiles[3 * tile + 1];
  const int nq = HEADS ? min(LT_TQ, H - hd) : tiles[3 * tile + 2];
  const int p0 = positions[t0], plast = HEADS ? p0 : p0 + nq - 1;
  const int lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
  const int nkeys = plast - lo + 1;
  const int nblk = (nkeys + LT_KB - 1) / LT_KB;
  const int* bt = block_tables + (int64_t)b * max_nb;
  const bool vec = (W % 8) == 0;

  // queries [latent | rotated], zero padded; key block area zeroed once
  for (int i = threadIdx.x; i < LT_TQ * Wp; i += blockDim.x) {
    const int q = i / Wp, k = i % Wp;
    float v = 0.f;
    if (q < nq) {
      const int tq = HEADS ? t0 : t0 + q, hq = HEADS ? hd + q : hd;
      if (k < r) v = to_f(q_lat[((int64_t)hq * Tn + tq) * r + k]);
      else if (k < W) v = q_rot[((int64_t)tq * H + hq) * rd + (k - r)];
    }
    q_lds[i] = __float2bfloat16(v);
  }
  for (int i = threadIdx.x; i < LT_KB * Wp; i += blockDim.x) c_lds[i] = __float2bfloat16(0.f);

  float m[4], lsum[4];
  #pragma unroll
  for (int rr = 0; rr < 4; ++rr) { m[rr] = -INFINITY; lsum[rr] = 0.f; }
  f32x4_t acc[LC_NT];
  #pragma unroll
  for (int i = 0; i < LC_NT; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int KS = (W + 31) / 32;
  const int ntiles_f = (r + 15) / 16;

  const int kb_lo = (int)(((int64_t)nblk * blockIdx.z) / ksplit);
  const int kb_hi = (int)(((int64_t)nblk * (blockIdx.z + 1)) / ksplit);
  // cache rows of a block's 32 keys: looked up by 32 lanes one block ahead,
  // so the copy below does not chain a block-table load before every piece
  __shared__ int krow[LT_KB];
  auto key_rows = [&](int kb2) {
    if (threadIdx.x < LT_KB) {
      const int j = min(lo + kb2 * LT_KB + (int)threadIdx.x, plast);
      krow[threadIdx.x] = bt[j / block_size] * block_size + j % block_size;
    }
  };
  if (kb_lo < kb_hi) key_rows(kb_lo);
  if (kb_hi == kb_lo) __syncthreads();     // the LDS fills above, before any exit
  for (int kb = kb_lo; kb < kb_hi; ++kb) {
    const int nk = min(LT_KB, nkeys - kb * LT_KB);
    __syncthreads();                       // the previous block is fully consumed
    if (vec) {
      const int w8 = W / 8;
      #pragma unroll 4
      for (int i = threadIdx.x; i < nk * w8; i += blockDim.x) {
        const int kk = i / w8, k = (i % w8) * 8;
        *reinterpret_cast<bf16v8_t*>(c_lds + kk * Wp + k) =
            *reinterpret_cast<const bf16v8_t*>(cache + (int64_t)krow[kk] * W + k);
      }
    } else {
      for (int i = threadIdx.x; i < nk * W; i += blockDim.x) {
        const int kk = i / W, k = i % W;
        c_lds[kk * Wp + k] = cache[(int64_t)krow[kk] * W + k];
      }
    }
    __syncthreads();
    if (kb + 1 < kb_hi) key_rows(kb + 1);  // read again only after the next barrier
    const int j0 = lo + kb * LT_KB;
    // scores of the 32 keys: wave w forms the 16-key tile (w & 1) over one
    // half (w >> 1) of the feature steps; the two halves are added through
    // LDS and every wave then holds the whole 16 x 32 score block
    {
      const int u = wave & 1, hf = wave >> 1;
      const int ksh = (KS + 1) / 2;
      const int ks0 = hf * ksh, ks1 = min(KS, ks0 + ksh);
      f32x4_t sp = {0.f, 0.f, 0.f, 0.f};
      for (int ks = ks0; ks < ks1; ++ks) {
        const int f0 = ks * 32 + lk * 8;
        const bf16v8_t a = *reinterpret_cast<const bf16v8_t*>(q_lds + lrow * Wp + f0);
        const bf16v8_t bk = *reinterpret_cast<const bf16v8_t*>(c_lds + (u * 16 + lrow) * Wp + f0);
        sp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bk, sp, 0, 0, 0);
      }
      #pragma unroll
      for (int rr = 0; rr < 4; ++rr)
        s_lds[(hf * LT_TQ + lk * 4 + rr) * LT_KB + u * 16 + lrow] = sp[rr];
    }
    __syncthreads();
    f32x4_t s0, s1;
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int q = lk * 4 + rr;
      s0[rr] = s_lds[q * LT_KB + lrow] + s_lds[(LT_TQ + q) * LT_KB + lrow];
      s1[rr] = s_lds[q * LT_KB + 16 + lrow] + s_lds[(LT_TQ + q) * LT_KB + 16 + lrow];
    }
    float cr[4];
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int q = lk * 4 + rr;
      const int pq = HEADS ? p0 : p0 + q;
      const int ja = j0 + lrow, jb = j0 + 16 + lrow;
      const bool oka = q < nq && ja <= pq && (window <= 0 || pq - ja < window);
      const bool okb = q < nq && jb <= pq && (window <= 0 || pq - jb < window);
      const float sa = oka ? s0[rr] * scale : -INFINITY;
      const float sb = okb ? s1[rr] * scale : -INFINITY;
      float bm = fmaxf(sa, sb);
      #pragma unroll
      for (int off = 8; off > 0; off >>= 1) bm = fmaxf(bm, __shfl_xor(bm, off, SM_WAVE));
      const float mn = fmaxf(m[rr], bm);
      const float c = (mn == -INFINITY) ? 1.0f : expf(m[rr] - mn);
      const float pa = oka ? expf(sa - mn) : 0.f;
      const float pb = okb ? expf(sb - mn) : 0.f;
      float ps = pa + pb;
      #pragma unroll
      for (int off = 8; off > 0; off >>= 1) ps += __shfl_xor(ps, off, SM_WAVE);
      lsum[rr] = lsum[rr] * c + ps;
      m[rr] = mn;
      cr[rr] = c;
      p_lds[q * LT_KB + lrow] = pa;
      p_lds[q * LT_KB + 16 + lrow] = pb;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
    // weights as the A operand: row = query lrow; the MFMA's k index runs
    // over the keys lk + 4 j (any order works as long as A and B agree; this
    // one puts the four lane groups on neighbouring LDS rows of the block)
    bf16v8_t a_hi, a_lo;
    #pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float pv = p_lds[lrow * LT_KB + lk + 4 * j];
      const __bf16 hi = (__bf16)pv;
      a_hi[j] = hi;
      a_lo[j] = (__bf16)(pv - (float)hi);
    }
    #pragma unroll
    for (int i = 0; i < LC_NT; ++i) {
      const int nt = wave + 4 * i;
      if (nt < ntiles_f) {
        const int f = nt * 16 + lrow;         // padding columns of c_lds are zero
        bf16v8_t bc;
        #pragma unroll
        for (int j = 0; j < 8; ++j) {
          const bf16_t v = c_lds[(lk + 4 * j) * Wp + f];
          bc[j] = *reinterpret_cast<const __bf16*>(&v);
        }
        f32x4_t a4 = acc[i];
        #pragma unroll
        for (int rr = 0; rr < 4; ++rr) a4[rr] *= cr[rr];
        a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bc, a4, 0, 0, 0);
        a4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bc, a4, 0, 0, 0);
        acc[i] = a4;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (ksplit > 1 && wave == 0 && lrow == 0) {
    #pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int q = lk * 4 + rr;
      if (q < nq) {
        const int tq = HEADS ? t0 : t0 + q, hq = HEADS ? hd + q : hd;
        part_ml[(((int64_t)tq * H + hq) * ksplit + blockIdx.z) * 2] = m[rr];
        part_ml[(((int64_t)tq * H + hq) * ksplit + blockIdx.z) * 2 + 1] = lsum[rr];
      }
    }
  }
  float fin[4];
  #pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int q = lk * 4 + rr;
    fin[rr] = 0.f;
    if (q < nq && ksplit <= 1)
      fin[rr] = lat_close(m[rr], lsum[rr], sink, gate, ldg, HEADS ? t0 : t0 + q,
                          HEADS ? hd + q : hd);
  }
  #pragma unroll
  for (int i = 0; i < LC_NT; ++i) {
    const int nt = wave + 4 * i;
    const int f = nt * 16 + lrow;
    if (nt < ntiles_f && f < r) {
      #pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const int q = lk * 4 + rr;
        if (q < nq) {
          const int tq = HEADS ? t0 : t0 + q, hq = HEADS ? hd + q : hd;
          if (ksplit > 1)
            part_acc[(((int64_t)tq * H + hq) * ksplit + blockIdx.z) * r + f] = acc[i][rr];
          else
            out[((int64_t)hq * Tn + tq) * r + f] = __float2bfloat16(acc[i][rr] * fin[rr]);
        }
      }
    }
  }
}

// Merge the key splits of one (token, head): out = sum_z acc_z e^(m_z - M) / L.
__global__ __launch_bounds__(256) void latent_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    int Tn, int H, int r, int ksplit, bf16_t* __restrict__ out,
    const float* __restrict__ sink, const bf16_t* __restrict__ gate, int64_t ldg) {
  const int t = blockIdx.x / H, hd = blockIdx.x % H;
  const float* ml = part_ml + (int64_t)blockIdx.x * ksplit * 2;
  float M = -INFINITY;
  for (int z = 0; z < ksplit; ++z) M = fmaxf(M, ml[z * 2]);
  float L = 0.f;
  for (int z = 0; z < ksplit; ++z)
    if (ml[z * 2] != -INFINITY) L += ml[z * 2 + 1] * expf(ml[z * 2] - M);
  const float invL = lat_close(M, L, sink, gate, ldg, t, hd);
  for (int f = threadIdx.x; f < r; f += blockDim.x) {
    float a = 0.f;
    for (int z = 0; z < ksplit; ++z)
      if (ml[z * 2] != -INFINITY)
        a += part_acc[((int64_t)blockIdx.x * ksplit + z) * r + f] * expf(ml[z * 2] - M);
    out[((int64_t)hd * Tn + t) * r + f] = __float2bfloat16(a * invL);
  }
}

}  // namespace

torch::Tensor latent_prepare(torch::Tensor q, c10::optional<torch::Tensor> dkv, int64_t heads,
                             int64_t dim, int64_t rot_dim, int64_t kv_rank,
                             c10::optional<torch::Tensor> norm_w, double eps,
                             torch::Tensor positions, double rope_base,
                             int64_t rope_dims, torch::Tensor page_slot,
                             torch::Tensor cache, c10::optional<torch::Tensor> freqs,
                             double mag, bool pairs) {
  SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  SM_CHECK_CUDA(page_slot); SM_CHECK_I32(page_slot); SM_CHECK_CUDA(cache);
  const int64_t T = q.size(0);
  const int64_t qs = heads * (dim + rot_dim);
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.stride(1) == 1 && q.size(1) == qs,
              "latent_prepare: query rows");
  TORCH_CHECK(rope_dims % 2 == 0 && rope_dims <= rot_dim, "latent_prepare: rope dims");
  TORCH_CHECK(positions.numel() == T && page_slot.numel() == T, "latent_prepare: batch layout");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == kv_rank + rot_dim &&
              cache.scalar_type() == q.scalar_type(), "latent_prepare: cache shape/dtype");
  const float* nw = nullptr;
  const void* dp = nullptr;
  int64_t ldd = 0;
  if (dkv.has_value()) {
    TORCH_CHECK(dkv->is_cuda() && dkv->dim() == 2 && dkv->stride(1) == 1 && dkv->size(0) == T &&
                dkv->size(1) == kv_rank + rot_dim && dkv->scalar_type() == q.scalar_type(),
                "latent_prepare: latent rows");
    TORCH_CHECK(norm_w.has_value(), "latent_prepare: norm weight missing");
    SM_CHECK_CUDA(*norm_w); SM_CHECK_F32(*norm_w);
    TORCH_CHECK(norm_w->numel() == kv_rank, "latent_prepare: norm weight size");
    nw = norm_w->data_ptr<float>();
    dp = dkv->data_ptr();
    ldd = dkv->stride(0);
  }
  const float* fp = nullptr;
  if (freqs.has_value()) {
    SM_CHECK_CUDA(*freqs); SM_CHECK_F32(*freqs);
    TORCH_CHECK(freqs->numel() == rope_dims / 2, "latent_prepare: one frequency per pair");
    fp = freqs->data_ptr<float>();
  } else {
    TORCH_CHECK(!pairs && mag == 1.0, "latent_prepare: pair layout and scaling need a frequency table");
  }
  auto q_rot = torch::empty({T, heads, rot_dim}, q.options().dtype(at::kFloat));
  if (T == 0) return q_rot;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (q.scalar_type() == at::kBFloat16)
    latent_prepare_kernel<bf16_t><<<T, 256, 0, stream>>>(
        reinterpret_cast<const bf16_t*>(q.data_ptr()), q.stride(0),
        reinterpret_cast<const bf16_t*>(dp), ldd, heads, dim, rot_dim, kv_rank, nw, (float)eps,
        positions.data_ptr<int>(), (float)rope_base, (int)rope_dims, fp, (float)mag, pairs ? 1 : 0,
        page_slot.data_ptr<int>(), reinterpret_cast<bf16_t*>(cache.data_ptr()),
        q_rot.data_ptr<float>());
  else {
    SM_CHECK_F32(q);
    latent_prepare_kernel<float><<<T, 256, 0, stream>>>(
        q.data_ptr<float>(), q.stride(0), reinterpret_cast<const float*>(dp), ldd, heads, dim,
        rot_dim, kv_rank, nw, (float)eps, positions.data_ptr<int>(), (float)rope_base,
        (int)rope_dims, fp, (float)mag, pairs ? 1 : 0, page_slot.data_ptr<int>(),
        cache.data_ptr<float>(), q_rot.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return q_rot;
}

torch::Tensor latent_window_attention(torch::Tensor q_lat, torch::Tensor q_rot,
                                      torch::Tensor cache, int64_t kv_rank,
                                      torch::Tensor block_tables, int64_t block_size,
                                      torch::Tensor tok_seq, torch::Tensor positions,
                                      int64_t window, double scale,
                                      c10::optional<torch::Tensor> tiles,
                                      int64_t max_tile_queries,
                                      c10::optional<torch::Tensor> sink,
                                      c10::optional<torch::Tensor> gate) {
  SM_CHECK_CUDA(q_lat); SM_CHECK_CUDA(q_rot); SM_CHECK_F32(q_rot); SM_CHECK_CUDA(cache);
  SM_CHECK_CUDA(block_tables); SM_CHECK_I32(block_tables);
  SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq); SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  TORCH_CHECK(q_lat.dim() == 3 && q_rot.dim() == 3 && block_tables.dim() == 2, "latent attention: ranks");
  const int H = q_lat.size(0);
  const int64_t T = q_lat.size(1);
  const int r = q_lat.size(2);
  const int rd = q_rot.size(2);
  TORCH_CHECK(r == kv_rank && r <= 64 * SM_LAT_REGS, "latent attention: kv_rank unsupported");
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H, "latent attention: q_rot shape");
  TORCH_CHECK(cache.size(1) == r + rd && cache.scalar_type() == q_lat.scalar_type(),
              "latent attention: cache shape/dtype");
  TORCH_CHECK(tok_seq.numel() == T && positions.numel() == T && block_size > 0, "latent attention: batch layout");
  const float* sinkp = nullptr;
  const void* gatep = nullptr;
  int64_t ldg = 0;
  if (sink.has_value()) {
    SM_CHECK_CUDA(*sink); SM_CHECK_F32(*sink);
    TORCH_CHECK(sink->numel() == H, "latent attention: one sink per head");
    sinkp = sink->data_ptr<float>();
  }
  if (gate.has_value()) {
    TORCH_CHECK(gate->is_cuda() && gate->dim() == 2 && gate->stride(1) == 1 && gate->size(0) == T &&
                gate->size(1) == H && gate->scalar_type() == q_lat.scalar_type(),
                "latent attention: gate is [T, H] in the model dtype");
    gatep = gate->data_ptr();
    ldg = gate->stride(0);
  }
  const bf16_t* gateb = reinterpret_cast<const bf16_t*>(gatep);
  auto out = torch::empty_like(q_lat);
  if (T == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  const size_t lds = (size_t)(r + rd + 64) * sizeof(float) + 64 * sizeof(int);
  if (q_lat.scalar_type() == at::kBFloat16 && tiles.has_value() && r <= 512) {
    // tiled MFMA path
    SM_CHECK_CUDA(*tiles); SM_CHECK_I32(*tiles);
    TORCH_CHECK(tiles->dim() == 2 && tiles->size(1) == 3, "latent attention: tiles shape");
    TORCH_CHECK(max_tile_queries >= 1 && max_tile_queries <= LT_TQ, "latent attention: tile size");
    const int ntiles = tiles->size(0);
    const int W = r + rd;
    const int Wp = ((W + 31) / 32) * 32 + 8;
    // decode-only batches (one query per row): a tile is one token with up
    // to 16 of its heads, and four waves split its keys
    const bool heads = max_tile_queries == 1 && H > 1;
    if (!heads && max_tile_queries > 4) {
      // prompt portions: the four-wave all-MFMA kernel
      const size_t ldsc = (size_t)(LT_TQ + LT_KB) * LC_ROW(W) * 2 + 6 * LT_TQ * LT_KB * 4;
      if (ldsc <= 78 * 1024) {              // two workgroups per CU
        static int raised = 0;
        if ((int)ldsc > raised) {
          TORCH_CHECK(hipFuncSetAttribute(
                          reinterpret_cast<const void*>(latent_attention_coop_kernel<false>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsc) == hipSuccess,
                      "latent attention: cannot raise the LDS limit");
          raised = (int)ldsc;
        }
        latent_attention_coop_kernel<false><<<dim3(ntiles, H), 256, ldsc, stream>>>(
            reinterpret_cast<const bf16_t*>(q_lat.data_ptr()), q_rot.data_ptr<float>(),
            reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),
            (int)block_tables.size(1), (int)block_size, tiles->data_ptr<int>(),
            positions.data_ptr<int>(), (int)T, H, r, rd, (int)window, (float)scale,
            reinterpret_cast<bf16_t*>(out.data_ptr()), 1, nullptr, nullptr, sinkp, gateb, ldg);
        SM_CHECK_LAUNCH();
        return out;
      }
    }
    if (heads) {
      // decoding: one token x up to 16 heads per workgroup, the key blocks
      // spread over blockIdx.z, merged by latent_combine
      const size_t ldsc = (size_t)(LT_TQ + LT_KB) * LC_ROW(W) * 2 + 6 * LT_TQ * LT_KB * 4;
      if (ldsc <= 78 * 1024) {
        static int raised = 0;
        if ((int)ldsc > raised) {
          TORCH_CHECK(hipFuncSetAttribute(
                          reinterpret_cast<const void*>(latent_attention_coop_kernel<true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsc) == hipSuccess,
                      "latent attention: cannot raise the LDS limit");
          raised = (int)ldsc;
        }
        const int64_t groups = (int64_t)ntiles * SM_CDIV(H, LT_TQ);
        int ks = (int)std::min<int64_t>(32, std::max<int64_t>(1, 1024 / groups));
        if (window > 0) ks = (int)std::min<int64_t>(ks, SM_CDIV(window, LT_KB) + 1);
        torch::Tensor pa, pm;
        float *pap = nullptr, *pmp = nullptr;
        if (ks > 1) {
          pa = torch::empty({T, H, ks, r}, q_rot.options());
          pm = torch::empty({T, H, ks, 2}, q_rot.options());
          pap = pa.data_ptr<float>();
          pmp = pm.data_ptr<float>();
        }
        latent_attention_coop_kernel<true><<<dim3(ntiles, SM_CDIV(H, LT_TQ), ks), 256, ldsc, stream>>>(
            reinterpret_cast<const bf16_t*>(q_lat.data_ptr()), q_rot.data_ptr<float>(),
            reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),
            (int)block_tables.size(1), (int)block_size, tiles->data_ptr<int>(),
            positions.data_ptr<int>(), (int)T, H, r, rd, (int)window, (float)scale,
            reinterpret_cast<bf16_t*>(out.data_ptr()), ks, pap, pmp, sinkp, gateb, ldg);
        SM_CHECK_LAUNCH();
        if (ks > 1) {
          latent_combine_kernel<<<(int)(T * H), 256, 0, stream>>>(
              pap, pmp, (int)T, H, r, ks, reinterpret_cast<bf16_t*>(out.data_ptr()), sinkp, gateb,
              ldg);
          SM_CHECK_LAUNCH();
        }
        return out;
      }
    }
    const int NW = (heads || (max_tile_queries <= 4 && (int64_t)ntiles * H < 4096)) ? 4 : 1;
    const int nq_cap = heads ? LT_TQ : (int)max_tile_queries;
    size_t lds2 = (size_t)LT_TQ * Wp * 2 + (size_t)NW * (LT_TQ * LT_KB + LT_KB + LT_TQ) * 4 +
                  (size_t)NW * LT_TQ * 2 * 4 + (size_t)(NW - 1) * nq_cap * r * 4;
    TORCH_CHECK(lds2 <= 150 * 1024, "latent attention: tile does not fit in LDS");
    // decode: enough key splits to fill the chip, at most one per wave pass
    int ksplit = 1;
    torch::Tensor part_acc, part_ml;
    float *pacc = nullptr, *pml = nullptr;
    if (heads) {
      const int64_t groups = (int64_t)ntiles * SM_CDIV(H, LT_TQ);
      ksplit = (int)std::min<int64_t>(16, std::max<int64_t>(1, 512 / groups));
      if (window > 0)
        ksplit = (int)std::min<int64_t>(ksplit, std::max<int64_t>(1, SM_CDIV(window, LT_KB * NW)));
      if (ksplit > 1) {
        part_acc = torch::empty({T, H, ksplit, r}, q_rot.options());
        part_ml = torch::empty({T, H, ksplit, 2}, q_rot.options());
        pacc = part_acc.data_ptr<float>();
        pml = part_ml.data_ptr<float>();
      }
    }
    dim3 g2(ntiles, heads ? SM_CDIV(H, LT_TQ) : H, ksplit);
    #define LT_LAUNCH(RPL, HD)                                                          \
      do {                                                                              \
        auto kern = latent_attention_tiled_kernel<RPL, HD>;                             \
        static int raised = 0;     /* per kernel variant; not repeated under graph capture */ \
        if (lds2 > 64 * 1024 && (int)lds2 > raised) {                                   \
          TORCH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),          \
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2) == hipSuccess, \
                      "latent attention: cannot raise the LDS limit");                  \
          raised = (int)lds2;                                                           \
        }                                                                               \
        kern<<<g2, 64 * NW, lds2, stream>>>(                                            \
          reinterpret_cast<const bf16_t*>(q_lat.data_ptr()), q_rot.data_ptr<float>(),   \
          reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(), \
          (int)block_tables.size(1), (int)block_size, tiles->data_ptr<int>(),            \
          positions.data_ptr<int>(), (int)T, H, r, rd, (int)window, (float)scale, nq_cap, \
          reinterpret_cast<bf16_t*>(out.data_ptr()), ksplit, pacc, pml, sinkp, gateb, ldg); \
      } while (0)
    if (heads) {
      if (r <= 128) LT_LAUNCH(2, true);
      else if (r <= 256) LT_LAUNCH(4, true);
      else LT_LAUNCH(8, true);
    } else {
      if (r <= 128) LT_LAUNCH(2, false);
      else if (r <= 256) LT_LAUNCH(4, false);
      else LT_LAUNCH(8, false);
    }
    #undef LT_LAUNCH
    if (ksplit > 1) {
      SM_CHECK_LAUNCH();
      latent_combine_kernel<<<(int)(T * H), 256, 0, stream>>>(
          pacc, pml, (int)T, H, r, ksplit, reinterpret_cast<bf16_t*>(out.data_ptr()), sinkp, gateb,
          ldg);
    }
    SM_CHECK_LAUNCH();
    return out;
  }
  dim3 grid(T, H);
  if (q_lat.scalar_type() == at::kBFloat16)
    latent_attention_kernel<bf16_t><<<grid, 64, lds, stream>>>(
        reinterpret_cast<const bf16_t*>(q_lat.data_ptr()), q_rot.data_ptr<float>(),
        reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),
        (int)block_tables.size(1), (int)block_size, tok_seq.data_ptr<int>(),
        positions.data_ptr<int>(), (int)T, H, r, rd, (int)window, (float)scale, sinkp, gateb, ldg,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else {
    SM_CHECK_F32(q_lat);
    latent_attention_kernel<float><<<grid, 64, lds, stream>>>(
        q_lat.data_ptr<float>(), q_rot.data_ptr<float>(), cache.data_ptr<float>(),
        block_tables.data_ptr<int>(), (int)block_tables.size(1), (int)block_size,
        tok_seq.data_ptr<int>(), positions.data_ptr<int>(), (int)T, H, r, rd,
        (int)window, (float)scale, sinkp, reinterpret_cast<const float*>(gatep), ldg,
        out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}
