// Tiled MFMA form of the windowed softmax attention for bf16 prompt portions.
//
// One workgroup (4 waves) per (tile of <= 64 consecutive queries of one
// sequence, query head); wave w owns queries 16 w .. 16 w + 15: their scores,
// their online softmax and their value sums. The keys a tile can see are one
// list: the kept first tokens that lie before the window of the tile's first
// query, then everything from that window's start to the tile's last query;
// the list is walked in blocks of KB keys (64; 32 for the wide key rows of
// folded queries, so that more than one workgroup fits a CU) whose key columns
// (the head's kv head, or the whole key row for folded queries) and V rows
// (transposed) are staged in LDS once per tile.
//   scores   MFMA 16x16x32: A = the wave's queries (registers, loaded once),
//            B = K rows from LDS
//   softmax  fp32 in the MFMA's result layout; distance bias and mask per
//            score; row reductions over the 16 lanes of a row by lane
//            permutes. The distance bias depends on (head, distance) only and
//            a wave's 16 queries meet a block's keys at KB + 15 distances:
//            the wave tabulates those once per block instead of taking a
//            logarithm per score
//   values   the fp32 weights go through a wave-private LDS tile to the A
//            layout and are split into two bf16 terms (p = hi + lo, error
//            <= 2^-17 p); B = V^T from LDS; fp32 accumulation
// The output gate's sigmoid multiplies the row where the softmax is closed.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16v8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {

// NT: 16-column value tiles per wave (vd <= 16 NT); KS: 32-entry steps of the
// query/key dot product held in registers (KD <= 32 KS); KB: keys per block;
// DIST: the distance bias is taken off the scores (r1, r2 given).
template <int NT, int KS, int KB, bool DIST>
__global__ __launch_bounds__(256, 2) void window_attention_mfma_kernel(
    const bf16_t* __restrict__ q, int KD,  // [Tn, H, KD]
    const bf16_t* __restrict__ cache,      // [rows, G (dk + vd)]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ positions,
    const int* __restrict__ tiles,         // [ntiles, 3] = (batch row, first token, queries)
    int H, int G, int dk, int vd, int whole_key, float scale, int window, int keep,
    const float* __restrict__ r1, const float* __restrict__ r2,
    const bf16_t* __restrict__ gate, int64_t ldg,
    bf16_t* __restrict__ out) {            // [Tn, H vd]
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int ksteps = (KD + 31) / 32;
  const int KP = ksteps * 32 + 8;                  // k_lds row pitch (bf16)
  const int NVp = (vd + 15) / 16 * 16;
  constexpr int WAM_KB = KB;
  constexpr int WAM_VP = KB + 8;                   // v_lds row pitch (bf16)
  constexpr int WAM_PP = KB + 4;                   // p_lds row pitch (floats)
  constexpr int WAM_TB = KB + 16;                  // distance-bias table per wave
  bf16_t* k_lds = reinterpret_cast<bf16_t*>(smem);                 // [KB][KP]
  bf16_t* v_lds = k_lds + WAM_KB * KP;                             // [NVp][WAM_VP]
  float* p_all = reinterpret_cast<float*>(v_lds + NVp * WAM_VP);   // [4][16][WAM_PP]
  int* krow = reinterpret_cast<int*>(p_all + 4 * 16 * WAM_PP);     // [KB]
  float* tb_all = reinterpret_cast<float*>(krow + KB);             // [4][WAM_TB], DIST only

  const int tile = blockIdx.x, hd = blockIdx.y;
  const int b = tiles[3 * tile], t0 = tiles[3 * tile + 1], nq = tiles[3 * tile + 2];
  const int tid = threadIdx.x, l = tid & 63, lrow = l & 15, lk = l >> 4;
  const int wave = tid >> 6;
  const int W = G * (dk + vd);
  const int grp = hd / (H / G);
  const int koff = whole_key ? 0 : grp * dk, voff = G * dk + grp * vd;
  const int p0 = positions[t0], plast = p0 + nq - 1;
  const int lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
  const int nf = (window > 0) ? min(keep, lo) : 0; // kept keys before the first window
  const int n = nf + (plast - lo + 1);             // keys in the tile's list
  const int nblk = (n + WAM_KB - 1) / WAM_KB;
  const int* bt = block_tables + (int64_t)b * max_nb;
  float* p_lds = p_all + wave * 16 * WAM_PP;
  float* tb = tb_all + wave * WAM_TB;
  const bool active = wave * 16 < nq;
  const float a1 = DIST ? r1[hd] : 0.f, a2 = DIST ? r2[hd] : 0.f;

  // the wave's queries as A fragments: row lrow, k = ks * 32 + lk * 8 ..
  bf16v8 qf[KS];
  {
    const int qi = wave * 16 + lrow;
    const bf16_t* qp = q + ((int64_t)(t0 + min(qi, nq - 1)) * H + hd) * KD;
    #pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      #pragma unroll
      for (int j = 0; j < 8; ++j) qf[ks][j] = (__bf16)0.0f;
      const int kk = ks * 32 + lk * 8;
      if (ks < ksteps && qi < nq && kk < KD) qf[ks] = *reinterpret_cast<const bf16v8*>(qp + kk);
    }
  }
  // padding rows of v_lds (value columns vd .. NVp) stay zero
  for (int i = tid; i < (NVp - vd) * WAM_VP; i += 256) v_lds[vd * WAM_VP + i] = __float2bfloat16(0.f);

  float m[4], lsum[4];
  f32x4 acc[NT];
  #pragma unroll
  for (int r = 0; r < 4; ++r) { m[r] = -INFINITY; lsum[r] = 0.f; }
  #pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kb = 0; kb < nblk; ++kb) {
    const int i0 = kb * WAM_KB;
    __syncthreads();                               // the previous block's LDS reads are done
    if (tid < WAM_KB) {
      const int i = min(i0 + tid, n - 1);          // list entries past the end are masked below
      const int j = (i < nf) ? i : lo + (i - nf);
      krow[tid] = bt[j / block_size] * block_size + j % block_size;
    }
    __syncthreads();
    // key columns: [key][KD], zero beyond KD
    for (int i = tid; i < WAM_KB * ksteps * 4; i += 256) {
      const int key = i / (ksteps * 4), c = (i % (ksteps * 4)) * 8;
      bf16v8 v;
      if (c < KD) {
        v = *reinterpret_cast<const bf16v8*>(cache + (int64_t)krow[key] * W + koff + c);
      } else {
        #pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (__bf16)0.0f;
      }
      *reinterpret_cast<bf16v8*>(k_lds + key * KP + c) = v;
    }
    // V rows, transposed: v_lds[column][key]
    for (int i = tid; i < WAM_KB * (vd / 8); i += 256) {
      const int key = i % WAM_KB, c = (i / WAM_KB) * 8;
      const bf16v8 v = *reinterpret_cast<const bf16v8*>(cache + (int64_t)krow[key] * W + voff + c);
      #pragma unroll
      for (int j = 0; j < 8; ++j)
        *reinterpret_cast<__bf16*>(v_lds + (c + j) * WAM_VP + key) = v[j];
    }
    __syncthreads();
    if (!active) continue;
    // a block of the window part that starts after the wave's last query, or
    // ends before the window of its first query, holds nothing the wave sees
    if (i0 >= nf) {
      const int jb0 = lo + (i0 - nf);
      const int wq_last = min(plast, p0 + wave * 16 + 15), wq_first = p0 + wave * 16;
      if (jb0 > wq_last) continue;
      if (window > 0 && jb0 + WAM_KB - 1 < wq_first - window + 1 && jb0 >= keep) continue;
    }

    // distance bias of this wave and block: the block's keys are consecutive
    // positions jb0 .. jb0 + KB - 1 once the list is past the kept tokens, and
    // tb[(query - 16 wave) + (KB - 1 - key column)] covers every pair
    const bool tabled = DIST && i0 >= nf;
    if (DIST && tabled) {
      const int dbase = p0 + wave * 16 - (lo + (i0 - nf)) - (KB - 1);
      for (int i = l; i < KB + 15; i += 64)
        tb[i] = a1 * log1pf(a2 * (float)max(dbase + i, 0));
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_s_waitcnt(0xc07f);
    }

    f32x4 s[KB / 16];
    #pragma unroll
    for (int ct = 0; ct < KB / 16; ++ct) {
      s[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
      #pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks < ksteps) {
          const bf16v8 kf = *reinterpret_cast<const bf16v8*>(
              k_lds + (ct * 16 + lrow) * KP + ks * 32 + lk * 8);
          s[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, s[ct], 0, 0, 0);
        }
      }
    }
    // result layout: reg r -> query lk * 4 + r, lane column lrow -> key ct * 16 + lrow
    float cr[4];
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int qi = wave * 16 + lk * 4 + r;
      const int prow = (qi < nq) ? p0 + qi : -1;
      float sv[KB / 16];
      float bm = -INFINITY;
      #pragma unroll
      for (int ct = 0; ct < KB / 16; ++ct) {
        const int i = i0 + ct * 16 + lrow;
        const int j = (i < nf) ? i : lo + (i - nf);
        const bool seen = i < n && j <= prow && (window <= 0 || prow - j < window || j < keep);
        float x = s[ct][r] * scale;
        if (DIST) {
          if (tabled) x -= tb[lk * 4 + r + (KB - 1) - (ct * 16 + lrow)];
          else if (seen) x -= a1 * log1pf(a2 * (float)(prow - j));
        }
        sv[ct] = seen ? x : -INFINITY;
        bm = fmaxf(bm, sv[ct]);
      }
      bm = sm_row16_max(bm);
      const float mn = fmaxf(m[r], bm);
      const float c = (mn == -INFINITY) ? 1.0f : expf(m[r] - mn);
      float ps = 0.f;
      #pragma unroll
      for (int ct = 0; ct < KB / 16; ++ct) {
        const float pv = (sv[ct] == -INFINITY) ? 0.f : expf(sv[ct] - mn);
        ps += pv;
        p_lds[(lk * 4 + r) * WAM_PP + ct * 16 + lrow] = pv;
      }
      ps = sm_row16_sum(ps);
      lsum[r] = lsum[r] * c + ps;
      m[r] = mn;
      cr[r] = c;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
    // weights as A fragments: row lrow, keys ks2 * 32 + lk * 8 ..
    bf16v8 a_hi[KB / 32], a_lo[KB / 32];
    #pragma unroll
    for (int ks2 = 0; ks2 < KB / 32; ++ks2) {
      const float4 w0 = *reinterpret_cast<const float4*>(p_lds + lrow * WAM_PP + ks2 * 32 + lk * 8);
      const float4 w1 = *reinterpret_cast<const float4*>(p_lds + lrow * WAM_PP + ks2 * 32 + lk * 8 + 4);
      const float pv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      #pragma unroll
      for (int j = 0; j < 8; ++j) {
        const __bf16 hi = (__bf16)pv[j];
        a_hi[ks2][j] = hi;
        a_lo[ks2][j] = (__bf16)(pv[j] - (float)hi);
      }
    }
    #pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (nt * 16 < vd) {
        f32x4 a = acc[nt];
        #pragma unroll
        for (int r = 0; r < 4; ++r) a[r] *= cr[r];
        #pragma unroll
        for (int ks2 = 0; ks2 < KB / 32; ++ks2) {
          const bf16v8 vf = *reinterpret_cast<const bf16v8*>(
              v_lds + (nt * 16 + lrow) * WAM_VP + ks2 * 32 + lk * 8);
          a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi[ks2], vf, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo[ks2], vf, a, 0, 0, 0);
        }
        acc[nt] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();               // p_lds is rewritten in the next block
  }

  if (!active) return;
  #pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int qi = wave * 16 + lk * 4 + r;
    if (qi >= nq) continue;
    float f = 1.0f / lsum[r];
    if (gate != nullptr) f *= sm_sigmoid(__bfloat162float(gate[(int64_t)(t0 + qi) * ldg + hd]));
    bf16_t* dst = out + ((int64_t)(t0 + qi) * H + hd) * vd;
    #pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int col = nt * 16 + lrow;
      if (col < vd) dst[col] = __float2bfloat16(acc[nt][r] * f);
    }
  }
}

#define WAM_KEYS 32   // keys per block

size_t wam_lds_bytes(int KD, int vd, bool dist) {
  const int ksteps = (KD + 31) / 32, KP = ksteps * 32 + 8, NVp = (vd + 15) / 16 * 16;
  const int KB = WAM_KEYS;
  return (size_t)KB * KP * 2 + (size_t)NVp * (KB + 8) * 2 + 4 * 16 * (KB + 4) * 4 + KB * 4 +
         (dist ? 4 * (KB + 16) * 4 : 0);
}

}  // namespace

// 16-byte pieces of the cache rows: the key columns a head meets (dim, or
// kv_heads * dim for folded queries) and the value size are multiples of 8
bool window_attention_mfma_fits(int KD, int vd) {
  return KD % 8 == 0 && vd % 8 == 0 && KD <= 512 && vd <= 256 &&
         wam_lds_bytes(KD, vd, true) <= 150 * 1024;
}

void window_attention_mfma(torch::Tensor q, int KD, torch::Tensor cache, int H, int G, int dk, int vd,
                           int whole_key, torch::Tensor block_tables, int block_size,
                           torch::Tensor positions, float scale, int window, int keep,
                           const float* r1, const float* r2, const void* gate, int64_t ldg,
                           torch::Tensor tiles, torch::Tensor out) {
  const int ntiles = tiles.size(0);
  if (q.size(0) == 0 || ntiles == 0) return;
  auto stream = at::cuda::getCurrentCUDAStream();
  const size_t lds = wam_lds_bytes(KD, vd, r1 != nullptr);
  dim3 grid(ntiles, H);
#define WAM_LAUNCH(NT, KS, KB, DIST)                                                           \
  do {                                                                                         \
    auto kern = window_attention_mfma_kernel<NT, KS, KB, DIST>;                                        \
    static int raised = 0;                                                                     \
    if (lds > 64 * 1024 && (int)lds > raised) {                                                \
      TORCH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                     \
                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,     \
                  "window attention: cannot raise the LDS limit");                             \
      raised = (int)lds;                                                                       \
    }                                                                                          \
    kern<<<grid, 256, lds, stream>>>(                                                          \
        reinterpret_cast<const bf16_t*>(q.data_ptr()), KD,                                     \
        reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),       \
        (int)block_tables.size(1), block_size, positions.data_ptr<int>(), tiles.data_ptr<int>(), \
        H, G, dk, vd, whole_key, scale, window, keep, r1, r2,                                  \
        reinterpret_cast<const bf16_t*>(gate), ldg, reinterpret_cast<bf16_t*>(out.data_ptr())); \
  } while (0)
#define WAM_BY_KS(NT, DIST)                            \
  do {                                                 \
    if (KD <= 128) WAM_LAUNCH(NT, 4, WAM_KEYS, DIST);        \
    else if (KD <= 256) WAM_LAUNCH(NT, 8, WAM_KEYS, DIST);   \
    else WAM_LAUNCH(NT, 16, WAM_KEYS, DIST);                 \
  } while (0)
#define WAM_BY_NT(DIST)                                \
  do {                                                 \
    if (vd <= 64) WAM_BY_KS(4, DIST);                  \
    else if (vd <= 128) WAM_BY_KS(8, DIST);            \
    else WAM_BY_KS(16, DIST);                          \
  } while (0)
  if (r1 != nullptr) WAM_BY_NT(true);
  else WAM_BY_NT(false);
#undef WAM_BY_NT
#undef WAM_BY_KS
#undef WAM_LAUNCH
  SM_CHECK_LAUNCH();
}
