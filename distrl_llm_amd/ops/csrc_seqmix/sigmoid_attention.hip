// Sigmoid attention over paged [k | v] rows: grouped-query attention whose
// weights are sigmoid(q.k * scale - slope_h (i - j) + bias_h), not normalised
// over the keys, under a sliding window that also keeps the first tokens.
//   qk_norm_kv_write   per token: RMS norm of every q and k head over the head
//                      size (plain shared weights), page write of [k | v]
//   sigmoid_attention_group  decode steps: one workgroup per (token, kv
//                      head, share of the keys) serves every query head of the
//                      kv head, so a K/V row is read once for all of them
//   sigmoid_attention  one wave per (token, head): any shape, the fallback
// (the tiled MFMA kernel for bf16 prompt portions is in
// sigmoid_attention_mfma.hip)
// A query at position p sees the keys [0, min(keep, lo)) and [lo, p] with
// lo = max(0, p - window + 1); the kernels walk the two ranges as one list.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

namespace {

// One workgroup per token; a wave takes q heads, then k heads, in turn.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_kv_write_kernel(
    const T* __restrict__ proj, int64_t ldp, int H, int G, int dk, int vd,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const int* __restrict__ page_slot, T* __restrict__ cache, T* __restrict__ q_out) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = proj + t * ldp;
  T* dst = cache + (int64_t)page_slot[t] * ((int64_t)G * (dk + vd));
  for (int job = wave; job < H + G; job += 4) {
    const bool is_k = job >= H;
    const T* src = row + (int64_t)job * dk;          // q heads, then k heads
    float ss = 0.f;
    for (int k = lane; k < dk; k += 64) {
      const float v = to_f(src[k]);
      ss += v * v;
    }
    ss = sm_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)dk + eps);
    const float* w = is_k ? kw : qw;
    T* o = is_k ? dst + (job - H) * dk : q_out + (t * H + job) * dk;
    for (int k = lane; k < dk; k += 64) o[k] = from_f<T>(to_f(src[k]) * inv * w[k]);
  }
  const T* v = row + (int64_t)(H + G) * dk;
  for (int k = threadIdx.x; k < G * vd; k += blockDim.x) dst[G * dk + k] = v[k];
}

#define SG_REGS 8   // value entries per lane: vdim <= 512
template <typename T>
__global__ __launch_bounds__(64) void sigmoid_attention_kernel(
    const T* __restrict__ q,          // [Tn, H, dk]
    const T* __restrict__ cache,      // [rows, G dk + G vd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int H, int G,
    int dk, int vd, float scale, int window, int keep,
    const float* __restrict__ slopes, const float* __restrict__ pos_bias,
    T* __restrict__ out) {            // [Tn, H vd]
  extern __shared__ float lds[];
  float* qs = lds;                                   // dk
  float* pw = lds + dk;                              // 64 weights
  int* krow = reinterpret_cast<int*>(pw + 64);       // 64 cache rows
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const int g = hd / (H / G);
  const int64_t W = (int64_t)G * (dk + vd);
  for (int k = lane; k < dk; k += 64) qs[k] = to_f(q[((int64_t)t * H + hd) * dk + k]);
  const int b = tok_seq[t], p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int nfirst = (window > 0) ? min(keep, lo) : 0;
  const int n = nfirst + (p - lo + 1);
  const int* bt = block_tables + (int64_t)b * max_nb;
  const float slope = slopes[hd], bias = pos_bias[hd];
  float acc[SG_REGS];
  #pragma unroll
  for (int i = 0; i < SG_REGS; ++i) acc[i] = 0.f;
  __syncthreads();
  for (int i0 = 0; i0 < n; i0 += 64) {
    const int i = i0 + lane;
    float w = 0.f;
    int row = 0;
    if (i < n) {
      const int j = (i < nfirst) ? i : lo + (i - nfirst);
      row = bt[j / block_size] * block_size + j % block_size;
      const T* kp = cache + (int64_t)row * W + g * dk;
      float dot = 0.f;
      for (int k = 0; k < dk; ++k) dot = fmaf(qs[k], to_f(kp[k]), dot);
      w = sm_sigmoid(dot * scale - slope * (float)(p - j) + bias);
    }
    __syncthreads();
    pw[lane] = w;
    krow[lane] = row;
    __syncthreads();
    const int nk = min(64, n - i0);
    #pragma unroll
    for (int r = 0; r < SG_REGS; ++r) {
      const int d = lane + 64 * r;
      if (d < vd) {
        float a = acc[r];
        for (int jj = 0; jj < nk; ++jj)
          a = fmaf(pw[jj], to_f(cache[(int64_t)krow[jj] * W + G * dk + g * vd + d]), a);
        acc[r] = a;
      }
    }
  }
  #pragma unroll
  for (int r = 0; r < SG_REGS; ++r) {
    const int d = lane + 64 * r;
    if (d < vd) out[((int64_t)t * H + hd) * vd + d] = from_f<T>(acc[r]);
  }
}

// ---- decode steps. One workgroup (4 waves) per (token, kv head g, key
// share z). The REP query heads of g sit in LDS as fp32; the visible keys (one
// list: kept first tokens before the window, then the window) are cut into
// blocks of 64, share z takes a contiguous run of blocks and its waves take
// them in turn. Per block: lane = key, the K row is read once in 16-byte
// pieces and dotted with all REP queries; the REP x 64 fp32 weights go through
// a wave-private LDS tile; then lane = pair of value columns, and every V row
// is read once (coalesced) for all REP heads. The waves' sums meet in LDS.
// Sigmoid weights are final as they are, so shares just add: with ksplit > 1
// the workgroup leaves an fp32 partial and sigmoid_attention_sum adds them in
// a fixed order.
#define SGG_CP 2     // value column pairs per lane: vdim <= 256
template <typename T> struct sg_vec;
template <> struct sg_vec<bf16_t> {
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
template <> struct sg_vec<float> {
  static constexpr int N = 4;
  SM_INLINE static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
  SM_INLINE static float2 load2(const float* p) { return *reinterpret_cast<const float2*>(p); }
};

template <typename T, int REP>
__global__ __launch_bounds__(256) void sigmoid_attention_group_kernel(
    const T* __restrict__ q,          // [Tn, H, dk]
    const T* __restrict__ cache,      // [rows, G dk + G vd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int H, int G,
    int dk, int vd, float scale, int window, int keep,
    const float* __restrict__ slopes, const float* __restrict__ pos_bias,
    int ksplit, float* __restrict__ part,   // [ksplit, Tn, H, vd] when ksplit > 1
    T* __restrict__ out) {                  // [Tn, H vd]
  extern __shared__ __attribute__((aligned(16))) float sgl[];
  constexpr int VN = sg_vec<T>::N;
  float* qs = sgl;                                   // [REP][dk]
  float* pw_all = qs + REP * dk;                     // [4][REP][64]
  int* krow_all = reinterpret_cast<int*>(pw_all + 4 * REP * 64);   // [4][64]
  float* red = reinterpret_cast<float*>(krow_all + 4 * 64);        // [3][REP][vd]
  const int t = blockIdx.x, g = blockIdx.y, z = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t W = (int64_t)G * (dk + vd);
  const int h0 = g * REP;
  for (int i = tid; i < REP * dk; i += 256)
    qs[i] = to_f(q[((int64_t)t * H + h0 + i / dk) * dk + i % dk]);
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
  float slope[REP], bias[REP];
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh) { slope[hh] = slopes[h0 + hh]; bias[hh] = pos_bias[h0 + hh]; }
  float acc[REP][SGG_CP][2];
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh)
    #pragma unroll
    for (int c = 0; c < SGG_CP; ++c) acc[hh][c][0] = acc[hh][c][1] = 0.f;
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
      const T* kp = cache + (int64_t)row * W + g * dk;
      for (int k = 0; k < dk; k += VN) {
        float kv[VN];
        sg_vec<T>::load(kp + k, kv);
        #pragma unroll
        for (int hh = 0; hh < REP; ++hh)
          #pragma unroll
          for (int e = 0; e < VN; ++e) s[hh] = fmaf(qs[hh * dk + k + e], kv[e], s[hh]);
      }
    }
    #pragma unroll
    for (int hh = 0; hh < REP; ++hh)
      pw[hh * 64 + lane] =
          (i < n) ? sm_sigmoid(s[hh] * scale - slope[hh] * (float)(p - j) + bias[hh]) : 0.f;
    krow[lane] = row;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);              // the wave's LDS writes have landed
    const int nk = min(64, n - kb * 64);
    for (int jj = 0; jj < nk; ++jj) {
      const T* vp = cache + (int64_t)krow[jj] * W + G * dk + g * vd;
      #pragma unroll
      for (int c = 0; c < SGG_CP; ++c) {
        const int d = 2 * lane + 128 * c;
        if (d < vd) {
          const float2 v = sg_vec<T>::load2(vp + d);
          #pragma unroll
          for (int hh = 0; hh < REP; ++hh) {
            const float w = pw[hh * 64 + jj];
            acc[hh][c][0] = fmaf(w, v.x, acc[hh][c][0]);
            acc[hh][c][1] = fmaf(w, v.y, acc[hh][c][1]);
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();                 // pw and krow are rewritten next round
  }
  // waves 1..3 leave their sums in LDS, wave 0 adds them in order and writes
  if (wave > 0) {
    #pragma unroll
    for (int hh = 0; hh < REP; ++hh)
      #pragma unroll
      for (int c = 0; c < SGG_CP; ++c) {
        const int d = 2 * lane + 128 * c;
        if (d < vd) {
          red[((wave - 1) * REP + hh) * vd + d] = acc[hh][c][0];
          red[((wave - 1) * REP + hh) * vd + d + 1] = acc[hh][c][1];
        }
      }
  }
  __syncthreads();
  if (wave > 0) return;
  #pragma unroll
  for (int hh = 0; hh < REP; ++hh)
    #pragma unroll
    for (int c = 0; c < SGG_CP; ++c) {
      const int d = 2 * lane + 128 * c;
      if (d < vd) {
        float a0 = acc[hh][c][0], a1 = acc[hh][c][1];
        for (int w = 0; w < 3; ++w) {
          a0 += red[(w * REP + hh) * vd + d];
          a1 += red[(w * REP + hh) * vd + d + 1];
        }
        if (ksplit > 1) {
          float* dst = part + (((int64_t)z * gridDim.x + t) * H + h0 + hh) * vd + d;
          dst[0] = a0; dst[1] = a1;
        } else {
          T* dst = out + ((int64_t)t * H + h0 + hh) * vd + d;
          dst[0] = from_f<T>(a0); dst[1] = from_f<T>(a1);
        }
      }
    }
}

// out = sum over the key shares, in order.
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_attention_sum_kernel(
    const float* __restrict__ part, int64_t n, int ksplit, T* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float a = 0.f;
  for (int z = 0; z < ksplit; ++z) a += part[z * n + i];
  out[i] = from_f<T>(a);
}

template <typename T>
bool launch_group(int rep, dim3 grid, size_t lds, hipStream_t stream, const T* q, const T* cache,
                  const int* bt, int max_nb, int bs, const int* tok_seq, const int* pos, int H,
                  int G, int dk, int vd, float scale, int window, int keep, const float* slopes,
                  const float* pb, int ksplit, float* part, T* out) {
#define SGG_CASE(R)                                                                         \
  if (rep == R) {                                                                           \
    sigmoid_attention_group_kernel<T, R><<<grid, 256, lds, stream>>>(                       \
        q, cache, bt, max_nb, bs, tok_seq, pos, H, G, dk, vd, scale, window, keep, slopes,  \
        pb, ksplit, part, out);                                                             \
    return true;                                                                            \
  }
  SGG_CASE(1) SGG_CASE(2) SGG_CASE(3) SGG_CASE(4) SGG_CASE(6) SGG_CASE(8)
#undef SGG_CASE
  return false;
}

}  // namespace

torch::Tensor qk_norm_kv_write(torch::Tensor proj, int64_t heads, int64_t kv_heads, int64_t dim,
                               int64_t vdim, torch::Tensor q_norm_w, torch::Tensor k_norm_w,
                               double eps, torch::Tensor page_slot, torch::Tensor cache) {
  SM_CHECK_CUDA(q_norm_w); SM_CHECK_F32(q_norm_w); SM_CHECK_CUDA(k_norm_w); SM_CHECK_F32(k_norm_w);
  SM_CHECK_CUDA(page_slot); SM_CHECK_I32(page_slot); SM_CHECK_CUDA(cache);
  const int64_t T = proj.size(0);
  const int64_t need = (heads + kv_heads) * dim + kv_heads * vdim;
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1 && proj.size(1) == need,
              "qk_norm_kv_write: rows are [q | k | v]");
  TORCH_CHECK(q_norm_w.numel() == dim && k_norm_w.numel() == dim && page_slot.numel() == T,
              "qk_norm_kv_write: weights / batch layout");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == kv_heads * (dim + vdim) &&
              cache.scalar_type() == proj.scalar_type(), "qk_norm_kv_write: cache shape/dtype");
  auto q = torch::empty({T, heads, dim}, proj.options());
  if (T == 0) return q;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (proj.scalar_type() == at::kBFloat16)
    qk_norm_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>(
        reinterpret_cast<const bf16_t*>(proj.data_ptr()), proj.stride(0), heads, kv_heads, dim, vdim,
        q_norm_w.data_ptr<float>(), k_norm_w.data_ptr<float>(), (float)eps,
        page_slot.data_ptr<int>(), reinterpret_cast<bf16_t*>(cache.data_ptr()),
        reinterpret_cast<bf16_t*>(q.data_ptr()));
  else {
    SM_CHECK_F32(proj);
    qk_norm_kv_write_kernel<float><<<T, 256, 0, stream>>>(
        proj.data_ptr<float>(), proj.stride(0), heads, kv_heads, dim, vdim,
        q_norm_w.data_ptr<float>(), k_norm_w.data_ptr<float>(), (float)eps,
        page_slot.data_ptr<int>(), cache.data_ptr<float>(), q.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return q;
}

// defined in sigmoid_attention_mfma.hip
bool sigmoid_attention_mfma_fits(int dk, int vd);
torch::Tensor sigmoid_attention_mfma(torch::Tensor q, torch::Tensor cache, int H, int G, int dk,
                                     int vd, torch::Tensor block_tables, int block_size,
                                     torch::Tensor positions, float scale, int window, int keep,
                                     torch::Tensor slopes, torch::Tensor pos_bias,
                                     torch::Tensor tiles);

torch::Tensor sigmoid_attention(torch::Tensor q, torch::Tensor cache, int64_t heads,
                                int64_t kv_heads, int64_t dim, int64_t vdim,
                                torch::Tensor block_tables, int64_t block_size,
                                torch::Tensor tok_seq, torch::Tensor positions, double scale,
                                int64_t window, int64_t keep_first, torch::Tensor slopes,
                                torch::Tensor pos_bias, c10::optional<torch::Tensor> tiles,
                                int64_t max_tile_queries) {
  SM_CHECK_CUDA(q); SM_CHECK_CUDA(cache); SM_CHECK_CUDA(block_tables); SM_CHECK_I32(block_tables);
  SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq); SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  SM_CHECK_CUDA(slopes); SM_CHECK_F32(slopes); SM_CHECK_CUDA(pos_bias); SM_CHECK_F32(pos_bias);
  const int H = heads, G = kv_heads, dk = dim, vd = vdim;
  const int64_t T = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0, "sigmoid_attention: heads must be a multiple of kv_heads");
  TORCH_CHECK(q.dim() == 3 && q.size(1) == H && q.size(2) == dk, "sigmoid_attention: q is [T, H, dim]");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == (int64_t)G * (dk + vd) &&
              cache.scalar_type() == q.scalar_type(), "sigmoid_attention: cache shape/dtype");
  TORCH_CHECK(block_tables.dim() == 2 && tok_seq.numel() == T && positions.numel() == T &&
              block_size > 0, "sigmoid_attention: batch layout");
  TORCH_CHECK(slopes.numel() == H && pos_bias.numel() == H, "sigmoid_attention: per-head tensors");
  TORCH_CHECK(vd <= 64 * SG_REGS, "sigmoid_attention: value size above 512");
  TORCH_CHECK(window >= 0 && keep_first >= 0, "sigmoid_attention: window");
  if (q.scalar_type() == at::kBFloat16 && tiles.has_value() && max_tile_queries > 4 &&
      sigmoid_attention_mfma_fits(dk, vd)) {
    SM_CHECK_CUDA(*tiles); SM_CHECK_I32(*tiles);
    TORCH_CHECK(tiles->dim() == 2 && tiles->size(1) == 3 && max_tile_queries <= 64,
                "sigmoid_attention: tiles");
    return sigmoid_attention_mfma(q, cache, H, G, dk, vd, block_tables, (int)block_size, positions,
                                  (float)scale, (int)window, (int)keep_first, slopes, pos_bias,
                                  *tiles);
  }
  auto out = torch::empty({T, (int64_t)H * vd}, q.options());
  if (T == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  const bool is_bf16 = q.scalar_type() == at::kBFloat16;
  const int rep = H / G, vn = is_bf16 ? 8 : 4;
  const bool rep_ok = rep <= 4 || rep == 6 || rep == 8;
  // steps of few tokens per row: the grouped kernel, when the head sizes
  // allow 16-byte pieces of K and column pairs of V
  if (rep_ok && dk % vn == 0 && vd % 2 == 0 && ((int64_t)G * (dk + vd)) % vn == 0 &&
      vd <= 128 * SGG_CP && (max_tile_queries <= 4 || !is_bf16) &&
      (size_t)(rep * dk + 4 * rep * 64 + 3 * rep * vd + 4 * 64) * 4 <= 64 * 1024) {
    if (!is_bf16) SM_CHECK_F32(q);
    const size_t ldsg = (size_t)(rep * dk + 4 * rep * 64 + 3 * rep * vd + 4 * 64) * 4;
    // enough key shares to fill the chip, at least four 64-key blocks each
    const int64_t longest = (window > 0) ? window + keep_first
                                         : (int64_t)block_tables.size(1) * block_size;
    int ksplit = (int)std::min<int64_t>(std::max<int64_t>(1, 512 / std::max<int64_t>(1, T * G)),
                                        std::max<int64_t>(1, longest / 256));
    ksplit = std::min(ksplit, 16);
    torch::Tensor part;
    float* pp = nullptr;
    if (ksplit > 1) {
      part = torch::empty({ksplit, T, (int64_t)H * vd}, q.options().dtype(at::kFloat));
      pp = part.data_ptr<float>();
    }
    dim3 gg(T, G, ksplit);
    bool ran;
    if (is_bf16)
      ran = launch_group<bf16_t>(rep, gg, ldsg, stream, reinterpret_cast<const bf16_t*>(q.data_ptr()),
                                 reinterpret_cast<const bf16_t*>(cache.data_ptr()),
                                 block_tables.data_ptr<int>(), (int)block_tables.size(1),
                                 (int)block_size, tok_seq.data_ptr<int>(), positions.data_ptr<int>(),
                                 H, G, dk, vd, (float)scale, (int)window, (int)keep_first,
                                 slopes.data_ptr<float>(), pos_bias.data_ptr<float>(), ksplit, pp,
                                 reinterpret_cast<bf16_t*>(out.data_ptr()));
    else
      ran = launch_group<float>(rep, gg, ldsg, stream, q.data_ptr<float>(), cache.data_ptr<float>(),
                                block_tables.data_ptr<int>(), (int)block_tables.size(1),
                                (int)block_size, tok_seq.data_ptr<int>(), positions.data_ptr<int>(),
                                H, G, dk, vd, (float)scale, (int)window, (int)keep_first,
                                slopes.data_ptr<float>(), pos_bias.data_ptr<float>(), ksplit, pp,
                                out.data_ptr<float>());
    TORCH_CHECK(ran, "sigmoid_attention: no grouped kernel for this head ratio");
    SM_CHECK_LAUNCH();
    if (ksplit > 1) {
      const int64_t nel = T * (int64_t)H * vd;
      if (is_bf16)
        sigmoid_attention_sum_kernel<bf16_t><<<SM_CDIV(nel, 256), 256, 0, stream>>>(
            pp, nel, ksplit, reinterpret_cast<bf16_t*>(out.data_ptr()));
      else
        sigmoid_attention_sum_kernel<float><<<SM_CDIV(nel, 256), 256, 0, stream>>>(
            pp, nel, ksplit, out.data_ptr<float>());
      SM_CHECK_LAUNCH();
    }
    return out;
  }
  const size_t lds = (size_t)(dk + 64) * sizeof(float) + 64 * sizeof(int);
  dim3 grid(T, H);
  if (q.scalar_type() == at::kBFloat16)
    sigmoid_attention_kernel<bf16_t><<<grid, 64, lds, stream>>>(
        reinterpret_cast<const bf16_t*>(q.data_ptr()), reinterpret_cast<const bf16_t*>(cache.data_ptr()),
        block_tables.data_ptr<int>(), (int)block_tables.size(1), (int)block_size,
        tok_seq.data_ptr<int>(), positions.data_ptr<int>(), H, G, dk, vd, (float)scale,
        (int)window, (int)keep_first, slopes.data_ptr<float>(), pos_bias.data_ptr<float>(),
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else {
    SM_CHECK_F32(q);
    sigmoid_attention_kernel<float><<<grid, 64, lds, stream>>>(
        q.data_ptr<float>(), cache.data_ptr<float>(), block_tables.data_ptr<int>(),
        (int)block_tables.size(1), (int)block_size, tok_seq.data_ptr<int>(),
        positions.data_ptr<int>(), H, G, dk, vd, (float)scale, (int)window, (int)keep_first,
        slopes.data_ptr<float>(), pos_bias.data_ptr<float>(), out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}
