// Sigmoid attention over paged [k | v] rows: grouped-query attention whose
// weights are sigmoid(q.k * scale - slope_h (i - j) + bias_h), not normalised
// over the keys, under a sliding window that also keeps the first tokens.
//   qk_norm_kv_write   per token: RMS norm of every q and k head over the head
//                      size (plain shared weights), page write of [k | v]
//   sigmoid_attention  one wave per (token, head): fp32 models, any shape,
//                      steps of few tokens
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
