// Offset-weight RMS norm, short causal depthwise convolution with per-slot
// tails (added to its input, or followed by SiLU), the gated
// parallel-residual update (alone, and fused with the next layer's norm),
// the sandwich residual update (closing norm of a sublayer, residual sum and
// the next opening norm in one pass; without a closing norm it is the
// pre-norm tail), the clamped GLU and tanh-GELU activations. Norms may be
// taken over equal consecutive groups of the row. One workgroup per token row
// for the row-wise ops.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

namespace {

// h = x / sqrt(mean(x^2) + eps) * (offset + w), the mean over each of ng
// equal consecutive parts of the row; written as fp32 and (if hb) as T. Input
// rows are ldx apart (a column slice of a wider matrix).
template <typename Tin, typename T>
__global__ __launch_bounds__(256) void offset_rmsnorm_kernel(
    const Tin* __restrict__ x, int64_t ldx, const float* __restrict__ w, float eps,
    float offset, int D, int ng, float* __restrict__ h32, T* __restrict__ hb) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const Tin* xr = x + row * ldx;
  const int n = D / ng;
  for (int g = 0; g < ng; ++g) {
    float ss = 0.f;
    for (int d = g * n + threadIdx.x; d < (g + 1) * n; d += blockDim.x) {
      const float v = to_f(xr[d]);
      ss += v * v;
    }
    ss = sm_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int d = g * n + threadIdx.x; d < (g + 1) * n; d += blockDim.x) {
      const float v = to_f(xr[d]) * inv * (offset + w[d]);
      h32[row * D + d] = v;
      if (hb != nullptr) hb[row * D + d] = from_f<T>(v);
    }
  }
}

// x += mult * (mix * sigmoid(g1 + b1) + ff * sigmoid(g2 + b2)); optionally
// followed by the next offset RMS norm of the new row.
template <typename T>
__global__ __launch_bounds__(256) void gated_residual_kernel(
    float* __restrict__ x, const T* __restrict__ mix, const float* __restrict__ ff,
    const T* __restrict__ gates, const float* __restrict__ gate_b, float mult,
    int D, int G, const float* __restrict__ next_w, float eps,
    float* __restrict__ h32, T* __restrict__ hb) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = to_f(mix[row * D + d]) * sm_sigmoid(to_f(gates[row * G + d]) + gate_b[d]);
    if (ff != nullptr)
      acc += ff[row * D + d] * sm_sigmoid(to_f(gates[row * G + D + d]) + gate_b[D + d]);
    const float v = x[row * D + d] + mult * acc;
    x[row * D + d] = v;
    ss += v * v;
  }
  if (next_w == nullptr) return;
  ss = sm_block_sum(ss, red);   // also orders the row's writes before the re-read
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = x[row * D + d] * inv * (1.0f + next_w[d]);
    h32[row * D + d] = v;
    if (hb != nullptr) hb[row * D + d] = from_f<T>(v);
  }
}

// acc = sum_j w[:, j] * h[t - taps + 1 + j] within the row's sequence;
// inputs before the portion come from tails[slot]. ADD_IN: out = h[t] + acc
// (input rows fp32); SILU: out = acc * sigmoid(acc). h rows are ld apart.
template <typename Tin, typename T, bool ADD_IN, bool SILU>
__global__ __launch_bounds__(256) void tap_conv_kernel(
    const Tin* __restrict__ h, int64_t ld, const float* __restrict__ w,
    const float* __restrict__ tails, const int* __restrict__ cu,
    const int* __restrict__ tok_seq, const int* __restrict__ slots, int D,
    int taps, T* __restrict__ out) {
  const int t = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const int b = tok_seq[t];
  const int start = cu[b];
  const int rel = t - start;
  const int64_t slot = slots[b];
  float acc = ADD_IN ? to_f(h[(int64_t)t * ld + d]) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = rel - taps + 1 + j;
    const float v = (src >= 0)
        ? to_f(h[(int64_t)(start + src) * ld + d])
        : tails[(slot * (taps - 1) + (taps - 1 + src)) * D + d];
    acc += w[d * taps + j] * v;
  }
  if (SILU) acc = acc * sm_sigmoid(acc);
  out[(int64_t)t * D + d] = from_f<T>(acc);
}

// Advance tails[slot] to the last taps-1 inputs of the row's sequence.
#define SM_MAX_TAILS 15
template <typename Tin>
__global__ __launch_bounds__(256) void tap_tail_kernel(
    const Tin* __restrict__ h, int64_t ld, float* __restrict__ tails,
    const int* __restrict__ cu, const int* __restrict__ slots, int D, int taps) {
  const int b = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const int start = cu[b], n = cu[b + 1] - start;
  if (n == 0) return;
  const int64_t slot = slots[b];
  const int keep = taps - 1;
  float nv[SM_MAX_TAILS];
  #pragma unroll
  for (int k = 0; k < SM_MAX_TAILS; ++k) {
    if (k < keep) {
      const int src = n - keep + k;
      nv[k] = (src >= 0) ? to_f(h[(int64_t)(start + src) * ld + d])
                         : tails[(slot * keep + (k + n)) * D + d];
    }
  }
  #pragma unroll
  for (int k = 0; k < SM_MAX_TAILS; ++k)
    if (k < keep) tails[(slot * keep + k) * D + d] = nv[k];
}

// Steps in which every row brings one token: conv and tail update in one
// kernel, one thread per (row, channel) (it alone touches that tail).
template <typename Tin, typename T, bool ADD_IN, bool SILU>
__global__ __launch_bounds__(256) void tap_conv_step_kernel(
    const Tin* __restrict__ h, int64_t ld, const float* __restrict__ w,
    float* __restrict__ tails, const int* __restrict__ slots, int D, int taps,
    T* __restrict__ out) {
  const int b = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const int keep = taps - 1;
  float* tl = tails + (int64_t)slots[b] * keep * D + d;
  const float x = to_f(h[(int64_t)b * ld + d]);
  float acc = (ADD_IN ? x : 0.f) + w[d * taps + keep] * x;
  float prev = x;                       // becomes the newest tail entry
  for (int j = keep - 1; j >= 0; --j) {
    const float v = tl[(int64_t)j * D];
    acc += w[d * taps + j] * v;
    tl[(int64_t)j * D] = prev;          // shift: entry j takes what entry j + 1 held
    prev = v;
  }
  if (SILU) acc = acc * sm_sigmoid(acc);
  out[(int64_t)b * D + d] = from_f<T>(acc);
}

// x += s / sqrt(mean(s^2) + eps) * (1 + post_w), s = y (+ y2), or x += s
// without post_w; then, with next_w, h = x / sqrt(mean(x^2) + eps) *
// (1 + next_w), the mean over each of ng equal parts of the row. y and y2 are
// bf16 or fp32 each (flags), h is T.
SM_INLINE float ld_any(const void* p, bool is_bf16, int64_t i) {
  return is_bf16 ? __bfloat162float(reinterpret_cast<const bf16_t*>(p)[i])
                 : reinterpret_cast<const float*>(p)[i];
}
template <typename T>
__global__ __launch_bounds__(256) void sandwich_residual_kernel(
    float* __restrict__ x, const void* __restrict__ y, bool y_bf16,
    const void* __restrict__ y2, bool y2_bf16, const float* __restrict__ post_w,
    const float* __restrict__ next_w, float eps, float offset, float ys, float y2s,
    int D, int ng, T* __restrict__ h) {
  // the closing norm is over s = ys * y (+ y2s * y2); h (when given) gets the
  // next norm of the new row, or, without next_w, the new row itself
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  float inv = 1.0f;
  if (post_w != nullptr) {
    float ss = 0.f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      float s = ys * ld_any(y, y_bf16, row * D + d);
      if (y2 != nullptr) s += y2s * ld_any(y2, y2_bf16, row * D + d);
      ss += s * s;
    }
    ss = sm_block_sum(ss, red);
    inv = 1.0f / sqrtf(ss / (float)D + eps);
  }
  float xx = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float s = ys * ld_any(y, y_bf16, row * D + d);
    if (y2 != nullptr) s += y2s * ld_any(y2, y2_bf16, row * D + d);
    const float v = x[row * D + d] + (post_w != nullptr ? s * inv * (offset + post_w[d]) : s);
    x[row * D + d] = v;
    xx += v * v;
    if (next_w == nullptr && h != nullptr) h[row * D + d] = from_f<T>(v);
  }
  if (next_w == nullptr) return;
  if (ng == 1) {
    xx = sm_block_sum(xx, red);   // also orders the row's writes before the re-read
    const float inv2 = 1.0f / sqrtf(xx / (float)D + eps);
    for (int d = threadIdx.x; d < D; d += blockDim.x)
      h[row * D + d] = from_f<T>(x[row * D + d] * inv2 * (offset + next_w[d]));
    return;
  }
  // grouped norm: another thread may have written what this one reads now
  __syncthreads();
  const int n = D / ng;
  for (int g = 0; g < ng; ++g) {
    float gs = 0.f;
    for (int d = g * n + threadIdx.x; d < (g + 1) * n; d += blockDim.x) {
      const float v = x[row * D + d];
      gs += v * v;
    }
    gs = sm_block_sum(gs, red);
    const float inv2 = 1.0f / sqrtf(gs / (float)n + eps);
    for (int d = g * n + threadIdx.x; d < (g + 1) * n; d += blockDim.x)
      h[row * D + d] = from_f<T>(x[row * D + d] * inv2 * (offset + next_w[d]));
  }
}

// 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))), fp32 inside.
template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_kernel(const T* __restrict__ x, int64_t n,
                                                        T* __restrict__ out) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= n) return;
  const float z = to_f(x[id]);
  out[id] = from_f<T>(0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))));
}

// gu rows = [gate (ff) | up (ff)]: g = min(gate, limit), u = clamp(up, +-limit),
// out = g * sigmoid(1.702 g) * (u + 1); SILU: out = gate * sigmoid(gate) * up.
template <typename T, bool SILU>
__global__ __launch_bounds__(256) void capped_glu_kernel(
    const T* __restrict__ gu, int64_t n, int ff, float limit, T* __restrict__ out) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= n) return;
  const int64_t t = id / ff;
  const int f = id % ff;
  const float g = to_f(gu[t * 2 * ff + f]), u = to_f(gu[t * 2 * ff + ff + f]);
  out[id] = from_f<T>(SILU ? g * sm_sigmoid(g) * u : sm_capped_glu(g, u, limit));
}

}  // namespace

std::vector<torch::Tensor> offset_rmsnorm(torch::Tensor x, torch::Tensor w,
                                          double eps, bool out_bf16, double offset,
                                          int64_t groups) {
  SM_CHECK_CUDA(w); SM_CHECK_F32(w);
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1 && w.numel() == x.size(1),
              "offset_rmsnorm: shapes");
  TORCH_CHECK(groups >= 1 && x.size(1) % groups == 0, "offset_rmsnorm: groups must divide the row");
  const int64_t ldx = x.stride(0);
  const int64_t T = x.size(0);
  const int D = x.size(1);
  auto h32 = torch::empty({T, D}, x.options().dtype(at::kFloat));
  torch::Tensor hb = out_bf16 ? torch::empty({T, D}, x.options().dtype(at::kBFloat16)) : h32;
  if (T == 0) return {h32, hb};
  auto stream = at::cuda::getCurrentCUDAStream();
  bf16_t* hbp = out_bf16 ? reinterpret_cast<bf16_t*>(hb.data_ptr()) : nullptr;
  if (x.scalar_type() == at::kBFloat16) {
    offset_rmsnorm_kernel<bf16_t, bf16_t><<<T, 256, 0, stream>>>(
        reinterpret_cast<const bf16_t*>(x.data_ptr()), ldx, w.data_ptr<float>(),
        (float)eps, (float)offset, D, (int)groups, h32.data_ptr<float>(), hbp);
  } else {
    SM_CHECK_F32(x);
    offset_rmsnorm_kernel<float, bf16_t><<<T, 256, 0, stream>>>(
        x.data_ptr<float>(), ldx, w.data_ptr<float>(), (float)eps, (float)offset, D,
        (int)groups, h32.data_ptr<float>(), hbp);
  }
  SM_CHECK_LAUNCH();
  return {h32, hb};
}

static std::vector<torch::Tensor> gated_residual_impl(
    torch::Tensor x, torch::Tensor mix, c10::optional<torch::Tensor> ff,
    torch::Tensor gates, torch::Tensor gate_b, double mult,
    c10::optional<torch::Tensor> next_w, double eps, bool out_bf16) {
  SM_CHECK_CUDA(x); SM_CHECK_F32(x); SM_CHECK_CUDA(mix); SM_CHECK_CUDA(gates);
  SM_CHECK_CUDA(gate_b); SM_CHECK_F32(gate_b);
  const int64_t T = x.size(0);
  const int D = x.size(1);
  const int G = gates.size(1);
  TORCH_CHECK(mix.size(0) == T && mix.size(1) == D && gates.size(0) == T, "gated_residual: shapes");
  TORCH_CHECK(G == (ff.has_value() ? 2 * D : D) && gate_b.numel() == G, "gated_residual: gate width");
  TORCH_CHECK(mix.scalar_type() == gates.scalar_type(), "gated_residual: dtypes");
  const float* ffp = nullptr;
  if (ff.has_value()) {
    SM_CHECK_CUDA(*ff); SM_CHECK_F32(*ff);
    TORCH_CHECK(ff->size(0) == T && ff->size(1) == D, "gated_residual: ff shape");
    ffp = ff->data_ptr<float>();
  }
  torch::Tensor h32, hb;
  const float* nw = nullptr;
  if (next_w.has_value()) {
    SM_CHECK_CUDA(*next_w); SM_CHECK_F32(*next_w);
    TORCH_CHECK(next_w->numel() == D, "gated_residual: norm weight");
    nw = next_w->data_ptr<float>();
    h32 = torch::empty({T, D}, x.options());
    hb = out_bf16 ? torch::empty({T, D}, x.options().dtype(at::kBFloat16)) : h32;
  }
  if (T == 0) return {h32, hb};
  auto stream = at::cuda::getCurrentCUDAStream();
  float* h32p = next_w.has_value() ? h32.data_ptr<float>() : nullptr;
  if (mix.scalar_type() == at::kBFloat16) {
    bf16_t* hbp = (next_w.has_value() && out_bf16) ? reinterpret_cast<bf16_t*>(hb.data_ptr()) : nullptr;
    gated_residual_kernel<bf16_t><<<T, 256, 0, stream>>>(
        x.data_ptr<float>(), reinterpret_cast<const bf16_t*>(mix.data_ptr()), ffp,
        reinterpret_cast<const bf16_t*>(gates.data_ptr()), gate_b.data_ptr<float>(),
        (float)mult, D, G, nw, (float)eps, h32p, hbp);
  } else {
    SM_CHECK_F32(mix);
    TORCH_CHECK(!out_bf16, "gated_residual: bf16 output needs bf16 inputs");
    gated_residual_kernel<float><<<T, 256, 0, stream>>>(
        x.data_ptr<float>(), mix.data_ptr<float>(), ffp, gates.data_ptr<float>(),
        gate_b.data_ptr<float>(), (float)mult, D, G, nw, (float)eps, h32p, nullptr);
  }
  SM_CHECK_LAUNCH();
  return {h32, hb};
}

void gated_residual_add(torch::Tensor x, torch::Tensor mix,
                        c10::optional<torch::Tensor> ff, torch::Tensor gates,
                        torch::Tensor gate_b, double mult) {
  gated_residual_impl(x, mix, ff, gates, gate_b, mult, c10::nullopt, 0.0, false);
}

std::vector<torch::Tensor> gated_residual_norm(
    torch::Tensor x, torch::Tensor mix, c10::optional<torch::Tensor> ff,
    torch::Tensor gates, torch::Tensor gate_b, double mult, torch::Tensor next_w,
    double eps, bool out_bf16) {
  return gated_residual_impl(x, mix, ff, gates, gate_b, mult, next_w, eps, out_bf16);
}

torch::Tensor causal_tap_conv(torch::Tensor h, torch::Tensor w, torch::Tensor tails,
                              torch::Tensor cu, torch::Tensor tok_seq,
                              torch::Tensor slots, bool out_bf16) {
  SM_CHECK_CUDA(h); SM_CHECK_F32(h); SM_CHECK_CUDA(w); SM_CHECK_F32(w);
  SM_CHECK_CUDA(tails); SM_CHECK_F32(tails);
  SM_CHECK_CUDA(cu); SM_CHECK_I32(cu); SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq);
  SM_CHECK_CUDA(slots); SM_CHECK_I32(slots);
  const int64_t T = h.size(0);
  const int D = h.size(1);
  const int taps = w.size(1);
  const int B = slots.numel();
  TORCH_CHECK(w.size(0) == D && taps >= 1 && taps - 1 <= SM_MAX_TAILS, "tap conv: weight shape");
  TORCH_CHECK(tails.dim() == 3 && tails.size(1) == taps - 1 && tails.size(2) == D, "tap conv: tails shape");
  TORCH_CHECK(cu.numel() == B + 1 && tok_seq.numel() == T, "tap conv: batch layout");
  auto out = torch::empty({T, D}, h.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  if (T == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  dim3 grid(T, SM_CDIV(D, 256));
  if (out_bf16)
    tap_conv_kernel<float, bf16_t, true, false><<<grid, 256, 0, stream>>>(
        h.data_ptr<float>(), (int64_t)D, w.data_ptr<float>(), tails.data_ptr<float>(),
        cu.data_ptr<int>(), tok_seq.data_ptr<int>(), slots.data_ptr<int>(), D, taps,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else
    tap_conv_kernel<float, float, true, false><<<grid, 256, 0, stream>>>(
        h.data_ptr<float>(), (int64_t)D, w.data_ptr<float>(), tails.data_ptr<float>(),
        cu.data_ptr<int>(), tok_seq.data_ptr<int>(), slots.data_ptr<int>(), D, taps,
        out.data_ptr<float>());
  SM_CHECK_LAUNCH();
  if (taps > 1) {
    dim3 g2(B, SM_CDIV(D, 256));
    tap_tail_kernel<float><<<g2, 256, 0, stream>>>(h.data_ptr<float>(), (int64_t)D,
                                                   tails.data_ptr<float>(), cu.data_ptr<int>(),
                                                   slots.data_ptr<int>(), D, taps);
    SM_CHECK_LAUNCH();
  }
  return out;
}

torch::Tensor tap_conv_silu(torch::Tensor x, torch::Tensor w, torch::Tensor tails,
                            torch::Tensor cu, torch::Tensor tok_seq,
                            torch::Tensor slots, bool out_bf16) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1, "tap_conv_silu: x must be row-major");
  SM_CHECK_CUDA(w); SM_CHECK_F32(w); SM_CHECK_CUDA(tails); SM_CHECK_F32(tails);
  SM_CHECK_CUDA(cu); SM_CHECK_I32(cu); SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq);
  SM_CHECK_CUDA(slots); SM_CHECK_I32(slots);
  const int64_t T = x.size(0);
  const int C = x.size(1);
  const int64_t ld = x.stride(0);
  const int taps = w.size(1);
  const int B = slots.numel();
  const bool in_bf16 = x.scalar_type() == at::kBFloat16;
  TORCH_CHECK(in_bf16 || x.scalar_type() == at::kFloat, "tap_conv_silu: dtype");
  TORCH_CHECK(in_bf16 == out_bf16, "tap_conv_silu: output dtype follows the input");
  TORCH_CHECK(w.size(0) == C && taps >= 1 && taps - 1 <= SM_MAX_TAILS, "tap_conv_silu: weight shape");
  TORCH_CHECK(tails.dim() == 3 && tails.size(1) == taps - 1 && tails.size(2) == C, "tap_conv_silu: tails shape");
  TORCH_CHECK(cu.numel() == B + 1 && tok_seq.numel() == T, "tap_conv_silu: batch layout");
  auto out = torch::empty({T, C}, x.options());
  if (T == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  dim3 grid(T, SM_CDIV(C, 256)), g2(B, SM_CDIV(C, 256));
  if (T == B) {
    // one token per row (cu is 0, 1, 2, ...: a step's rows are never empty)
    if (in_bf16)
      tap_conv_step_kernel<bf16_t, bf16_t, false, true><<<g2, 256, 0, stream>>>(
          reinterpret_cast<const bf16_t*>(x.data_ptr()), ld, w.data_ptr<float>(),
          tails.data_ptr<float>(), slots.data_ptr<int>(), C, taps,
          reinterpret_cast<bf16_t*>(out.data_ptr()));
    else
      tap_conv_step_kernel<float, float, false, true><<<g2, 256, 0, stream>>>(
          x.data_ptr<float>(), ld, w.data_ptr<float>(), tails.data_ptr<float>(),
          slots.data_ptr<int>(), C, taps, out.data_ptr<float>());
    SM_CHECK_LAUNCH();
    return out;
  }
  if (in_bf16) {
    const bf16_t* xp = reinterpret_cast<const bf16_t*>(x.data_ptr());
    tap_conv_kernel<bf16_t, bf16_t, false, true><<<grid, 256, 0, stream>>>(
        xp, ld, w.data_ptr<float>(), tails.data_ptr<float>(), cu.data_ptr<int>(),
        tok_seq.data_ptr<int>(), slots.data_ptr<int>(), C, taps,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
    SM_CHECK_LAUNCH();
    if (taps > 1)
      tap_tail_kernel<bf16_t><<<g2, 256, 0, stream>>>(xp, ld, tails.data_ptr<float>(),
                                                      cu.data_ptr<int>(), slots.data_ptr<int>(), C, taps);
  } else {
    tap_conv_kernel<float, float, false, true><<<grid, 256, 0, stream>>>(
        x.data_ptr<float>(), ld, w.data_ptr<float>(), tails.data_ptr<float>(), cu.data_ptr<int>(),
        tok_seq.data_ptr<int>(), slots.data_ptr<int>(), C, taps, out.data_ptr<float>());
    SM_CHECK_LAUNCH();
    if (taps > 1)
      tap_tail_kernel<float><<<g2, 256, 0, stream>>>(x.data_ptr<float>(), ld, tails.data_ptr<float>(),
                                                     cu.data_ptr<int>(), slots.data_ptr<int>(), C, taps);
  }
  SM_CHECK_LAUNCH();
  return out;
}

c10::optional<torch::Tensor> sandwich_residual_norm(
    torch::Tensor x, torch::Tensor y, c10::optional<torch::Tensor> y2,
    c10::optional<torch::Tensor> post_w, c10::optional<torch::Tensor> next_w, double eps,
    bool out_bf16, double offset, double y_scale, double y2_scale, bool cast_next,
    int64_t groups) {
  SM_CHECK_CUDA(x); SM_CHECK_F32(x); SM_CHECK_CUDA(y);
  const float* pw = nullptr;
  if (post_w.has_value()) {
    SM_CHECK_CUDA(*post_w); SM_CHECK_F32(*post_w);
    TORCH_CHECK(post_w->numel() == x.size(1), "sandwich_residual_norm: closing norm weight");
    pw = post_w->data_ptr<float>();
  }
  TORCH_CHECK(groups >= 1 && x.size(1) % groups == 0,
              "sandwich_residual_norm: groups must divide the row");
  const int64_t T = x.size(0);
  const int D = x.size(1);
  auto kind = [](const torch::Tensor& t) {
    TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat,
                "sandwich_residual_norm: addends are bf16 or fp32");
    return t.scalar_type() == at::kBFloat16;
  };
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && y.size(0) == T && y.size(1) == D,
              "sandwich_residual_norm: shapes");
  const bool yb = kind(y);
  const void* y2p = nullptr;
  bool y2b = false;
  if (y2.has_value()) {
    SM_CHECK_CUDA(*y2);
    TORCH_CHECK(y2->dim() == 2 && y2->size(0) == T && y2->size(1) == D, "sandwich_residual_norm: y2 shape");
    y2b = kind(*y2);
    y2p = y2->data_ptr();
  }
  const float* nw = nullptr;
  c10::optional<torch::Tensor> h;
  if (next_w.has_value()) {
    SM_CHECK_CUDA(*next_w); SM_CHECK_F32(*next_w);
    TORCH_CHECK(next_w->numel() == D, "sandwich_residual_norm: norm weight");
    nw = next_w->data_ptr<float>();
    h = torch::empty({T, D}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  } else if (cast_next) {
    TORCH_CHECK(out_bf16, "sandwich_residual_norm: a copy of the residual is made in bf16 only");
    h = torch::empty({T, D}, x.options().dtype(at::kBFloat16));
  }
  if (T == 0) return h;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (out_bf16)
    sandwich_residual_kernel<bf16_t><<<T, 256, 0, stream>>>(
        x.data_ptr<float>(), y.data_ptr(), yb, y2p, y2b, pw, nw, (float)eps,
        (float)offset, (float)y_scale, (float)y2_scale, D, (int)groups,
        h.has_value() ? reinterpret_cast<bf16_t*>(h->data_ptr()) : nullptr);
  else
    sandwich_residual_kernel<float><<<T, 256, 0, stream>>>(
        x.data_ptr<float>(), y.data_ptr(), yb, y2p, y2b, pw, nw, (float)eps,
        (float)offset, (float)y_scale, (float)y2_scale, D, (int)groups,
        h.has_value() ? h->data_ptr<float>() : nullptr);
  SM_CHECK_LAUNCH();
  return h;
}

template <bool SILU>
static torch::Tensor glu_impl(torch::Tensor gu, double limit) {
  SM_CHECK_CUDA(gu);
  TORCH_CHECK(gu.dim() == 2 && gu.size(1) % 2 == 0, "glu: rows are [gate | up]");
  const int64_t T = gu.size(0);
  const int ff = gu.size(1) / 2;
  auto out = torch::empty({T, ff}, gu.options());
  const int64_t n = T * ff;
  if (n == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (gu.scalar_type() == at::kBFloat16)
    capped_glu_kernel<bf16_t, SILU><<<SM_CDIV(n, 256), 256, 0, stream>>>(
        reinterpret_cast<const bf16_t*>(gu.data_ptr()), n, ff, (float)limit,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else {
    SM_CHECK_F32(gu);
    capped_glu_kernel<float, SILU><<<SM_CDIV(n, 256), 256, 0, stream>>>(
        gu.data_ptr<float>(), n, ff, (float)limit, out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}

torch::Tensor capped_glu(torch::Tensor gu, double limit) { return glu_impl<false>(gu, limit); }
torch::Tensor silu_glu(torch::Tensor gu) { return glu_impl<true>(gu, 0.0); }

torch::Tensor gelu_tanh(torch::Tensor x) {
  SM_CHECK_CUDA(x);
  auto out = torch::empty_like(x);
  const int64_t n = x.numel();
  if (n == 0) return out;
  auto stream = at::cuda::getCurrentCUDAStream();
  if (x.scalar_type() == at::kBFloat16)
    gelu_tanh_kernel<bf16_t><<<SM_CDIV(n, 256), 256, 0, stream>>>(
        reinterpret_cast<const bf16_t*>(x.data_ptr()), n, reinterpret_cast<bf16_t*>(out.data_ptr()));
  else {
    SM_CHECK_F32(x);
    gelu_tanh_kernel<float><<<SM_CDIV(n, 256), 256, 0, stream>>>(x.data_ptr<float>(), n,
                                                                 out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}
