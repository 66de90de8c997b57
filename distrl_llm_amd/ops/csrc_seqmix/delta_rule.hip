// Gated delta rule over a flat varlen batch, fp32 matrix state per (slot,
// head). Three kernels:
//   delta_prepare   per token: q, k of every q/k head made unit vectors (q
//                   also / sqrt(dim)), write strength beta = sigmoid(b) and
//                   decay = exp(-exp(a_log) softplus(a + dt_bias)), all fp32;
//                   b and a are given, or projected here from the mixer input
//   delta_scan      per (sequence row, head, block of value columns): walks
//                   the row's tokens in order with the state in registers
//                   (8 key rows of one value column per lane),
//                   S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q;
//                   inputs arrive in chunks through LDS, one chunk ahead
//   delta_finish    per (token, head): o / rms(o) * norm_w * silu(gate)
//                   (or * sigmoid(gate))
// With a decay per head and key channel (delta_channel_decay forms it from a
// low-rank input) the scan multiplies every state row by its own factor.
// The scan is strictly sequential over a row's tokens, so a prompt cut into
// portions gives bit-identical states and outputs.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

namespace {


// qkv row = [q (G dk) | k (G dk) | v (H vd)] after convolution and SiLU.
// One workgroup per token; wave w normalises q/k heads w, w + 4, ...
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const T* __restrict__ qkv, int C, const float* __restrict__ ab,
    const T* __restrict__ hin, int64_t ldh, const float* __restrict__ ab_w, int D,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, int H, int G,
    int dk, int dkp, float* __restrict__ qn, float* __restrict__ kn,
    float* __restrict__ beta, float* __restrict__ decay) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = qkv + t * C;
  if (blockIdx.y > 0) {
    // the [strength; step] projection of the mixer input, fp32: one wave per
    // output, four outputs per workgroup (blockIdx.y - 1 counts the groups)
    const int j = (blockIdx.y - 1) * 4 + wave;
    if (j >= 2 * H) return;
    const float* wr = ab_w + (int64_t)j * D;
    float a0 = 0.f, a1 = 0.f;
    int d = lane;
    for (; d + 64 < D; d += 128) {
      a0 = fmaf(to_f(hin[t * ldh + d]), wr[d], a0);
      a1 = fmaf(to_f(hin[t * ldh + d + 64]), wr[d + 64], a1);
    }
    if (d < D) a0 = fmaf(to_f(hin[t * ldh + d]), wr[d], a0);
    const float z = sm_wave_sum(a0 + a1);
    if (lane == 0) {
      if (j < H) {
        beta[t * H + j] = sm_sigmoid(z);
      } else {
        const float y = z + dt_bias[j - H];
        const float sp = (y > 20.f) ? y : log1pf(expf(y));
        decay[t * H + j - H] = expf(-expf(a_log[j - H]) * sp);
      }
    }
    return;
  }
  for (int job = wave; job < 2 * G; job += 4) {
    const bool is_k = job >= G;
    const int g = is_k ? job - G : job;
    const T* src = row + (is_k ? G * dk : 0) + g * dk;
    float ss = 0.f;
    for (int k = lane; k < dk; k += 64) {
      const float v = to_f(src[k]);
      ss += v * v;
    }
    ss = sm_wave_sum(ss);
    float inv = 1.0f / sqrtf(ss + 1e-6f);
    if (!is_k) inv *= 1.0f / sqrtf((float)dk);
    float* dst = (is_k ? kn : qn) + (t * G + g) * dkp;
    for (int k = lane; k < dkp; k += 64) dst[k] = (k < dk) ? to_f(src[k]) * inv : 0.f;
  }
  if (ab != nullptr) for (int h = threadIdx.x; h < H; h += blockDim.x) {
    beta[t * H + h] = sm_sigmoid(ab[t * 2 * H + h]);
    const float z = ab[t * 2 * H + H + h] + dt_bias[h];
    const float sp = (z > 20.f) ? z : log1pf(expf(z));
    decay[t * H + h] = expf(-expf(a_log[h]) * sp);
  }
}

// Per-channel decays: ab row = [strength (H) | low-rank decay input (R)],
// pre [T, H dk] = the decay input through its up-projection (a vendor GEMM);
// step = softplus(pre + dt_bias), decay[t, h, k] = exp(-exp(a_log[h]) step)
// for k < dk, 1 in the padding; beta[t, h] = sigmoid(strength).
__global__ __launch_bounds__(256) void delta_channel_decay_kernel(
    const float* __restrict__ ab, int abw, const float* __restrict__ pre, int H,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, int dk, int dkp,
    float* __restrict__ beta, float* __restrict__ decay) {
  const int64_t t = blockIdx.x;
  for (int h = threadIdx.x; h < H; h += blockDim.x) beta[t * H + h] = sm_sigmoid(ab[t * abw + h]);
  for (int i = threadIdx.x; i < H * dkp; i += blockDim.x) {
    const int h = i / dkp, k = i % dkp;
    float d = 1.0f;
    if (k < dk) {
      const float z = pre[t * H * dk + h * dk + k] + dt_bias[h * dk + k];
      const float sp = (z > 20.f) ? z : log1pf(expf(z));
      d = expf(-expf(a_log[h]) * sp);
    }
    decay[(t * H + h) * dkp + k] = d;
  }
}

// One workgroup (4 waves) per (row, head, block of 256 / KS value columns).
// Lane = (column, ks): it holds DR_ROWS state rows (8 or 32) of its column,
// starting at ks * DR_ROWS (few rows per lane when there are few sequence
// rows and heads: the walk is a dependent chain, so it is spread over more
// lanes and waves rather than made long); dot products over the key axis
// are finished with lane moves over the KS lanes of a column. The tokens come
// in chunks of DR_CH: a chunk's unit q/k rows, decays and strengths sit in
// LDS, shared by the four waves (every lane reads the same few addresses),
// the lane's own v entries in registers, and the next chunk is fetched into
// registers while the current one is walked. The state is stored value-major
// ([head][column][key]): a lane's rows are contiguous and the KS lanes of a
// column read one contiguous run.
#define DR_CH 16

// Sum over the KS adjacent lanes of a column (KS a power of two, groups
// aligned) with data-parallel lane moves: swaps inside a quad, then a mirror
// of 8 and of 16 lanes (after the quad steps every lane of a quad holds the
// quad's sum, so the mirrored lane brings the other half's). These are plain
// vector instructions; a cross-lane read through LDS per step would put
// several hundred cycles on the walk's dependent chain.
template <int CTRL>
SM_INLINE float dr_lane_move(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
template <int KS>
SM_INLINE float dr_column_sum(float x) {
  if (KS >= 2) x += dr_lane_move<0xB1>(x);     // quad lanes [1, 0, 3, 2]
  if (KS >= 4) x += dr_lane_move<0x4E>(x);     // quad lanes [2, 3, 0, 1]
  if (KS >= 8) x += dr_lane_move<0x141>(x);    // mirror within 8 lanes
  if (KS >= 16) x += dr_lane_move<0x140>(x);   // mirror within 16 lanes
  if (KS >= 32) x += __shfl_xor(x, 16, SM_WAVE);
  return x;
}

// CH: the decay is a row of DKP factors per (token, head), staged beside the
// token's k and q rows, instead of one factor per (token, head).
template <typename T, int KS, int DR_ROWS, bool CH>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    const T* __restrict__ qkv, int C, const float* __restrict__ qn,
    const float* __restrict__ kn, const float* __restrict__ beta,
    const float* __restrict__ decay, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ slots, int H, int G, int dk,
    int vd, float* __restrict__ o) {
  constexpr int COLS = 64 / KS;                 // columns per wave
  constexpr int DKP = KS * DR_ROWS;
  constexpr int ROW4 = DKP / 4;                 // float4 per q or k row
  constexpr int NR = CH ? 3 : 2;                // staged rows per token
  constexpr int NSTAGE = DR_CH * NR * ROW4;
  constexpr int NPRE = (NSTAGE + 255) / 256;    // float4 per thread and chunk
  __shared__ float4 kq4[NSTAGE];                // [token][k | q (| decay)][DKP]
  __shared__ float sc[DR_CH * 2];               // [token][decay | beta]
  const int b = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63;
  const int ks = lane % KS;
  const int col = (blockIdx.z * 4 + (tid >> 6)) * COLS + lane / KS;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 == t0) return;                         // uniform over the workgroup
  const bool live = col < vd;
  const int g = h / (H / G);
  const int64_t slot = slots[b];
  float* Sp = state + ((slot * H + h) * vd + (live ? col : 0)) * dk + ks * DR_ROWS;
  const bool vec = (dk % 4) == 0;               // a lane's rows as 16-byte pieces
  float S[DR_ROWS];
  #pragma unroll
  for (int r = 0; r < DR_ROWS; r += 4) {
    const int k = ks * DR_ROWS + r;
    if (vec) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (live && k < dk) v = *reinterpret_cast<const float4*>(Sp + r);
      S[r] = v.x; S[r + 1] = v.y; S[r + 2] = v.z; S[r + 3] = v.w;
    } else {
      #pragma unroll
      for (int j = 0; j < 4; ++j) S[r + j] = (live && k + j < dk) ? Sp[r + j] : 0.f;
    }
  }
  const int voff = 2 * G * dk + h * vd + (live ? col : 0);

  float4 pre[NPRE];
  float pv[DR_CH], pvn[DR_CH];
  float psc = 0.f;
  // fetch a chunk into registers: q/k rows (linear float4 index = LDS index),
  // the lane's v entries, and decay/beta of token tid / 2
  auto fetch = [&](int tb, int n, float* vout) {
    #pragma unroll
    for (int j = 0; j < NPRE; ++j) {
      const int i = tid + 256 * j;
      if (NSTAGE % 256 != 0 && i >= NSTAGE) break;
      const int tok = i / (NR * ROW4), rem = i % (NR * ROW4);
      const int64_t tt = tb + min(tok, n - 1);
      const float* src = (rem >= 2 * ROW4) ? decay + (tt * H + h) * DKP
                                           : (rem >= ROW4 ? qn : kn) + (tt * G + g) * DKP;
      pre[j] = reinterpret_cast<const float4*>(src)[rem % ROW4];
    }
    #pragma unroll
    for (int i = 0; i < DR_CH; ++i)
      vout[i] = to_f(qkv[(int64_t)(tb + min(i, n - 1)) * C + voff]);
    if (tid < 2 * DR_CH) {
      const int64_t t = tb + min(tid >> 1, n - 1);
      psc = (tid & 1) ? beta[t * H + h] : (CH ? 1.0f : decay[t * H + h]);
    }
  };
  auto stash = [&]() {
    #pragma unroll
    for (int j = 0; j < NPRE; ++j)
      if (NSTAGE % 256 == 0 || tid + 256 * j < NSTAGE) kq4[tid + 256 * j] = pre[j];
    if (tid < 2 * DR_CH) sc[tid] = psc;
  };

  fetch(t0, min(DR_CH, t1 - t0), pv);
  stash();
  __syncthreads();
  for (int tb = t0; tb < t1; tb += DR_CH) {
    const int n = min(DR_CH, t1 - tb);
    const int nn = min(DR_CH, t1 - tb - DR_CH);
    if (nn > 0) fetch(tb + DR_CH, nn, pvn);
    #pragma unroll
    for (int i = 0; i < DR_CH; ++i) {
      if (i >= n) break;
      const float4* kp = kq4 + (i * NR) * ROW4 + ks * (DR_ROWS / 4);
      const float4* qp = kp + ROW4;
      const float dec = sc[2 * i], bt = sc[2 * i + 1];
      float4 kk[DR_ROWS / 4];
      float sk0 = 0.f, sk1 = 0.f;
      #pragma unroll
      for (int r = 0; r < DR_ROWS; r += 4) {
        const float4 k4 = kk[r / 4] = kp[r / 4];
        if (CH) {
          const float4 d4 = kp[2 * ROW4 + r / 4];
          S[r] *= d4.x; S[r + 1] *= d4.y; S[r + 2] *= d4.z; S[r + 3] *= d4.w;
        } else {
          S[r] *= dec; S[r + 1] *= dec; S[r + 2] *= dec; S[r + 3] *= dec;
        }
        sk0 = fmaf(S[r], k4.x, sk0);
        sk1 = fmaf(S[r + 1], k4.y, sk1);
        sk0 = fmaf(S[r + 2], k4.z, sk0);
        sk1 = fmaf(S[r + 3], k4.w, sk1);
      }
      const float sk = dr_column_sum<KS>(sk0 + sk1);
      const float u = bt * (pv[i] - sk);
      float so0 = 0.f, so1 = 0.f;
      #pragma unroll
      for (int r = 0; r < DR_ROWS; r += 4) {
        const float4 k4 = kk[r / 4];
        const float4 q4 = qp[r / 4];
        S[r] = fmaf(k4.x, u, S[r]);
        S[r + 1] = fmaf(k4.y, u, S[r + 1]);
        S[r + 2] = fmaf(k4.z, u, S[r + 2]);
        S[r + 3] = fmaf(k4.w, u, S[r + 3]);
        so0 = fmaf(S[r], q4.x, so0);
        so1 = fmaf(S[r + 1], q4.y, so1);
        so0 = fmaf(S[r + 2], q4.z, so0);
        so1 = fmaf(S[r + 3], q4.w, so1);
      }
      const float so = dr_column_sum<KS>(so0 + so1);
      if (live && ks == 0) o[((int64_t)(tb + i) * H + h) * vd + col] = so;
    }
    __syncthreads();
    if (nn > 0) {
      stash();
      #pragma unroll
      for (int i = 0; i < DR_CH; ++i) pv[i] = pvn[i];
    }
    __syncthreads();
  }
  #pragma unroll
  for (int r = 0; r < DR_ROWS; r += 4) {
    const int k = ks * DR_ROWS + r;
    if (vec) {
      if (live && k < dk)
        *reinterpret_cast<float4*>(Sp + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
    } else {
      #pragma unroll
      for (int j = 0; j < 4; ++j)
        if (live && k + j < dk) Sp[r + j] = S[r + j];
    }
  }
}

// One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void delta_finish_kernel(
    const float* __restrict__ o, const T* __restrict__ gate, int64_t ldg,
    const float* __restrict__ norm_w, float eps, int H, int vd, int gate_sigmoid,
    T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* src = o + (t * H + h) * vd;
  float ss = 0.f;
  for (int d = lane; d < vd; d += 64) ss += src[d] * src[d];
  ss = sm_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vd + eps);
  for (int d = lane; d < vd; d += 64) {
    const float gt = to_f(gate[t * ldg + h * vd + d]);
    const float act = gate_sigmoid ? sm_sigmoid(gt) : gt * sm_sigmoid(gt);
    out[(t * H + h) * vd + d] = from_f<T>(src[d] * inv * norm_w[d] * act);
  }
}

template <typename T, bool CH>
void launch_scan(int KS, int R, dim3 grid, hipStream_t stream, const T* qkv, int C, const float* qn,
                 const float* kn, const float* beta, const float* decay, float* state,
                 const int* cu, const int* slots, int H, int G, int dk, int vd, float* o) {
#define DR_CASE(N, RR)                                                                        \
  if (KS == N && R == RR) {                                                                   \
    delta_scan_kernel<T, N, RR, CH><<<dim3(grid.x, grid.y, SM_CDIV(vd, 256 / N)), 256, 0, stream>>>( \
        qkv, C, qn, kn, beta, decay, state, cu, slots, H, G, dk, vd, o);                      \
    return;                                                                                   \
  }
  DR_CASE(4, 8) DR_CASE(8, 8) DR_CASE(16, 8) DR_CASE(32, 8)
  DR_CASE(1, 32) DR_CASE(2, 32) DR_CASE(4, 32) DR_CASE(8, 32)
#undef DR_CASE
  TORCH_CHECK(false, "gated_delta_rule: key dim too large");
}

}  // namespace

torch::Tensor gated_delta_rule(torch::Tensor qkv, torch::Tensor gate,
                               c10::optional<torch::Tensor> ab_opt,
                               c10::optional<torch::Tensor> h_opt,
                               c10::optional<torch::Tensor> ab_w_opt,
                               torch::Tensor a_log, torch::Tensor dt_bias, torch::Tensor onorm_w,
                               double eps, torch::Tensor state, torch::Tensor cu,
                               torch::Tensor slots, int64_t heads, int64_t kv_heads,
                               int64_t dim, int64_t vdim,
                               c10::optional<torch::Tensor> decay_up, bool gate_sigmoid) {
  SM_CHECK_CUDA(qkv);
  SM_CHECK_CUDA(a_log); SM_CHECK_F32(a_log); SM_CHECK_CUDA(dt_bias); SM_CHECK_F32(dt_bias);
  SM_CHECK_CUDA(onorm_w); SM_CHECK_F32(onorm_w); SM_CHECK_CUDA(state); SM_CHECK_F32(state);
  SM_CHECK_CUDA(cu); SM_CHECK_I32(cu); SM_CHECK_CUDA(slots); SM_CHECK_I32(slots);
  const int H = heads, G = kv_heads, dk = dim, vd = vdim;
  const int64_t T = qkv.size(0);
  const int C = 2 * G * dk + H * vd;
  const int B = slots.numel();
  TORCH_CHECK(G >= 1 && H % G == 0, "gated_delta_rule: heads must be a multiple of kv_heads");
  TORCH_CHECK(qkv.dim() == 2 && qkv.size(1) == C, "gated_delta_rule: qkv width");
  TORCH_CHECK(gate.is_cuda() && gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == T &&
              gate.size(1) == H * vd && gate.scalar_type() == qkv.scalar_type(), "gated_delta_rule: gate layout");
  // the write strength / step inputs: given as [T, 2H] fp32, or computed here
  // from the mixer input h [T, D] and the fp32 matrix ab_w [2H, D]
  const bool chan = decay_up.has_value();
  const int Rk = chan ? (int)decay_up->size(1) : 0;       // low-rank decay inputs
  const int abw = chan ? H + Rk : 2 * H;
  if (chan) {
    SM_CHECK_CUDA(*decay_up); SM_CHECK_F32(*decay_up);
    TORCH_CHECK(decay_up->dim() == 2 && decay_up->size(0) == (int64_t)H * dk && Rk >= 1 &&
                ab_opt.has_value(),
                "gated_delta_rule: channel decays need decay_up [H dim, R] and ab [T, H + R]");
  }
  const float* abp = nullptr;
  const float* abwp = nullptr;
  const void* hp = nullptr;
  int64_t ldh = 0;
  int Dh = 0;
  if (ab_opt.has_value()) {
    const torch::Tensor& ab = *ab_opt;
    SM_CHECK_CUDA(ab); SM_CHECK_F32(ab);
    TORCH_CHECK(ab.dim() == 2 && ab.size(0) == T && ab.size(1) == abw, "gated_delta_rule: ab width");
    abp = ab.data_ptr<float>();
  } else {
    TORCH_CHECK(h_opt.has_value() && ab_w_opt.has_value(), "gated_delta_rule: ab, or h with ab_w");
    const torch::Tensor& hh = *h_opt;
    const torch::Tensor& w = *ab_w_opt;
    SM_CHECK_CUDA(w); SM_CHECK_F32(w);
    TORCH_CHECK(hh.is_cuda() && hh.dim() == 2 && hh.stride(1) == 1 && hh.size(0) == T &&
                hh.scalar_type() == qkv.scalar_type(), "gated_delta_rule: h layout");
    TORCH_CHECK(w.dim() == 2 && w.size(0) == 2 * H && w.size(1) == hh.size(1), "gated_delta_rule: ab_w is [2H, D]");
    hp = hh.data_ptr();
    ldh = hh.stride(0);
    Dh = hh.size(1);
    abwp = w.data_ptr<float>();
  }
  TORCH_CHECK(a_log.numel() == H && dt_bias.numel() == (chan ? (int64_t)H * dk : H) &&
              onorm_w.numel() == vd, "gated_delta_rule: per-head tensors");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == (int64_t)H * dk * vd && cu.numel() == B + 1,
              "gated_delta_rule: state/batch layout");
  TORCH_CHECK(dk <= 256, "gated_delta_rule: key dim above 256");
  int dkp = 32;
  while (dkp < dk) dkp *= 2;
  // 32 state rows per lane once that gives every SIMD of the chip a wave
  // (fewer lane moves and LDS reads per multiply-add); 8 rows, four times the
  // lanes, below that
  // (measured crossover on 256 CUs: 1024 waves). Steps of a few tokens per
  // row are bound by reading and writing the state: 8 rows per lane make the
  // KS lanes of a column one contiguous run of 16-byte pieces.
  const int64_t waves32 = (int64_t)B * H * SM_CDIV(vd * (dkp / 32), 64);
  const int R = (waves32 >= 1024 && T >= 8 * (int64_t)B) ? 32 : 8;
  const int KS = dkp / R;
  auto out = torch::empty({T, (int64_t)H * vd}, qkv.options());
  if (T == 0 || B == 0) return out;
  auto f32 = qkv.options().dtype(at::kFloat);
  auto qn = torch::empty({T, G, dkp}, f32), kn = torch::empty({T, G, dkp}, f32);
  auto beta = torch::empty({T, H}, f32);
  auto decay = chan ? torch::empty({T, H, dkp}, f32) : torch::empty({T, H}, f32);
  auto o = torch::empty({T, H, vd}, f32);
  auto stream = at::cuda::getCurrentCUDAStream();
  const bool bf16 = qkv.scalar_type() == at::kBFloat16;
  if (!bf16) SM_CHECK_F32(qkv);
  dim3 gscan(B, H), gfin(T, H);
  dim3 gprep(T, abp != nullptr ? 1 : 1 + SM_CDIV(2 * H, 4));
  // channel decays: the unit q/k rows come from delta_prepare (which then
  // leaves beta/decay alone), strengths and decays from their own kernel
  const float* abq = chan ? nullptr : abp;
  if (chan) {
    auto pre = at::linear(ab_opt->slice(1, H, H + Rk), *decay_up);   // fp32 [T, H dk]
    delta_channel_decay_kernel<<<T, 256, 0, stream>>>(
        abp, abw, pre.data_ptr<float>(), H, a_log.data_ptr<float>(), dt_bias.data_ptr<float>(),
        dk, dkp, beta.data_ptr<float>(), decay.data_ptr<float>());
    SM_CHECK_LAUNCH();
  }
  if (bf16) {
    const bf16_t* xp = reinterpret_cast<const bf16_t*>(qkv.data_ptr());
    delta_prepare_kernel<bf16_t><<<gprep, 256, 0, stream>>>(
        xp, C, abq, reinterpret_cast<const bf16_t*>(hp), ldh, abwp, Dh, a_log.data_ptr<float>(),
        dt_bias.data_ptr<float>(), H, G, dk, dkp,
        qn.data_ptr<float>(), kn.data_ptr<float>(), beta.data_ptr<float>(), decay.data_ptr<float>());
    SM_CHECK_LAUNCH();
    if (chan)
      launch_scan<bf16_t, true>(KS, R, gscan, stream, xp, C, qn.data_ptr<float>(), kn.data_ptr<float>(),
                        beta.data_ptr<float>(), decay.data_ptr<float>(), state.data_ptr<float>(),
                        cu.data_ptr<int>(), slots.data_ptr<int>(), H, G, dk, vd, o.data_ptr<float>());
    else
      launch_scan<bf16_t, false>(KS, R, gscan, stream, xp, C, qn.data_ptr<float>(), kn.data_ptr<float>(),
                        beta.data_ptr<float>(), decay.data_ptr<float>(), state.data_ptr<float>(),
                        cu.data_ptr<int>(), slots.data_ptr<int>(), H, G, dk, vd, o.data_ptr<float>());
    SM_CHECK_LAUNCH();
    delta_finish_kernel<bf16_t><<<gfin, 64, 0, stream>>>(
        o.data_ptr<float>(), reinterpret_cast<const bf16_t*>(gate.data_ptr()), gate.stride(0),
        onorm_w.data_ptr<float>(), (float)eps, H, vd, gate_sigmoid ? 1 : 0,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  } else {
    const float* xp = qkv.data_ptr<float>();
    delta_prepare_kernel<float><<<gprep, 256, 0, stream>>>(
        xp, C, abq, reinterpret_cast<const float*>(hp), ldh, abwp, Dh, a_log.data_ptr<float>(),
        dt_bias.data_ptr<float>(), H, G, dk, dkp,
        qn.data_ptr<float>(), kn.data_ptr<float>(), beta.data_ptr<float>(), decay.data_ptr<float>());
    SM_CHECK_LAUNCH();
    if (chan)
      launch_scan<float, true>(KS, R, gscan, stream, xp, C, qn.data_ptr<float>(), kn.data_ptr<float>(),
                       beta.data_ptr<float>(), decay.data_ptr<float>(), state.data_ptr<float>(),
                       cu.data_ptr<int>(), slots.data_ptr<int>(), H, G, dk, vd, o.data_ptr<float>());
    else
      launch_scan<float, false>(KS, R, gscan, stream, xp, C, qn.data_ptr<float>(), kn.data_ptr<float>(),
                       beta.data_ptr<float>(), decay.data_ptr<float>(), state.data_ptr<float>(),
                       cu.data_ptr<int>(), slots.data_ptr<int>(), H, G, dk, vd, o.data_ptr<float>());
    SM_CHECK_LAUNCH();
    delta_finish_kernel<float><<<gfin, 64, 0, stream>>>(
        o.data_ptr<float>(), gate.data_ptr<float>(), gate.stride(0), onorm_w.data_ptr<float>(),
        (float)eps, H, vd, gate_sigmoid ? 1 : 0, out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}
