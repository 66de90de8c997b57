// Shared device helpers of the sequence-mixing kernels (gfx950, wave64).
// Kernels are templated on the matrix dtype T (bf16 or float); everything
// that carries state, a norm, a score or the residual is float.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <cstdint>

#define SM_WAVE 64
#define SM_INLINE __device__ __forceinline__

typedef __hip_bfloat16 bf16_t;

SM_INLINE float to_f(float x) { return x; }
SM_INLINE float to_f(bf16_t x) { return __bfloat162float(x); }
template <typename T> SM_INLINE T from_f(float x);
template <> SM_INLINE float from_f<float>(float x) { return x; }
template <> SM_INLINE bf16_t from_f<bf16_t>(float x) { return __float2bfloat16(x); }

SM_INLINE float sm_wave_sum(float x) {
  #pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, SM_WAVE);
  return x;
}
SM_INLINE float sm_wave_max(float x) {
  #pragma unroll
  for (int off = 32; off > 0; off >>= 1) x = fmaxf(x, __shfl_xor(x, off, SM_WAVE));
  return x;
}
// Reductions over the 16 lanes of a row (lanes that share lane >> 4) on the
// VALU's lane-permute path: the two quad swaps, then the mirrors of 8 and of
// 16 lanes; afterwards every lane of the row holds the result.
template <int CTRL> SM_INLINE float sm_dpp(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
SM_INLINE float sm_row16_max(float x) {
  x = fmaxf(x, sm_dpp<0xB1>(x));    // quad_perm [1, 0, 3, 2]
  x = fmaxf(x, sm_dpp<0x4E>(x));    // quad_perm [2, 3, 0, 1]
  x = fmaxf(x, sm_dpp<0x141>(x));   // row_half_mirror
  return fmaxf(x, sm_dpp<0x140>(x));   // row_mirror
}
SM_INLINE float sm_row16_sum(float x) {
  x += sm_dpp<0xB1>(x);
  x += sm_dpp<0x4E>(x);
  x += sm_dpp<0x141>(x);
  return x + sm_dpp<0x140>(x);
}
// Sum over a block of up to 1024 threads; red needs blockDim.x / 64 floats.
SM_INLINE float sm_block_sum(float x, float* red) {
  const int lane = threadIdx.x & (SM_WAVE - 1), wid = threadIdx.x / SM_WAVE;
  const int nw = (blockDim.x + SM_WAVE - 1) / SM_WAVE;
  x = sm_wave_sum(x);
  __syncthreads();
  if (lane == 0) red[wid] = x;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}
SM_INLINE float sm_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
// clamped GLU: g = min(gate, limit), u = clamp(up, +-limit), g sigmoid(1.702 g) (u + 1)
SM_INLINE float sm_capped_glu(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sm_sigmoid(1.702f * g) * (u + 1.0f);
}

#define SM_CHECK_LAUNCH()                                                  \
  do {                                                                     \
    hipError_t e_ = hipGetLastError();                                     \
    TORCH_CHECK(e_ == hipSuccess, "HIP kernel launch failed: ",            \
                hipGetErrorString(e_));                                    \
  } while (0)

#define SM_CDIV(a, b) (((a) + (b) - 1) / (b))

#define SM_CHECK_CUDA(t) TORCH_CHECK((t).is_cuda() && (t).is_contiguous(), #t " must be a contiguous GPU tensor")
#define SM_CHECK_F32(t) TORCH_CHECK((t).scalar_type() == at::kFloat, #t " must be float32")
#define SM_CHECK_I32(t) TORCH_CHECK((t).scalar_type() == at::kInt, #t " must be int32")
