// Row kernels of a sandwich-norm layer (an RMS norm before AND after every
// sublayer) on an fp32 residual stream (gfx950):
//
//   add_normed_rmsnorm   residual += rmsnorm(delta) * w_post   (in place)
//                        out = rmsnorm(residual) * w_pre, or the residual
//                        itself in the activation type when w_pre is absent
//   gelu_mul_rows        gelu_tanh(z) * table[token, col0 : col0 + W]
//
// One 256-thread block per row; both statistics are fp32 block reductions.
#include "../csrc_hybrid/act_types.h"

namespace igw {

template <typename TD, typename TO>
__global__ __launch_bounds__(256) void add_normed_rmsnorm_kernel(
    TO* __restrict__ out, float* __restrict__ residual,
    const TD* __restrict__ delta, int64_t delta_rs,
    const float* __restrict__ w_post, const float* __restrict__ w_pre, int D,
    float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x, tid = threadIdx.x;
  float* res = residual + (int64_t)t * D;
  TO* o = out + (int64_t)t * D;
  float ss = 0.0f;
  if (delta) {
    const TD* dl = delta + (int64_t)t * delta_rs;
    float sd = 0.0f;
    for (int d = tid; d < D; d += 256) {
      const float x = Act<TD>::ld(dl + d);
      sd += x * x;
    }
    sd = block_reduce_sum<256>(sd, red);
    const float r1 = 1.0f / sqrtf(sd / (float)D + eps);
    __syncthreads();
    for (int d = tid; d < D; d += 256) {
      const float x = res[d] + Act<TD>::ld(dl + d) * r1 * w_post[d];
      res[d] = x;
      ss += x * x;
    }
  } else {
    for (int d = tid; d < D; d += 256) {
      const float x = res[d];
      ss += x * x;
    }
  }
  if (!w_pre) {
    for (int d = tid; d < D; d += 256) Act<TO>::st(o + d, res[d]);
    return;
  }
  ss = block_reduce_sum<256>(ss, red);
  const float r2 = 1.0f / sqrtf(ss / (float)D + eps);
  for (int d = tid; d < D; d += 256)
    Act<TO>::st(o + d, res[d] * r2 * w_pre[d]);
}

void add_normed_rmsnorm(torch::Tensor out, torch::Tensor residual,
                        c10::optional<torch::Tensor> delta,
                        c10::optional<torch::Tensor> w_post,
                        c10::optional<torch::Tensor> w_pre, double eps) {
  TORCH_CHECK(residual.is_cuda() && residual.dtype() == torch::kFloat32 &&
              residual.is_contiguous() && residual.dim() == 2);
  const int T = residual.size(0), D = residual.size(1);
  TORCH_CHECK(out.is_contiguous() && out.numel() == residual.numel());
  if (delta.has_value()) {
    TORCH_CHECK(delta->dim() == 2 && delta->size(0) == T &&
                delta->size(1) == D && delta->stride(1) == 1);
    TORCH_CHECK(w_post.has_value() && w_post->dtype() == torch::kFloat32 &&
                w_post->is_contiguous() && w_post->numel() == D);
  }
  if (w_pre.has_value())
    TORCH_CHECK(w_pre->dtype() == torch::kFloat32 && w_pre->is_contiguous() &&
                w_pre->numel() == D);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const float* wp = delta.has_value() ? (const float*)w_post->data_ptr()
                                      : nullptr;
  const float* wn = w_pre.has_value() ? (const float*)w_pre->data_ptr()
                                      : nullptr;
  const int64_t drs = delta.has_value() ? (int64_t)delta->stride(0) : 0;
#define LAUNCH_ANR(TD, TO)                                                    \
  hipLaunchKernelGGL((add_normed_rmsnorm_kernel<TD, TO>), dim3(T), dim3(256), \
                     0, stream, (TO*)out.data_ptr(),                          \
                     (float*)residual.data_ptr(),                             \
                     delta.has_value() ? (const TD*)delta->data_ptr()         \
                                       : nullptr,                             \
                     drs, wp, wn, D, (float)eps)
  const bool d16 = delta.has_value() &&
                   delta->scalar_type() == torch::kBFloat16;
  if (delta.has_value())
    TORCH_CHECK(d16 || delta->scalar_type() == torch::kFloat32,
                "delta must be bfloat16 or float32");
  IGW_DISPATCH_ACT(out, {
    if (d16) LAUNCH_ANR(uint16_t, act_t);
    else LAUNCH_ANR(float, act_t);
  });
#undef LAUNCH_ANR
  HIP_CHECK_KERNEL();
}

DEVINLINE float gelu_tanh_f32(float z) {
  const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.0f + tanhf(u));
}

template <typename T>
__global__ void gelu_mul_rows_kernel(T* __restrict__ out,
                                     const T* __restrict__ z,
                                     const T* __restrict__ table,
                                     int64_t table_rs,
                                     const int64_t* __restrict__ tokens,
                                     int64_t total, int W, int col0) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / W;
  const int c = (int)(i - t * W);
  const float e = Act<T>::ld(table + tokens[t] * table_rs + col0 + c);
  Act<T>::st(out + i, gelu_tanh_f32(Act<T>::ld(z + i)) * e);
}

void gelu_mul_rows(torch::Tensor out, torch::Tensor z, torch::Tensor table,
                   torch::Tensor tokens, int64_t col0) {
  TORCH_CHECK(z.is_cuda() && z.is_contiguous() && z.dim() == 2 &&
              out.is_contiguous() && out.dtype() == z.dtype() &&
              out.numel() == z.numel());
  const int64_t T = z.size(0);
  const int W = z.size(1);
  TORCH_CHECK(table.dim() == 2 && table.stride(1) == 1 &&
              table.dtype() == z.dtype() && col0 >= 0 &&
              col0 + W <= table.size(1));
  TORCH_CHECK(tokens.dtype() == torch::kInt64 && tokens.is_contiguous() &&
              tokens.numel() == T);
  if (T == 0 || W == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int64_t total = T * W;
  IGW_DISPATCH_ACT(z, {
    hipLaunchKernelGGL((gelu_mul_rows_kernel<act_t>),
                       dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       stream, (act_t*)out.data_ptr(),
                       (const act_t*)z.data_ptr(),
                       (const act_t*)table.data_ptr(),
                       (int64_t)table.stride(0),
                       (const int64_t*)tokens.data_ptr(), total, W,
                       (int)col0);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace igw
