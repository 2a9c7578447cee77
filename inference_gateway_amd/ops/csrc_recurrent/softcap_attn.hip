// Causal softmax attention over paged keys and values with a score cap
// (gfx950).  For query row t (position p, sequence s) and head h on
// key/value head g = h / (H / G):
//
//   score_j = (q[t,h] . K_j[g]) * scale * temp(p),   lo <= j <= p
//   temp(p) = 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)
//   score_j <- softcap * tanh(score_j / softcap)      (softcap > 0)
//   score_j <- score_j - slope[h] * (p - j)            (slopes given)
//   out[t,h] = sum_j softmax_j(score) V_j[g]          [P]
//
// lo = max(0, p - window + 1) with a window, 0 without; with chunk > 0 also
// lo >= floor(p / chunk) * chunk (keys of the row's own position chunk).
// With sinks, exp(sink[h]) joins the softmax denominator (a key of that
// score without a value); with a gate, out[t,h] *= sigmoid(gate[t,h]).  Keys are
// [blocks, G, block, N], values [blocks, G, block, P]; N and P need not be
// equal.  Scores, probabilities and the accumulator are fp32.
//
// softcap_attention_rows: one wave per (row, head); lanes are keys for the
// scores and value entries for the weighted sum.  Works for any sizes and
// both activation types; rows of a prompt portion and decoded rows look
// the same to it (each row carries its own position and sequence).
#include "../csrc_hybrid/act_types.h"

namespace igw {

template <typename T, int NACC>
__global__ __launch_bounds__(64) void softcap_attention_rows_kernel(
    T* __restrict__ out, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions,
    float scale, float softcap, float temp_coef, int temp_every, int window,
    const float* __restrict__ slopes, int chunk,
    const float* __restrict__ sinks, const T* __restrict__ gate,
    int64_t gate_stride, int H, int G, int N, int P, int block_size) {
  extern __shared__ float lds[];
  float* ql = lds;                            // [N], pre-scaled
  float* p_lds = lds + N;                     // [64]
  int32_t* row_lds = (int32_t*)(p_lds + 64);  // [64] key's row inside cache
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  const int pos = positions[t];
  const int32_t* bt = block_table + (int64_t)row_seq[t] * max_blocks;
  int lo = window > 0 ? max(0, pos - window + 1) : 0;
  if (chunk > 0) lo = max(lo, pos / chunk * chunk);
  const float slope = slopes ? slopes[h] : 0.0f;
  const float temp =
      1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  const float qs = scale * temp;
  for (int d = lane; d < N; d += 64)
    ql[d] = Act<T>::ld(q + (int64_t)t * q_stride + h * N + d) * qs;
  __syncthreads();
  const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
  float m = -INFINITY, l = 0.0f;
  float acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc[i] = 0.0f;
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    int32_t prow = 0;
    if (valid) {
      // row index of (page, key/value head, slot) in a [.., N|P] matrix
      prow = (bt[j / block_size] * G + g) * block_size + j % block_size;
      const T* row = kcache + (int64_t)prow * N;
      float a = 0.0f;
      for (int d = 0; d < N; ++d) a += ql[d] * Act<T>::ld(row + d);
      s = softcap > 0.0f ? softcap * tanhf(a * inv_cap) : a;
      s -= slope * (float)(pos - j);
    }
    const float m_new = fmaxf(m, wave_reduce_max(s));
    const float corr = expf(m - m_new);
    const float pr = valid ? expf(s - m_new) : 0.0f;
    l = l * corr + wave_reduce_sum(pr);
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] *= corr;
    m = m_new;
    __syncthreads();
    p_lds[lane] = pr;
    row_lds[lane] = prow;
    __syncthreads();
    const int n = min(64, pos - j0 + 1);
    for (int kx = 0; kx < n; ++kx) {
      const float pk = p_lds[kx];
      const T* row = vcache + (int64_t)row_lds[kx] * P;
#pragma unroll
      for (int i = 0; i < NACC; ++i) {
        const int d = lane + 64 * i;
        if (d < P) acc[i] += pk * Act<T>::ld(row + d);
      }
    }
  }
  // the sink's term relative to the running maximum (an overflow to
  // infinity gives the right limit, an all-zero row)
  if (sinks) l += expf(sinks[h] - m);
  const float inv = 1.0f / l;
  T* o = out + ((int64_t)t * H + h) * P;
  const T* gt = gate ? gate + (int64_t)t * gate_stride + h * P : nullptr;
#pragma unroll
  for (int i = 0; i < NACC; ++i) {
    const int d = lane + 64 * i;
    if (d < P) {
      float y = acc[i] * inv;
      if (gt) y *= sigmoid_f32(Act<T>::ld(gt + d));
      Act<T>::st(o + d, y);
    }
  }
}

void softcap_attention(torch::Tensor out, torch::Tensor q, torch::Tensor kcache,
                       torch::Tensor vcache, torch::Tensor block_table,
                       torch::Tensor row_seq, torch::Tensor positions,
                       double scale, double softcap, double temp_coef,
                       int64_t temp_every, int64_t window,
                       c10::optional<torch::Tensor> slopes, int64_t chunk,
                       c10::optional<torch::Tensor> sinks,
                       c10::optional<torch::Tensor> gate) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.stride(1) == 1);
  TORCH_CHECK(kcache.is_contiguous() && kcache.dim() == 4 &&
              vcache.is_contiguous() && vcache.dim() == 4 &&
              kcache.dtype() == q.dtype() && vcache.dtype() == q.dtype());
  const int T = q.size(0), G = kcache.size(1), bs = kcache.size(2);
  const int N = kcache.size(3), P = vcache.size(3);
  TORCH_CHECK(q.size(1) % N == 0);
  const int H = q.size(1) / N;
  TORCH_CHECK(H % G == 0 && vcache.size(0) == kcache.size(0) &&
              vcache.size(1) == G && vcache.size(2) == bs);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.numel() == (int64_t)T * H * P);
  TORCH_CHECK(block_table.dtype() == torch::kInt32 &&
              block_table.is_contiguous() && block_table.dim() == 2);
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
  TORCH_CHECK(P <= 1024, "value width above 1024 is not supported");
  TORCH_CHECK(temp_every >= 1 && chunk >= 0);
  if (slopes.has_value())
    TORCH_CHECK(slopes->dtype() == torch::kFloat32 &&
                slopes->is_contiguous() && slopes->numel() == H);
  if (sinks.has_value())
    TORCH_CHECK(sinks->dtype() == torch::kFloat32 && sinks->is_contiguous() &&
                sinks->numel() == H);
  if (gate.has_value())
    TORCH_CHECK(gate->dtype() == q.dtype() && gate->dim() == 2 &&
                gate->stride(1) == 1 && gate->size(0) == T &&
                gate->size(1) == (int64_t)H * P);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const size_t shmem = (size_t)(N + 128) * sizeof(float);
  const int nacc = (P + 63) / 64;
#define LAUNCH_ROWS(NA)                                                      \
  hipLaunchKernelGGL(                                                        \
      (softcap_attention_rows_kernel<act_t, NA>), dim3(T, H), dim3(64),      \
      shmem, stream, (act_t*)out.data_ptr(), (const act_t*)q.data_ptr(),     \
      (int64_t)q.stride(0), (const act_t*)kcache.data_ptr(),                 \
      (const act_t*)vcache.data_ptr(),                                       \
      (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),      \
      (const int32_t*)row_seq.data_ptr(),                                    \
      (const int32_t*)positions.data_ptr(), (float)scale, (float)softcap,    \
      (float)temp_coef, (int)temp_every, (int)window,                        \
      slopes.has_value() ? (const float*)slopes->data_ptr() : nullptr,       \
      (int)chunk,                                                            \
      sinks.has_value() ? (const float*)sinks->data_ptr() : nullptr,         \
      gate.has_value() ? (const act_t*)gate->data_ptr() : nullptr,           \
      gate.has_value() ? (int64_t)gate->stride(0) : 0, H, G, N, P, bs)
  IGW_DISPATCH_ACT(q, {
    if (nacc <= 1) LAUNCH_ROWS(1);
    else if (nacc <= 2) LAUNCH_ROWS(2);
    else if (nacc <= 4) LAUNCH_ROWS(4);
    else if (nacc <= 8) LAUNCH_ROWS(8);
    else LAUNCH_ROWS(16);
  });
#undef LAUNCH_ROWS
  HIP_CHECK_KERNEL();
}

}  // namespace igw
