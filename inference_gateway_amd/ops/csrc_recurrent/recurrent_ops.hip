// Row-wise kernels of the recurrent mixers (gfx950).
//
//   embed_pair_norm    token row * scale + hashed (previous, current) pair
//                      row + position row, RMS norm -> fp32 residual
//   causal_conv        short per-channel causal filter over ragged
//                      sequences, history in a slot buffer
//   token_shift_mix    h + (h_prev - h) * mu for several mixing vectors
//   mlstm_gates        capped exponential gates with a running maximum
//   ssm_gates          softplus step sizes and their decays
//   head_norm_gate     read-out epilogue: normaliser division, grouped
//                      RMS norm, sigmoid / silu gate
//   append_paged_kv    keys and values of unequal width into pages
//   rmsnorm_pair_mean  average of two RMS-normed branches
//
// A batch is ragged: rows of sequence s are [seq_cu[s], seq_cu[s+1]), its
// first row sits at position seq_start[s], its state in row seq_slots[s]
// of a slot buffer.  A sequence that starts at position 0 reads no state.
// All arithmetic is fp32; loads and stores are in the activation type.
#include "../csrc_hybrid/act_types.h"

namespace igw {

constexpr int RROW_BLOCK = 256;

DEVINLINE float rrow_block_sum(float x, float* lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  x = wave_reduce_sum(x);
  __syncthreads();  // lds may still be read from a previous reduction
  if (lane == 0) lds[wave] = x;
  __syncthreads();
  float r = 0.0f;
#pragma unroll
  for (int w = 0; w < RROW_BLOCK / 64; ++w) r += lds[w];
  return r;
}

DEVINLINE float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// 4 consecutive activations <-> 4 floats
template <typename T>
struct Val4;
template <>
struct Val4<float> {
  static DEVINLINE float4 ld(const float* p) { return *(const float4*)p; }
  static DEVINLINE void st(float* p, float4 v) { *(float4*)p = v; }
};
template <>
struct Val4<uint16_t> {
  static DEVINLINE float4 ld(const uint16_t* p) {
    const ushort4x r = *(const ushort4x*)p;
    return make_float4(bf16_to_f32(r.v[0]), bf16_to_f32(r.v[1]),
                       bf16_to_f32(r.v[2]), bf16_to_f32(r.v[3]));
  }
  static DEVINLINE void st(uint16_t* p, float4 v) {
    ushort4x r;
    r.v[0] = f32_to_bf16(v.x);
    r.v[1] = f32_to_bf16(v.y);
    r.v[2] = f32_to_bf16(v.z);
    r.v[3] = f32_to_bf16(v.w);
    *(ushort4x*)p = r;
  }
};

// ---------------------------------------------------------------------------
// embedding
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(RROW_BLOCK) void embed_pair_norm_kernel(
    float* __restrict__ out, const int64_t* __restrict__ tokens,
    const int32_t* __restrict__ positions, int32_t* __restrict__ prev_tok,
    const int32_t* __restrict__ seq_cu, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ row_seq,
    const T* __restrict__ embed, const T* __restrict__ pair,
    const T* __restrict__ pos, const float* __restrict__ w, int D,
    int pos_rows, float scale, int64_t buckets, int64_t mul_prev,
    int64_t mul_cur, float eps) {
  __shared__ float lds[RROW_BLOCK / 64];
  const int t = blockIdx.x;
  const int s = row_seq[t];
  const int r0 = seq_cu[s], r1 = seq_cu[s + 1];
  const int64_t tok = tokens[t];
  int64_t prow;
  if (t > r0) {
    prow = (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets;
  } else {
    // the sequence's first row of this step: the only reader of the slot,
    // and its writer (the step's last token)
    const int slot = seq_slots[s];
    if (seq_start[s] > 0)
      prow = ((int64_t)prev_tok[slot] * mul_prev + tok * mul_cur) % buckets;
    else
      prow = buckets;
    __syncthreads();
    if (threadIdx.x == 0) prev_tok[slot] = (int32_t)tokens[r1 - 1];
  }
  const int p = min(positions[t], pos_rows - 1);
  const T* e = embed + tok * D;
  const T* b = pair + prow * D;
  const T* q = pos + (int64_t)p * D;
  float* o = out + (int64_t)t * D;
  float sq = 0.0f;
  for (int d = threadIdx.x; d < D; d += RROW_BLOCK) {
    const float x = Act<T>::ld(e + d) * scale + Act<T>::ld(b + d) +
                    Act<T>::ld(q + d);
    o[d] = x;
    sq += x * x;
  }
  const float rstd = 1.0f / sqrtf(rrow_block_sum(sq, lds) / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += RROW_BLOCK) o[d] = o[d] * rstd * w[d];
}

void embed_pair_norm(torch::Tensor out, torch::Tensor tokens,
                     torch::Tensor positions, torch::Tensor prev_tok,
                     torch::Tensor seq_cu, torch::Tensor seq_start,
                     torch::Tensor seq_slots, torch::Tensor row_seq,
                     torch::Tensor embed, torch::Tensor pair, torch::Tensor pos,
                     torch::Tensor w, double scale, int64_t buckets,
                     int64_t mul_prev, int64_t mul_cur, double eps) {
  const int T = tokens.numel(), D = embed.size(1);
  TORCH_CHECK(out.is_cuda() && out.dtype() == torch::kFloat32 &&
              out.is_contiguous() && out.size(0) == T && out.size(1) == D);
  TORCH_CHECK(tokens.dtype() == torch::kInt64 && tokens.is_contiguous());
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T);
  TORCH_CHECK(prev_tok.dtype() == torch::kInt32 && prev_tok.is_contiguous());
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 &&
              seq_start.dtype() == torch::kInt32 &&
              seq_slots.dtype() == torch::kInt32);
  TORCH_CHECK(embed.is_contiguous() && pair.is_contiguous() &&
              pos.is_contiguous() && pair.size(1) == D && pos.size(1) == D &&
              pair.dtype() == embed.dtype() && pos.dtype() == embed.dtype());
  TORCH_CHECK(pair.size(0) == buckets + 1, "pair table needs buckets+1 rows");
  TORCH_CHECK(w.dtype() == torch::kFloat32 && w.numel() == D);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(embed, {
    hipLaunchKernelGGL(
        (embed_pair_norm_kernel<act_t>), dim3(T), dim3(RROW_BLOCK), 0, stream,
        (float*)out.data_ptr(), (const int64_t*)tokens.data_ptr(),
        (const int32_t*)positions.data_ptr(), (int32_t*)prev_tok.data_ptr(),
        (const int32_t*)seq_cu.data_ptr(), (const int32_t*)seq_start.data_ptr(),
        (const int32_t*)seq_slots.data_ptr(),
        (const int32_t*)row_seq.data_ptr(), (const act_t*)embed.data_ptr(),
        (const act_t*)pair.data_ptr(), (const act_t*)pos.data_ptr(),
        (const float*)w.data_ptr(), D, (int)pos.size(0), (float)scale, buckets,
        mul_prev, mul_cur, (float)eps);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// short causal convolution
// ---------------------------------------------------------------------------
constexpr int CONV_MAX_TAPS = 8;

// one thread per (row, channel): y = sum_j w[c, j] * u[t - taps + 1 + j]
// with u = this step's rows, the slot history before them, zeros before
// the sequence's start
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ row_seq,
    int C, int taps, int silu) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = row_seq[t];
  const int r0 = seq_cu[s];
  const bool has_hist = seq_start[s] > 0;
  const float* hist = state + (int64_t)seq_slots[s] * (taps - 1) * C;
  float acc = bias ? bias[c] : 0.0f;
  for (int j = 0; j < taps; ++j) {
    const int r = t - taps + 1 + j;
    float u = 0.0f;
    if (r >= r0) {
      u = Act<T>::ld(x + (int64_t)r * x_stride + c);
    } else if (has_hist) {
      // history row index: taps-1 rows, oldest first; row r0-1 is the last
      u = hist[(int64_t)(taps - 1 - (r0 - r)) * C + c];
    }
    acc += w[c * taps + j] * u;
  }
  if (silu) acc = silu_f32(acc);
  Act<T>::st(out + (int64_t)t * C + c, acc);
}

// 8 consecutive activations <-> 8 floats (16-byte accesses for bf16)
template <typename T>
struct Row8;
template <>
struct Row8<float> {
  static DEVINLINE void ld(const float* p, float* o) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
  static DEVINLINE void st(float* p, const float* v) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <>
struct Row8<uint16_t> {
  static DEVINLINE void ld(const uint16_t* p, float* o) {
    const ushort8 r = *(const ushort8*)p;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = bf16_to_f32(r.v[e]);
  }
  static DEVINLINE void st(uint16_t* p, const float* v) {
    ushort8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r.v[e] = f32_to_bf16(v[e]);
    *(ushort8*)p = r;
  }
};

// the same filter, one thread per (row, 8 channels): C % 8 == 0 and every
// row 16-byte aligned
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_vec8_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ row_seq,
    int C, int taps, int silu) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  const int s = row_seq[t];
  const int r0 = seq_cu[s];
  const bool has_hist = seq_start[s] > 0;
  const float* hist = state + (int64_t)seq_slots[s] * (taps - 1) * C;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = bias ? bias[c + e] : 0.0f;
  for (int j = 0; j < taps; ++j) {
    const int r = t - taps + 1 + j;
    float u[8];
    if (r >= r0) {
      Row8<T>::ld(x + (int64_t)r * x_stride + c, u);
    } else if (has_hist) {
      Row8<float>::ld(hist + (int64_t)(taps - 1 - (r0 - r)) * C + c, u);
    } else {
      continue;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += w[(c + e) * taps + j] * u[e];
  }
  if (silu) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = silu_f32(acc[e]);
  }
  Row8<T>::st(out + (int64_t)t * C + c, acc);
}

// one thread per (ROWS consecutive rows, 8 channels), filter length known
// at compile time: the rows' inputs and the filter are loaded once and
// shared by the ROWS outputs
template <typename T, int TAPS, int ROWS>
__global__ __launch_bounds__(256) void causal_conv_tile_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ row_seq,
    int Trows, int C, int silu) {
  const int t0 = blockIdx.x * ROWS;
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  float wr[8][TAPS];
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wr[e][j] = w[(c + e) * TAPS + j];
  float xr[TAPS - 1 + ROWS][8];
#pragma unroll
  for (int k = 0; k < TAPS - 1 + ROWS; ++k) {
    const int r = t0 - (TAPS - 1) + k;
    if (r >= 0 && r < Trows) {
      Row8<T>::ld(x + (int64_t)r * x_stride + c, xr[k]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) xr[k][e] = 0.0f;
    }
  }
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int t = t0 + i;
    if (t >= Trows) break;
    const int s = row_seq[t];
    const int r0 = seq_cu[s];
    const bool has_hist = seq_start[s] > 0;
    const float* hist = state + (int64_t)seq_slots[s] * (TAPS - 1) * C;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = bias ? bias[c + e] : 0.0f;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int r = t - TAPS + 1 + j;
      if (r >= r0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += wr[e][j] * xr[i + j][e];
      } else if (has_hist) {
        float u[8];
        Row8<float>::ld(hist + (int64_t)(TAPS - 1 - (r0 - r)) * C + c, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += wr[e][j] * u[e];
      }
    }
    if (silu) {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] *= sigmoid_for<T>(acc[e]);
    }
    Row8<T>::st(out + (int64_t)t * C + c, acc);
  }
}

// one thread per (sequence, channel): history <- last taps-1 inputs
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(
    const T* __restrict__ x, int64_t x_stride, float* __restrict__ state,
    const int32_t* __restrict__ seq_cu, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, int C, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = seq_cu[s], r1 = seq_cu[s + 1];
  const int n = r1 - r0;
  if (n == 0) return;
  float* hist = state + (int64_t)seq_slots[s] * (taps - 1) * C;
  const bool has_hist = seq_start[s] > 0;
  float old[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j)
    old[j] = (j < taps - 1 && has_hist) ? hist[(int64_t)j * C + c] : 0.0f;
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    if (j >= taps - 1) break;
    // new history row j is input index n - (taps-1) + j of this step
    const int i = n - (taps - 1) + j;
    float v;
    if (i >= 0) {
      v = Act<T>::ld(x + (int64_t)(r0 + i) * x_stride + c);
    } else {
      const int k = j + n;  // old row j + n (shifted by the new rows)
      v = 0.0f;
#pragma unroll
      for (int m = 0; m < CONV_MAX_TAPS; ++m)
        if (m == k) v = old[m];
    }
    hist[(int64_t)j * C + c] = v;
  }
}

void causal_conv(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                 c10::optional<torch::Tensor> bias, torch::Tensor state,
                 torch::Tensor seq_cu, torch::Tensor seq_start,
                 torch::Tensor seq_slots, torch::Tensor row_seq, bool silu) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.stride(1) == 1);
  const int T = x.size(0), C = x.size(1), taps = w.size(1);
  const int S = seq_slots.numel();
  TORCH_CHECK(out.is_contiguous() && out.dtype() == x.dtype() &&
              out.size(0) == T && out.size(1) == C);
  TORCH_CHECK(w.dtype() == torch::kFloat32 && w.is_contiguous() &&
              w.size(0) == C);
  TORCH_CHECK(taps >= 1 && taps <= CONV_MAX_TAPS + 1, "taps out of range");
  if (bias.has_value())
    TORCH_CHECK(bias->dtype() == torch::kFloat32 && bias->numel() == C);
  TORCH_CHECK(state.dtype() == torch::kFloat32 && state.is_contiguous() &&
              state.size(1) >= (int64_t)(taps - 1) * C);
  TORCH_CHECK(state.size(1) == (int64_t)(taps - 1) * C || taps == 1,
              "history buffer width must be (taps-1)*channels");
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 && seq_cu.numel() == S + 1 &&
              seq_start.dtype() == torch::kInt32 && seq_start.numel() == S &&
              seq_slots.dtype() == torch::kInt32);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const bool vec8 =
      C % 8 == 0 && (x.stride(0) * x.element_size()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(state.data_ptr()) % 16 == 0;
#define LAUNCH_CONV_TILE(TP)                                                  \
  hipLaunchKernelGGL(                                                        \
      (causal_conv_tile_kernel<act_t, TP, 4>),                               \
      dim3((T + 3) / 4, (C / 8 + 255) / 256), dim3(256), 0, stream,          \
      (act_t*)out.data_ptr(), (const act_t*)x.data_ptr(),                    \
      (int64_t)x.stride(0), (const float*)w.data_ptr(),                      \
      bias.has_value() ? (const float*)bias->data_ptr() : nullptr,           \
      (const float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),     \
      (const int32_t*)seq_start.data_ptr(),                                  \
      (const int32_t*)seq_slots.data_ptr(),                                  \
      (const int32_t*)row_seq.data_ptr(), T, C, silu ? 1 : 0)
  IGW_DISPATCH_ACT(x, {
    if (vec8 && taps == 4) LAUNCH_CONV_TILE(4);
    else if (vec8 && taps == 3) LAUNCH_CONV_TILE(3);
    else if (vec8 && taps == 2) LAUNCH_CONV_TILE(2);
    else if (vec8)
      hipLaunchKernelGGL(
          (causal_conv_vec8_kernel<act_t>), dim3(T, (C / 8 + 255) / 256),
          dim3(256), 0, stream, (act_t*)out.data_ptr(),
          (const act_t*)x.data_ptr(), (int64_t)x.stride(0),
          (const float*)w.data_ptr(),
          bias.has_value() ? (const float*)bias->data_ptr() : nullptr,
          (const float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),
          (const int32_t*)seq_start.data_ptr(),
          (const int32_t*)seq_slots.data_ptr(),
          (const int32_t*)row_seq.data_ptr(), C, taps, silu ? 1 : 0);
    else
    hipLaunchKernelGGL(
        (causal_conv_kernel<act_t>), dim3(T, (C + 255) / 256), dim3(256), 0,
        stream, (act_t*)out.data_ptr(), (const act_t*)x.data_ptr(),
        (int64_t)x.stride(0), (const float*)w.data_ptr(),
        bias.has_value() ? (const float*)bias->data_ptr() : nullptr,
        (const float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),
        (const int32_t*)seq_start.data_ptr(),
        (const int32_t*)seq_slots.data_ptr(),
        (const int32_t*)row_seq.data_ptr(), C, taps, silu ? 1 : 0);
    if (taps > 1)
      hipLaunchKernelGGL(
          (conv_state_kernel<act_t>), dim3((C + 255) / 256, S), dim3(256), 0,
          stream, (const act_t*)x.data_ptr(), (int64_t)x.stride(0),
          (float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),
          (const int32_t*)seq_start.data_ptr(),
          (const int32_t*)seq_slots.data_ptr(), C, taps);
  });
#undef LAUNCH_CONV_TILE
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// token shift
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(
    T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
    float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ row_seq,
    int Trows, int D, int M) {
  const int t = blockIdx.x;
  const int d = blockIdx.y * 256 + threadIdx.x;
  if (d >= D) return;
  const int s = row_seq[t];
  const int r0 = seq_cu[s];
  const float cur = Act<T>::ld(h + (int64_t)t * D + d);
  float prev;
  if (t > r0) {
    prev = Act<T>::ld(h + (int64_t)(t - 1) * D + d);
  } else {
    // first row of the sequence in this step: sole reader and writer of
    // the slot entry
    float* st = state + (int64_t)seq_slots[s] * D + d;
    prev = seq_start[s] > 0 ? *st : 0.0f;
    *st = Act<T>::ld(h + (int64_t)(seq_cu[s + 1] - 1) * D + d);
  }
  const float diff = prev - cur;
  for (int m = 0; m < M; ++m)
    Act<T>::st(out + ((int64_t)m * Trows + t) * D + d,
               cur + diff * mu[m * D + d]);
}

// D % 8 == 0: one thread per (row, 8 channels), 16-byte accesses
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_vec8_kernel(
    T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
    float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ row_seq,
    int Trows, int D, int M) {
  const int t = blockIdx.x;
  const int d = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (d >= D) return;
  const int s = row_seq[t];
  const int r0 = seq_cu[s];
  float cur[8], prev[8];
  Row8<T>::ld(h + (int64_t)t * D + d, cur);
  if (t > r0) {
    Row8<T>::ld(h + (int64_t)(t - 1) * D + d, prev);
  } else {
    float* st = state + (int64_t)seq_slots[s] * D + d;
    if (seq_start[s] > 0) {
      Row8<float>::ld(st, prev);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) prev[e] = 0.0f;
    }
    float last[8];
    Row8<T>::ld(h + (int64_t)(seq_cu[s + 1] - 1) * D + d, last);
    Row8<float>::st(st, last);
  }
  for (int m = 0; m < M; ++m) {
    float w[8], y[8];
    Row8<float>::ld(mu + (int64_t)m * D + d, w);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = cur[e] + (prev[e] - cur[e]) * w[e];
    Row8<T>::st(out + ((int64_t)m * Trows + t) * D + d, y);
  }
}

void token_shift_mix(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                     torch::Tensor state, torch::Tensor seq_cu,
                     torch::Tensor seq_start, torch::Tensor seq_slots,
                     torch::Tensor row_seq) {
  TORCH_CHECK(h.is_cuda() && h.is_contiguous() && h.dim() == 2);
  const int T = h.size(0), D = h.size(1), M = mu.size(0);
  TORCH_CHECK(out.is_contiguous() && out.dtype() == h.dtype() &&
              out.numel() == (int64_t)M * T * D);
  TORCH_CHECK(mu.dtype() == torch::kFloat32 && mu.is_contiguous() &&
              mu.size(1) == D);
  TORCH_CHECK(state.dtype() == torch::kFloat32 && state.is_contiguous() &&
              state.size(1) == D);
  TORCH_CHECK(row_seq.dtype() == torch::kInt32 && row_seq.numel() == T);
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 &&
              seq_start.dtype() == torch::kInt32 &&
              seq_slots.dtype() == torch::kInt32);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(h, {
    if (D % 8 == 0)
      hipLaunchKernelGGL(
          (token_shift_mix_vec8_kernel<act_t>), dim3(T, (D / 8 + 255) / 256),
          dim3(256), 0, stream, (act_t*)out.data_ptr(),
          (const act_t*)h.data_ptr(), (const float*)mu.data_ptr(),
          (float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),
          (const int32_t*)seq_start.data_ptr(),
          (const int32_t*)seq_slots.data_ptr(),
          (const int32_t*)row_seq.data_ptr(), T, D, M);
    else
    hipLaunchKernelGGL(
        (token_shift_mix_kernel<act_t>), dim3(T, (D + 255) / 256), dim3(256),
        0, stream, (act_t*)out.data_ptr(), (const act_t*)h.data_ptr(),
        (const float*)mu.data_ptr(), (float*)state.data_ptr(),
        (const int32_t*)seq_cu.data_ptr(), (const int32_t*)seq_start.data_ptr(),
        (const int32_t*)seq_slots.data_ptr(),
        (const int32_t*)row_seq.data_ptr(), T, D, M);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// gates
// ---------------------------------------------------------------------------
DEVINLINE float logsigmoid_f32(float x) {
  // -softplus(-x), stable on both sides
  return fminf(x, 0.0f) - log1pf(expf(-fabsf(x)));
}

// One wave per (sequence, head), 64 rows per pass.  The recurrence m_t =
// max(f_t + m_(t-1), i_t) is the composition of the maps m -> max(m + a, b)
// with (a, b) = (f_t, i_t); composing (a1, b1) then (a2, b2) gives (a1 +
// a2, max(b1 + a2, b2)), an associative operator, so the rows of a pass are
// combined by a shuffle scan and m_t = max(m_start + A_t, B_t).  No
// difference of large sums is ever formed.
__global__ __launch_bounds__(64) void mlstm_gates_kernel(
    float* __restrict__ out, const float* __restrict__ pre,
    float* __restrict__ m_state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, int T, int H, int S, float cap) {
  const int s = blockIdx.x / H, h = blockIdx.x % H, lane = threadIdx.x;
  const int r0 = seq_cu[s], r1 = seq_cu[s + 1];
  if (r1 == r0) return;
  float* ms = m_state + (int64_t)seq_slots[s] * H + h;
  float m = seq_start[s] > 0 ? *ms : 0.0f;
  const float inv_cap = 1.0f / cap;
  float* decay = out;
  float* kscale = out + (int64_t)T * H;
  float* floor_ = out + (int64_t)2 * T * H;
  for (int c0 = r0; c0 < r1; c0 += 64) {
    const int t = c0 + lane;
    const bool valid = t < r1;
    float gi = -INFINITY, gf = 0.0f;
    if (valid) {
      gi = cap * tanhf(pre[(int64_t)t * 2 * H + h] * inv_cap);
      gf = logsigmoid_f32(cap *
                          tanhf(pre[(int64_t)t * 2 * H + H + h] * inv_cap));
    }
    float a = gf, b = gi;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float pa = __shfl_up(a, off, 64), pb = __shfl_up(b, off, 64);
      if (lane >= off) {
        b = fmaxf(pb + a, b);
        a = pa + a;
      }
    }
    const float m_t = fmaxf(m + a, b);
    float m_prev = __shfl_up(m_t, 1, 64);
    if (lane == 0) m_prev = m;
    if (valid) {
      decay[(int64_t)t * H + h] = expf(gf + m_prev - m_t);
      kscale[(int64_t)t * H + h] = expf(gi - m_t);
      floor_[(int64_t)t * H + h] = expf(-m_t);
    }
    m = __shfl(m_t, min(63, r1 - c0 - 1), 64);
  }
  if (lane == 0) *ms = m;
}

void mlstm_gates(torch::Tensor out, torch::Tensor pre, double cap,
                 torch::Tensor m_state, torch::Tensor seq_cu,
                 torch::Tensor seq_start, torch::Tensor seq_slots) {
  TORCH_CHECK(pre.is_cuda() && pre.dtype() == torch::kFloat32 &&
              pre.is_contiguous() && pre.dim() == 2 && pre.size(1) % 2 == 0);
  const int T = pre.size(0), H = pre.size(1) / 2, S = seq_slots.numel();
  TORCH_CHECK(out.dtype() == torch::kFloat32 && out.is_contiguous() &&
              out.numel() == (int64_t)3 * T * H);
  TORCH_CHECK(m_state.dtype() == torch::kFloat32 && m_state.is_contiguous() &&
              m_state.size(1) == H);
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 && seq_cu.numel() == S + 1 &&
              seq_start.dtype() == torch::kInt32 &&
              seq_slots.dtype() == torch::kInt32);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3(S * H), dim3(64), 0, stream, (float*)out.data_ptr(),
                     (const float*)pre.data_ptr(), (float*)m_state.data_ptr(),
                     (const int32_t*)seq_cu.data_ptr(),
                     (const int32_t*)seq_start.data_ptr(),
                     (const int32_t*)seq_slots.data_ptr(), T, H, S, (float)cap);
  HIP_CHECK_KERNEL();
}

__global__ __launch_bounds__(256) void ssm_gates_kernel(
    float* __restrict__ out, const float* __restrict__ dt_pre,
    const float* __restrict__ a_log, int64_t n, int H) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float x = dt_pre[i];
  // softplus, stable on both sides
  const float dt = fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x)));
  out[i] = expf(-expf(a_log[i % H]) * dt);
  out[n + i] = dt;
}

void ssm_gates(torch::Tensor out, torch::Tensor dt_pre, torch::Tensor a_log) {
  TORCH_CHECK(dt_pre.is_cuda() && dt_pre.dtype() == torch::kFloat32 &&
              dt_pre.is_contiguous() && dt_pre.dim() == 2);
  const int64_t n = dt_pre.numel();
  const int H = dt_pre.size(1);
  TORCH_CHECK(out.dtype() == torch::kFloat32 && out.is_contiguous() &&
              out.numel() == 2 * n);
  TORCH_CHECK(a_log.dtype() == torch::kFloat32 && a_log.numel() == H);
  if (n == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(ssm_gates_kernel, dim3((n + 255) / 256), dim3(256), 0,
                     stream, (float*)out.data_ptr(),
                     (const float*)dt_pre.data_ptr(),
                     (const float*)a_log.data_ptr(), n, H);
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// read-out epilogue over o fp32 [T, C], C = H * P: optional division of
// every head by max(|den|, floor) + 1e-6 (den, floor [T, H]), RMS norm in
// groups of `group` channels times w, sigmoid / silu gate before or after.
// A wave takes HNG_PAIRS consecutive (row, group) pairs at once (all their
// loads are in flight together; the values wait in registers between the
// statistic and the store), four waves per workgroup; a lane holds VPL
// runs of VW consecutive channels (16-byte loads when VW = 4):
// group <= 64 * VPL * VW.
// ---------------------------------------------------------------------------
constexpr int HNG_PAIRS = 4;

template <typename T, int VW>
DEVINLINE void hng_load(const float* o, const T* g, float* v, float* z) {
  if constexpr (VW == 4) {
    const float4 a = *(const float4*)o;
    const float4 b = Val4<T>::ld(g);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    z[0] = b.x; z[1] = b.y; z[2] = b.z; z[3] = b.w;
  } else if constexpr (VW == 2) {
    const float2 a = *(const float2*)o;
    v[0] = a.x; v[1] = a.y;
    z[0] = Act<T>::ld(g);
    z[1] = Act<T>::ld(g + 1);
  } else {
    v[0] = *o;
    z[0] = Act<T>::ld(g);
  }
}

// gate value in the activation type's precision class: exact functions
// for fp32 activations, the hardware exp / rcp for bf16
template <typename T>
DEVINLINE float gate_value(float z, int silu) {
  const float s = sigmoid_for<T>(z);
  return silu ? z * s : s;
}

template <typename T, int VPL, int VW>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(
    T* __restrict__ out, const float* __restrict__ o,
    const T* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ w, const float* __restrict__ den,
    const float* __restrict__ floor_, int H, int P, int group, float eps,
    int gate_silu, int gate_first, int64_t npairs) {
  const int lane = threadIdx.x & 63;
  const int C = H * P;
  const int ng = C / group;
  // pairs are numbered row-major (row, group); npairs < 2^31 (host check)
  const int first = (blockIdx.x * 4 + (threadIdx.x >> 6)) * HNG_PAIRS;
  const int np = (int)npairs;
  const int t0 = first / ng, g0 = first - t0 * ng;
  const bool one_head = group == P;
  int tj[HNG_PAIRS], gj[HNG_PAIRS];
#pragma unroll
  for (int j = 0; j < HNG_PAIRS; ++j) {
    // HNG_PAIRS <= ng or not: walk (row, group) forward, clamp at the end
    int g = g0 + j, t = t0;
    while (g >= ng) { g -= ng; ++t; }
    if (first + j >= np) { t = (np - 1) / ng; g = (np - 1) - t * ng; }
    tj[j] = t;
    gj[j] = g;
  }
  float val[HNG_PAIRS][VPL][VW], gz[HNG_PAIRS][VPL][VW];
  float scl[HNG_PAIRS][VPL];
#pragma unroll
  for (int j = 0; j < HNG_PAIRS; ++j) {
    const int t = tj[j], c0 = gj[j] * group;
#pragma unroll
    for (int e = 0; e < VPL; ++e) {
      const int i = (lane + 64 * e) * VW;
      scl[j][e] = 1.0f;
#pragma unroll
      for (int x = 0; x < VW; ++x) val[j][e][x] = gz[j][e][x] = 0.0f;
      if (i < group) {
        const int c = c0 + i;
        hng_load<T, VW>(o + (int64_t)t * C + c,
                        gate + (int64_t)t * gate_stride + c, val[j][e],
                        gz[j][e]);
        if (den != nullptr) {
          // VW channels never straddle a head: P % VW == 0
          const int h = one_head ? gj[j] : c / P;
          const float d = fabsf(den[(int64_t)t * H + h]);
          const float f = floor_ ? floor_[(int64_t)t * H + h] : 0.0f;
          scl[j][e] = 1.0f / (fmaxf(d, f) + 1e-6f);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < HNG_PAIRS; ++j) {
    float sq = 0.0f;
#pragma unroll
    for (int e = 0; e < VPL; ++e)
#pragma unroll
      for (int x = 0; x < VW; ++x) {
        const float z = gz[j][e][x];
        const float a = gate_value<T>(z, gate_silu);
        float v = val[j][e][x] * scl[j][e];
        if (gate_first) v *= a;
        gz[j][e][x] = a;
        val[j][e][x] = v;
        sq += v * v;        // entries past the group are zero
      }
    const float rstd = 1.0f / sqrtf(wave_reduce_sum(sq) / (float)group + eps);
    if (first + j >= np) continue;
    const int t = tj[j], c0 = gj[j] * group;
#pragma unroll
    for (int e = 0; e < VPL; ++e) {
      const int i = (lane + 64 * e) * VW;
      if (i >= group) continue;
      float r[VW];
#pragma unroll
      for (int x = 0; x < VW; ++x) {
        r[x] = val[j][e][x] * rstd * w[c0 + i + x];
        if (!gate_first) r[x] *= gz[j][e][x];
      }
      T* dst = out + (int64_t)t * C + c0 + i;
      if constexpr (VW == 4) {
        Val4<T>::st(dst, make_float4(r[0], r[1], r[2], r[3]));
      } else {
#pragma unroll
        for (int x = 0; x < VW; ++x) Act<T>::st(dst + x, r[x]);
      }
    }
  }
}

// any group size: one (row, group) pair per wave at a time, two passes
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_wide_kernel(
    T* __restrict__ out, const float* __restrict__ o,
    const T* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ w, const float* __restrict__ den,
    const float* __restrict__ floor_, int H, int P, int group, float eps,
    int gate_silu, int gate_first, int64_t npairs) {
  const int lane = threadIdx.x & 63;
  const int C = H * P;
  const int ng = C / group;
  const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= npairs) return;
  const int t = (int)(pair / ng), g = (int)(pair % ng);
  const int c0 = g * group;
  const float* orow = o + (int64_t)t * C;
  const T* grow = gate + (int64_t)t * gate_stride;
  auto value = [&](int i) {
    const int c = c0 + i;
    float v = orow[c];
    if (den != nullptr) {
      const int h = c / P;
      const float f = floor_ ? floor_[(int64_t)t * H + h] : 0.0f;
      v = v / (fmaxf(fabsf(den[(int64_t)t * H + h]), f) + 1e-6f);
    }
    return v;
  };
  float sq = 0.0f;
  for (int i = lane; i < group; i += 64) {
    float v = value(i);
    if (gate_first) {
      const float z = Act<T>::ld(grow + c0 + i);
      v *= gate_silu ? silu_f32(z) : 1.0f / (1.0f + expf(-z));
    }
    sq += v * v;
  }
  const float rstd = 1.0f / sqrtf(wave_reduce_sum(sq) / (float)group + eps);
  for (int i = lane; i < group; i += 64) {
    const int c = c0 + i;
    float v = value(i);
    const float z = Act<T>::ld(grow + c);
    const float gzv = gate_silu ? silu_f32(z) : 1.0f / (1.0f + expf(-z));
    if (gate_first) v *= gzv;
    v = v * rstd * w[c];
    if (!gate_first) v *= gzv;
    Act<T>::st(out + (int64_t)t * C + c, v);
  }
}

void head_norm_gate(torch::Tensor out, torch::Tensor o, torch::Tensor gate,
                    torch::Tensor w, double eps, int64_t group,
                    int64_t gate_act, bool gate_first,
                    c10::optional<torch::Tensor> den,
                    c10::optional<torch::Tensor> floor_) {
  TORCH_CHECK(o.is_cuda() && o.dtype() == torch::kFloat32 &&
              o.is_contiguous() && o.dim() == 3);
  const int T = o.size(0), H = o.size(1), P = o.size(2);
  const int C = H * P;
  TORCH_CHECK(P >= 1 && group >= 1 && C % group == 0,
              "norm groups must divide the channels");
  TORCH_CHECK(out.is_contiguous() && out.size(0) == T && out.size(1) == C);
  TORCH_CHECK(gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == T &&
              gate.size(1) == C && gate.dtype() == out.dtype());
  TORCH_CHECK(w.dtype() == torch::kFloat32 && w.numel() == C &&
              w.is_contiguous());
  TORCH_CHECK(den.has_value() || !floor_.has_value(),
              "a floor needs the normaliser it bounds");
  for (const auto* x : {&den, &floor_})
    if (x->has_value())
      TORCH_CHECK((*x)->dtype() == torch::kFloat32 && (*x)->is_contiguous() &&
                  (*x)->numel() == (int64_t)T * H);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int64_t npairs = (int64_t)T * (C / group);
  TORCH_CHECK(npairs < (int64_t)1 << 31, "too many (row, group) pairs");
  const int64_t ge = gate.element_size();
  const bool vec4 = P % 4 == 0 && group % 4 == 0 &&
                    (gate.stride(0) * ge) % (4 * ge) == 0 &&
                    reinterpret_cast<uintptr_t>(gate.data_ptr()) % (4 * ge) ==
                        0;
#define HNG_ARGS                                                              \
  (act_t*)out.data_ptr(), (const float*)o.data_ptr(),                         \
      (const act_t*)gate.data_ptr(), (int64_t)gate.stride(0),                 \
      (const float*)w.data_ptr(),                                             \
      den.has_value() ? (const float*)den->data_ptr() : nullptr,              \
      floor_.has_value() ? (const float*)floor_->data_ptr() : nullptr, H, P,  \
      (int)group, (float)eps, gate_act == 1 ? 1 : 0, gate_first ? 1 : 0,      \
      npairs
#define LAUNCH_HNG(VPL, VW)                                                   \
  hipLaunchKernelGGL((head_norm_gate_kernel<act_t, VPL, VW>),                 \
                     dim3((npairs + 4 * HNG_PAIRS - 1) / (4 * HNG_PAIRS)),    \
                     dim3(256), 0, stream, HNG_ARGS)
  IGW_DISPATCH_ACT(out, {
    if (vec4 && group <= 64) LAUNCH_HNG(1, 1);
    else if (vec4 && group <= 128) LAUNCH_HNG(1, 2);
    else if (vec4 && group <= 256) LAUNCH_HNG(1, 4);
    else if (vec4 && group <= 512) LAUNCH_HNG(2, 4);
    else if (vec4 && group <= 1024) LAUNCH_HNG(4, 4);
    else if (group <= 64) LAUNCH_HNG(1, 1);
    else if (group <= 128) LAUNCH_HNG(2, 1);
    else if (group <= 256) LAUNCH_HNG(4, 1);
    else
      hipLaunchKernelGGL((head_norm_gate_wide_kernel<act_t>),
                         dim3((npairs + 3) / 4), dim3(256), 0, stream,
                         HNG_ARGS);
  });
#undef LAUNCH_HNG
#undef HNG_ARGS
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// paged append, keys and values of unequal width
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void append_paged_kv_kernel(
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, T* __restrict__ kcache, T* __restrict__ vcache,
    const int32_t* __restrict__ slot_mapping, int G, int N, int P,
    int block_size) {
  const int t = blockIdx.x;
  const int slot = slot_mapping[t];
  const int64_t blk = slot / block_size, off = slot % block_size;
  for (int i = threadIdx.x; i < G * N; i += 256) {
    const int g = i / N, n = i % N;
    kcache[((blk * G + g) * block_size + off) * N + n] = k[t * k_stride + i];
  }
  for (int i = threadIdx.x; i < G * P; i += 256) {
    const int g = i / P, p = i % P;
    vcache[((blk * G + g) * block_size + off) * P + p] = v[t * v_stride + i];
  }
}

// N % 8 == 0, P % 8 == 0, rows 16-byte aligned
template <typename T>
__global__ __launch_bounds__(256) void append_paged_kv_vec8_kernel(
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, T* __restrict__ kcache, T* __restrict__ vcache,
    const int32_t* __restrict__ slot_mapping, int G, int N, int P,
    int block_size) {
  const int t = blockIdx.x;
  const int slot = slot_mapping[t];
  const int64_t blk = slot / block_size, off = slot % block_size;
  struct alignas(16) Vec { T v[8]; };
  for (int i = threadIdx.x * 8; i < G * N; i += 256 * 8) {
    const int g = i / N, n = i % N;
    *(Vec*)(kcache + ((blk * G + g) * block_size + off) * N + n) =
        *(const Vec*)(k + t * k_stride + i);
  }
  for (int i = threadIdx.x * 8; i < G * P; i += 256 * 8) {
    const int g = i / P, p = i % P;
    *(Vec*)(vcache + ((blk * G + g) * block_size + off) * P + p) =
        *(const Vec*)(v + t * v_stride + i);
  }
}

void append_paged_kv(torch::Tensor k, torch::Tensor v, torch::Tensor kcache,
                     torch::Tensor vcache, torch::Tensor slot_mapping) {
  TORCH_CHECK(k.is_cuda() && k.dim() == 2 && k.stride(1) == 1 &&
              v.dim() == 2 && v.stride(1) == 1 && k.dtype() == v.dtype());
  TORCH_CHECK(kcache.is_contiguous() && vcache.is_contiguous() &&
              kcache.dim() == 4 && vcache.dim() == 4 &&
              kcache.dtype() == k.dtype() && vcache.dtype() == k.dtype());
  const int T = k.size(0), G = kcache.size(1), bs = kcache.size(2);
  const int N = kcache.size(3), P = vcache.size(3);
  TORCH_CHECK(vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
              vcache.size(2) == bs);
  TORCH_CHECK(k.size(1) == G * N && v.size(1) == G * P && v.size(0) == T);
  TORCH_CHECK(slot_mapping.dtype() == torch::kInt32 &&
              slot_mapping.numel() == T);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int64_t es = k.element_size();
  const bool vec8 = N % 8 == 0 && P % 8 == 0 &&
                    (k.stride(0) * es) % 16 == 0 &&
                    (v.stride(0) * es) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(k.data_ptr()) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(v.data_ptr()) % 16 == 0;
  IGW_DISPATCH_ACT(k, {
    if (vec8)
      hipLaunchKernelGGL(
          (append_paged_kv_vec8_kernel<act_t>), dim3(T), dim3(256), 0, stream,
          (const act_t*)k.data_ptr(), (int64_t)k.stride(0),
          (const act_t*)v.data_ptr(), (int64_t)v.stride(0),
          (act_t*)kcache.data_ptr(), (act_t*)vcache.data_ptr(),
          (const int32_t*)slot_mapping.data_ptr(), G, N, P, bs);
    else
    hipLaunchKernelGGL(
        (append_paged_kv_kernel<act_t>), dim3(T), dim3(256), 0, stream,
        (const act_t*)k.data_ptr(), (int64_t)k.stride(0),
        (const act_t*)v.data_ptr(), (int64_t)v.stride(0),
        (act_t*)kcache.data_ptr(), (act_t*)vcache.data_ptr(),
        (const int32_t*)slot_mapping.data_ptr(), G, N, P, bs);
  });
  HIP_CHECK_KERNEL();
}

// ---------------------------------------------------------------------------
// average of two normed branches
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(RROW_BLOCK) void rmsnorm_pair_mean_kernel(
    T* __restrict__ out, const T* __restrict__ a, const T* __restrict__ b,
    const float* __restrict__ wa, const float* __restrict__ wb, int D,
    float eps) {
  __shared__ float lds[RROW_BLOCK / 64];
  const int64_t row = blockIdx.x;
  const T* ar = a + row * D;
  const T* br = b + row * D;
  float sa = 0.0f, sb = 0.0f;
  if (D % 8 == 0) {
    for (int d = threadIdx.x * 8; d < D; d += RROW_BLOCK * 8) {
      float x[8], y[8];
      Row8<T>::ld(ar + d, x);
      Row8<T>::ld(br + d, y);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sa += x[e] * x[e];
        sb += y[e] * y[e];
      }
    }
  } else {
    for (int d = threadIdx.x; d < D; d += RROW_BLOCK) {
      const float x = Act<T>::ld(ar + d), y = Act<T>::ld(br + d);
      sa += x * x;
      sb += y * y;
    }
  }
  const float ra = 1.0f / sqrtf(rrow_block_sum(sa, lds) / (float)D + eps);
  const float rb = 1.0f / sqrtf(rrow_block_sum(sb, lds) / (float)D + eps);
  if (D % 8 == 0) {
    for (int d = threadIdx.x * 8; d < D; d += RROW_BLOCK * 8) {
      float x[8], y[8], u[8], v[8], r[8];
      Row8<T>::ld(ar + d, x);
      Row8<T>::ld(br + d, y);
      Row8<float>::ld(wa + d, u);
      Row8<float>::ld(wb + d, v);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        r[e] = 0.5f * (x[e] * ra * u[e] + y[e] * rb * v[e]);
      Row8<T>::st(out + row * D + d, r);
    }
  } else {
    for (int d = threadIdx.x; d < D; d += RROW_BLOCK)
      Act<T>::st(out + row * D + d,
                 0.5f * (Act<T>::ld(ar + d) * ra * wa[d] +
                         Act<T>::ld(br + d) * rb * wb[d]));
  }
}

void rmsnorm_pair_mean(torch::Tensor out, torch::Tensor a, torch::Tensor b,
                       torch::Tensor wa, torch::Tensor wb, double eps) {
  TORCH_CHECK(a.is_cuda() && a.is_contiguous() && b.is_contiguous() &&
              a.dim() == 2 && a.sizes() == b.sizes() &&
              a.dtype() == b.dtype());
  const int T = a.size(0), D = a.size(1);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == a.sizes() &&
              out.dtype() == a.dtype());
  TORCH_CHECK(wa.dtype() == torch::kFloat32 && wa.numel() == D &&
              wb.dtype() == torch::kFloat32 && wb.numel() == D);
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  IGW_DISPATCH_ACT(a, {
    hipLaunchKernelGGL((rmsnorm_pair_mean_kernel<act_t>), dim3(T),
                       dim3(RROW_BLOCK), 0, stream, (act_t*)out.data_ptr(),
                       (const act_t*)a.data_ptr(), (const act_t*)b.data_ptr(),
                       (const float*)wa.data_ptr(), (const float*)wb.data_ptr(),
                       D, (float)eps);
  });
  HIP_CHECK_KERNEL();
}

}  // namespace igw
