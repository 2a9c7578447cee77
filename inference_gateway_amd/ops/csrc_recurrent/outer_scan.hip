// Outer-product memory scan (gfx950): the one recurrence behind matrix
// memories (mLSTM), state-space layers (Mamba-2) and decayed memories
// (RWKV-style), per (sequence, head):
//
//   S' = diag(a_t) S + (c_t k_t) v_t^T            S [N, PP] fp32
//   POST  (no bonus):  o_t = S'^T q_t
//   PRE   (bonus u):   o_t = (S + diag(u) k_t v_t^T)^T q_t
//   out_t = o_t * qscale + skip_h v_t
//
// a_t is a scalar per head (VEC_DECAY = false) or one factor per key entry,
// given either directly or as x with a = exp(-exp(x)).  With ones_col the
// memory has one more column fed with v = 1 (the normaliser n_t = a n +
// c k); its read-out n_t . q_t goes to a tensor of its own.
//
// One workgroup per (run of value tiles, head, sequence); each of its up to
// four waves takes 64 value columns, and a lane owns ONE column of S in
// registers (NMAX fp32) for the whole run of rows, so the state is read and
// written once per step of the engine, not per token.  q, k and a of a
// chunk of rows are converted to fp32 once per workgroup (16-byte loads
// when the layout allows) and staged in LDS; the inner loop reads them as
// broadcasts (every lane the same address) in 16-byte pieces and is bound
// by the vector ALU: three multiply-adds per (row, key entry, column).
// Rows of a sequence are taken in order; sequences, heads and value tiles
// fill the chip.
#include "../csrc_hybrid/act_types.h"

namespace igw {

constexpr int SCAN_CHUNK = 16;  // rows staged per pass

// 8 consecutive activations -> 8 floats
template <typename T>
struct Act8;
template <>
struct Act8<float> {
  static DEVINLINE void ld(const float* p, float* o) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
};
template <>
struct Act8<uint16_t> {
  static DEVINLINE void ld(const uint16_t* p, float* o) {
    const ushort8 r = *(const ushort8*)p;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = bf16_to_f32(r.v[e]);
  }
};

constexpr int SCAN_MAX_WAVES = 4;

template <typename T, int NMAX, bool VEC_DECAY, bool BONUS, bool VEC8>
__global__ __launch_bounds__(64 * SCAN_MAX_WAVES) void outer_scan_kernel(
    float* __restrict__ out, float* __restrict__ norm_out,
    const T* __restrict__ q, int64_t q_s0,
    int64_t q_s1, const T* __restrict__ k, int64_t k_s0, int64_t k_s1,
    const T* __restrict__ v, int64_t v_s0, int64_t v_s1,
    const float* __restrict__ decay, const float* __restrict__ kscale,
    const float* __restrict__ bonus, const float* __restrict__ skip,
    float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, int H, int G, int N, int P,
    int ones_col, int exp_neg_exp, float qscale) {
  __shared__ __attribute__((aligned(16))) float lds_q[SCAN_CHUNK * NMAX];
  __shared__ __attribute__((aligned(16))) float lds_k[SCAN_CHUNK * NMAX];
  __shared__ __attribute__((aligned(16))) float
      lds_a[VEC_DECAY ? SCAN_CHUNK * NMAX : SCAN_CHUNK];
  __shared__ __attribute__((aligned(16))) float lds_u[BONUS ? NMAX : 4];
  // sum_n q_n u_n k_n per row: the bonus term of every column is this
  // number times v
  __shared__ float lds_c[SCAN_CHUNK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tid = threadIdx.x, nthr = blockDim.x;
  const int h = blockIdx.y, s = blockIdx.z;
  const int g = h / (H / G);
  const int r0 = seq_cu[s], r1 = seq_cu[s + 1];
  if (r1 == r0) return;
  const int PP = P + ones_col;
  const int p = (blockIdx.x * (nthr >> 6) + wave) * 64 + lane;
  const bool active = p < P;
  // the normaliser column is kept by one wave of the whole launch row
  const bool keeps_norm = ones_col && blockIdx.x == 0 && wave == 0;
  const bool fresh = seq_start[s] == 0;
  float* st = state + ((int64_t)seq_slots[s] * H + h) * N * PP;
  constexpr int NL = (NMAX + 63) / 64;  // normaliser entries per lane

  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n)
    S[n] = (n < N && active && !fresh) ? st[(int64_t)n * PP + p] : 0.0f;
  float nrm[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int n = lane + 64 * i;
    nrm[i] = (keeps_norm && n < N && !fresh) ? st[(int64_t)n * PP + P] : 0.0f;
  }
  // entries past N stay zero for the whole run
  for (int i = tid; i < SCAN_CHUNK * NMAX; i += nthr) {
    lds_q[i] = 0.0f;
    lds_k[i] = 0.0f;
    if (VEC_DECAY) lds_a[i] = 0.0f;
  }
  if (BONUS)
    for (int n = tid; n < NMAX; n += nthr)
      lds_u[n] = n < N ? bonus[h * N + n] : 0.0f;
  const float sk = skip ? skip[h] : 0.0f;

  for (int c0 = r0; c0 < r1; c0 += SCAN_CHUNK) {
    const int tc = min(SCAN_CHUNK, r1 - c0);
    __syncthreads();
    if (VEC8) {
      // N % 8 == 0, rows 16-byte aligned: 8 entries per thread and pass
      const int n8 = N >> 3;
      for (int i = tid; i < tc * n8; i += nthr) {
        const int t = i / n8, n = (i - t * n8) * 8;
        const int64_t row = c0 + t;
        float kk[8], qq[8];
        Act8<T>::ld(k + row * k_s0 + g * k_s1 + n, kk);
        Act8<T>::ld(q + row * q_s0 + g * q_s1 + n, qq);
        const float c = kscale ? kscale[row * H + h] : 1.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          lds_k[t * NMAX + n + e] = kk[e] * c;
          lds_q[t * NMAX + n + e] = qq[e];
        }
        if (VEC_DECAY) {
          float aa[8];
          Act8<float>::ld(decay + (row * H + h) * N + n, aa);
#pragma unroll
          for (int e = 0; e < 8; ++e)
            lds_a[t * NMAX + n + e] =
                exp_neg_exp ? expf(-expf(aa[e])) : aa[e];
        }
      }
    } else {
      for (int i = tid; i < tc * N; i += nthr) {
        const int t = i / N, n = i - t * N;
        const int64_t row = c0 + t;
        float kk = Act<T>::ld(k + row * k_s0 + g * k_s1 + n);
        if (kscale) kk *= kscale[row * H + h];
        lds_k[t * NMAX + n] = kk;
        lds_q[t * NMAX + n] = Act<T>::ld(q + row * q_s0 + g * q_s1 + n);
        if (VEC_DECAY) {
          float a = decay[(row * H + h) * N + n];
          if (exp_neg_exp) a = expf(-expf(a));
          lds_a[t * NMAX + n] = a;
        }
      }
    }
    if (!VEC_DECAY && tid < tc) {
      float a = decay[(int64_t)(c0 + tid) * H + h];
      if (exp_neg_exp) a = expf(-expf(a));
      lds_a[tid] = a;
    }
    __syncthreads();
    if (keeps_norm) {
      // the normaliser column: lanes over key entries, rows in order
      for (int t = 0; t < tc; ++t) {
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
          const int n = lane + 64 * i;
          if (n < NMAX) {
            const float a = VEC_DECAY ? lds_a[t * NMAX + n] : lds_a[t];
            const float kk = lds_k[t * NMAX + n];
            const float qq = lds_q[t * NMAX + n];
            if (BONUS) {
              dot += qq * (nrm[i] + lds_u[n] * kk);
              nrm[i] = a * nrm[i] + kk;
            } else {
              nrm[i] = a * nrm[i] + kk;
              dot += qq * nrm[i];
            }
          }
        }
        dot = wave_reduce_sum(dot);
        if (lane == 0)
          norm_out[(int64_t)(c0 + t) * H + h] = dot * qscale;
      }
    }
    if (BONUS) {
      for (int t = wave; t < tc; t += nthr >> 6) {
        float part = 0.0f;
        for (int n = lane; n < NMAX; n += 64)
          part += lds_q[t * NMAX + n] * lds_u[n] * lds_k[t * NMAX + n];
        part = wave_reduce_sum(part);
        if (lane == 0) lds_c[t] = part;
      }
      __syncthreads();
    }
    // the next row's value is requested before this row's arithmetic
    float vnext =
        active ? Act<T>::ld(v + (int64_t)c0 * v_s0 + h * v_s1 + p) : 0.0f;
    for (int t = 0; t < tc; ++t) {
      const int64_t row = c0 + t;
      const float vv = vnext;
      if (active && t + 1 < tc)
        vnext = Act<T>::ld(v + (row + 1) * v_s0 + h * v_s1 + p);
      const float4* q4 = (const float4*)(lds_q + t * NMAX);
      const float4* k4 = (const float4*)(lds_k + t * NMAX);
      const float4* a4 = (const float4*)(lds_a + (VEC_DECAY ? t * NMAX : 0));
      const float as = VEC_DECAY ? 0.0f : lds_a[t];
      float o = BONUS ? lds_c[t] * vv : 0.0f;
#pragma unroll
      for (int n4 = 0; n4 < NMAX / 4; ++n4) {
        const float4 qq = q4[n4], kk = k4[n4];
        float4 aa = make_float4(as, as, as, as);
        if (VEC_DECAY) aa = a4[n4];
        const float qa[4] = {qq.x, qq.y, qq.z, qq.w};
        const float ka[4] = {kk.x, kk.y, kk.z, kk.w};
        const float da[4] = {aa.x, aa.y, aa.z, aa.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = n4 * 4 + j;
          if (BONUS) {
            o += qa[j] * S[n];
            S[n] = da[j] * S[n] + ka[j] * vv;
          } else {
            S[n] = da[j] * S[n] + ka[j] * vv;
            o += qa[j] * S[n];
          }
        }
      }
      if (active) out[(row * H + h) * P + p] = o * qscale + sk * vv;
    }
  }
  if (active) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) st[(int64_t)n * PP + p] = S[n];
  }
  if (keeps_norm) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int n = lane + 64 * i;
      if (n < N) st[(int64_t)n * PP + P] = nrm[i];
    }
  }
}

void outer_scan(torch::Tensor out, c10::optional<torch::Tensor> norm_out,
                torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor decay,
                c10::optional<torch::Tensor> kscale,
                c10::optional<torch::Tensor> bonus,
                c10::optional<torch::Tensor> skip, torch::Tensor state,
                torch::Tensor seq_cu, torch::Tensor seq_start,
                torch::Tensor seq_slots, int64_t decay_mode, bool ones_col,
                double qscale) {
  TORCH_CHECK(v.is_cuda() && v.dim() == 3 && v.stride(2) == 1);
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && k.dim() == 3 &&
              k.stride(2) == 1 && q.dtype() == v.dtype() &&
              k.dtype() == v.dtype() && q.sizes() == k.sizes());
  const int T = v.size(0), H = v.size(1), P = v.size(2);
  const int G = q.size(1), N = q.size(2);
  const int S = seq_slots.numel();
  const int PP = P + (ones_col ? 1 : 0);
  TORCH_CHECK(q.size(0) == T && G >= 1 && H % G == 0);
  TORCH_CHECK(out.dtype() == torch::kFloat32 && out.is_contiguous() &&
              out.numel() == (int64_t)T * H * P);
  TORCH_CHECK(norm_out.has_value() == ones_col,
              "the normaliser read-out goes with the ones column");
  if (ones_col)
    TORCH_CHECK(norm_out->dtype() == torch::kFloat32 &&
                norm_out->is_contiguous() &&
                norm_out->numel() == (int64_t)T * H);
  TORCH_CHECK(decay.dtype() == torch::kFloat32 && decay.is_contiguous() &&
              decay.dim() == 3 && decay.size(0) == T && decay.size(1) == H &&
              (decay.size(2) == 1 || decay.size(2) == N));
  const bool vec = decay.size(2) == N && N > 1;
  if (kscale.has_value())
    TORCH_CHECK(kscale->dtype() == torch::kFloat32 &&
                kscale->is_contiguous() && kscale->numel() == (int64_t)T * H);
  if (bonus.has_value())
    TORCH_CHECK(bonus->dtype() == torch::kFloat32 && bonus->is_contiguous() &&
                bonus->numel() == (int64_t)H * N);
  if (skip.has_value())
    TORCH_CHECK(skip->dtype() == torch::kFloat32 && skip->numel() == H);
  TORCH_CHECK(state.dtype() == torch::kFloat32 && state.is_contiguous() &&
              state.size(1) == (int64_t)H * N * PP,
              "memory slot width must be heads * keys * columns");
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 && seq_cu.numel() == S + 1 &&
              seq_start.dtype() == torch::kInt32 && seq_start.numel() == S &&
              seq_slots.dtype() == torch::kInt32);
  TORCH_CHECK(N <= 256, "key width above 256 is not supported");
  TORCH_CHECK(vec == bonus.has_value() || (N == 1 && !vec),
              "supported forms: scalar decay without bonus, per-entry decay "
              "with bonus");
  if (T == 0 || S == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int tiles = (P + 63) / 64;
  const int waves = std::min(tiles, SCAN_MAX_WAVES);
  const dim3 grid((tiles + waves - 1) / waves, H, S);
  const dim3 block(64 * waves);
  // 16-byte staging loads: 8 entries at a time from aligned rows
  const int64_t es = q.element_size();
  auto aligned = [&](const torch::Tensor& t) {
    return (reinterpret_cast<uintptr_t>(t.data_ptr()) % 16) == 0 &&
           (t.stride(0) * es) % 16 == 0 && (t.stride(1) * es) % 16 == 0;
  };
  const bool vec8 = N % 8 == 0 && aligned(q) && aligned(k) &&
                    (reinterpret_cast<uintptr_t>(decay.data_ptr()) % 16) == 0;
#define LAUNCH_SCAN_V(NM, VD, BO, V8)                                         \
  hipLaunchKernelGGL(                                                         \
      (outer_scan_kernel<act_t, NM, VD, BO, V8>), grid, block, 0, stream,     \
      (float*)out.data_ptr(),                                                 \
      ones_col ? (float*)norm_out->data_ptr() : nullptr,                      \
      (const act_t*)q.data_ptr(),                                             \
      (int64_t)q.stride(0), (int64_t)q.stride(1),                             \
      (const act_t*)k.data_ptr(), (int64_t)k.stride(0),                       \
      (int64_t)k.stride(1), (const act_t*)v.data_ptr(),                       \
      (int64_t)v.stride(0), (int64_t)v.stride(1),                             \
      (const float*)decay.data_ptr(),                                         \
      kscale.has_value() ? (const float*)kscale->data_ptr() : nullptr,        \
      bonus.has_value() ? (const float*)bonus->data_ptr() : nullptr,          \
      skip.has_value() ? (const float*)skip->data_ptr() : nullptr,            \
      (float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),            \
      (const int32_t*)seq_start.data_ptr(),                                   \
      (const int32_t*)seq_slots.data_ptr(), H, G, N, P, ones_col ? 1 : 0,     \
      decay_mode == 1 ? 1 : 0, (float)qscale)
#define LAUNCH_SCAN(NM, VD, BO)                                               \
  do {                                                                        \
    if (vec8) LAUNCH_SCAN_V(NM, VD, BO, true);                                \
    else LAUNCH_SCAN_V(NM, VD, BO, false);                                    \
  } while (0)
#define LAUNCH_SCAN_N(VD, BO)                                                 \
  do {                                                                        \
    if (N <= 16) LAUNCH_SCAN(16, VD, BO);                                     \
    else if (N <= 32) LAUNCH_SCAN(32, VD, BO);                                \
    else if (N <= 64) LAUNCH_SCAN(64, VD, BO);                                \
    else if (N <= 128) LAUNCH_SCAN(128, VD, BO);                              \
    else LAUNCH_SCAN(256, VD, BO);                                            \
  } while (0)
  IGW_DISPATCH_ACT(v, {
    if (bonus.has_value()) {
      if (vec) LAUNCH_SCAN_N(true, true);
      else LAUNCH_SCAN_V(16, false, true, false);   // N == 1
    } else {
      LAUNCH_SCAN_N(false, false);
    }
  });
#undef LAUNCH_SCAN_N
#undef LAUNCH_SCAN
#undef LAUNCH_SCAN_V
  HIP_CHECK_KERNEL();
}

}  // namespace igw
