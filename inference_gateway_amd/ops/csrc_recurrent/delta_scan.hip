// Gated delta-rule memory scan (gfx950), per (sequence, head):
//
//   S <- a_t S                          S [N, P] fp32, a_t scalar per head
//   u  = b_t (v_t - S^T k_t)            what the memory does not yet return
//   S <- S + k_t u^T                    for k_t, written with strength b_t
//   o_t = S^T q_t                       the read-out sees the row's own write
//
// With unit_eps > 0, q_t and k_t are first scaled to unit length per head,
// x / sqrt(sum x^2 + unit_eps), in fp32; q_t is multiplied by qscale.
//
// Same layout as the outer-product scan: one workgroup per (run of value
// tiles, head, sequence); each of its up to four waves takes 64 value
// columns and a lane owns ONE column of S in registers (NMAX fp32) for the
// whole run of rows, so the state is read and written once per engine step.
// A column's update needs only that column (S^T k and S^T q are per-column
// dot products), so no lane talks to another inside the row loop.  q, k of
// a chunk of rows are converted to fp32, normalised once per workgroup and
// staged in LDS; the inner loop reads them as broadcasts in 16-byte pieces:
// four multiply-adds per (row, key entry, column).
#include "../csrc_hybrid/act_types.h"

namespace igw {

constexpr int DSCAN_CHUNK = 16;  // rows staged per pass
constexpr int DSCAN_MAX_WAVES = 4;

// MINB = workgroups per compute unit the register budget must allow.
// Decoded rows (one row per sequence: load the state, one update, store it)
// are latency-bound and gain from three waves per SIMD (168 registers at
// 128 key entries: 144 -> 99 us for 256 sequences of 16 heads); long runs of
// rows lose to the few spills that budget causes (4.6 -> 5.6 ms) and keep
// the compiler's own choice (232 registers, two waves).
template <typename T, int NMAX, int MINB>
__global__ __launch_bounds__(64 * DSCAN_MAX_WAVES, MINB)
void delta_scan_kernel(
    float* __restrict__ out, const T* __restrict__ q, int64_t q_s0,
    int64_t q_s1, const T* __restrict__ k, int64_t k_s0, int64_t k_s1,
    const T* __restrict__ v, int64_t v_s0, int64_t v_s1,
    const float* __restrict__ decay, const float* __restrict__ beta,
    float* __restrict__ state, const int32_t* __restrict__ seq_cu,
    const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ seq_slots, int H, int G, int N, int P,
    float unit_eps, float qscale) {
  __shared__ __attribute__((aligned(16))) float lds_q[DSCAN_CHUNK * NMAX];
  __shared__ __attribute__((aligned(16))) float lds_k[DSCAN_CHUNK * NMAX];
  __shared__ float lds_a[DSCAN_CHUNK];
  __shared__ float lds_b[DSCAN_CHUNK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tid = threadIdx.x, nthr = blockDim.x, nwaves = nthr >> 6;
  const int h = blockIdx.y, s = blockIdx.z;
  const int g = h / (H / G);
  const int r0 = seq_cu[s], r1 = seq_cu[s + 1];
  if (r1 == r0) return;
  const int p = (blockIdx.x * nwaves + wave) * 64 + lane;
  const bool active = p < P;
  const bool fresh = seq_start[s] == 0;
  float* st = state + ((int64_t)seq_slots[s] * H + h) * N * P;

  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n)
    S[n] = (n < N && active && !fresh) ? st[(int64_t)n * P + p] : 0.0f;
  // entries past N stay zero for the whole run
  for (int i = tid; i < DSCAN_CHUNK * NMAX; i += nthr) {
    lds_q[i] = 0.0f;
    lds_k[i] = 0.0f;
  }

  for (int c0 = r0; c0 < r1; c0 += DSCAN_CHUNK) {
    const int tc = min(DSCAN_CHUNK, r1 - c0);
    __syncthreads();
    for (int i = tid; i < tc * N; i += nthr) {
      const int t = i / N, n = i - t * N;
      const int64_t row = c0 + t;
      lds_k[t * NMAX + n] = Act<T>::ld(k + row * k_s0 + g * k_s1 + n);
      lds_q[t * NMAX + n] = Act<T>::ld(q + row * q_s0 + g * q_s1 + n);
    }
    if (tid < tc) {
      lds_a[tid] = decay[(int64_t)(c0 + tid) * H + h];
      lds_b[tid] = beta[(int64_t)(c0 + tid) * H + h];
    }
    __syncthreads();
    // unit length per (row, head) and the query factor: a wave per row
    for (int t = wave; t < tc; t += nwaves) {
      float sq = 0.0f, sk = 0.0f;
      for (int n = lane; n < N; n += 64) {
        const float a = lds_q[t * NMAX + n], b = lds_k[t * NMAX + n];
        sq += a * a;
        sk += b * b;
      }
      float fq = qscale, fk = 1.0f;
      if (unit_eps > 0.0f) {
        fq = qscale / sqrtf(wave_reduce_sum(sq) + unit_eps);
        fk = 1.0f / sqrtf(wave_reduce_sum(sk) + unit_eps);
      }
      for (int n = lane; n < N; n += 64) {
        lds_q[t * NMAX + n] *= fq;
        lds_k[t * NMAX + n] *= fk;
      }
    }
    __syncthreads();
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
      const float a = lds_a[t];
      // what the decayed memory returns for this key
      float r = 0.0f;
#pragma unroll
      for (int n4 = 0; n4 < NMAX / 4; ++n4) {
        const float4 kk = k4[n4];
        r += kk.x * S[n4 * 4] + kk.y * S[n4 * 4 + 1] + kk.z * S[n4 * 4 + 2] +
             kk.w * S[n4 * 4 + 3];
      }
      const float u = lds_b[t] * (vv - a * r);
      float o = 0.0f;
      // the second pass must READ k again: if the compiler sees the same
      // addresses it keeps the first pass's 128 loaded values in registers
      // beside the state, which halves the occupancy
      asm volatile("" : "+v"(k4), "+v"(q4));
#pragma unroll
      for (int n4 = 0; n4 < NMAX / 4; ++n4) {
        const float4 qq = q4[n4], kk = k4[n4];
        const float qa[4] = {qq.x, qq.y, qq.z, qq.w};
        const float ka[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = n4 * 4 + j;
          S[n] = a * S[n] + ka[j] * u;
          o += qa[j] * S[n];
        }
      }
      if (active) out[(row * H + h) * P + p] = o;
    }
  }
  if (active) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) st[(int64_t)n * P + p] = S[n];
  }
}

void delta_scan(torch::Tensor out, torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor decay, torch::Tensor beta,
                torch::Tensor state, torch::Tensor seq_cu,
                torch::Tensor seq_start, torch::Tensor seq_slots,
                double unit_eps, double qscale) {
  TORCH_CHECK(v.is_cuda() && v.dim() == 3 && v.stride(2) == 1);
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && k.dim() == 3 &&
              k.stride(2) == 1 && q.dtype() == v.dtype() &&
              k.dtype() == v.dtype() && q.sizes() == k.sizes());
  const int T = v.size(0), H = v.size(1), P = v.size(2);
  const int G = q.size(1), N = q.size(2);
  const int S = seq_slots.numel();
  TORCH_CHECK(q.size(0) == T && G >= 1 && H % G == 0);
  TORCH_CHECK(out.dtype() == torch::kFloat32 && out.is_contiguous() &&
              out.numel() == (int64_t)T * H * P);
  TORCH_CHECK(decay.dtype() == torch::kFloat32 && decay.is_contiguous() &&
              decay.numel() == (int64_t)T * H &&
              beta.dtype() == torch::kFloat32 && beta.is_contiguous() &&
              beta.numel() == (int64_t)T * H);
  TORCH_CHECK(state.dtype() == torch::kFloat32 && state.is_contiguous() &&
              state.dim() == 2 && state.size(1) == (int64_t)H * N * P,
              "memory slot width must be heads * keys * values");
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 && seq_cu.numel() == S + 1 &&
              seq_start.dtype() == torch::kInt32 && seq_start.numel() == S &&
              seq_slots.dtype() == torch::kInt32);
  TORCH_CHECK(N <= 256, "key width above 256 is not supported");
  if (T == 0 || S == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  const int tiles = (P + 63) / 64;
  const int waves = std::min(tiles, DSCAN_MAX_WAVES);
  const dim3 grid((tiles + waves - 1) / waves, H, S);
  const dim3 block(64 * waves);
  // mostly single rows: the three-wave build
  const bool lean = T <= 2 * S;
#define LAUNCH_DSCAN_B(NM, MB)                                                \
  hipLaunchKernelGGL(                                                         \
      (delta_scan_kernel<act_t, NM, MB>), grid, block, 0, stream,             \
      (float*)out.data_ptr(), (const act_t*)q.data_ptr(),                     \
      (int64_t)q.stride(0), (int64_t)q.stride(1),                             \
      (const act_t*)k.data_ptr(), (int64_t)k.stride(0),                       \
      (int64_t)k.stride(1), (const act_t*)v.data_ptr(),                       \
      (int64_t)v.stride(0), (int64_t)v.stride(1),                             \
      (const float*)decay.data_ptr(), (const float*)beta.data_ptr(),          \
      (float*)state.data_ptr(), (const int32_t*)seq_cu.data_ptr(),            \
      (const int32_t*)seq_start.data_ptr(),                                   \
      (const int32_t*)seq_slots.data_ptr(), H, G, N, P, (float)unit_eps,      \
      (float)qscale)
#define LAUNCH_DSCAN(NM)                                                      \
  do {                                                                        \
    if (lean) LAUNCH_DSCAN_B(NM, 3);                                          \
    else LAUNCH_DSCAN_B(NM, 1);                                               \
  } while (0)
  IGW_DISPATCH_ACT(v, {
    if (N <= 16) LAUNCH_DSCAN(16);
    else if (N <= 32) LAUNCH_DSCAN(32);
    else if (N <= 64) LAUNCH_DSCAN(64);
    else if (N <= 128) LAUNCH_DSCAN(128);
    else LAUNCH_DSCAN_B(256, 1);
  });
#undef LAUNCH_DSCAN
#undef LAUNCH_DSCAN_B
  HIP_CHECK_KERNEL();
}

// decay = exp(-exp(a_log) * softplus(step + dt_bias)), beta =
// sigmoid(strength) from pre [T, 2H] fp32 = (step | strength); out [2, T, H]
__global__ void decay_beta_gates_kernel(float* __restrict__ out,
                                        const float* __restrict__ pre,
                                        const float* __restrict__ a_log,
                                        const float* __restrict__ dt_bias,
                                        int64_t T, int H) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * H) return;
  const int64_t t = i / H;
  const int h = (int)(i - t * H);
  const float x = pre[t * 2 * H + h] + dt_bias[h];
  // softplus without overflow: max(x, 0) + log1p(exp(-|x|))
  const float sp = fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x)));
  out[i] = expf(-expf(a_log[h]) * sp);
  out[T * H + i] = sigmoid_f32(pre[t * 2 * H + H + h]);
}

void decay_beta_gates(torch::Tensor out, torch::Tensor pre,
                      torch::Tensor a_log, torch::Tensor dt_bias) {
  TORCH_CHECK(pre.is_cuda() && pre.dtype() == torch::kFloat32 &&
              pre.is_contiguous() && pre.dim() == 2 && pre.size(1) % 2 == 0);
  const int64_t T = pre.size(0);
  const int H = pre.size(1) / 2;
  TORCH_CHECK(out.dtype() == torch::kFloat32 && out.is_contiguous() &&
              out.numel() == 2 * T * H);
  TORCH_CHECK(a_log.dtype() == torch::kFloat32 && a_log.numel() == H &&
              dt_bias.dtype() == torch::kFloat32 && dt_bias.numel() == H &&
              a_log.is_contiguous() && dt_bias.is_contiguous());
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(decay_beta_gates_kernel,
                     dim3((unsigned)((T * H + 255) / 256)), dim3(256), 0,
                     stream, (float*)out.data_ptr(),
                     (const float*)pre.data_ptr(),
                     (const float*)a_log.data_ptr(),
                     (const float*)dt_bias.data_ptr(), T, H);
  HIP_CHECK_KERNEL();
}

}  // namespace igw
