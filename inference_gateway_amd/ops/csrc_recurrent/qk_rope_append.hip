// Query/key post-processing of a fused projection (gfx950): per-head RMS
// norm, partial interleaved-pair rotation with scaled cos/sin, and the
// append of keys and values to the paged caches, in one launch.
//
//   proj [T, H*N | G*N | G*P | ...]   (row stride of its own)
//   x = head of q or k;  x <- x / sqrt(mean(x^2) + eps) * w      (w given)
//   pairs (2i, 2i+1), i < R:  angle = position * inv_freq[i]
//     (x_2i, x_2i+1) <- (x_2i c - x_2i+1 s, x_2i+1 c + x_2i s),
//     c = cos(angle) * mag, s = sin(angle) * mag
//   q -> out [T, H*N];  k -> kcache [blocks, G, block, N] at slot;
//   v -> vcache [blocks, G, block, P] at slot (copied)
//
// One 256-thread workgroup per row; its four waves take the row's units in
// turn: the H query heads, then the G key heads, then the G value heads.
// Lanes own entry pairs (one 4- or 8-byte access per pair when the layout
// allows); norms, angles and the rotation are fp32 (cosf / sinf with full
// range reduction, evaluated once per row and shared through LDS).
#include "../csrc_hybrid/act_types.h"

namespace igw {

// two consecutive activations
template <typename T>
struct Act2;
template <>
struct Act2<float> {
  static DEVINLINE void ld(const float* p, float& a, float& b) {
    const float2 x = *(const float2*)p;
    a = x.x;
    b = x.y;
  }
  static DEVINLINE void st(float* p, float a, float b) {
    *(float2*)p = make_float2(a, b);
  }
};
template <>
struct Act2<uint16_t> {
  static DEVINLINE void ld(const uint16_t* p, float& a, float& b) {
    const uint32_t x = *(const uint32_t*)p;
    a = bf16_to_f32((uint16_t)(x & 0xffffu));
    b = bf16_to_f32((uint16_t)(x >> 16));
  }
  static DEVINLINE void st(uint16_t* p, float a, float b) {
    *(uint32_t*)p = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
  }
};

// PAIRED: every head starts on an even element and N, P are even, so a
// pair is one aligned access
template <typename T, bool PAIRED>
__global__ __launch_bounds__(256) void qk_norm_rope_append_kernel(
    T* __restrict__ qout, const T* __restrict__ proj, int64_t proj_rs,
    const int32_t* __restrict__ positions,
    const int32_t* __restrict__ slot_mapping, T* __restrict__ kcache,
    T* __restrict__ vcache, const float* __restrict__ qnorm_w,
    const float* __restrict__ knorm_w, const float* __restrict__ inv_freq,
    int R, float mag, float eps, int H, int G, int N, int P, int BS) {
  // cos | sin of the row's R angles, shared by all its heads
  extern __shared__ float cs_lds[];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = proj + (int64_t)t * proj_rs;
  const int slot = slot_mapping[t];
  const int64_t blk = slot / BS, off = slot % BS;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < R; i += 256) {
    const float ang = pos * inv_freq[i];
    cs_lds[i] = cosf(ang) * mag;
    cs_lds[R + i] = sinf(ang) * mag;
  }
  __syncthreads();
  for (int unit = wave; unit < H + 2 * G; unit += 4) {
    if (unit >= H + G) {
      // value head: plain copy into its page
      const int gv = unit - H - G;
      const T* src = row + (int64_t)(H + G) * N + gv * P;
      T* dst = vcache + ((blk * G + gv) * BS + off) * P;
      if (PAIRED) {
        for (int i = lane; i < P / 2; i += 64) {
          float a, b;
          Act2<T>::ld(src + 2 * i, a, b);
          Act2<T>::st(dst + 2 * i, a, b);
        }
      } else {
        for (int d = lane; d < P; d += 64) dst[d] = src[d];
      }
      continue;
    }
    const bool is_q = unit < H;
    const T* src = row + (int64_t)unit * N;     // q heads then k heads
    T* dst = is_q ? qout + ((int64_t)t * H + unit) * N
                  : kcache + ((blk * G + (unit - H)) * BS + off) * N;
    const float* w = is_q ? qnorm_w : knorm_w;
    const int npairs = (N + 1) / 2;
    // a head of up to 128 entries sits in one pair per lane; wider heads
    // are read again after the statistic
    float a0 = 0.0f, b0 = 0.0f;
    const bool first = lane < npairs;
    if (first) {
      if (PAIRED) {
        Act2<T>::ld(src + 2 * lane, a0, b0);
      } else {
        a0 = Act<T>::ld(src + 2 * lane);
        b0 = 2 * lane + 1 < N ? Act<T>::ld(src + 2 * lane + 1) : 0.0f;
      }
    }
    float scale = 1.0f;
    if (w) {
      float ss = a0 * a0 + b0 * b0;
      for (int i = lane + 64; i < npairs; i += 64) {
        const float x = Act<T>::ld(src + 2 * i);
        const float y = 2 * i + 1 < N ? Act<T>::ld(src + 2 * i + 1) : 0.0f;
        ss += x * x + y * y;
      }
      scale = 1.0f / sqrtf(wave_reduce_sum(ss) / (float)N + eps);
    }
    for (int i = lane; i < npairs; i += 64) {
      const int d0 = 2 * i, d1 = 2 * i + 1;
      float a, b;
      if (i == lane) {
        a = a0;
        b = b0;
      } else {
        a = Act<T>::ld(src + d0);
        b = d1 < N ? Act<T>::ld(src + d1) : 0.0f;
      }
      a *= scale;
      b *= scale;
      if (w) {
        a *= w[d0];
        if (d1 < N) b *= w[d1];
      }
      if (i < R) {
        const float c = cs_lds[i], s = cs_lds[R + i];
        const float ra = a * c - b * s, rb = b * c + a * s;
        a = ra;
        b = rb;
      }
      if (PAIRED) {
        Act2<T>::st(dst + d0, a, b);
      } else {
        Act<T>::st(dst + d0, a);
        if (d1 < N) Act<T>::st(dst + d1, b);
      }
    }
  }
}

void qk_norm_rope_append(torch::Tensor qout, torch::Tensor proj,
                         torch::Tensor positions, torch::Tensor slot_mapping,
                         torch::Tensor kcache, torch::Tensor vcache,
                         c10::optional<torch::Tensor> qnorm_w,
                         c10::optional<torch::Tensor> knorm_w,
                         c10::optional<torch::Tensor> inv_freq, double mag,
                         double eps, int64_t heads, int64_t kv_heads,
                         int64_t dim, int64_t vdim) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1);
  const int T = proj.size(0), H = heads, G = kv_heads, N = dim, P = vdim;
  TORCH_CHECK(proj.size(1) >= (int64_t)(H + G) * N + (int64_t)G * P);
  TORCH_CHECK(kcache.is_contiguous() && kcache.dim() == 4 &&
              vcache.is_contiguous() && vcache.dim() == 4 &&
              kcache.dtype() == proj.dtype() && vcache.dtype() == proj.dtype());
  const int BS = kcache.size(2);
  TORCH_CHECK(kcache.size(1) == G && kcache.size(3) == N &&
              vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
              vcache.size(2) == BS && vcache.size(3) == P);
  TORCH_CHECK(qout.is_contiguous() && qout.dtype() == proj.dtype() &&
              qout.numel() == (int64_t)T * H * N);
  TORCH_CHECK(positions.dtype() == torch::kInt32 && positions.numel() == T &&
              slot_mapping.dtype() == torch::kInt32 &&
              slot_mapping.numel() == T);
  auto fvec = [&](const c10::optional<torch::Tensor>& t, int64_t n) {
    if (t.has_value())
      TORCH_CHECK(t->dtype() == torch::kFloat32 && t->is_contiguous() &&
                  t->numel() == n);
  };
  fvec(qnorm_w, N);
  fvec(knorm_w, N);
  TORCH_CHECK(qnorm_w.has_value() == knorm_w.has_value());
  int R = 0;
  if (inv_freq.has_value()) {
    R = inv_freq->numel();
    fvec(inv_freq, R);
    TORCH_CHECK(2 * R <= N, "more rotated entries than a head has");
  }
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  // pair accesses need even sizes and an aligned start of every row
  const int64_t es = proj.element_size();
  const bool paired =
      N % 2 == 0 && P % 2 == 0 && proj.stride(0) % 2 == 0 &&
      reinterpret_cast<uintptr_t>(proj.data_ptr()) % (2 * es) == 0;
#define LAUNCH_QKR(PA)                                                        \
  hipLaunchKernelGGL(                                                         \
      (qk_norm_rope_append_kernel<act_t, PA>), dim3(T), dim3(256),            \
      (size_t)(2 * R) * sizeof(float), stream,                                \
      (act_t*)qout.data_ptr(), (const act_t*)proj.data_ptr(),                 \
      (int64_t)proj.stride(0), (const int32_t*)positions.data_ptr(),          \
      (const int32_t*)slot_mapping.data_ptr(), (act_t*)kcache.data_ptr(),     \
      (act_t*)vcache.data_ptr(),                                              \
      qnorm_w.has_value() ? (const float*)qnorm_w->data_ptr() : nullptr,      \
      knorm_w.has_value() ? (const float*)knorm_w->data_ptr() : nullptr,      \
      R ? (const float*)inv_freq->data_ptr() : nullptr, R, (float)mag,        \
      (float)eps, H, G, N, P, BS)
  IGW_DISPATCH_ACT(proj, {
    if (paired) LAUNCH_QKR(true);
    else LAUNCH_QKR(false);
  });
#undef LAUNCH_QKR
  HIP_CHECK_KERNEL();
}

}  // namespace igw
