// Group-limited sigmoid routing for mixtures of experts (gfx950).
//
//   s_e = sigmoid(logit_e)                  the weight of a chosen expert
//   c_e = s_e + correction_e                the score experts are chosen by
//   The E experts are `groups` equal runs of neighbours; a group scores the
//   sum of its two largest c (its only one if it has a single expert); only
//   experts of the `keep` best groups can be chosen.  The K largest c among
//   them are taken (ties to the lower index), weights s, not renormalised.
//
// One thread per token (E <= 64); its choice scores sit in a padded LDS row.
// With dst given, the padded-dispatch row of every assignment (expert *
// capacity + arrival rank) comes from the same launch.
#include "../csrc_hybrid/act_types.h"

namespace igw {

__global__ __launch_bounds__(64) void moe_group_route_kernel(
    float* __restrict__ weights, int32_t* __restrict__ idx,
    int64_t* __restrict__ dst, int32_t* __restrict__ counts,
    const float* __restrict__ logits, const float* __restrict__ correction,
    int T, int E, int K, int capacity, int groups, int keep) {
  __shared__ float cs[64][65];
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* row = logits + (int64_t)t * E;
  float* c = cs[threadIdx.x];
  for (int e = 0; e < E; ++e) c[e] = sigmoid_f32(row[e]) + correction[e];
  uint64_t allowed = E >= 64 ? ~0ull : ((1ull << E) - 1ull);
  if (groups > 1) {
    const int size = E / groups;
    allowed = 0;
    uint64_t kept = 0;
    for (int kk = 0; kk < keep; ++kk) {
      int best = -1;
      float bv = 0.0f;
      for (int g = 0; g < groups; ++g) {
        if ((kept >> g) & 1ull) continue;
        // sum of the group's two largest choice scores
        float m1 = -INFINITY, m2 = -INFINITY;
        for (int e = g * size; e < (g + 1) * size; ++e) {
          const float x = c[e];
          if (x > m1) {
            m2 = m1;
            m1 = x;
          } else if (x > m2) {
            m2 = x;
          }
        }
        const float gs = size > 1 ? m1 + m2 : m1;
        if (best < 0 || gs > bv) {
          bv = gs;
          best = g;
        }
      }
      kept |= 1ull << best;
      const uint64_t run = size >= 64 ? ~0ull : ((1ull << size) - 1ull);
      allowed |= run << (best * size);
    }
  }
  float* w = weights + (int64_t)t * K;
  int32_t* id = idx + (int64_t)t * K;
  uint64_t taken = 0;
  for (int k = 0; k < K; ++k) {
    int best = -1;
    float bv = 0.0f;
    for (int e = 0; e < E; ++e) {
      if (!((allowed >> e) & 1ull) || ((taken >> e) & 1ull)) continue;
      if (best < 0 || c[e] > bv) {
        bv = c[e];
        best = e;
      }
    }
    taken |= 1ull << best;
    id[k] = best;
    w[k] = sigmoid_f32(row[best]);
  }
  if (dst != nullptr) {
    for (int k = 0; k < K; ++k) {
      const int e = id[k];
      const int r = atomicAdd(counts + e, 1);
      dst[(int64_t)t * K + k] = (int64_t)e * capacity + r;
    }
  }
}

void moe_group_route(torch::Tensor weights, torch::Tensor idx,
                     torch::Tensor logits, torch::Tensor correction,
                     c10::optional<torch::Tensor> dst,
                     c10::optional<torch::Tensor> counts, int64_t capacity,
                     int64_t groups, int64_t keep) {
  TORCH_CHECK(logits.is_cuda() && logits.dtype() == torch::kFloat32 &&
              logits.is_contiguous() && logits.dim() == 2);
  const int T = logits.size(0), E = logits.size(1), K = weights.size(1);
  TORCH_CHECK(E <= 64 && K >= 1, "moe_group_route: E <= 64");
  TORCH_CHECK(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups,
              "moe_group_route: experts must split into equal groups");
  TORCH_CHECK(K <= (groups > 1 ? keep * (E / groups) : E),
              "moe_group_route: more experts asked for than can be chosen");
  TORCH_CHECK(correction.dtype() == torch::kFloat32 &&
              correction.is_contiguous() && correction.numel() == E);
  TORCH_CHECK(weights.is_contiguous() && weights.dtype() == torch::kFloat32 &&
              weights.size(0) == T);
  TORCH_CHECK(idx.is_contiguous() && idx.dtype() == torch::kInt32 &&
              idx.size(0) == T && idx.size(1) == K);
  if (dst.has_value()) {
    TORCH_CHECK(counts.has_value() && capacity >= T);
    TORCH_CHECK(dst->is_contiguous() && dst->dtype() == torch::kInt64 &&
                dst->numel() == (int64_t)T * K);
    TORCH_CHECK(counts->is_contiguous() && counts->dtype() == torch::kInt32 &&
                counts->numel() == E);   // zeroed by the caller
  }
  if (T == 0) return;
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
  hipLaunchKernelGGL(moe_group_route_kernel, dim3((T + 63) / 64), dim3(64), 0,
                     stream, (float*)weights.data_ptr(),
                     (int32_t*)idx.data_ptr(),
                     dst.has_value() ? (int64_t*)dst->data_ptr() : nullptr,
                     dst.has_value() ? (int32_t*)counts->data_ptr() : nullptr,
                     (const float*)logits.data_ptr(),
                     (const float*)correction.data_ptr(), T, E, K,
                     (int)capacity, (int)groups, (int)keep);
  HIP_CHECK_KERNEL();
}

}  // namespace igw
