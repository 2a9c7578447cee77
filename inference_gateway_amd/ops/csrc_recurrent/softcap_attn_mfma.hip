// Causal softmax attention with a score cap on MFMA tiles (gfx950, bf16):
// the serving path of softcap_attention.  Same tiling as the engine's
// paged flash-attention prefill (64 query rows x 64 keys per step, 4
// waves of 16 rows, mfma_f32_16x16x32_bf16 for Q.K^T and P.V, K staged
// row-major and V transposed in swizzled LDS, probabilities through a
// per-wave LDS tile, online softmax in fp32 registers), generalised to
//
//   * key width N and value width P of their own, each padded with zeros
//     to the template's NP / PP (N, P multiples of 8);
//   * any page size;
//   * score = q.k * scale * temp(position), then cap * tanh(. / cap);
//   * an optional sliding window, an optional restriction to the row's
//     own chunk of positions, an optional linear distance bias per head
//     (slope * (row position - key position) is taken off the score), an
//     optional sink term per head in the softmax denominator and an
//     optional sigmoid output gate;
//   * two row maps.  Prompt tiles: rows are 64 consecutive tokens of one
//     head (grid = tiles x heads).  Decoded rows (HEADS_ROWS): the rows of
//     a tile are the query heads that share one key/value head, so every
//     K/V page is staged once per group instead of once per head
//     (grid = decoded rows x key/value heads).
//
// Everything is read from the paged cache; a row's own key is already
// appended.  Sequence s has rows [seq_cu[s], seq_cu[s+1]) whose first sits
// at position seq_start[s].
#include "../csrc_hybrid/act_types.h"

namespace igw {

typedef __attribute__((ext_vector_type(8))) short short8v;
typedef __attribute__((ext_vector_type(4))) float float4v;

// XOR byte swizzle inside a row of ROWB bytes: 16-lane 16-byte fragment
// reads of consecutive rows land in different banks
template <int ROWB>
DEVINLINE int swz(int row, int colbyte) {
  return colbyte ^ ((row & (ROWB >= 256 ? 15 : 7)) << 4);
}

// The transposed V tile (rows = value entries, 128 bytes of keys each) is
// WRITTEN by lanes whose rows differ by multiples of 8 and READ by lanes on
// 16 consecutive rows; folding both the low and the next three row bits
// into the 16-byte chunk index keeps either access to two lanes per bank.
DEVINLINE int swz_vt(int row, int colbyte) {
  return colbyte ^ ((((row & 7) ^ ((row >> 3) & 7))) << 4);
}

DEVINLINE float tanh_fast(float x) {
  return 1.0f - 2.0f * __frcp_rn(1.0f + __expf(2.0f * x));
}

constexpr int SA_BM = 64;
constexpr int SA_BN = 64;
constexpr int SA_BT_LDS = 1024;   // page numbers kept in LDS per sequence

template <int NP, int PP, bool HEADS_ROWS>
__global__ __launch_bounds__(256, 2) void softcap_attention_mfma_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ q, int64_t q_rs,
    const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ seq_cu, const int32_t* __restrict__ seq_start,
    const int32_t* __restrict__ tile_seq, const int32_t* __restrict__ tile_off,
    int H, int G, int N, int P, int BS, float scale, float softcap,
    float temp_coef, int temp_every, int window,
    const float* __restrict__ slopes, int chunk,
    const float* __restrict__ sinks, const uint16_t* __restrict__ gate,
    int64_t gate_rs) {
  constexpr int BM = SA_BM, BN = SA_BN;
  constexpr int KROWB = NP * 2;          // bytes per staged Q / K row
  // K tile (shared with the Q staging) | V^T tile | per-wave P tiles
  __shared__ __attribute__((aligned(16)))
  uint16_t smem[BN * NP + PP * BN + 4 * 16 * BN];
  uint16_t* k_s = smem;
  uint16_t* vt_s = smem + BN * NP;
  uint16_t* p_s = vt_s + PP * BN;

  const int tile = blockIdx.x;
  const int seq = tile_seq[tile];
  const int q0 = seq_cu[seq];
  const int Lq = HEADS_ROWS ? 1 : seq_cu[seq + 1] - q0;
  const int P0 = seq_start[seq];
  const int KVL = P0 + Lq;
  const int qoff = HEADS_ROWS ? 0 : tile_off[tile];
  const int rep = H / G;
  const int kvh = HEADS_ROWS ? blockIdx.y : blockIdx.y / rep;
  const int nrows = HEADS_ROWS ? rep : min(BM, Lq - qoff);  // valid rows
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  uint16_t* pw_s = p_s + wave * 16 * BN;
  // the sequence's page numbers sit in LDS when they fit, so that a K/V
  // address does not wait on a second global load
  __shared__ int32_t bt_s[SA_BT_LDS];
  const int32_t* bt_row = block_table + (int64_t)seq * max_blocks;
  const int nblk = (KVL + BS - 1) / BS;
  if (nblk <= SA_BT_LDS) {
    for (int i = tid; i < nblk; i += 256) bt_s[i] = bt_row[i];
    bt_row = bt_s;      // visible after the barrier that follows Q staging
  }

  // ---- Q tile -> LDS (the K region) -> A fragments ----
  for (int it = 0; it < BM * NP / 8 / 256; ++it) {
    const int idx = tid + it * 256;
    const int row = idx / (NP / 8);
    const int d8 = (idx % (NP / 8)) * 8;
    const int r = min(row, nrows - 1);
    const int64_t tok = HEADS_ROWS ? q0 : q0 + qoff + r;
    const int head = HEADS_ROWS ? kvh * rep + r : blockIdx.y;
    ushort8 val;
    if (d8 < N) {
      val = *reinterpret_cast<const ushort8*>(q + tok * q_rs + head * N + d8);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) val.v[e] = 0;
    }
    *reinterpret_cast<ushort8*>(reinterpret_cast<char*>(k_s) + row * KROWB +
                                swz<KROWB>(row, d8 * 2)) = val;
  }
  const int frag_m = lane & 15;
  const int frag_k8 = (lane >> 4) * 8;
  const int crow0 = (lane >> 4) * 4;
  const int ccol = lane & 15;
  __syncthreads();
  short8v qfrag[NP / 32];
  {
    const int row = wave * 16 + frag_m;
#pragma unroll
    for (int kk = 0; kk < NP / 32; ++kk)
      qfrag[kk] = *reinterpret_cast<const short8v*>(
          reinterpret_cast<char*>(k_s) + row * KROWB +
          swz<KROWB>(row, (kk * 32 + frag_k8) * 2));
  }

  float m[4], l[4], rscale[4], slope[4];
  int qpos[4], klo[4];
  float4v acc_o[PP / 16];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.0f;
    qpos[r] = HEADS_ROWS ? P0 : P0 + qoff + wave * 16 + crow0 + r;
    rscale[r] = scale * (1.0f + temp_coef * logf((float)((qpos[r] + 1) /
                                                         temp_every) + 1.0f));
    // first visible key of the row: window and position chunk
    klo[r] = window > 0 ? qpos[r] - window + 1 : 0;
    if (chunk > 0) klo[r] = max(klo[r], qpos[r] / chunk * chunk);
    const int head_r =
        HEADS_ROWS ? kvh * rep + min(wave * 16 + crow0 + r, rep - 1)
                   : (int)blockIdx.y;
    slope[r] = slopes ? slopes[head_r] : 0.0f;
  }
#pragma unroll
  for (int nt = 0; nt < PP / 16; ++nt) acc_o[nt] = {0.f, 0.f, 0.f, 0.f};
  const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;

  // keys [kfirst, kend): up to the tile's last row, from its first row's
  // window start
  const int kend = HEADS_ROWS ? KVL : min(KVL, P0 + qoff + BM);
  int kfirst = window > 0 ? max(0, P0 + qoff - window + 1) : 0;
  if (chunk > 0) kfirst = max(kfirst, (P0 + qoff) / chunk * chunk);
  kfirst = kfirst / BN * BN;

  // the next K/V tile travels in registers while the current one is used
  // (a second tile in flight costs more in occupancy than it hides)
  constexpr int KIT = BN * NP / 8 / 256, VIT = BN * PP / 8 / 256;
  ushort8 kreg[KIT], vreg[VIT];
  auto fetch = [&](int kbase) {
#pragma unroll
    for (int it = 0; it < KIT; ++it) {
      const int idx = tid + it * 256;
      const int row = idx / (NP / 8);
      const int d8 = (idx % (NP / 8)) * 8;
      if (d8 < N) {
        const int gpos = min(kbase + row, KVL - 1);
        const int64_t blk = bt_row[gpos / BS];
        kreg[it] = *reinterpret_cast<const ushort8*>(
            kcache + ((blk * G + kvh) * BS + (gpos % BS)) * N + d8);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) kreg[it].v[e] = 0;
      }
    }
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      const int idx = tid + it * 256;
      const int key = idx / (PP / 8);
      const int d8 = (idx % (PP / 8)) * 8;
      if (d8 < P) {
        const int gpos = min(kbase + key, KVL - 1);
        const int64_t blk = bt_row[gpos / BS];
        vreg[it] = *reinterpret_cast<const ushort8*>(
            vcache + ((blk * G + kvh) * BS + (gpos % BS)) * P + d8);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) vreg[it].v[e] = 0;
      }
    }
  };
  if (kfirst < kend) fetch(kfirst);

  for (int kbase = kfirst; kbase < kend; kbase += BN) {
    __syncthreads();
#pragma unroll
    for (int it = 0; it < KIT; ++it) {
      const int idx = tid + it * 256;
      const int row = idx / (NP / 8);
      const int d8 = (idx % (NP / 8)) * 8;
      *reinterpret_cast<ushort8*>(reinterpret_cast<char*>(k_s) + row * KROWB +
                                  swz<KROWB>(row, d8 * 2)) = kreg[it];
    }
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      const int idx = tid + it * 256;
      const int key = idx / (PP / 8);
      const int d8 = (idx % (PP / 8)) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(vt_s) +
                                     (d8 + e) * (BN * 2) +
                                     swz_vt(d8 + e, key * 2)) =
            vreg[it].v[e];
    }
    __syncthreads();
    if (kbase + BN < kend) fetch(kbase + BN);
    // a wave none of whose 16 rows exists only helps with the staging
    if (wave * 16 >= nrows) continue;

    float4v acc_s[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      acc_s[nt] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NP / 32; ++kk) {
        const int krow = nt * 16 + frag_m;
        short8v bfrag = *reinterpret_cast<const short8v*>(
            reinterpret_cast<char*>(k_s) + krow * KROWB +
            swz<KROWB>(krow, (kk * 32 + frag_k8) * 2));
        acc_s[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[kk], bfrag,
                                                            acc_s[nt], 0, 0, 0);
      }
    }

    float pmax[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int lo = klo[r];
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int kpos = kbase + nt * 16 + ccol;
        float s = acc_s[nt][r] * rscale[r];
        if (softcap > 0.0f) s = softcap * tanh_fast(s * inv_cap);
        s -= slope[r] * (float)(qpos[r] - kpos);
        if (kpos > qpos[r] || kpos >= KVL || kpos < lo) s = -INFINITY;
        acc_s[nt][r] = s;
        mx = fmaxf(mx, s);
      }
      pmax[r] = group_reduce_max<16>(mx);
    }
    float alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float mn = fmaxf(m[r], pmax[r]);
      alpha[r] = (m[r] == -INFINITY) ? 0.0f : __expf(m[r] - mn);
      m[r] = mn;
      float rowsum = 0.0f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const float s = acc_s[nt][r];
        const float p = (s == -INFINITY) ? 0.0f : __expf(s - mn);
        rowsum += p;
        const int prow = crow0 + r;
        *reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(pw_s) +
                                     prow * (BN * 2) +
                                     swz<128>(prow, (nt * 16 + ccol) * 2)) =
            f32_to_bf16(p);
      }
      l[r] = l[r] * alpha[r] + group_reduce_sum<16>(rowsum);
    }
#pragma unroll
    for (int nt = 0; nt < PP / 16; ++nt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc_o[nt][r] *= alpha[r];
    }
#pragma unroll
    for (int kk2 = 0; kk2 < BN / 32; ++kk2) {
      short8v pfrag = *reinterpret_cast<const short8v*>(
          reinterpret_cast<char*>(pw_s) + frag_m * (BN * 2) +
          swz<128>(frag_m, (kk2 * 32 + frag_k8) * 2));
#pragma unroll
      for (int nt = 0; nt < PP / 16; ++nt) {
        const int vrow = nt * 16 + frag_m;
        short8v vfrag = *reinterpret_cast<const short8v*>(
            reinterpret_cast<char*>(vt_s) + vrow * (BN * 2) +
            swz_vt(vrow, (kk2 * 32 + frag_k8) * 2));
        acc_o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pfrag, vfrag,
                                                            acc_o[nt], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = wave * 16 + crow0 + r;
    if (row >= nrows) continue;
    const int64_t tok = HEADS_ROWS ? q0 : q0 + qoff + row;
    const int head = HEADS_ROWS ? kvh * rep + row : blockIdx.y;
    // the sink's term relative to the running maximum (an overflow to
    // infinity gives the right limit, an all-zero row)
    const float lsum = sinks ? l[r] + __expf(sinks[head] - m[r]) : l[r];
    const float inv = 1.0f / lsum;
    uint16_t* o = out + (tok * H + head) * P;
    const uint16_t* gt = gate ? gate + tok * gate_rs + head * P : nullptr;
#pragma unroll
    for (int nt = 0; nt < PP / 16; ++nt) {
      const int c = nt * 16 + ccol;
      if (c < P) {
        float y = acc_o[nt][r] * inv;
        if (gt) y *= sigmoid_fast(bf16_to_f32(gt[c]));
        o[c] = f32_to_bf16(y);
      }
    }
  }
}

int64_t softcap_attention_tile_rows() { return SA_BM; }

// prompt tiles: (tile_seq, tile_off) over the first sequences of the
// batch; decoded rows: dec_seq lists the sequences that bring one row.
// Returns false when the sizes do not fit the tile kernel.
bool softcap_attention_mfma(torch::Tensor out, torch::Tensor q,
                            torch::Tensor kcache, torch::Tensor vcache,
                            torch::Tensor block_table, torch::Tensor seq_cu,
                            torch::Tensor seq_start, torch::Tensor tile_seq,
                            torch::Tensor tile_off, torch::Tensor dec_seq,
                            double scale, double softcap, double temp_coef,
                            int64_t temp_every, int64_t window,
                            c10::optional<torch::Tensor> slopes,
                            int64_t chunk, c10::optional<torch::Tensor> sinks,
                            c10::optional<torch::Tensor> gate) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 2 && q.stride(1) == 1);
  if (q.scalar_type() != torch::kBFloat16) return false;
  TORCH_CHECK(kcache.is_contiguous() && kcache.dim() == 4 &&
              vcache.is_contiguous() && vcache.dim() == 4 &&
              kcache.dtype() == q.dtype() && vcache.dtype() == q.dtype());
  const int T = q.size(0), G = kcache.size(1), BS = kcache.size(2);
  const int N = kcache.size(3), P = vcache.size(3);
  TORCH_CHECK(q.size(1) % N == 0);
  const int H = q.size(1) / N;
  TORCH_CHECK(H % G == 0 && vcache.size(0) == kcache.size(0) &&
              vcache.size(1) == G && vcache.size(2) == BS);
  const int ndec = dec_seq.numel(), ntile = tile_seq.numel();
  if (N % 8 || P % 8 || N > 128 || P > 256 || q.stride(0) % 8 ||
      (reinterpret_cast<uintptr_t>(q.data_ptr()) & 15) ||
      (ndec > 0 && H / G > SA_BM))
    return false;
  TORCH_CHECK(out.is_contiguous() && out.dtype() == q.dtype() &&
              out.numel() == (int64_t)T * H * P);
  TORCH_CHECK(block_table.dtype() == torch::kInt32 &&
              block_table.is_contiguous() && block_table.dim() == 2);
  const int S = seq_start.numel();
  TORCH_CHECK(seq_cu.dtype() == torch::kInt32 && seq_cu.numel() == S + 1 &&
              seq_start.dtype() == torch::kInt32 && block_table.size(0) >= S);
  TORCH_CHECK(tile_seq.dtype() == torch::kInt32 &&
              tile_off.dtype() == torch::kInt32 &&
              tile_off.numel() == ntile && dec_seq.dtype() == torch::kInt32);
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
  hipStream_t stream = at::cuda::getCurrentCUDAStream();
#define LAUNCH_SA(NPV, PPV, HR, GRID, TSEQ)                                   \
  hipLaunchKernelGGL(                                                         \
      (softcap_attention_mfma_kernel<NPV, PPV, HR>), GRID, dim3(256), 0,      \
      stream, (uint16_t*)out.data_ptr(), (const uint16_t*)q.data_ptr(),       \
      (int64_t)q.stride(0), (const uint16_t*)kcache.data_ptr(),               \
      (const uint16_t*)vcache.data_ptr(),                                     \
      (const int32_t*)block_table.data_ptr(), (int)block_table.size(1),       \
      (const int32_t*)seq_cu.data_ptr(), (const int32_t*)seq_start.data_ptr(), \
      (const int32_t*)TSEQ.data_ptr(), (const int32_t*)tile_off.data_ptr(),   \
      H, G, N, P, BS, (float)scale, (float)softcap, (float)temp_coef,         \
      (int)temp_every, (int)window,                                           \
      slopes.has_value() ? (const float*)slopes->data_ptr() : nullptr,        \
      (int)chunk,                                                             \
      sinks.has_value() ? (const float*)sinks->data_ptr() : nullptr,          \
      gate.has_value() ? (const uint16_t*)gate->data_ptr() : nullptr,         \
      gate.has_value() ? (int64_t)gate->stride(0) : 0)
#define LAUNCH_SA_SIZES(HR, GRID, TSEQ)                                       \
  do {                                                                        \
    if (N <= 64 && P <= 64) LAUNCH_SA(64, 64, HR, GRID, TSEQ);                \
    else if (N <= 64 && P <= 128) LAUNCH_SA(64, 128, HR, GRID, TSEQ);         \
    else if (N <= 64) LAUNCH_SA(64, 256, HR, GRID, TSEQ);                     \
    else if (P <= 64) LAUNCH_SA(128, 64, HR, GRID, TSEQ);                     \
    else if (P <= 128) LAUNCH_SA(128, 128, HR, GRID, TSEQ);                   \
    else LAUNCH_SA(128, 256, HR, GRID, TSEQ);                                 \
  } while (0)
  if (ntile > 0) LAUNCH_SA_SIZES(false, dim3(ntile, H), tile_seq);
  if (ndec > 0) LAUNCH_SA_SIZES(true, dim3(ndec, G), dec_seq);
#undef LAUNCH_SA_SIZES
#undef LAUNCH_SA
  HIP_CHECK_KERNEL();
  return true;
}

}  // namespace igw
