// Shared-key/value rotary attention over the paged cache.
//
//  * rope_unitnorm_cache: interleaved-pair rotary on the leading rot dims
//    of every q/k head (fp32 angle = position * inv_freq), each head then
//    divided by its RMS; processed q to a dense buffer, processed k to
//    the paged k cache and the UNPROCESSED k to the paged v cache.
//  * ranged_paged_attention (row-per-wave form): each (row, head) wave
//    walks the row's visible key range [lo, p] of its own sequence —
//    lo from the chunk and/or window mask — 64 keys per step with an
//    online fp32 softmax. One-row (decode) groups and short rows use it.
//
// Cache layout: [num_blocks, kv_heads, block_size, head_dim].

#include "seqmix.h"

namespace fi {

constexpr int kMaxPairsPerLane = 4;  // head_dim <= 512

template <typename A>
__global__ __launch_bounds__(64) void rope_unitnorm_cache_kernel(
    A* __restrict__ q_out,            // [T, H, D] dense
    const A* __restrict__ q, int64_t q_stride,
    const A* __restrict__ k, int64_t k_stride,
    const int* __restrict__ positions, const float* __restrict__ inv_freq,
    A* __restrict__ k_cache, A* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, int H, int G, int D, int rot_dims,
    int block_size, float eps) {
  const int t = blockIdx.x;
  const int hh = blockIdx.y;  // 0..H-1: q heads, H..H+G-1: k heads
  const int lane = threadIdx.x;
  const bool is_q = hh < H;
  const A* src = is_q ? q + t * q_stride + static_cast<int64_t>(hh) * D
                      : k + t * k_stride + static_cast<int64_t>(hh - H) * D;
  const float pos = static_cast<float>(positions[t]);
  const int npairs = (D + 1) / 2;
  float u[kMaxPairsPerLane], w[kMaxPairsPerLane];
  float ru[kMaxPairsPerLane], rw[kMaxPairsPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    u[i] = w[i] = ru[i] = rw[i] = 0.f;
    if (j < npairs) {
      u[i] = Act<A>::ld(src + 2 * j);
      const bool has_w = 2 * j + 1 < D;
      w[i] = has_w ? Act<A>::ld(src + 2 * j + 1) : 0.f;
      if (2 * j + 1 < rot_dims) {
        const float ang = pos * inv_freq[j];
        float sn, cs;
        sincosf(ang, &sn, &cs);
        ru[i] = u[i] * cs - w[i] * sn;
        rw[i] = w[i] * cs + u[i] * sn;
      } else {
        ru[i] = u[i];
        rw[i] = w[i];
      }
      ss += ru[i] * ru[i] + rw[i] * rw[i];
    }
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / D + eps);
  A* dst;
  A* raw = nullptr;
  if (is_q) {
    dst = q_out + (static_cast<int64_t>(t) * H + hh) * D;
  } else {
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    const int64_t off =
        ((static_cast<int64_t>(slot / block_size) * G + (hh - H)) * block_size +
         slot % block_size) * D;
    dst = k_cache + off;
    raw = v_cache + off;
  }
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    if (j < npairs) {
      Act<A>::st(dst + 2 * j, ru[i] * inv);
      if (raw) Act<A>::st(raw + 2 * j, u[i]);
      if (2 * j + 1 < D) {
        Act<A>::st(dst + 2 * j + 1, rw[i] * inv);
        if (raw) Act<A>::st(raw + 2 * j + 1, w[i]);
      }
    }
  }
}

constexpr int kAttnWaves = 4;        // (row, head) pairs per workgroup
constexpr int kMaxDPerLane = 8;      // head_dim <= 512

template <typename A>
__global__ __launch_bounds__(64 * kAttnWaves) void ranged_attention_row_kernel(
    A* __restrict__ out,              // [T, H, D]
    const A* __restrict__ q,          // [T, H, D]
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ seq_bt, int bt_stride,
    const int* __restrict__ row_seq, const int* __restrict__ positions,
    int T, int H, int G, int D, int block_size, float scale, int chunk,
    int window) {
  extern __shared__ float smem[];     // kAttnWaves * D floats of q
  const int wave = threadIdx.x / 64;
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kAttnWaves + wave;
  const bool live = item < static_cast<int64_t>(T) * H;
  const int t = live ? static_cast<int>(item / H) : 0;
  const int h = live ? static_cast<int>(item % H) : 0;
  float* qs = smem + wave * D;
  if (live) {
    const A* qp = q + (static_cast<int64_t>(t) * H + h) * D;
    for (int d = lane; d < D; d += 64) qs[d] = Act<A>::ld(qp + d);
  }
  __syncthreads();
  if (!live) return;
  const int p = positions[t];
  int lo = 0;
  if (chunk > 0) lo = (p / chunk) * chunk;
  if (window > 0) lo = max(lo, p - window + 1);
  const int g = h / (H / G);
  const int* bt = seq_bt + static_cast<int64_t>(row_seq[t]) * bt_stride;

  float m = -INFINITY, l = 0.f;
  float acc[kMaxDPerLane];
#pragma unroll
  for (int i = 0; i < kMaxDPerLane; ++i) acc[i] = 0.f;

  for (int j0 = lo; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= p) {
      const int blk = bt[j / block_size];
      const A* kp = k_cache +
          ((static_cast<int64_t>(blk) * G + g) * block_size + j % block_size) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * Act<A>::ld(kp + d);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_reduce_max(s));
    const float corr = expf(m - m_new);      // m = -inf first: exp(-inf) = 0
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    l = l * corr + wave_reduce_sum(pj);
#pragma unroll
    for (int i = 0; i < kMaxDPerLane; ++i) acc[i] *= corr;
    m = m_new;
    const int n = min(64, p - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const float pv = __shfl(pj, jj, 64);
      const int key = j0 + jj;
      const int blk = bt[key / block_size];
      const A* vp = v_cache +
          ((static_cast<int64_t>(blk) * G + g) * block_size + key % block_size) * D;
#pragma unroll
      for (int i = 0; i < kMaxDPerLane; ++i) {
        const int d = lane + 64 * i;
        if (d < D) acc[i] += pv * Act<A>::ld(vp + d);
      }
    }
  }
  const float inv_l = 1.0f / l;
  A* op = out + (static_cast<int64_t>(t) * H + h) * D;
#pragma unroll
  for (int i = 0; i < kMaxDPerLane; ++i) {
    const int d = lane + 64 * i;
    if (d < D) Act<A>::st(op + d, acc[i] * inv_l);
  }
}

template <typename A>
void launch_rope_unitnorm_cache(A* q_out, const A* q, int64_t q_stride,
                                const A* k, int64_t k_stride,
                                const int* positions, const float* inv_freq,
                                A* k_cache, A* v_cache,
                                const int* slot_mapping, int T, int H, int G,
                                int D, int rot_dims, int block_size, float eps,
                                hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(rope_unitnorm_cache_kernel<A>, dim3(T, H + G), dim3(64), 0,
                     s, q_out, q, q_stride, k, k_stride, positions, inv_freq,
                     k_cache, v_cache, slot_mapping, H, G, D, rot_dims,
                     block_size, eps);
}

template <typename A>
void launch_ranged_attention_rows(A* out, const A* q, const A* k_cache,
                                  const A* v_cache, const int* seq_bt,
                                  int bt_stride, const int* row_seq,
                                  const int* positions, int T, int H, int G,
                                  int D, int block_size, float scale,
                                  int chunk, int window, hipStream_t s) {
  if (T == 0) return;
  const int64_t items = static_cast<int64_t>(T) * H;
  const int blocks = static_cast<int>((items + kAttnWaves - 1) / kAttnWaves);
  hipLaunchKernelGGL(ranged_attention_row_kernel<A>, dim3(blocks),
                     dim3(64 * kAttnWaves), kAttnWaves * D * sizeof(float), s,
                     out, q, k_cache, v_cache, seq_bt, bt_stride, row_seq,
                     positions, T, H, G, D, block_size, scale, chunk, window);
}

#define FI_INST(A)                                                             \
  template void launch_rope_unitnorm_cache<A>(                                 \
      A*, const A*, int64_t, const A*, int64_t, const int*, const float*, A*,  \
      A*, const int*, int, int, int, int, int, int, float, hipStream_t);       \
  template void launch_ranged_attention_rows<A>(                               \
      A*, const A*, const A*, const A*, const int*, int, const int*,           \
      const int*, int, int, int, int, int, float, int, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
