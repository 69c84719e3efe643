// Row kernels of a layer-normed fp32 residual stream with sigmoid-gated
// sublayer results, grouped unit-RMS output gates, and the plain paged
// cache write.
//
//  * layer_norm:  out = (x - mean) / sqrt(var + eps) * w   (biased var)
//  * gated_residual_layer_norm:
//        x += (s1*y1 + s2*y2) * sigmoid(gate_lin + gate_bias)   (fp32)
//        out = layer_norm(x) * w_next                           (optional)
//    one workgroup per row; the row is re-read from L2 for the second
//    statistic (mean first, then squared deviations) so any width works.
//  * group_rms_gate: rows of fp32 read-outs cut into equal groups, each
//    divided by its RMS, times a gain (per coordinate or per position in
//    the group) and sigmoid/silu of a gate projection. One wave per
//    (row, group).
//  * paged_cache_write: k/v rows into [blocks, heads, block, size] caches.

#include "seqmix.h"

namespace fi {

namespace {

// mean and 1/sqrt(var + eps) of a fp32 row, by a 256-thread workgroup
FI_DEV void row_moments(const float* row, int W, float eps, float* scratch,
                        float& mean, float& rstd) {
  float s = 0.f, dummy = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) s += row[i];
  block_reduce_sum2_256(s, dummy, scratch);
  mean = s / W;
  float q = 0.f;
  dummy = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float d = row[i] - mean;
    q += d * d;
  }
  block_reduce_sum2_256(q, dummy, scratch);
  rstd = rsqrtf(q / W + eps);
}

template <typename A>
__global__ __launch_bounds__(256) void layer_norm_kernel(
    A* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ w, float eps, int W) {
  __shared__ float scratch[8];
  const float* row = x + static_cast<int64_t>(blockIdx.x) * W;
  float mean, rstd;
  row_moments(row, W, eps, scratch, mean, rstd);
  A* o = out + static_cast<int64_t>(blockIdx.x) * W;
  for (int i = threadIdx.x; i < W; i += 256)
    Act<A>::st(o + i, (row[i] - mean) * rstd * w[i]);
}

template <typename A>
__global__ __launch_bounds__(256) void gated_residual_layer_norm_kernel(
    float* __restrict__ resid, const A* __restrict__ y1, float s1,
    const A* __restrict__ y2, float s2, const A* __restrict__ gate_lin,
    int64_t g_stride, const float* __restrict__ gate_bias,
    const float* __restrict__ w_next, A* __restrict__ out, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t t = blockIdx.x;
  float* row = resid + t * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    float y = s1 * Act<A>::ld(y1 + t * W + i);
    if (y2 != nullptr) y += s2 * Act<A>::ld(y2 + t * W + i);
    const float g =
        sigmoidf_acc(Act<A>::ld(gate_lin + t * g_stride + i) + gate_bias[i]);
    row[i] += y * g;     // each element is read and written by one thread
  }
  if (w_next == nullptr) return;
  __syncthreads();
  float mean, rstd;
  row_moments(row, W, eps, scratch, mean, rstd);
  A* o = out + t * W;
  for (int i = threadIdx.x; i < W; i += 256)
    Act<A>::st(o + i, (row[i] - mean) * rstd * w_next[i]);
}

template <typename A>
__global__ __launch_bounds__(256) void group_rms_gate_kernel(
    A* __restrict__ out, const float* __restrict__ o_raw,
    const A* __restrict__ glin, int64_t g_stride, const float* __restrict__ w,
    int w_shared, int T, int groups, int part, float eps, bool silu) {
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / 64;
  if (item >= static_cast<int64_t>(T) * groups) return;
  const int64_t t = item / groups;
  const int grp = static_cast<int>(item % groups);
  const int64_t base = t * groups * part + static_cast<int64_t>(grp) * part;
  float ss = 0.f;
  for (int d = lane; d < part; d += 64) {
    const float o = o_raw[base + d];
    ss += o * o;
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / part + eps);
  for (int d = lane; d < part; d += 64) {
    const float g = Act<A>::ld(glin + t * g_stride + grp * part + d);
    const float gate = silu ? g * sigmoidf_acc(g) : sigmoidf_acc(g);
    const float gain = w[w_shared ? d : grp * part + d];
    Act<A>::st(out + base + d, o_raw[base + d] * inv * gain * gate);
  }
}

template <typename A>
__global__ __launch_bounds__(256) void paged_cache_write_kernel(
    A* __restrict__ k_cache, A* __restrict__ v_cache, const A* __restrict__ k,
    int64_t k_stride, const A* __restrict__ v, int64_t v_stride,
    const int* __restrict__ slot_mapping, int G, int bs, int D, int V) {
  const int t = blockIdx.x;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t blk = slot / bs;
  const int off = slot % bs;
  for (int i = threadIdx.x; i < G * D; i += 256) {
    const int g = i / D, d = i % D;
    k_cache[((blk * G + g) * bs + off) * D + d] = k[t * k_stride + i];
  }
  for (int i = threadIdx.x; i < G * V; i += 256) {
    const int g = i / V, d = i % V;
    v_cache[((blk * G + g) * bs + off) * V + d] = v[t * v_stride + i];
  }
}

}  // namespace

template <typename A>
void launch_layer_norm(A* out, const float* x, const float* w, float eps,
                       int T, int W, hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(layer_norm_kernel<A>, dim3(T), dim3(256), 0, st, out, x,
                     w, eps, W);
}

template <typename A>
void launch_gated_residual_layer_norm(float* resid, const A* y1, float s1,
                                      const A* y2, float s2, const A* gate_lin,
                                      int64_t g_stride, const float* gate_bias,
                                      const float* w_next, A* out, float eps,
                                      int T, int W, hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(gated_residual_layer_norm_kernel<A>, dim3(T), dim3(256),
                     0, st, resid, y1, s1, y2, s2, gate_lin, g_stride,
                     gate_bias, w_next, out, eps, W);
}

template <typename A>
void launch_group_rms_gate(A* out, const float* o_raw, const A* glin,
                           int64_t g_stride, const float* w, bool w_shared,
                           int T, int groups, int part, float eps, bool silu,
                           hipStream_t st) {
  if (T == 0) return;
  const int64_t items = static_cast<int64_t>(T) * groups;
  hipLaunchKernelGGL(group_rms_gate_kernel<A>,
                     dim3(static_cast<int>((items + 3) / 4)), dim3(256), 0, st,
                     out, o_raw, glin, g_stride, w, w_shared ? 1 : 0, T,
                     groups, part, eps, silu);
}

template <typename A>
void launch_paged_cache_write(A* k_cache, A* v_cache, const A* k,
                              int64_t k_stride, const A* v, int64_t v_stride,
                              const int* slot_mapping, int T, int G, int bs,
                              int D, int V, hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(paged_cache_write_kernel<A>, dim3(T), dim3(256), 0, st,
                     k_cache, v_cache, k, k_stride, v, v_stride, slot_mapping,
                     G, bs, D, V);
}

#define FI_INST(A)                                                             \
  template void launch_layer_norm<A>(A*, const float*, const float*, float,    \
                                     int, int, hipStream_t);                   \
  template void launch_gated_residual_layer_norm<A>(                           \
      float*, const A*, float, const A*, float, const A*, int64_t,             \
      const float*, const float*, A*, float, int, int, hipStream_t);           \
  template void launch_group_rms_gate<A>(A*, const float*, const A*, int64_t,  \
                                         const float*, bool, int, int, int,    \
                                         float, bool, hipStream_t);            \
  template void launch_paged_cache_write<A>(A*, A*, const A*, int64_t,         \
                                            const A*, int64_t, const int*,     \
                                            int, int, int, int, int,           \
                                            hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
