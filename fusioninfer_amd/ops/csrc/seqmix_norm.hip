// Row kernels on the fp32 residual stream: scalar-gain RMS norms, the
// fused residual updates around a sublayer, the norm + token shift in
// front of a mixer, and the tanh-GELU gated activation.
//
// One 256-thread workgroup per token row; a row is re-read from L2 for
// the second pass instead of being held in registers, so any width works.

#include "seqmix.h"

namespace fi {

constexpr int kRowThreads = 256;

// out = x * rsqrt(mean(x^2) + eps) * g
template <typename A>
__global__ __launch_bounds__(kRowThreads) void scalar_rms_norm_kernel(
    A* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ g, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f, zero = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float v = x[base + c];
    ss += v * v;
  }
  block_reduce_sum2_256(ss, zero, scratch);
  const float sc = rsqrtf(ss / W + eps) * g[0];
  for (int c = threadIdx.x; c < W; c += kRowThreads)
    Act<A>::st(out + base + c, x[base + c] * sc);
}

// resid += y * rsqrt(mean(y^2)+eps) * g_post; optionally
// out = resid * rsqrt(mean(resid^2)+eps) * g_next
template <typename A>
__global__ __launch_bounds__(kRowThreads) void residual_add_scalar_norm_kernel(
    float* __restrict__ resid, const A* __restrict__ y,
    const float* __restrict__ g_post, const float* __restrict__ g_next,
    A* __restrict__ out, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f, zero = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float v = Act<A>::ld(y + base + c);
    ss += v * v;
  }
  block_reduce_sum2_256(ss, zero, scratch);
  const float sc = rsqrtf(ss / W + eps) * g_post[0];
  float rs = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float r = resid[base + c] + Act<A>::ld(y + base + c) * sc;
    resid[base + c] = r;
    rs += r * r;
  }
  if (g_next == nullptr) return;
  zero = 0.f;
  block_reduce_sum2_256(rs, zero, scratch);
  const float sn = rsqrtf(rs / W + eps) * g_next[0];
  for (int c = threadIdx.x; c < W; c += kRowThreads)
    Act<A>::st(out + base + c, resid[base + c] * sn);
}

// y = (yl*rms^-1(yl)*wl + yr*rms^-1(yr)*wr)/2; resid += y*rms^-1(y)*g_post;
// optionally out = resid * rms^-1(resid) * g_next
template <typename A>
__global__ __launch_bounds__(kRowThreads) void dual_norm_combine_residual_kernel(
    float* __restrict__ resid, const A* __restrict__ yl,
    const A* __restrict__ yr, const float* __restrict__ wl,
    const float* __restrict__ wr, const float* __restrict__ g_post,
    const float* __restrict__ g_next, A* __restrict__ out, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float sl = 0.f, sr = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float a = Act<A>::ld(yl + base + c);
    const float b = Act<A>::ld(yr + base + c);
    sl += a * a;
    sr += b * b;
  }
  block_reduce_sum2_256(sl, sr, scratch);
  const float il = rsqrtf(sl / W + eps), ir = rsqrtf(sr / W + eps);
  float sy = 0.f, zero = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float v = 0.5f * (Act<A>::ld(yl + base + c) * il * wl[c] +
                            Act<A>::ld(yr + base + c) * ir * wr[c]);
    sy += v * v;
  }
  block_reduce_sum2_256(sy, zero, scratch);
  const float iy = rsqrtf(sy / W + eps) * g_post[0];
  float rs = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float v = 0.5f * (Act<A>::ld(yl + base + c) * il * wl[c] +
                            Act<A>::ld(yr + base + c) * ir * wr[c]);
    const float r = resid[base + c] + v * iy;
    resid[base + c] = r;
    rs += r * r;
  }
  if (g_next == nullptr) return;
  zero = 0.f;
  block_reduce_sum2_256(rs, zero, scratch);
  const float sn = rsqrtf(rs / W + eps) * g_next[0];
  for (int c = threadIdx.x; c < W; c += kRowThreads)
    Act<A>::st(out + base + c, resid[base + c] * sn);
}

// h_t = rms-norm(resid_t) * g; out_t = h_t + (h_prev - h_t) * shift.
// h_prev of a group's first row is the slot's saved vector (zero at
// position 0 or without a slot); that same workgroup then saves the
// group's LAST h into the slot, after its own read of every element, so
// no other workgroup touches the slot concurrently.
template <typename A>
__global__ __launch_bounds__(kRowThreads) void norm_token_shift_kernel(
    A* __restrict__ out, const float* __restrict__ resid,
    const float* __restrict__ g, const float* __restrict__ shift,
    float* __restrict__ state, const int* __restrict__ seq_cu,
    const int* __restrict__ row_seq, const int* __restrict__ positions,
    const int* __restrict__ seq_slots, float eps, int W) {
  __shared__ float scratch[8];
  const int t = blockIdx.x;
  const int s = row_seq[t];
  const int first_row = seq_cu[s];
  const int last_row = seq_cu[s + 1] - 1;
  const bool first = (t == first_row);
  const int slot = seq_slots[s];
  const int64_t base = static_cast<int64_t>(t) * W;
  // the second row this workgroup needs statistics of
  const int other = first ? last_row : t - 1;
  const int64_t obase = static_cast<int64_t>(other) * W;
  float ss = 0.f, so = 0.f;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float v = resid[base + c];
    const float o = resid[obase + c];
    ss += v * v;
    so += o * o;
  }
  block_reduce_sum2_256(ss, so, scratch);
  const float gg = g[0];
  const float sc = rsqrtf(ss / W + eps) * gg;
  const float oc = rsqrtf(so / W + eps) * gg;
  if (!first) {
    for (int c = threadIdx.x; c < W; c += kRowThreads) {
      const float h = resid[base + c] * sc;
      const float hp = resid[obase + c] * oc;
      Act<A>::st(out + base + c, h + (hp - h) * shift[c]);
    }
    return;
  }
  const bool carry = slot >= 0 && positions[t] > 0;
  float* st = slot >= 0 ? state + static_cast<int64_t>(slot) * W : nullptr;
  for (int c = threadIdx.x; c < W; c += kRowThreads) {
    const float h = resid[base + c] * sc;
    const float hp = carry ? st[c] : 0.f;
    Act<A>::st(out + base + c, h + (hp - h) * shift[c]);
    if (st != nullptr) st[c] = resid[obase + c] * oc;
  }
}

// out[t, f] = gelu_tanh(gu[t, f]) * gu[t, F + f]
template <typename A>
__global__ __launch_bounds__(kRowThreads) void gelu_tanh_and_mul_kernel(
    A* __restrict__ out, const A* __restrict__ gu, int F) {
  const int64_t ib = static_cast<int64_t>(blockIdx.x) * 2 * F;
  const int64_t ob = static_cast<int64_t>(blockIdx.x) * F;
  for (int c = blockIdx.y * kRowThreads + threadIdx.x; c < F;
       c += gridDim.y * kRowThreads) {
    const float z = Act<A>::ld(gu + ib + c);
    const float u = Act<A>::ld(gu + ib + F + c);
    const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    Act<A>::st(out + ob + c, 0.5f * z * (1.0f + tanhf(inner)) * u);
  }
}

template <typename A>
void launch_scalar_rms_norm(A* out, const float* x, const float* g, float eps,
                            int T, int W, hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(scalar_rms_norm_kernel<A>, dim3(T), dim3(kRowThreads), 0,
                     s, out, x, g, eps, W);
}

template <typename A>
void launch_residual_add_scalar_norm(float* resid, const A* y,
                                     const float* g_post, const float* g_next,
                                     A* out, float eps, int T, int W,
                                     hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(residual_add_scalar_norm_kernel<A>, dim3(T),
                     dim3(kRowThreads), 0, s, resid, y, g_post, g_next, out,
                     eps, W);
}

template <typename A>
void launch_dual_norm_combine_residual(float* resid, const A* yl, const A* yr,
                                       const float* wl, const float* wr,
                                       const float* g_post,
                                       const float* g_next, A* out, float eps,
                                       int T, int W, hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(dual_norm_combine_residual_kernel<A>, dim3(T),
                     dim3(kRowThreads), 0, s, resid, yl, yr, wl, wr, g_post,
                     g_next, out, eps, W);
}

template <typename A>
void launch_norm_token_shift(A* out, const float* resid, const float* g,
                             const float* shift, float* state,
                             const int* seq_cu, const int* row_seq,
                             const int* positions, const int* seq_slots,
                             float eps, int T, int W, hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(norm_token_shift_kernel<A>, dim3(T), dim3(kRowThreads), 0,
                     s, out, resid, g, shift, state, seq_cu, row_seq,
                     positions, seq_slots, eps, W);
}

template <typename A>
void launch_gelu_tanh_and_mul(A* out, const A* gu, int T, int F,
                              hipStream_t s) {
  if (T == 0) return;
  const int gy = std::min(ceil_div(F, kRowThreads * 4), 64);
  hipLaunchKernelGGL(gelu_tanh_and_mul_kernel<A>, dim3(T, std::max(gy, 1)),
                     dim3(kRowThreads), 0, s, out, gu, F);
}

#define FI_INST(A)                                                             \
  template void launch_scalar_rms_norm<A>(A*, const float*, const float*,      \
                                          float, int, int, hipStream_t);       \
  template void launch_residual_add_scalar_norm<A>(                            \
      float*, const A*, const float*, const float*, A*, float, int, int,       \
      hipStream_t);                                                            \
  template void launch_dual_norm_combine_residual<A>(                          \
      float*, const A*, const A*, const float*, const float*, const float*,    \
      const float*, A*, float, int, int, hipStream_t);                         \
  template void launch_norm_token_shift<A>(                                    \
      A*, const float*, const float*, const float*, float*, const int*,        \
      const int*, const int*, const int*, float, int, int, hipStream_t);       \
  template void launch_gelu_tanh_and_mul<A>(A*, const A*, int, int,            \
                                            hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
