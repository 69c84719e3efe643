// Row kernels on the fp32 residual stream: scalar-gain RMS norms, the
// fused residual updates around a sublayer, the norm + token shift in
// front of a mixer, and the tanh-GELU gated activation.
//
// One 256-thread workgroup per token row; a row is re-read from L2 for
// every pass instead of being held in registers, so any width works.
// Rows whose width is a multiple of 4 move 4 elements per access (VW = 4:
// 16-byte fp32, 8-byte bf16); other widths take the scalar form (VW = 1).

#include "seqmix.h"

namespace fi {

constexpr int kRowThreads = 256;

#define FI_ROW_LOOP(c) \
  for (int c = threadIdx.x * VW; c < W; c += kRowThreads * VW)

// out = x * rsqrt(mean(x^2) + eps) * g
template <typename A, int VW>
__global__ __launch_bounds__(kRowThreads) void scalar_rms_norm_kernel(
    A* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ g, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f, zero = 0.f;
  FI_ROW_LOOP(c) {
    float v[VW];
    ldv<float, VW>(x + base + c, v);
#pragma unroll
    for (int i = 0; i < VW; ++i) ss += v[i] * v[i];
  }
  block_reduce_sum2_256(ss, zero, scratch);
  const float sc = rsqrtf(ss / W + eps) * g[0];
  FI_ROW_LOOP(c) {
    float v[VW];
    ldv<float, VW>(x + base + c, v);
#pragma unroll
    for (int i = 0; i < VW; ++i) v[i] *= sc;
    stv<A, VW>(out + base + c, v);
  }
}

// resid += y * rsqrt(mean(y^2)+eps) * g_post; optionally
// out = resid * rsqrt(mean(resid^2)+eps) * g_next
template <typename A, int VW>
__global__ __launch_bounds__(kRowThreads) void residual_add_scalar_norm_kernel(
    float* __restrict__ resid, const A* __restrict__ y,
    const float* __restrict__ g_post, const float* __restrict__ g_next,
    A* __restrict__ out, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f, zero = 0.f;
  FI_ROW_LOOP(c) {
    float v[VW];
    ldv<A, VW>(y + base + c, v);
#pragma unroll
    for (int i = 0; i < VW; ++i) ss += v[i] * v[i];
  }
  block_reduce_sum2_256(ss, zero, scratch);
  const float sc = rsqrtf(ss / W + eps) * g_post[0];
  float rs = 0.f;
  FI_ROW_LOOP(c) {
    float v[VW], r[VW];
    ldv<A, VW>(y + base + c, v);
    ldv<float, VW>(resid + base + c, r);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      r[i] += v[i] * sc;
      rs += r[i] * r[i];
    }
    stv<float, VW>(resid + base + c, r);
  }
  if (g_next == nullptr) return;
  zero = 0.f;
  block_reduce_sum2_256(rs, zero, scratch);
  const float sn = rsqrtf(rs / W + eps) * g_next[0];
  FI_ROW_LOOP(c) {
    float r[VW];
    ldv<float, VW>(resid + base + c, r);   // this thread's own stores
#pragma unroll
    for (int i = 0; i < VW; ++i) r[i] *= sn;
    stv<A, VW>(out + base + c, r);
  }
}

// y = (yl*rms^-1(yl)*wl + yr*rms^-1(yr)*wr)/2; resid += y*rms^-1(y)*g_post;
// optionally out = resid * rms^-1(resid) * g_next
template <typename A, int VW>
__global__ __launch_bounds__(kRowThreads) void dual_norm_combine_residual_kernel(
    float* __restrict__ resid, const A* __restrict__ yl,
    const A* __restrict__ yr, const float* __restrict__ wl,
    const float* __restrict__ wr, const float* __restrict__ g_post,
    const float* __restrict__ g_next, A* __restrict__ out, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float sl = 0.f, sr = 0.f;
  FI_ROW_LOOP(c) {
    float a[VW], b[VW];
    ldv<A, VW>(yl + base + c, a);
    ldv<A, VW>(yr + base + c, b);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      sl += a[i] * a[i];
      sr += b[i] * b[i];
    }
  }
  block_reduce_sum2_256(sl, sr, scratch);
  const float il = 0.5f * rsqrtf(sl / W + eps);
  const float ir = 0.5f * rsqrtf(sr / W + eps);
  float sy = 0.f, zero = 0.f;
  FI_ROW_LOOP(c) {
    float a[VW], b[VW], p[VW], q[VW];
    ldv<A, VW>(yl + base + c, a);
    ldv<A, VW>(yr + base + c, b);
    ldv<float, VW>(wl + c, p);
    ldv<float, VW>(wr + c, q);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      const float v = a[i] * il * p[i] + b[i] * ir * q[i];
      sy += v * v;
    }
  }
  block_reduce_sum2_256(sy, zero, scratch);
  const float iy = rsqrtf(sy / W + eps) * g_post[0];
  float rs = 0.f;
  FI_ROW_LOOP(c) {
    float a[VW], b[VW], p[VW], q[VW], r[VW];
    ldv<A, VW>(yl + base + c, a);
    ldv<A, VW>(yr + base + c, b);
    ldv<float, VW>(wl + c, p);
    ldv<float, VW>(wr + c, q);
    ldv<float, VW>(resid + base + c, r);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      r[i] += (a[i] * il * p[i] + b[i] * ir * q[i]) * iy;
      rs += r[i] * r[i];
    }
    stv<float, VW>(resid + base + c, r);
  }
  if (g_next == nullptr) return;
  zero = 0.f;
  block_reduce_sum2_256(rs, zero, scratch);
  const float sn = rsqrtf(rs / W + eps) * g_next[0];
  FI_ROW_LOOP(c) {
    float r[VW];
    ldv<float, VW>(resid + base + c, r);
#pragma unroll
    for (int i = 0; i < VW; ++i) r[i] *= sn;
    stv<A, VW>(out + base + c, r);
  }
}

// h_t = rms-norm(resid_t) * g; out_t = h_t + (h_prev - h_t) * shift.
// h_prev of a group's first row is the slot's saved vector (zero at
// position 0 or without a slot); that same workgroup then saves the
// group's LAST h into the slot, after its own read of every element, so
// no other workgroup touches the slot concurrently.
template <typename A, int VW>
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
  FI_ROW_LOOP(c) {
    float v[VW], o[VW];
    ldv<float, VW>(resid + base + c, v);
    ldv<float, VW>(resid + obase + c, o);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      ss += v[i] * v[i];
      so += o[i] * o[i];
    }
  }
  block_reduce_sum2_256(ss, so, scratch);
  const float gg = g[0];
  const float sc = rsqrtf(ss / W + eps) * gg;
  const float oc = rsqrtf(so / W + eps) * gg;
  if (!first) {
    FI_ROW_LOOP(c) {
      float v[VW], o[VW], m[VW];
      ldv<float, VW>(resid + base + c, v);
      ldv<float, VW>(resid + obase + c, o);
      ldv<float, VW>(shift + c, m);
#pragma unroll
      for (int i = 0; i < VW; ++i) {
        const float h = v[i] * sc;
        v[i] = h + (o[i] * oc - h) * m[i];
      }
      stv<A, VW>(out + base + c, v);
    }
    return;
  }
  const bool carry = slot >= 0 && positions[t] > 0;
  float* st = slot >= 0 ? state + static_cast<int64_t>(slot) * W : nullptr;
  FI_ROW_LOOP(c) {
    float v[VW], o[VW], m[VW], hp[VW];
    ldv<float, VW>(resid + base + c, v);
    ldv<float, VW>(resid + obase + c, o);
    ldv<float, VW>(shift + c, m);
#pragma unroll
    for (int i = 0; i < VW; ++i) hp[i] = 0.f;
    if (carry) ldv<float, VW>(st + c, hp);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      const float h = v[i] * sc;
      v[i] = h + (hp[i] - h) * m[i];
      o[i] *= oc;
    }
    stv<A, VW>(out + base + c, v);
    if (st != nullptr) stv<float, VW>(st + c, o);
  }
}

// out[t, f] = gelu_tanh(gu[t, f]) * gu[t, F + f]
template <typename A, int VW>
__global__ __launch_bounds__(kRowThreads) void gelu_tanh_and_mul_kernel(
    A* __restrict__ out, const A* __restrict__ gu, int F) {
  const int64_t ib = static_cast<int64_t>(blockIdx.x) * 2 * F;
  const int64_t ob = static_cast<int64_t>(blockIdx.x) * F;
  for (int c = (blockIdx.y * kRowThreads + threadIdx.x) * VW; c < F;
       c += gridDim.y * kRowThreads * VW) {
    float z[VW], u[VW];
    ldv<A, VW>(gu + ib + c, z);
    ldv<A, VW>(gu + ib + F + c, u);
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      const float inner =
          0.7978845608028654f * (z[i] + 0.044715f * z[i] * z[i] * z[i]);
      z[i] = 0.5f * z[i] * (1.0f + tanhf(inner)) * u[i];
    }
    stv<A, VW>(out + ob + c, z);
  }
}

#undef FI_ROW_LOOP

// VW = 4 needs every row start 16-byte (fp32) / 8-byte (bf16) aligned
#define FI_VW_LAUNCH(KERNEL, vec_ok, grid, ...)                            \
  if (vec_ok) {                                                            \
    hipLaunchKernelGGL((KERNEL<A, 4>), grid, dim3(kRowThreads), 0, s,      \
                       __VA_ARGS__);                                       \
  } else {                                                                 \
    hipLaunchKernelGGL((KERNEL<A, 1>), grid, dim3(kRowThreads), 0, s,      \
                       __VA_ARGS__);                                       \
  }

template <typename A>
void launch_scalar_rms_norm(A* out, const float* x, const float* g, float eps,
                            int T, int W, hipStream_t s) {
  if (T == 0) return;
  FI_VW_LAUNCH(scalar_rms_norm_kernel, W % 4 == 0, dim3(T), out, x, g, eps, W);
}

template <typename A>
void launch_residual_add_scalar_norm(float* resid, const A* y,
                                     const float* g_post, const float* g_next,
                                     A* out, float eps, int T, int W,
                                     hipStream_t s) {
  if (T == 0) return;
  FI_VW_LAUNCH(residual_add_scalar_norm_kernel, W % 4 == 0, dim3(T), resid, y,
               g_post, g_next, out, eps, W);
}

template <typename A>
void launch_dual_norm_combine_residual(float* resid, const A* yl, const A* yr,
                                       const float* wl, const float* wr,
                                       const float* g_post,
                                       const float* g_next, A* out, float eps,
                                       int T, int W, hipStream_t s) {
  if (T == 0) return;
  FI_VW_LAUNCH(dual_norm_combine_residual_kernel, W % 4 == 0, dim3(T), resid,
               yl, yr, wl, wr, g_post, g_next, out, eps, W);
}

template <typename A>
void launch_norm_token_shift(A* out, const float* resid, const float* g,
                             const float* shift, float* state,
                             const int* seq_cu, const int* row_seq,
                             const int* positions, const int* seq_slots,
                             float eps, int T, int W, hipStream_t s) {
  if (T == 0) return;
  FI_VW_LAUNCH(norm_token_shift_kernel, W % 4 == 0, dim3(T), out, resid, g,
               shift, state, seq_cu, row_seq, positions, seq_slots, eps, W);
}

template <typename A>
void launch_gelu_tanh_and_mul(A* out, const A* gu, int T, int F,
                              hipStream_t s) {
  if (T == 0) return;
  const int gy = std::max(std::min(ceil_div(F, kRowThreads * 8), 64), 1);
  FI_VW_LAUNCH(gelu_tanh_and_mul_kernel, F % 4 == 0, dim3(T, gy), out, gu, F);
}

#undef FI_VW_LAUNCH

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
