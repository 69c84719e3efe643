// Generalized delta rule, recurrent form, with its output stage fused.
//
// Per (sequence, head) one workgroup walks the sequence's rows in order.
// Thread c owns column c of the head's state S [dim x dim] (fp32, in
// registers, DK = compile-time row capacity >= dim):
//
//   u   = k / sqrt(|k|^2 + 1e-6)
//   w   = exp(-decay_scale * sigmoid(wlin + w0))
//   a   = sigmoid(alin + a_bias)
//   tc  = sum_i u_i S[i][c]                         (old state)
//   S[i][c] <- w_i S[i][c] - a_i u_i tc + k_i v_c
//   o_c = sum_i S[i][c] r_i
//   out_c = o_c * rsqrt(mean_c(o^2) + eps) * norm_w * sigmoid(glin)
//
// The per-row vectors (w, a*u, u, k, r) are computed once by threads
// i < dim and broadcast through LDS. The state is read from the
// sequence's slot unless the group starts at position 0 (or has no slot)
// and written back at the end.

#include "seqmix.h"

namespace fi {

template <int NW>
FI_DEV float block_sum(float v, float* scratch) {
  v = wave_reduce_sum(v);
  const int wave = threadIdx.x / kWaveSize;
  const int lane = threadIdx.x % kWaveSize;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) tot += scratch[i];
  return tot;
}

template <typename A, int DK>
__global__ __launch_bounds__(DK) void delta_rule_kernel(
    A* __restrict__ out,                        // [T, heads*dim]
    const A* __restrict__ r, const A* __restrict__ k, const A* __restrict__ v,
    const A* __restrict__ wlin, const A* __restrict__ alin,
    const A* __restrict__ glin, int64_t r_stride, int64_t k_stride,
    int64_t v_stride, int64_t w_stride, int64_t a_stride, int64_t g_stride,
    const float* __restrict__ w0, const float* __restrict__ a_bias,
    const float* __restrict__ norm_w, float* __restrict__ state,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int heads, int dim, float eps,
    float decay_scale) {
  constexpr int NW = DK / 64;
  __shared__ float sw[DK], sau[DK], su[DK], sk[DK], sr[DK];
  __shared__ float scratch[NW];
  const int head = blockIdx.x;
  const int s = blockIdx.y;
  const int c = threadIdx.x;
  const int row0 = seq_cu[s], row1 = seq_cu[s + 1];
  if (row1 <= row0) return;
  const int slot = seq_slots[s];
  const bool active = c < dim;
  const int hc = head * dim + c;

  float S[DK];
#pragma unroll
  for (int i = 0; i < DK; ++i) S[i] = 0.f;
  float* sp = nullptr;
  if (slot >= 0)
    sp = state + (static_cast<int64_t>(slot) * heads + head) * dim * dim;
  if (sp != nullptr && positions[row0] > 0 && active) {
#pragma unroll
    for (int i = 0; i < DK; ++i)
      if (i < dim) S[i] = sp[static_cast<int64_t>(i) * dim + c];
  }
  const float w0c = active ? w0[hc] : 0.f;
  const float abc = active ? a_bias[hc] : 0.f;
  const float nwc = active ? norm_w[hc] : 0.f;

  for (int t = row0; t < row1; ++t) {
    float kc = 0.f, rc = 0.f, vc = 0.f, wc = 1.f, ac = 0.f, gc = 0.f;
    if (active) {
      kc = Act<A>::ld(k + t * k_stride + hc);
      rc = Act<A>::ld(r + t * r_stride + hc);
      vc = Act<A>::ld(v + t * v_stride + hc);
      wc = expf(-decay_scale *
                sigmoidf_acc(Act<A>::ld(wlin + t * w_stride + hc) + w0c));
      ac = sigmoidf_acc(Act<A>::ld(alin + t * a_stride + hc) + abc);
      gc = Act<A>::ld(glin + t * g_stride + hc);
    }
    const float ksq = block_sum<NW>(kc * kc, scratch);
    const float uc = kc * rsqrtf(ksq + 1e-6f);
    // previous row's readers of the broadcast vectors passed the barriers
    // inside block_sum
    sw[c] = wc;
    sau[c] = ac * uc;
    su[c] = uc;
    sk[c] = kc;
    sr[c] = rc;
    __syncthreads();
    float tc = 0.f;
#pragma unroll
    for (int i = 0; i < DK; ++i) tc += su[i] * S[i];
    float oc = 0.f;
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      S[i] = sw[i] * S[i] - sau[i] * tc + sk[i] * vc;
      oc += S[i] * sr[i];
    }
    if (!active) oc = 0.f;
    const float osq = block_sum<NW>(oc * oc, scratch);
    if (active) {
      const float y = oc * rsqrtf(osq / dim + eps) * nwc * sigmoidf_acc(gc);
      Act<A>::st(out + static_cast<int64_t>(t) * heads * dim + hc, y);
    }
  }
  if (sp != nullptr && active) {
#pragma unroll
    for (int i = 0; i < DK; ++i)
      if (i < dim) sp[static_cast<int64_t>(i) * dim + c] = S[i];
  }
}

template <typename A>
void launch_delta_rule(A* out, const A* r, const A* k, const A* v,
                       const A* wlin, const A* alin, const A* glin,
                       int64_t r_stride, int64_t k_stride, int64_t v_stride,
                       int64_t w_stride, int64_t a_stride, int64_t g_stride,
                       const float* w0, const float* a_bias,
                       const float* norm_w, float* state, const int* seq_cu,
                       const int* seq_slots, const int* positions, int S,
                       int heads, int dim, float eps, float decay_scale,
                       hipStream_t st) {
  if (S == 0) return;
  dim3 grid(heads, S);
#define FI_LAUNCH(DK)                                                          \
  hipLaunchKernelGGL((delta_rule_kernel<A, DK>), grid, dim3(DK), 0, st, out,   \
                     r, k, v, wlin, alin, glin, r_stride, k_stride, v_stride,  \
                     w_stride, a_stride, g_stride, w0, a_bias, norm_w, state,  \
                     seq_cu, seq_slots, positions, heads, dim, eps,            \
                     decay_scale)
  if (dim <= 64) {
    FI_LAUNCH(64);
  } else if (dim <= 128) {
    FI_LAUNCH(128);
  } else {
    FI_LAUNCH(256);
  }
#undef FI_LAUNCH
}

#define FI_INST(A)                                                             \
  template void launch_delta_rule<A>(                                          \
      A*, const A*, const A*, const A*, const A*, const A*, const A*, int64_t, \
      int64_t, int64_t, int64_t, int64_t, int64_t, const float*, const float*, \
      const float*, float*, const int*, const int*, const int*, int, int, int, \
      float, float, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
