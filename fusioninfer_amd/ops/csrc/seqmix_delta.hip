// Generalized delta rule, recurrent form.
//
// Per head the state S [dim x dim] (key rows x value columns, fp32)
// follows, token by token,
//
//   u   = k / sqrt(|k|^2 + 1e-6)
//   w   = exp(-decay_scale * sigmoid(wlin + w0))
//   a   = sigmoid(alin + a_bias)
//   tc  = sum_i u_i S[i][c]                         (old state)
//   S[i][c] <- w_i S[i][c] - a_i u_i tc + k_i v_c
//   o_c = sum_i S[i][c] r_i
//
// Value columns never mix, so the work is cut into (column tile, head,
// sequence) items of 16 columns, one 64-lane wave each: lane = (column,
// row quarter) keeps its quarter of the column in registers (DK = row
// capacity >= dim, compile time). The per-token vectors (w, a*u, u, k, r)
// are computed once by the wave and broadcast through LDS; the next
// token's inputs are fetched while the current one is applied. The state
// is read from the sequence's slot unless the group starts at position 0
// (or has no slot) and written back at the end.
//
// A second kernel turns the raw o into the mixer output: per-head
// unit-RMS, gain, sigmoid gate.

#include "seqmix.h"

namespace fi {

constexpr int kColsPerWave = 16;

template <typename A, int DK>
__global__ __launch_bounds__(64) void delta_rule_wave_kernel(
    float* __restrict__ o_raw,                  // [T, heads*dim] fp32
    const A* __restrict__ r, const A* __restrict__ k, const A* __restrict__ v,
    const A* __restrict__ wlin, const A* __restrict__ alin, int64_t r_stride,
    int64_t k_stride, int64_t v_stride, int64_t w_stride, int64_t a_stride,
    const float* __restrict__ w0, const float* __restrict__ a_bias,
    float* __restrict__ state, const int* __restrict__ seq_cu,
    const int* __restrict__ seq_slots, const int* __restrict__ positions,
    int heads, int dim, float decay_scale) {
  constexpr int RS = DK / 4;       // rows per lane
  constexpr int EPL = DK / 64;     // vector elements per lane
  __shared__ __attribute__((aligned(16))) float sw[DK];
  __shared__ __attribute__((aligned(16))) float sau[DK];
  __shared__ __attribute__((aligned(16))) float su[DK];
  __shared__ __attribute__((aligned(16))) float sk[DK];
  __shared__ __attribute__((aligned(16))) float sr[DK];
  const int lane = threadIdx.x;
  const int col = lane % kColsPerWave;
  const int slice = lane / kColsPerWave;
  const int c = blockIdx.x * kColsPerWave + col;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  const int row0 = seq_cu[s], row1 = seq_cu[s + 1];
  if (row1 <= row0) return;
  const int slot = seq_slots[s];
  const bool col_ok = c < dim;
  const int hbase = head * dim;

  float S[RS];
#pragma unroll
  for (int j = 0; j < RS; ++j) S[j] = 0.f;
  float* sp = nullptr;
  if (slot >= 0)
    sp = state + (static_cast<int64_t>(slot) * heads + head) * dim * dim;
  if (sp != nullptr && positions[row0] > 0 && col_ok) {
#pragma unroll
    for (int j = 0; j < RS; ++j) {
      const int i = slice * RS + j;
      if (i < dim) S[j] = sp[static_cast<int64_t>(i) * dim + c];
    }
  }
  float w0e[EPL], abe[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const int i = lane + 64 * e;
    w0e[e] = i < dim ? w0[hbase + i] : 0.f;
    abe[e] = i < dim ? a_bias[hbase + i] : 0.f;
  }

  // raw inputs of the token about to be applied
  float ke[EPL], re[EPL], we[EPL], ae[EPL], vc;
  auto fetch = [&](int t) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int i = lane + 64 * e;
      const bool ok = i < dim;
      ke[e] = ok ? Act<A>::ld(k + t * k_stride + hbase + i) : 0.f;
      re[e] = ok ? Act<A>::ld(r + t * r_stride + hbase + i) : 0.f;
      we[e] = ok ? Act<A>::ld(wlin + t * w_stride + hbase + i) : 0.f;
      ae[e] = ok ? Act<A>::ld(alin + t * a_stride + hbase + i) : 0.f;
    }
    vc = col_ok ? Act<A>::ld(v + t * v_stride + hbase + c) : 0.f;
  };
  fetch(row0);

  for (int t = row0; t < row1; ++t) {
    float ksq = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) ksq += ke[e] * ke[e];
    ksq = wave_reduce_sum(ksq);
    const float kinv = rsqrtf(ksq + 1e-6f);
    __syncthreads();   // single-wave workgroup: previous readers are done
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      const int i = lane + 64 * e;
      const bool ok = i < dim;
      const float uu = ke[e] * kinv;
      const float ww =
          ok ? expf(-decay_scale * sigmoidf_acc(we[e] + w0e[e])) : 1.f;
      const float aa = ok ? sigmoidf_acc(ae[e] + abe[e]) : 0.f;
      sw[i] = ww;
      sau[i] = aa * uu;
      su[i] = uu;
      sk[i] = ke[e];
      sr[i] = re[e];
    }
    const float vcur = vc;
    if (t + 1 < row1) fetch(t + 1);
    __syncthreads();
    const int i0 = slice * RS;
    float tc = 0.f;
#pragma unroll
    for (int j = 0; j < RS; j += 4) {
      const float4 uu = *reinterpret_cast<const float4*>(su + i0 + j);
      tc += uu.x * S[j] + uu.y * S[j + 1] + uu.z * S[j + 2] + uu.w * S[j + 3];
    }
    tc += __shfl_xor(tc, 16, 64);
    tc += __shfl_xor(tc, 32, 64);
    float oc = 0.f;
#pragma unroll
    for (int j = 0; j < RS; j += 4) {
      const float4 ww = *reinterpret_cast<const float4*>(sw + i0 + j);
      const float4 au = *reinterpret_cast<const float4*>(sau + i0 + j);
      const float4 kk = *reinterpret_cast<const float4*>(sk + i0 + j);
      const float4 rr = *reinterpret_cast<const float4*>(sr + i0 + j);
      S[j] = ww.x * S[j] - au.x * tc + kk.x * vcur;
      S[j + 1] = ww.y * S[j + 1] - au.y * tc + kk.y * vcur;
      S[j + 2] = ww.z * S[j + 2] - au.z * tc + kk.z * vcur;
      S[j + 3] = ww.w * S[j + 3] - au.w * tc + kk.w * vcur;
      oc += S[j] * rr.x + S[j + 1] * rr.y + S[j + 2] * rr.z + S[j + 3] * rr.w;
    }
    oc += __shfl_xor(oc, 16, 64);
    oc += __shfl_xor(oc, 32, 64);
    if (slice == 0 && col_ok)
      o_raw[static_cast<int64_t>(t) * heads * dim + hbase + c] = oc;
  }
  if (sp != nullptr && col_ok) {
#pragma unroll
    for (int j = 0; j < RS; ++j) {
      const int i = slice * RS + j;
      if (i < dim) sp[static_cast<int64_t>(i) * dim + c] = S[j];
    }
  }
}

// out = o * rsqrt(mean_head(o^2) + eps) * norm_w * sigmoid(glin);
// one wave per (row, head)
template <typename A>
__global__ __launch_bounds__(256) void delta_out_gate_kernel(
    A* __restrict__ out, const float* __restrict__ o_raw,
    const A* __restrict__ glin, int64_t g_stride,
    const float* __restrict__ norm_w, int T, int heads, int dim, float eps) {
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / 64;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads);
  const int head = static_cast<int>(item % heads);
  const int64_t base = static_cast<int64_t>(t) * heads * dim + head * dim;
  float ss = 0.f;
  for (int d = lane; d < dim; d += 64) {
    const float o = o_raw[base + d];
    ss += o * o;
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / dim + eps);
  for (int d = lane; d < dim; d += 64) {
    const float g = Act<A>::ld(glin + t * g_stride + head * dim + d);
    Act<A>::st(out + base + d,
               o_raw[base + d] * inv * norm_w[head * dim + d] * sigmoidf_acc(g));
  }
}

template <typename A>
void launch_delta_rule(A* out, float* o_raw, const A* r, const A* k,
                       const A* v, const A* wlin, const A* alin,
                       const A* glin, int64_t r_stride, int64_t k_stride,
                       int64_t v_stride, int64_t w_stride, int64_t a_stride,
                       int64_t g_stride, const float* w0, const float* a_bias,
                       const float* norm_w, float* state, const int* seq_cu,
                       const int* seq_slots, const int* positions, int T,
                       int S, int heads, int dim, float eps, float decay_scale,
                       hipStream_t st) {
  if (S == 0 || T == 0) return;
  dim3 grid(ceil_div(dim, kColsPerWave), heads, S);
#define FI_LAUNCH(DK)                                                          \
  hipLaunchKernelGGL((delta_rule_wave_kernel<A, DK>), grid, dim3(64), 0, st,   \
                     o_raw, r, k, v, wlin, alin, r_stride, k_stride, v_stride, \
                     w_stride, a_stride, w0, a_bias, state, seq_cu, seq_slots, \
                     positions, heads, dim, decay_scale)
  if (dim <= 64) {
    FI_LAUNCH(64);
  } else if (dim <= 128) {
    FI_LAUNCH(128);
  } else {
    FI_LAUNCH(256);
  }
#undef FI_LAUNCH
  const int64_t items = static_cast<int64_t>(T) * heads;
  hipLaunchKernelGGL(delta_out_gate_kernel<A>,
                     dim3(static_cast<int>((items + 3) / 4)), dim3(256), 0, st,
                     out, o_raw, glin, g_stride, norm_w, T, heads, dim, eps);
}

#define FI_INST(A)                                                             \
  template void launch_delta_rule<A>(                                          \
      A*, float*, const A*, const A*, const A*, const A*, const A*, const A*,  \
      int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, const float*,      \
      const float*, const float*, float*, const int*, const int*, const int*,  \
      int, int, int, int, float, float, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
