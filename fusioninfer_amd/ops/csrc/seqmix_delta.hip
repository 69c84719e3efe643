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
// Three kernels:
//  1. delta_prep: everything per token that does not depend on the state
//     — the fp32 vectors (w, a*u, u, k, r) of every (token, head), padded
//     to the row capacity DK — fully parallel, one wave per (token, head).
//  2. delta_rule_wave: the recurrence. Value columns never mix, so the
//     work is cut into (column tile, head, sequence) items, one 64-lane
//     wave each, four waves to a workgroup: lane = (column, row slice)
//     keeps its slice of the column in registers (DK = row capacity >=
//     dim, SL = slices per column, compile time; a wave covers 64/SL
//     columns). Slices of one column sit in adjacent lanes, so the two
//     per-token reductions over rows are DPP lane swaps. Tokens are
//     staged in blocks of TB: the block's vectors go global -> registers
//     -> LDS (double-buffered, shared by the four waves, one barrier per
//     block) while the previous block is applied from LDS, so no global
//     round trip sits on the token-to-token chain.
//     The state is read from the sequence's slot unless the group starts
//     at position 0 (or has no slot) and written back at the end.
//  3. delta_out_gate: per-head unit-RMS of o, gain, sigmoid gate.

#include "seqmix.h"

namespace fi {

template <int CTRL>
FI_DEV float dpp_move(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL,
                                         0xF, 0xF, true));
}

// sum over the SL adjacent lanes that hold one column (SL = 4, 8, 16);
// every lane of the group ends with the total
template <int SL>
FI_DEV float slice_sum(float x) {
  x += dpp_move<0xB1>(x);              // quad_perm [1,0,3,2]
  x += dpp_move<0x4E>(x);              // quad_perm [2,3,0,1]
  if (SL >= 8) x += dpp_move<0x141>(x);   // row_half_mirror: other quad
  if (SL == 16) x += dpp_move<0x140>(x);  // row_mirror: other half row
  return x;
}

// vecs[t][head][0..4][DK] = (w, a*u, u, k, r); entries >= dim are the
// identity (w = 1, rest 0) so padded state rows stay zero
template <typename A>
__global__ __launch_bounds__(256) void delta_prep_kernel(
    float* __restrict__ vecs, const A* __restrict__ r, const A* __restrict__ k,
    const A* __restrict__ wlin, const A* __restrict__ alin, int64_t r_stride,
    int64_t k_stride, int64_t w_stride, int64_t a_stride,
    const float* __restrict__ w0, const float* __restrict__ a_bias, int T,
    int heads, int dim, int DK, float decay_scale) {
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / 64;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads);
  const int head = static_cast<int>(item % heads);
  const int hbase = head * dim;
  float* dst = vecs + item * 5 * DK;
  float ksq = 0.f;
  for (int i = lane; i < dim; i += 64) {
    const float kk = Act<A>::ld(k + t * k_stride + hbase + i);
    ksq += kk * kk;
  }
  ksq = wave_reduce_sum(ksq);
  const float kinv = rsqrtf(ksq + 1e-6f);
  for (int i = lane; i < DK; i += 64) {
    float ww = 1.f, au = 0.f, uu = 0.f, kk = 0.f, rr = 0.f;
    if (i < dim) {
      kk = Act<A>::ld(k + t * k_stride + hbase + i);
      rr = Act<A>::ld(r + t * r_stride + hbase + i);
      uu = kk * kinv;
      ww = expf(-decay_scale *
                sigmoidf_acc(Act<A>::ld(wlin + t * w_stride + hbase + i) +
                             w0[hbase + i]));
      au = sigmoidf_acc(Act<A>::ld(alin + t * a_stride + hbase + i) +
                        a_bias[hbase + i]) * uu;
    }
    dst[i] = ww;
    dst[DK + i] = au;
    dst[2 * DK + i] = uu;
    dst[3 * DK + i] = kk;
    dst[4 * DK + i] = rr;
  }
}

constexpr int kDeltaWaves = 4;   // waves (column tiles) per workgroup

template <typename A, int DK, int SL, int TB>
__global__ __launch_bounds__(64 * kDeltaWaves) void delta_rule_wave_kernel(
    float* __restrict__ o_raw,                  // [T, heads*dim] fp32
    const float* __restrict__ vecs,             // [T, heads, 5, DK]
    const A* __restrict__ v, int64_t v_stride, float* __restrict__ state,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int heads, int dim) {
  constexpr int RS = DK / SL;      // rows per lane
  constexpr int R4 = RS / 4;
  constexpr int COLS = 64 / SL;    // columns per wave
  constexpr int NT = 64 * kDeltaWaves;
  constexpr int TOKF4 = 5 * DK / 4;            // float4 per token
  constexpr int BLKF4 = TB * TOKF4;            // float4 per block
  constexpr int LPB = (BLKF4 + NT - 1) / NT;   // float4 per thread per block
  static_assert(RS % 4 == 0, "row slices are float4 multiples");
  __shared__ __attribute__((aligned(16))) float lds[2][TB * 5 * DK];
  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int col = lane / SL;
  const int slice = lane % SL;
  const int c = (blockIdx.x * kDeltaWaves + tid / 64) * COLS + col;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  const int row0 = seq_cu[s], row1 = seq_cu[s + 1];
  if (row1 <= row0) return;
  const int slot = seq_slots[s];
  const bool col_ok = c < dim;
  const int hbase = head * dim;
  const int64_t tok_stride = static_cast<int64_t>(heads) * 5 * DK;
  const float* vhead = vecs + static_cast<int64_t>(head) * 5 * DK;

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

  // the NEXT block's vectors and values, in flight while the current
  // block is applied
  float4 nx[LPB];
  float nv[TB];
  auto fetch_block = [&](int tb0) {
#pragma unroll
    for (int x = 0; x < LPB; ++x) {
      const int f = tid + NT * x;              // float4 index in the block
      if (f < BLKF4) {
        const int tt = f / TOKF4, within = f % TOKF4;
        const int t = tb0 + tt;
        if (t < row1) {
          nx[x] = *reinterpret_cast<const float4*>(vhead + t * tok_stride +
                                                   within * 4);
        } else {
          // past the group's end: the identity token (w = 1, rest 0)
          // leaves the state untouched, so the apply loop needs no branch
          const float one = within < DK / 4 ? 1.f : 0.f;
          nx[x] = float4{one, one, one, one};
        }
      }
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      const int t = min(tb0 + tt, row1 - 1);
      nv[tt] = col_ok ? Act<A>::ld(v + t * v_stride + hbase + c) : 0.f;
    }
  };
  fetch_block(row0);

  const int i0 = slice * RS;
  int buf = 0;
  for (int tb0 = row0; tb0 < row1; tb0 += TB, buf ^= 1) {
    // Buffer `buf` was last read two blocks ago; every wave has passed
    // the barrier of the block in between since, so it is free.
    float vb[TB];
#pragma unroll
    for (int x = 0; x < LPB; ++x) {
      const int f = tid + NT * x;
      if (f < BLKF4) *reinterpret_cast<float4*>(&lds[buf][f * 4]) = nx[x];
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) vb[tt] = nv[tt];
    __syncthreads();
    // issued after the barrier (which drains outstanding loads): these
    // have the whole apply phase to land
    if (tb0 + TB < row1) fetch_block(tb0 + TB);

    const int nt = min(TB, row1 - tb0);
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      {
        const float* base = &lds[buf][tt * 5 * DK + i0];
        float4 ww[R4], au[R4], uu[R4], kk[R4], rr[R4];
#pragma unroll
        for (int x = 0; x < R4; ++x) {
          uu[x] = *reinterpret_cast<const float4*>(base + 2 * DK + 4 * x);
          ww[x] = *reinterpret_cast<const float4*>(base + 4 * x);
          au[x] = *reinterpret_cast<const float4*>(base + DK + 4 * x);
          kk[x] = *reinterpret_cast<const float4*>(base + 3 * DK + 4 * x);
          rr[x] = *reinterpret_cast<const float4*>(base + 4 * DK + 4 * x);
        }
        const float vcur = vb[tt];
        float t0 = 0.f, t1 = 0.f, t2 = 0.f, t3 = 0.f;
#pragma unroll
        for (int x = 0; x < R4; ++x) {
          t0 += uu[x].x * S[4 * x];
          t1 += uu[x].y * S[4 * x + 1];
          t2 += uu[x].z * S[4 * x + 2];
          t3 += uu[x].w * S[4 * x + 3];
        }
        const float tc = slice_sum<SL>((t0 + t1) + (t2 + t3));
        float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
        for (int x = 0; x < R4; ++x) {
          S[4 * x] = ww[x].x * S[4 * x] + (kk[x].x * vcur - au[x].x * tc);
          S[4 * x + 1] =
              ww[x].y * S[4 * x + 1] + (kk[x].y * vcur - au[x].y * tc);
          S[4 * x + 2] =
              ww[x].z * S[4 * x + 2] + (kk[x].z * vcur - au[x].z * tc);
          S[4 * x + 3] =
              ww[x].w * S[4 * x + 3] + (kk[x].w * vcur - au[x].w * tc);
          o0 += S[4 * x] * rr[x].x;
          o1 += S[4 * x + 1] * rr[x].y;
          o2 += S[4 * x + 2] * rr[x].z;
          o3 += S[4 * x + 3] * rr[x].w;
        }
        const float oc = slice_sum<SL>((o0 + o1) + (o2 + o3));
        if (slice == 0 && col_ok && tt < nt)
          o_raw[static_cast<int64_t>(tb0 + tt) * heads * dim + hbase + c] = oc;
      }
    }
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

inline int delta_row_capacity(int dim) {
  return dim <= 64 ? 64 : (dim <= 128 ? 128 : 256);
}

template <typename A>
void launch_delta_rule(A* out, float* o_raw, float* vecs, const A* r,
                       const A* k, const A* v, const A* wlin, const A* alin,
                       const A* glin, int64_t r_stride, int64_t k_stride,
                       int64_t v_stride, int64_t w_stride, int64_t a_stride,
                       int64_t g_stride, const float* w0, const float* a_bias,
                       const float* norm_w, float* state, const int* seq_cu,
                       const int* seq_slots, const int* positions, int T,
                       int S, int heads, int dim, float eps, float decay_scale,
                       hipStream_t st) {
  if (S == 0 || T == 0) return;
  const int64_t items = static_cast<int64_t>(T) * heads;
  const int nblk = static_cast<int>((items + 3) / 4);
  const int DK = delta_row_capacity(dim);
  hipLaunchKernelGGL(delta_prep_kernel<A>, dim3(nblk), dim3(256), 0, st, vecs,
                     r, k, wlin, alin, r_stride, k_stride, w_stride, a_stride,
                     w0, a_bias, T, heads, dim, DK, decay_scale);
#define FI_LAUNCH(DKK, SL, TB)                                                 \
  hipLaunchKernelGGL(                                                          \
      (delta_rule_wave_kernel<A, DKK, SL, TB>),                                \
      dim3(ceil_div(dim, kDeltaWaves * 64 / SL), heads, S),                    \
      dim3(64 * kDeltaWaves), 0, st, o_raw, vecs, v, v_stride, state, seq_cu,  \
      seq_slots, positions, heads, dim)
  if (DK == 64) {
    FI_LAUNCH(64, 8, 8);
  } else if (DK == 128) {
    FI_LAUNCH(128, 16, 8);
  } else {
    FI_LAUNCH(256, 16, 4);
  }
#undef FI_LAUNCH
  hipLaunchKernelGGL(delta_out_gate_kernel<A>, dim3(nblk), dim3(256), 0, st,
                     out, o_raw, glin, g_stride, norm_w, T, heads, dim, eps);
}

#define FI_INST(A)                                                             \
  template void launch_delta_rule<A>(                                          \
      A*, float*, float*, const A*, const A*, const A*, const A*, const A*,    \
      const A*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t,          \
      const float*, const float*, const float*, float*, const int*,            \
      const int*, const int*, int, int, int, int, float, float, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
