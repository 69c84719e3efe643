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

// The state is [dim x vdim] per head (key rows x value columns); v and
// o_raw rows hold heads*vdim values.
template <typename A, int DK, int SL, int TB>
__global__ __launch_bounds__(64 * kDeltaWaves) void delta_rule_wave_kernel(
    float* __restrict__ o_raw,                  // [T, heads*vdim] fp32
    const float* __restrict__ vecs,             // [T, heads, 5, DK]
    const A* __restrict__ v, int64_t v_stride, float* __restrict__ state,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int heads, int dim, int vdim,
    int max_rows) {
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
  // longer groups may belong to another kernel (chunk-parallel forms)
  if (row1 <= row0 || row1 - row0 > max_rows) return;
  const int slot = seq_slots[s];
  const bool col_ok = c < vdim;
  const int hbase = head * vdim;
  const int64_t tok_stride = static_cast<int64_t>(heads) * 5 * DK;
  const float* vhead = vecs + static_cast<int64_t>(head) * 5 * DK;

  float S[RS];
#pragma unroll
  for (int j = 0; j < RS; ++j) S[j] = 0.f;
  float* sp = nullptr;
  if (slot >= 0)
    sp = state + (static_cast<int64_t>(slot) * heads + head) * dim * vdim;
  if (sp != nullptr && positions[row0] > 0 && col_ok) {
#pragma unroll
    for (int j = 0; j < RS; ++j) {
      const int i = slice * RS + j;
      if (i < dim) S[j] = sp[static_cast<int64_t>(i) * vdim + c];
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
          o_raw[static_cast<int64_t>(tb0 + tt) * heads * vdim + hbase + c] = oc;
      }
    }
  }
  if (sp != nullptr && col_ok) {
#pragma unroll
    for (int j = 0; j < RS; ++j) {
      const int i = slice * RS + j;
      if (i < dim) sp[static_cast<int64_t>(i) * vdim + c] = S[j];
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

// The recurrence alone, on prepared vectors: S <- diag(w) S - (a*u)(u^T S)
// + k v^T per token, o = S^T r. v rows are of type VT (activations, or
// fp32 when a preparation kernel has already transformed them).
template <typename VT>
void launch_recurrence(float* o_raw, const float* vecs, const VT* v,
                       int64_t v_stride, float* state, const int* seq_cu,
                       const int* seq_slots, const int* positions, int S,
                       int heads, int dim, int vdim, hipStream_t st,
                       int max_rows = 0x7fffffff) {
  const int DK = delta_row_capacity(dim);
#define FI_LAUNCH(DKK, SL, TB)                                                 \
  hipLaunchKernelGGL(                                                          \
      (delta_rule_wave_kernel<VT, DKK, SL, TB>),                               \
      dim3(ceil_div(vdim, kDeltaWaves * 64 / SL), heads, S),                   \
      dim3(64 * kDeltaWaves), 0, st, o_raw, vecs, v, v_stride, state, seq_cu,  \
      seq_slots, positions, heads, dim, vdim, max_rows)
  if (DK == 64) {
    FI_LAUNCH(64, 8, 8);
  } else if (DK == 128) {
    FI_LAUNCH(128, 16, 8);
  } else {
    FI_LAUNCH(256, 16, 4);
  }
#undef FI_LAUNCH
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
  launch_recurrence<A>(o_raw, vecs, v, v_stride, state, seq_cu, seq_slots,
                       positions, S, heads, dim, dim, st);
  hipLaunchKernelGGL(delta_out_gate_kernel<A>, dim3(nblk), dim3(256), 0, st,
                     out, o_raw, glin, g_stride, norm_w, T, heads, dim, eps);
}

// ---------------------------------------------------------------------
// Linear attention with one scalar decay per head, as a case of the same
// recurrence: w = decay_h on every row, nothing removed (a*u = 0),
// k and r = silu of the key/query projections, v = silu of the value
// projection (fp32 scratch).
template <typename A>
__global__ __launch_bounds__(256) void decay_linear_prep_kernel(
    float* __restrict__ vecs, float* __restrict__ vbuf,
    const A* __restrict__ q, const A* __restrict__ k, const A* __restrict__ v,
    int64_t q_stride, int64_t k_stride, int64_t v_stride,
    const float* __restrict__ decay, int T, int heads, int dim, int vdim,
    int DK, bool silu) {
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / 64;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads);
  const int head = static_cast<int>(item % heads);
  float* dst = vecs + item * 5 * DK;
  const float lam = decay[head];
  for (int i = lane; i < DK; i += 64) {
    float ww = 1.f, kk = 0.f, rr = 0.f;
    if (i < dim) {
      ww = lam;
      kk = Act<A>::ld(k + t * k_stride + head * dim + i);
      rr = Act<A>::ld(q + t * q_stride + head * dim + i);
      if (silu) {
        kk = kk * sigmoidf_acc(kk);
        rr = rr * sigmoidf_acc(rr);
      }
    }
    dst[i] = ww;
    dst[DK + i] = 0.f;
    dst[2 * DK + i] = 0.f;
    dst[3 * DK + i] = kk;
    dst[4 * DK + i] = rr;
  }
  for (int c = lane; c < vdim; c += 64) {
    float vv = Act<A>::ld(v + t * v_stride + head * vdim + c);
    if (silu) vv = vv * sigmoidf_acc(vv);
    vbuf[(static_cast<int64_t>(t) * heads + head) * vdim + c] = vv;
  }
}

bool launch_decay_linear_chunks(float*, const float*, int, const float*,
                                const float*, float*, const int*, const int*,
                                const int*, int, int, int, int, int,
                                hipStream_t);

// The preparation kernel runs for every row; groups of two or more rows
// (prompt portions) then take the chunk-parallel kernel where the key size
// has a variant and the row -> group map is given, one-row groups (decoded
// tokens) and everything else the serial recurrence.
template <typename A>
void launch_decay_linear_attention(float* o_raw, float* vecs, float* vbuf,
                                   const A* q, const A* k, const A* v,
                                   int64_t q_stride, int64_t k_stride,
                                   int64_t v_stride, const float* decay,
                                   float* state, const int* seq_cu,
                                   const int* seq_slots, const int* positions,
                                   const int* row_seq, int T, int S, int heads,
                                   int dim, int vdim, bool silu,
                                   hipStream_t st) {
  if (S == 0 || T == 0) return;
  const int64_t items = static_cast<int64_t>(T) * heads;
  const int nblk = static_cast<int>((items + 3) / 4);
  const int DK = delta_row_capacity(dim);
  hipLaunchKernelGGL(decay_linear_prep_kernel<A>, dim3(nblk), dim3(256), 0, st,
                     vecs, vbuf, q, k, v, q_stride, k_stride, v_stride, decay,
                     T, heads, dim, vdim, DK, silu);
  int max_rows = 0x7fffffff;
  if (row_seq != nullptr && T > S &&
      launch_decay_linear_chunks(o_raw, vecs, DK, vbuf, decay, state, seq_cu,
                                 seq_slots, positions, S, heads, dim, vdim, 2,
                                 st))
    max_rows = 1;
  launch_recurrence<float>(o_raw, vecs, vbuf,
                           static_cast<int64_t>(heads) * vdim, state, seq_cu,
                           seq_slots, positions, S, heads, dim, vdim, st,
                           max_rows);
}

// ---------------------------------------------------------------------
// Gated delta rule behind a short causal convolution, again as a case of
// the recurrence. With g the head's decay and beta its write strength,
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// equals S <- g S - (beta g k)(k^T S_old) + k (beta v)^T, i.e. the
// recurrence with w = g, a*u = beta g k, u = k, v' = beta v, r = q.
//
// x rows hold the projections q | k | v (C = 2*kv_heads*dim + heads*vdim
// channels). y_t[c] = silu(sum_j conv_w[c][j] * x_(t-(taps-1-j))[c]), with
// inputs from before the step's first row taken from the slot's
// conv_state [taps-1, C] (oldest first) and zeros before position 0.
template <typename A>
struct ConvSrc {
  const A* x;
  int64_t x_stride;
  const float* conv_w;
  const float* hist;   // slot's conv state or nullptr
  int taps, C, row0, t, pos;
  // convolved + silu value of channel c at row t
  FI_DEV float at(int c) const {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      if (back > pos) continue;              // before the sequence start
      const int src = t - back;
      float xv;
      if (src >= row0) {
        xv = Act<A>::ld(x + src * x_stride + c);
      } else if (hist != nullptr) {
        // hist[i] is the input at row0 - (taps-1) + i
        xv = hist[static_cast<int64_t>(taps - 1 - (row0 - src)) * C + c];
      } else {
        xv = 0.f;
      }
      acc += conv_w[c * taps + j] * xv;
    }
    return acc * sigmoidf_acc(acc);
  }
};

template <typename A>
__global__ __launch_bounds__(256) void gated_delta_prep_kernel(
    float* __restrict__ vecs, float* __restrict__ vbuf,
    const A* __restrict__ x, int64_t x_stride,
    const float* __restrict__ conv_w, const A* __restrict__ alin,
    int64_t a_stride, const A* __restrict__ blin, int64_t b_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    const float* __restrict__ conv_state, const int* __restrict__ seq_cu,
    const int* __restrict__ seq_slots, const int* __restrict__ positions,
    const int* __restrict__ row_seq, int T, int heads, int kv_heads, int dim,
    int vdim, int taps, int DK) {
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / 64;
  if (item >= static_cast<int64_t>(T) * heads) return;
  const int t = static_cast<int>(item / heads);
  const int head = static_cast<int>(item % heads);
  const int kvh = head / (heads / kv_heads);
  const int s = row_seq[t];
  const int slot = seq_slots[s];
  const int nq = kv_heads * dim;
  ConvSrc<A> cs;
  cs.x = x;
  cs.x_stride = x_stride;
  cs.conv_w = conv_w;
  cs.taps = taps;
  cs.C = 2 * nq + heads * vdim;
  cs.row0 = seq_cu[s];
  cs.t = t;
  cs.pos = positions[t];
  cs.hist = (slot >= 0 && taps > 1)
      ? conv_state + static_cast<int64_t>(slot) * (taps - 1) * cs.C
      : nullptr;

  const float beta = sigmoidf_acc(Act<A>::ld(blin + t * b_stride + head));
  const float z = Act<A>::ld(alin + t * a_stride + head) + dt_bias[head];
  const float sp = z > 20.f ? z : log1pf(expf(z));
  const float g = expf(-expf(a_log[head]) * sp);

  // convolved q/k of this lane's rows (DK <= 256: at most four per lane),
  // evaluated once
  float qc[4], kc[4];
  float qsq = 0.f, ksq = 0.f;
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int i = lane + 64 * x;
    qc[x] = kc[x] = 0.f;
    if (i < dim) {
      qc[x] = cs.at(kvh * dim + i);
      kc[x] = cs.at(nq + kvh * dim + i);
      qsq += qc[x] * qc[x];
      ksq += kc[x] * kc[x];
    }
  }
  qsq = wave_reduce_sum(qsq);
  ksq = wave_reduce_sum(ksq);
  const float qinv = rsqrtf(qsq + 1e-6f) * rsqrtf(static_cast<float>(dim));
  const float kinv = rsqrtf(ksq + 1e-6f);
  float* dst = vecs + item * 5 * DK;
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int i = lane + 64 * x;
    if (i >= DK) break;
    float ww = 1.f, au = 0.f, uu = 0.f, rr = 0.f;
    if (i < dim) {
      uu = kc[x] * kinv;
      rr = qc[x] * qinv;
      ww = g;
      au = beta * g * uu;
    }
    dst[i] = ww;
    dst[DK + i] = au;
    dst[2 * DK + i] = uu;
    dst[3 * DK + i] = uu;
    dst[4 * DK + i] = rr;
  }
  for (int c = lane; c < vdim; c += 64)
    vbuf[(static_cast<int64_t>(t) * heads + head) * vdim + c] =
        beta * cs.at(2 * nq + head * vdim + c);
}

// New conv state of every sequence group: the last taps-1 inputs, taken
// from the step's rows or shifted from the old state when the group is
// shorter; inputs before position 0 are stored as zeros. One thread per
// (group, channel) reads its old entries before it overwrites them
// (ascending order: entry j only needs old entries >= j).
template <typename A>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    float* __restrict__ conv_state, const A* __restrict__ x, int64_t x_stride,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int C, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = seq_slots[s];
  const int row0 = seq_cu[s], row1 = seq_cu[s + 1];
  if (slot < 0 || row1 <= row0) return;
  const int n = row1 - row0;
  const int pos_end = positions[row0] + n;   // position after the last row
  float* st = conv_state + static_cast<int64_t>(slot) * (taps - 1) * C + c;
  for (int j = 0; j < taps - 1; ++j) {
    // entry j <- input at row index row1 - (taps-1) + j
    const int back = taps - 1 - j;           // tokens before the end
    float val;
    if (back > pos_end) {
      val = 0.f;                             // before the sequence start
    } else if (back <= n) {
      val = Act<A>::ld(x + (row1 - back) * x_stride + c);
    } else {
      val = st[static_cast<int64_t>(j + n) * C];   // old entry, j + n > j
    }
    st[static_cast<int64_t>(j) * C] = val;
  }
}

template <typename A>
void launch_gated_delta_rule(float* o_raw, float* vecs, float* vbuf,
                             const A* x, int64_t x_stride, const float* conv_w,
                             const A* alin, int64_t a_stride, const A* blin,
                             int64_t b_stride, const float* a_log,
                             const float* dt_bias, float* conv_state,
                             float* state, const int* seq_cu,
                             const int* seq_slots, const int* positions,
                             const int* row_seq, int T, int S, int heads,
                             int kv_heads, int dim, int vdim, int taps,
                             hipStream_t st) {
  if (S == 0 || T == 0) return;
  const int64_t items = static_cast<int64_t>(T) * heads;
  const int nblk = static_cast<int>((items + 3) / 4);
  const int DK = delta_row_capacity(dim);
  const int C = 2 * kv_heads * dim + heads * vdim;
  hipLaunchKernelGGL(gated_delta_prep_kernel<A>, dim3(nblk), dim3(256), 0, st,
                     vecs, vbuf, x, x_stride, conv_w, alin, a_stride, blin,
                     b_stride, a_log, dt_bias, conv_state, seq_cu, seq_slots,
                     positions, row_seq, T, heads, kv_heads, dim, vdim, taps,
                     DK);
  if (taps > 1)
    hipLaunchKernelGGL(conv_state_update_kernel<A>, dim3(ceil_div(C, 256), S),
                       dim3(256), 0, st, conv_state, x, x_stride, seq_cu,
                       seq_slots, positions, C, taps);
  launch_recurrence<float>(o_raw, vecs, vbuf,
                           static_cast<int64_t>(heads) * vdim, state, seq_cu,
                           seq_slots, positions, S, heads, dim, vdim, st);
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

#define FI_INST(A)                                                             \
  template void launch_decay_linear_attention<A>(                              \
      float*, float*, float*, const A*, const A*, const A*, int64_t, int64_t,  \
      int64_t, const float*, float*, const int*, const int*, const int*,       \
      const int*, int, int, int, int, int, bool, hipStream_t);                 \
  template void launch_gated_delta_rule<A>(                                    \
      float*, float*, float*, const A*, int64_t, const float*, const A*,       \
      int64_t, const A*, int64_t, const float*, const float*, float*, float*,  \
      const int*, const int*, const int*, const int*, int, int, int, int, int, \
      int, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
