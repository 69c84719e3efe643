// Linear attention with one scalar decay per head, chunk-parallel form
// for prompt portions.
//
// Per head, S_t = lam S_(t-1) + k_t v_t^T and o_t = S_t^T q_t. For a chunk
// of n <= C consecutive tokens with incoming state S0,
//
//   o_i   = lam^(i+1) S0^T q_i + sum_{j<=i} lam^(i-j) (q_i . k_j) v_j
//   S_out = lam^n S0 + sum_j lam^(n-1-j) k_j v_j^T
//
// so a chunk is four matrix products. Value columns never mix, so the
// work is cut into (64 value columns, head, sequence group) workgroups of
// four waves, 16 columns per wave; chunks of one group run one after the
// other with the state slice [D x 16] of every wave held in MFMA
// accumulators. Everything is true fp32 (v_mfma_f32_16x16x4_f32) whatever
// the activation type: the state, the scores and the decay powers must be,
// and the inputs are staged through LDS as fp32 (silu applied on the way).
//
// The state accumulators double as the B operand of S0^T q: in step (t, r)
// lane (g4, c16) holds S[16t + 4 g4 + r][c16], so the contraction runs over
// d = 16t + 4 g4 + r with the matching q element read from LDS.

#include <math.h>

#include "seqmix.h"

namespace fi {

namespace {

typedef __attribute__((ext_vector_type(4))) float floatx4;

// lam^m for m >= 0, exact for m = 0 and for lam = 0
FI_DEV float decay_pow(float lam, float log2lam, int m) {
  if (m == 0) return 1.f;
  if (lam <= 0.f) return 0.f;
  return exp2f(static_cast<float>(m) * log2lam);
}

// q and k come from the preparation kernel's fp32 vectors
// (vecs [T, heads, 5, DK]: entry 3 = k, entry 4 = q, activation applied),
// v from its fp32 value buffer [T, heads*V].
template <int D, int C>
__global__ __launch_bounds__(256) void decay_linear_chunk_kernel(
    float* __restrict__ o_raw,               // [T, heads*V] fp32
    const float* __restrict__ vecs, int DK, const float* __restrict__ vbuf,
    const float* __restrict__ decay, float* __restrict__ state,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int heads, int V, int min_rows) {
  constexpr int DT = D / 16;                 // state row tiles
  constexpr int CT = C / 16;                 // chunk row tiles
  constexpr int QP = D + 4;                  // pitch of the q / k tiles
  constexpr int VP = 64 + 4;                 // pitch of the v tile
  constexpr int AP = C + 4;                  // pitch of the score tile
  __shared__ __attribute__((aligned(16))) float Qs[C * QP];
  __shared__ __attribute__((aligned(16))) float Ks[C * QP];
  __shared__ __attribute__((aligned(16))) float Vs[C * VP];
  __shared__ __attribute__((aligned(16))) float As[C * AP];
  __shared__ float pw[C + 2];                // lam^m, m = 0..C

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int g4 = lane / 16, c16 = lane % 16;
  const int head = blockIdx.y;
  const int s = blockIdx.z;
  const int row0 = seq_cu[s], row1 = seq_cu[s + 1];
  if (row1 - row0 < min_rows) return;
  const int slot = seq_slots[s];
  const int col0 = blockIdx.x * 64;          // first value column of the WG
  const int col = col0 + wave * 16 + c16;    // this lane's column
  const bool col_ok = col < V;
  const float lam = decay[head];
  const float log2lam = lam > 0.f ? log2f(lam) : 0.f;
  for (int m = tid; m <= C; m += 256) pw[m] = decay_pow(lam, log2lam, m);

  floatx4 S[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) S[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  float* sp = nullptr;
  if (slot >= 0)
    sp = state + (static_cast<int64_t>(slot) * heads + head) * D * V;
  if (sp != nullptr && positions[row0] > 0 && col_ok) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        S[t][r] = sp[static_cast<int64_t>(16 * t + 4 * g4 + r) * V + col];
  }

  // chunk tiles travel global -> registers -> LDS; the next chunk's loads
  // are issued before the current chunk is computed
  constexpr int NQ = C * D / 4 / 256;        // float4 of q (and of k) per thread
  constexpr int NV = C * 64 / 256;           // floats of v per thread
  float4 nq[NQ], nk[NQ];
  float nv[NV];
  auto fetch = [&](int t0) {
    const int n = min(C, row1 - t0);
#pragma unroll
    for (int x = 0; x < NQ; ++x) {
      const int i = tid + 256 * x;           // float4 index in the [C][D] tile
      const int r = i / (D / 4), d = (i % (D / 4)) * 4;
      nq[x] = nk[x] = float4{0.f, 0.f, 0.f, 0.f};
      if (r < n) {
        const float* base =
            vecs + (static_cast<int64_t>(t0 + r) * heads + head) * 5 * DK + d;
        nk[x] = *reinterpret_cast<const float4*>(base + 3 * DK);
        nq[x] = *reinterpret_cast<const float4*>(base + 4 * DK);
      }
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int i = tid + 256 * x;
      const int r = i / 64, c = i % 64;
      nv[x] = 0.f;
      if (r < n && col0 + c < V)
        nv[x] = vbuf[(static_cast<int64_t>(t0 + r) * heads + head) * V + col0 + c];
    }
  };
  fetch(row0);

  for (int t0 = row0; t0 < row1; t0 += C) {
    const int n = min(C, row1 - t0);
    __syncthreads();                         // previous chunk's tiles are done
#pragma unroll
    for (int x = 0; x < NQ; ++x) {
      const int i = tid + 256 * x;
      const int r = i / (D / 4), d = (i % (D / 4)) * 4;
      *reinterpret_cast<float4*>(Qs + r * QP + d) = nq[x];
      *reinterpret_cast<float4*>(Ks + r * QP + d) = nk[x];
    }
#pragma unroll
    for (int x = 0; x < NV; ++x) {
      const int i = tid + 256 * x;
      Vs[(i / 64) * VP + i % 64] = nv[x];
    }
    __syncthreads();
    if (t0 + C < row1) fetch(t0 + C);

    // Operands are read from LDS into registers in batches ahead of the
    // MFMA chains (one wait per batch instead of one per instruction).
    //
    // (1) decayed causal scores A[i][j] = lam^(i-j) (q_i . k_j), j <= i;
    // the (C/16)^2 tiles are spread over the waves. The contraction index
    // is arbitrary as long as both operands agree: lane group g4 takes the
    // contiguous quarter d = g4*D/4 + kk of the rows (vector reads).
#pragma unroll
    for (int x = 0; x < (CT * CT + 3) / 4; ++x) {
      const int tile = wave + 4 * x;
      if (tile >= CT * CT) break;
      const int rt = tile / CT, ct = tile % CT;
      floatx4 acc = {0.f, 0.f, 0.f, 0.f};
      if (ct <= rt) {
        constexpr int Q4 = D / 16;           // float4 per lane and row
        float4 aq[Q4], bk[Q4];
        const float* qrow = Qs + (16 * rt + c16) * QP + g4 * (D / 4);
        const float* krow = Ks + (16 * ct + c16) * QP + g4 * (D / 4);
#pragma unroll
        for (int u = 0; u < Q4; ++u) {
          aq[u] = *reinterpret_cast<const float4*>(qrow + 4 * u);
          bk[u] = *reinterpret_cast<const float4*>(krow + 4 * u);
        }
#pragma unroll
        for (int u = 0; u < Q4; ++u) {
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[u].x, bk[u].x, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[u].y, bk[u].y, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[u].z, bk[u].z, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[u].w, bk[u].w, acc, 0, 0, 0);
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * rt + 4 * g4 + r, j = 16 * ct + c16;
        As[i * AP + j] = j <= i ? acc[r] * pw[i - j] : 0.f;
      }
    }
    // this lane's value column, keys j = 4 kk + g4
    float vreg[C / 4];
#pragma unroll
    for (int kk = 0; kk < C / 4; ++kk)
      vreg[kk] = Vs[(4 * kk + g4) * VP + wave * 16 + c16];
    __syncthreads();

    // (2) o = A v + lam^(i+1) q S0 for this wave's 16 columns
#pragma unroll
    for (int rt = 0; rt < CT; ++rt) {
      float ar[C / 4];
#pragma unroll
      for (int kk = 0; kk < C / 4; ++kk)
        if (kk < 4 * (rt + 1)) ar[kk] = As[(16 * rt + c16) * AP + 4 * kk + g4];
      float4 qr[DT];
#pragma unroll
      for (int t = 0; t < DT; ++t)
        qr[t] = *reinterpret_cast<const float4*>(
            Qs + (16 * rt + c16) * QP + 16 * t + 4 * g4);
      floatx4 acc = {0.f, 0.f, 0.f, 0.f};
      // keys beyond row tile rt have zero scores
#pragma unroll
      for (int kk = 0; kk < C / 4; ++kk)
        if (kk < 4 * (rt + 1))
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[kk], vreg[kk], acc, 0,
                                                     0, 0);
      floatx4 inter = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        inter = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[t].x, S[t][0], inter, 0, 0, 0);
        inter = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[t].y, S[t][1], inter, 0, 0, 0);
        inter = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[t].z, S[t][2], inter, 0, 0, 0);
        inter = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[t].w, S[t][3], inter, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * rt + 4 * g4 + r;
        if (i < n && col_ok)
          o_raw[static_cast<int64_t>(t0 + i) * heads * V + head * V + col] =
              acc[r] + pw[i + 1] * inter[r];
      }
    }

    // (3) S <- lam^n S + sum_j k_j (lam^(n-1-j) v_j)^T
#pragma unroll
    for (int kk = 0; kk < C / 4; ++kk) {
      const int j = 4 * kk + g4;
      vreg[kk] = j < n ? vreg[kk] * pw[n - 1 - j] : 0.f;
    }
    const float ln = pw[n];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      float kr[C / 4];
#pragma unroll
      for (int kk = 0; kk < C / 4; ++kk)
        kr[kk] = Ks[(4 * kk + g4) * QP + 16 * t + c16];
      floatx4 acc = {S[t][0] * ln, S[t][1] * ln, S[t][2] * ln, S[t][3] * ln};
#pragma unroll
      for (int kk = 0; kk < C / 4; ++kk)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kr[kk], vreg[kk], acc, 0, 0,
                                                   0);
      S[t] = acc;
    }
  }
  if (sp != nullptr && col_ok) {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        sp[static_cast<int64_t>(16 * t + 4 * g4 + r) * V + col] = S[t][r];
  }
}

}  // namespace

// Groups of at least min_rows rows through the chunk kernel, on the
// preparation kernel's vectors. Returns false when the key size has no
// variant (the caller keeps the serial kernel).
bool launch_decay_linear_chunks(float* o_raw, const float* vecs, int DK,
                                const float* vbuf, const float* decay,
                                float* state, const int* seq_cu,
                                const int* seq_slots, const int* positions,
                                int S, int heads, int D, int V, int min_rows,
                                hipStream_t st) {
  if (S == 0) return true;
  const dim3 grid(ceil_div(V, 64), heads, S);
#define FI_CHUNK(DD, CC)                                                      \
  case DD:                                                                    \
    hipLaunchKernelGGL((decay_linear_chunk_kernel<DD, CC>), grid, dim3(256),  \
                       0, st, o_raw, vecs, DK, vbuf, decay, state, seq_cu,    \
                       seq_slots, positions, heads, V, min_rows);             \
    return true;
  switch (D) {
    FI_CHUNK(16, 64)
    FI_CHUNK(32, 64)
    FI_CHUNK(64, 32)
    FI_CHUNK(128, 32)
    default:
      return false;
  }
#undef FI_CHUNK
}

}  // namespace fi
