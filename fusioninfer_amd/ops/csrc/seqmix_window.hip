// Sliding-window softmax attention over the paged cache with a
// log-distance score penalty and score mixing across heads.
//
// For query row t at position p of its sequence, keys j with
// lo <= j <= p, lo = max(0, p - window + 1) (window <= 0: lo = 0):
//
//   raw_g[j]   = (q_g . k_kv(g)[j]) * scale - r1_g * ln(1 + r2_g (p - j))
//   mixed_h[j] = sum_g talk[h][g] raw_g[j]
//   o_h        = softmax_j(mixed_h) . v_kv(h)[j]
//
// Because every head's softmax needs all heads' raw scores of a key, one
// workgroup owns ALL heads of a query row (row kernel) or of a tile of
// query rows (tile kernel). Scores, the mixing, the softmax and the
// weighted sum are fp32; keys/values are read in the cache's type.
//
// Row kernel (decode rows, and any row when no tile table is given):
// 256 threads per row, key tiles of KT keys, five phases per tile: raw
// scores -> LDS, mixing -> LDS, per-head running maximum, exponentials
// and running sums, weighted value sum with every thread owning
// (head, value column) outputs in registers.

#include <math.h>

#include "seqmix.h"

namespace fi {

namespace {

constexpr int kRowKT = 64;   // keys per tile of the row kernel

template <typename A, int NACC>
__global__ __launch_bounds__(256) void talking_window_row_kernel(
    A* __restrict__ out,                 // [T, H, V]
    const A* __restrict__ q, int64_t q_stride,   // [T, H*D]
    const A* __restrict__ k_cache,       // [B, G, bs, D]
    const A* __restrict__ v_cache,       // [B, G, bs, V]
    const int* __restrict__ seq_bt, int bt_width,
    const int* __restrict__ row_seq, const int* __restrict__ positions,
    const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ talk, int row_begin, int H, int G, int D, int V,
    int bs, float scale, int window) {
  extern __shared__ float smem[];
  float* qs = smem;                      // [H*D]
  float* raw = qs + H * D;               // [H][KT]
  float* mix = raw + H * kRowKT;         // [H][KT]
  float* tk = mix + H * kRowKT;          // [H][H]
  float* mrun = tk + H * H;              // [H] running max
  float* lrun = mrun + H;                // [H] running sum
  float* alpha = lrun + H;               // [H] rescale of this tile
  float* pen1 = alpha + H;               // [H]
  float* pen2 = pen1 + H;                // [H]

  const int t = row_begin + blockIdx.x;
  const int tid = threadIdx.x;
  const int s = row_seq[t];
  const int p = positions[t];
  const int lo = window > 0 ? max(p - window + 1, 0) : 0;
  const int* bt = seq_bt + static_cast<int64_t>(s) * bt_width;
  const int rep = H / G;

  for (int i = tid; i < H * D; i += 256)
    qs[i] = Act<A>::ld(q + t * q_stride + i);
  for (int i = tid; i < H * H; i += 256) tk[i] = talk[i];
  for (int i = tid; i < H; i += 256) {
    mrun[i] = -INFINITY;
    lrun[i] = 0.f;
    pen1[i] = r1[i];
    pen2[i] = r2[i];
  }
  float acc[NACC];
#pragma unroll
  for (int x = 0; x < NACC; ++x) acc[x] = 0.f;
  __syncthreads();

  for (int j0 = lo; j0 <= p; j0 += kRowKT) {
    // raw scores of (head g, key jj)
    for (int it = tid; it < H * kRowKT; it += 256) {
      const int g = it / kRowKT, jj = it % kRowKT;
      const int j = j0 + jj;
      float sc = 0.f;
      if (j <= p) {
        const int64_t blk = bt[j / bs];
        const A* kr = k_cache + ((blk * G + g / rep) * bs + j % bs) * D;
        const float* qr = qs + g * D;
        float d0 = 0.f, d1 = 0.f;
        int d = 0;
        for (; d + 1 < D; d += 2) {
          d0 += qr[d] * Act<A>::ld(kr + d);
          d1 += qr[d + 1] * Act<A>::ld(kr + d + 1);
        }
        if (d < D) d0 += qr[d] * Act<A>::ld(kr + d);
        sc = (d0 + d1) * scale -
             pen1[g] * log1pf(pen2[g] * static_cast<float>(p - j));
      }
      raw[it] = sc;
    }
    __syncthreads();
    // mixing across heads; keys past p are masked out
    for (int it = tid; it < H * kRowKT; it += 256) {
      const int h = it / kRowKT, jj = it % kRowKT;
      float m = -INFINITY;
      if (j0 + jj <= p) {
        m = 0.f;
        for (int g = 0; g < H; ++g) m += tk[h * H + g] * raw[g * kRowKT + jj];
      }
      mix[it] = m;
    }
    __syncthreads();
    if (tid < H) {
      float m = mrun[tid];
      for (int jj = 0; jj < kRowKT; ++jj) m = fmaxf(m, mix[tid * kRowKT + jj]);
      alpha[tid] = expf(mrun[tid] - m);    // 0 on the first tile
      mrun[tid] = m;
    }
    __syncthreads();
    for (int it = tid; it < H * kRowKT; it += 256)
      mix[it] = expf(mix[it] - mrun[it / kRowKT]);
    __syncthreads();
    if (tid < H) {
      float l = 0.f;
      for (int jj = 0; jj < kRowKT; ++jj) l += mix[tid * kRowKT + jj];
      lrun[tid] = lrun[tid] * alpha[tid] + l;
    }
    const int nk = min(kRowKT, p - j0 + 1);
#pragma unroll
    for (int x = 0; x < NACC; ++x) {
      const int o = tid + 256 * x;
      if (o < H * V) {
        const int h = o / V, c = o % V;
        float a = acc[x] * alpha[h];
        const float* pw = mix + h * kRowKT;
        for (int jj = 0; jj < nk; ++jj) {
          const int j = j0 + jj;
          const int64_t blk = bt[j / bs];
          a += pw[jj] *
               Act<A>::ld(v_cache + ((blk * G + h / rep) * bs + j % bs) * V + c);
        }
        acc[x] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int x = 0; x < NACC; ++x) {
    const int o = tid + 256 * x;
    if (o < H * V)
      Act<A>::st(out + static_cast<int64_t>(t) * H * V + o,
                 acc[x] / lrun[o / V]);
  }
}

}  // namespace

size_t talking_window_row_smem(int H, int D) {
  return sizeof(float) *
         (static_cast<size_t>(H) * D + 2 * H * kRowKT + H * H + 5 * H);
}

template <typename A>
void launch_talking_window_rows(A* out, const A* q, int64_t q_stride,
                                const A* k_cache, const A* v_cache,
                                const int* seq_bt, int bt_width,
                                const int* row_seq, const int* positions,
                                const float* r1, const float* r2,
                                const float* talk, int row_begin, int rows,
                                int H, int G, int D, int V, int bs,
                                float scale, int window, hipStream_t st) {
  if (rows <= 0) return;
  const size_t smem = talking_window_row_smem(H, D);
  const int per = ceil_div(H * V, 256);
#define FI_LAUNCH(N)                                                          \
  hipLaunchKernelGGL((talking_window_row_kernel<A, N>), dim3(rows),           \
                     dim3(256), smem, st, out, q, q_stride, k_cache, v_cache, \
                     seq_bt, bt_width, row_seq, positions, r1, r2, talk,      \
                     row_begin, H, G, D, V, bs, scale, window)
  if (per <= 2) {
    FI_LAUNCH(2);
  } else if (per <= 4) {
    FI_LAUNCH(4);
  } else if (per <= 8) {
    FI_LAUNCH(8);
  } else if (per <= 16) {
    FI_LAUNCH(16);
  } else {
    FI_LAUNCH(32);
  }
#undef FI_LAUNCH
}

#define FI_INST(A)                                                            \
  template void launch_talking_window_rows<A>(                                \
      A*, const A*, int64_t, const A*, const A*, const int*, int, const int*, \
      const int*, const float*, const float*, const float*, int, int, int,    \
      int, int, int, int, float, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
