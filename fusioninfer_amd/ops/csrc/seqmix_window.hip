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
// Tile kernel (prompt portions): the mixing is linear in the queries, so
// it is folded into them first,
//
//   mixed_h[j] = scale * sum_kv (q'_(h,kv) . k_kv[j]) - pen'_h(p - j),
//   q'_(h,kv)  = sum_{g in kv} talk[h][g] q_g          (fp32 sum)
//   pen'_h(d)  = sum_g talk[h][g] r1_g ln(1 + r2_g d)   (fp32 table)
//
// which is ordinary attention of head h with one query segment per kv
// head. A 4-wave workgroup takes 128 consecutive rows of one (sequence,
// head), 32 per wave, walks the key range in LDS-staged tiles, and for
// every tile accumulates S^T = sum_kv K_kv Q'_kv^T on the matrix cores
// (bf16 16x16x16, or true-fp32 16x16x4), one kv head's key tile in LDS at
// a time; the value tile of the head's own kv head is staged with the
// first segment. Softmax statistics stay fp32 per lane (one query per
// lane column). O^T += V^T P^T as in the shared-key/value tile kernel.
//
// Row kernel (decode rows, and any row when no tile table is given):
// 256 threads per row, key tiles of KT keys, five phases per tile: raw
// scores -> LDS, mixing -> LDS, per-head running maximum, exponentials
// and running sums, weighted value sum with every thread owning
// (head, value column) outputs in registers.

#include <math.h>

#include <type_traits>

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



// Row kernel, thread-per-key form (decode rows when the sizes allow 4-wide
// accesses): 64 keys per wave and pass, one per thread. A thread reads its key's
// rows of all kv heads once (vector loads), forms the raw scores of all
// heads against the query held in LDS (broadcast reads), mixes them in
// registers, and the block then takes per-head maxima and sums across
// threads (wave shuffles + one LDS hop). For the weighted value sum the
// threads switch to owning (head, 4 value columns) outputs and walk the
// pass's weights in LDS.
constexpr int kFastWaves = 4;       // waves per workgroup of the fast row kernel
constexpr int kFastKT = 64 * kFastWaves;
constexpr int kFastMaxRep = 8;
constexpr int kFastItems = 4;      // (head, 4 columns) outputs per thread

template <typename A, int MAXH>
__global__ __launch_bounds__(kFastKT) void talking_window_row_fast_kernel(
    float* __restrict__ part_ml,         // [rows, nsplit, 2, H] max, sum
    float* __restrict__ part_o,          // [rows, nsplit, H*V]
    const A* __restrict__ q, int64_t q_stride,
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ seq_bt, int bt_width,
    const int* __restrict__ row_seq, const int* __restrict__ positions,
    const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ talk, int row_begin, int H, int G, int D, int V,
    int bs, float scale, int window) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* qs = smem;                      // [H*D]
  float* pbuf = qs + H * D;              // [H][KT] weights of this pass
  float* tk = pbuf + H * kFastKT;        // [H][H]
  float* wred = tk + H * H;              // [waves][H] per-wave partials
  int* kblk = reinterpret_cast<int*>(wred + kFastWaves * H);   // [KT] key's row base

  const int t = row_begin + blockIdx.x;
  const int split = blockIdx.y, nsplit = gridDim.y;
  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int s = row_seq[t];
  const int p = positions[t];
  const int lo = window > 0 ? max(p - window + 1, 0) : 0;
  const int* bt = seq_bt + static_cast<int64_t>(s) * bt_width;
  const int rep = H / G;
  const int nitems = H * V / 4;
  const int64_t pslot = static_cast<int64_t>(blockIdx.x) * nsplit + split;
  float* pml = part_ml + pslot * 2 * H;
  float* po = part_o + pslot * H * V;

  // the keys of this pass, one per thread
  const int j0 = lo + split * kFastKT;
  if (j0 > p) {                          // nothing to see: an empty partial
    if (tid < H) {
      pml[tid] = -INFINITY;
      pml[H + tid] = 0.f;
    }
    return;
  }
  for (int i = tid; i < H * D; i += kFastKT)
    qs[i] = Act<A>::ld(q + t * q_stride + i);
  for (int i = tid; i < H * H; i += kFastKT) tk[i] = talk[i];
  __syncthreads();

  const int j = j0 + tid;
  const bool live = j <= p;
  float raw[MAXH];
#pragma unroll
  for (int g = 0; g < MAXH; ++g) raw[g] = 0.f;
  if (live) {
    const int64_t blk = bt[j / bs];
    // row index of kv head 0 of this key; head kv adds kv * bs rows
    kblk[tid] = static_cast<int>(blk * G * bs + j % bs);
    const float dist = static_cast<float>(p - j);
    for (int kv = 0; kv < G; ++kv) {
      const A* kr = k_cache + ((blk * G + kv) * bs + j % bs) * D;
      float part[kFastMaxRep];
#pragma unroll
      for (int r = 0; r < kFastMaxRep; ++r) part[r] = 0.f;
#pragma unroll 4
      for (int d = 0; d < D; d += 4) {
        float k4[4];
        ldv<A, 4>(kr + d, k4);
#pragma unroll
        for (int r = 0; r < kFastMaxRep; ++r) {
          if (r < rep) {
            const float4 q4 = *reinterpret_cast<const float4*>(
                qs + (kv * rep + r) * D + d);
            part[r] += q4.x * k4[0] + q4.y * k4[1] + q4.z * k4[2] +
                       q4.w * k4[3];
          }
        }
      }
      // hand the group's scores to their (statically indexed) slots
#pragma unroll
      for (int g = 0; g < MAXH; ++g) {
        const int r = g - kv * rep;
        if (g < H && r >= 0 && r < rep) {
          float pv = part[0];
#pragma unroll
          for (int rr = 1; rr < kFastMaxRep; ++rr)
            if (rr == r) pv = part[rr];
          raw[g] = pv * scale - r1[g] * log1pf(r2[g] * dist);
        }
      }
    }
  }
  // mixing, per-head maxima over the pass
  float mh[MAXH];
#pragma unroll
  for (int h = 0; h < MAXH; ++h) {
    mh[h] = -INFINITY;
    if (h < H) {
      if (live) {
        float m = 0.f;
#pragma unroll
        for (int g = 0; g < MAXH; ++g)
          if (g < H) m += tk[h * H + g] * raw[g];
        mh[h] = m;
      }
      const float wm = wave_reduce_max(mh[h]);
      if (lane == 0) wred[wave * H + h] = wm;
    }
  }
  __syncthreads();
  float wsum[MAXH];
#pragma unroll
  for (int h = 0; h < MAXH; ++h) {
    if (h < H) {
      // finite: key j0 is live
      float mt = wred[h];
#pragma unroll
      for (int w = 1; w < kFastWaves; ++w) mt = fmaxf(mt, wred[w * H + h]);
      const float pw = live ? expf(mh[h] - mt) : 0.f;
      pbuf[h * kFastKT + tid] = pw;
      wsum[h] = wave_reduce_sum(pw);
      if (tid == 0) pml[h] = mt;
    }
  }
  __syncthreads();       // everyone has read the maxima; weights are in LDS
#pragma unroll
  for (int h = 0; h < MAXH; ++h)
    if (h < H && lane == 0) wred[wave * H + h] = wsum[h];
  const int nk = min(kFastKT, p - j0 + 1);
#pragma unroll
  for (int x = 0; x < kFastItems; ++x) {
    const int it = tid + kFastKT * x;
    if (it < nitems) {
      const int h = it / (V / 4), c = (it % (V / 4)) * 4;
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      const float* pw = pbuf + h * kFastKT;
      const A* vbase = v_cache + static_cast<int64_t>(h / rep) * bs * V + c;
#pragma unroll 4
      for (int jj = 0; jj < nk; ++jj) {
        float v4[4];
        ldv<A, 4>(vbase + static_cast<int64_t>(kblk[jj]) * V, v4);
        const float w = pw[jj];
        a0 += w * v4[0];
        a1 += w * v4[1];
        a2 += w * v4[2];
        a3 += w * v4[3];
      }
      *reinterpret_cast<float4*>(po + h * V + c) = float4{a0, a1, a2, a3};
    }
  }
  __syncthreads();
  if (tid < H) {
    float l = wred[tid];
#pragma unroll
    for (int w = 1; w < kFastWaves; ++w) l += wred[w * H + tid];
    pml[H + tid] = l;
  }
}

// out[h][c] = sum_s e^(m_s - M) o_s[h][c] / sum_s e^(m_s - M) l_s
template <typename A>
__global__ __launch_bounds__(256) void talking_window_combine_kernel(
    A* __restrict__ out, const float* __restrict__ part_ml,
    const float* __restrict__ part_o, int row_begin, int nsplit, int H,
    int V) {
  const int64_t r = blockIdx.x;
  const float* ml = part_ml + r * nsplit * 2 * H;
  const float* po = part_o + r * nsplit * H * V;
  for (int o = threadIdx.x; o < H * V; o += 256) {
    const int h = o / V;
    float M = -INFINITY;
    for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, ml[sp * 2 * H + h]);
    float num = 0.f, den = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) {
      const float m = ml[sp * 2 * H + h];
      if (m == -INFINITY) continue;
      const float f = expf(m - M);
      num += f * po[static_cast<int64_t>(sp) * H * V + o];
      den += f * ml[sp * 2 * H + H + h];
    }
    Act<A>::st(out + (row_begin + r) * H * V + o, num / den);
  }
}

typedef __attribute__((ext_vector_type(4))) short short4v;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int kQSets = 2;               // 16-row query sets per wave
constexpr int kTileRows = 64 * kQSets;  // q rows per workgroup (4 waves)

// q' [T, H, G, D] = sum over the q heads g of kv head kv of talk[h][g] q_g
template <typename A>
__global__ __launch_bounds__(256) void talking_fold_queries_kernel(
    A* __restrict__ qf, const A* __restrict__ q, int64_t q_stride,
    const float* __restrict__ talk, int H, int G, int D) {
  const int64_t t = blockIdx.x;
  const int rep = H / G;
  const int n = H * G * D;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int d = i % D;
    const int kv = (i / D) % G;
    const int h = i / (D * G);
    float acc = 0.f;
    for (int r = 0; r < rep; ++r) {
      const int g = kv * rep + r;
      acc += talk[h * H + g] * Act<A>::ld(q + t * q_stride + g * D + d);
    }
    Act<A>::st(qf + t * n + i, acc);
  }
}

// pen' [H, maxd]
__global__ __launch_bounds__(256) void talking_penalty_table_kernel(
    float* __restrict__ pen, const float* __restrict__ r1,
    const float* __restrict__ r2, const float* __restrict__ talk, int H,
    int maxd) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= H * maxd) return;
  const int h = i / maxd;
  const float d = static_cast<float>(i % maxd);
  float acc = 0.f;
  for (int g = 0; g < H; ++g)
    acc += talk[h * H + g] * r1[g] * log1pf(r2[g] * d);
  pen[i] = acc;
}

template <typename A, int D, int DV, int BN>
__global__ __launch_bounds__(256) void talking_window_tile_kernel(
    A* __restrict__ out,                 // [T, H, DV]
    const A* __restrict__ qf,            // [T, H, G, D] folded queries
    const A* __restrict__ k_cache,       // [B, G, bs, D]
    const A* __restrict__ v_cache,       // [B, G, bs, DV]
    const float* __restrict__ pen, int maxd,   // [H, maxd]
    const int* __restrict__ seq_bt, int bt_stride,
    const int* __restrict__ seq_cu, const int* __restrict__ positions,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_row0, int H,
    int G, int block_size, float scale, int window) {
  constexpr bool BF = std::is_same<A, u16>::value;
  constexpr int QS = kQSets;
  constexpr int VEC = BF ? 8 : 4;               // elements per 16-byte load
  constexpr int KP = D + (BF ? 8 : 4);          // K tile [BN][KP]
  constexpr int VP = BF ? BN + 8 : DV + 4;      // bf16: V^T [DV][VP]; fp32: V [BN][VP]
  constexpr int NB = BN / 16;
  constexpr int DB = D / 16;
  constexpr int VB = DV / 16;
  __shared__ __attribute__((aligned(16))) A k_lds[BN * KP];
  __shared__ __attribute__((aligned(16))) A v_lds[BF ? DV * VP : BN * VP];

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int g4 = lane / 16, c16 = lane % 16;
  const int h = blockIdx.y;
  const int gv = h / (H / G);                   // the head's value kv head
  const int s = tile_seq[blockIdx.x];
  const int row_first = seq_cu[s] + tile_row0[blockIdx.x];
  const int nrows = min(kTileRows, seq_cu[s + 1] - row_first);
  const int* bt = seq_bt + static_cast<int64_t>(s) * bt_stride;
  const float* pen_h = pen + static_cast<int64_t>(h) * maxd;

  auto range_lo = [&](int p) { return window > 0 ? max(p - window + 1, 0) : 0; };
  const int p_first = positions[row_first];
  const int kv_lo = range_lo(p_first);
  const int kv_hi = p_first + nrows - 1;   // positions in a group ascend by 1

  // this lane's queries: column c16 of each of the wave's 16-row sets
  int my_row[QS], my_pos[QS], my_lo[QS];
  bool row_ok[QS];
  const A* my_q[QS];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    my_row[qs] = (wave * QS + qs) * 16 + c16;
    row_ok[qs] = my_row[qs] < nrows;
    my_pos[qs] = row_ok[qs] ? p_first + my_row[qs] : -1;
    my_lo[qs] = row_ok[qs] ? range_lo(my_pos[qs]) : 0;
    my_q[qs] = qf + (static_cast<int64_t>(row_first +
                                          (row_ok[qs] ? my_row[qs] : 0)) * H +
                     h) * G * D;
  }

  floatx4 o[QS][VB];
  float m[QS], l[QS];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    m[qs] = -INFINITY;
    l[qs] = 0.f;
#pragma unroll
    for (int vb = 0; vb < VB; ++vb) o[qs][vb] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // short groups (a decoded row is a group of one): waves and query sets
  // without rows only help staging (wave-uniform flags)
  bool set_on[QS];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs) set_on[qs] = (wave * QS + qs) * 16 < nrows;
  const bool wave_on = set_on[0];

  for (int j0 = kv_lo; j0 <= kv_hi; j0 += BN) {
    floatx4 sacc[QS][NB];
#pragma unroll
    for (int qs = 0; qs < QS; ++qs)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) sacc[qs][nb] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int kv = 0; kv < G; ++kv) {
      // ---- stage this kv head's K tile (and, once, the V tile) ----
      constexpr int KPR = D / VEC;               // vectors per key row
      constexpr int VPR = DV / VEC;
      for (int vid = tid; vid < BN * KPR; vid += 256) {
        const int key_l = vid / KPR, dv = vid % KPR;
        const int key = j0 + key_l;
        u32x4 k4 = {0u, 0u, 0u, 0u};
        if (key <= kv_hi) {
          const int64_t off =
              ((static_cast<int64_t>(bt[key / block_size]) * G + kv) *
                   block_size + key % block_size) * D + dv * VEC;
          k4 = *reinterpret_cast<const u32x4*>(k_cache + off);
        }
        *reinterpret_cast<u32x4*>(k_lds + key_l * KP + dv * VEC) = k4;
      }
      if (kv == 0) {
        if constexpr (BF) {
          // two adjacent keys per thread: the transposed V tile is written
          // with 4-byte stores (one (key, key+1) pair per value column)
          for (int pid = tid; pid < (BN / 2) * VPR; pid += 256) {
            const int kp = pid / VPR, dv = pid % VPR;
            u32x4 v4[2];
#pragma unroll
            for (int e2 = 0; e2 < 2; ++e2) {
              const int key = j0 + 2 * kp + e2;
              v4[e2] = u32x4{0u, 0u, 0u, 0u};
              if (key <= kv_hi) {
                const int64_t off =
                    ((static_cast<int64_t>(bt[key / block_size]) * G + gv) *
                         block_size + key % block_size) * DV + dv * VEC;
                v4[e2] = *reinterpret_cast<const u32x4*>(v_cache + off);
              }
            }
            const u16* va = reinterpret_cast<const u16*>(&v4[0]);
            const u16* vb = reinterpret_cast<const u16*>(&v4[1]);
#pragma unroll
            for (int e = 0; e < 8; ++e)
              *reinterpret_cast<u32*>(v_lds + (dv * 8 + e) * VP + 2 * kp) =
                  static_cast<u32>(va[e]) | (static_cast<u32>(vb[e]) << 16);
          }
        } else {
          for (int vid = tid; vid < BN * VPR; vid += 256) {
            const int key_l = vid / VPR, dv = vid % VPR;
            const int key = j0 + key_l;
            u32x4 vv4 = {0u, 0u, 0u, 0u};
            if (key <= kv_hi) {
              const int64_t off =
                  ((static_cast<int64_t>(bt[key / block_size]) * G + gv) *
                       block_size + key % block_size) * DV + dv * VEC;
              vv4 = *reinterpret_cast<const u32x4*>(v_cache + off);
            }
            *reinterpret_cast<u32x4*>(v_lds + key_l * VP + dv * VEC) = vv4;
          }
        }
      }
      __syncthreads();

      // ---- S^T += K_kv Q'_kv^T ----
      if (!wave_on) {
        // nothing to compute for this wave
      } else if constexpr (BF) {
        short4v qfr[QS][DB];
#pragma unroll
        for (int qs = 0; qs < QS; ++qs)
#pragma unroll
          for (int kk = 0; kk < DB; ++kk)
            qfr[qs][kk] = row_ok[qs]
                ? *reinterpret_cast<const short4v*>(my_q[qs] + kv * D +
                                                    16 * kk + 4 * g4)
                : short4v{0, 0, 0, 0};
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const A* kr = k_lds + (nb * 16 + c16) * KP;
#pragma unroll
          for (int kk = 0; kk < DB; ++kk) {
            const short4v a =
                *reinterpret_cast<const short4v*>(kr + 16 * kk + 4 * g4);
#pragma unroll
            for (int qs = 0; qs < QS; ++qs)
              if (set_on[qs])
                sacc[qs][nb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                    a, qfr[qs][kk], sacc[qs][nb], 0, 0, 0);
          }
        }
      } else {
#pragma unroll 4
        for (int kk = 0; kk < D / 4; ++kk) {
          float qv[QS];
#pragma unroll
          for (int qs = 0; qs < QS; ++qs)
            qv[qs] = row_ok[qs] ? my_q[qs][kv * D + 4 * kk + g4] : 0.f;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const float a = k_lds[(nb * 16 + c16) * KP + 4 * kk + g4];
#pragma unroll
            for (int qs = 0; qs < QS; ++qs)
              if (set_on[qs])
                sacc[qs][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                    a, qv[qs], sacc[qs][nb], 0, 0, 0);
          }
        }
      }
      // the next segment overwrites the K tile
      if (kv + 1 < G) __syncthreads();
    }

    // ---- scale, distance penalty, mask, online softmax ----
    if (!wave_on) {
      __syncthreads();
      continue;
    }
    float sv[QS][NB][4];
#pragma unroll
    for (int qs = 0; qs < QS; ++qs) {
      float tmax = -INFINITY;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = j0 + nb * 16 + 4 * g4 + i;
          const bool vis = key <= my_pos[qs] && key >= my_lo[qs];
          float x = -INFINITY;
          if (vis) x = sacc[qs][nb][i] * scale - pen_h[my_pos[qs] - key];
          sv[qs][nb][i] = x;
          tmax = fmaxf(tmax, x);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m[qs], tmax);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float corr = expf(m[qs] - m_safe);     // m = -inf -> 0
      float psum = 0.f;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sv[qs][nb][i] = expf(sv[qs][nb][i] - m_safe);  // masked -> 0
          psum += sv[qs][nb][i];
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l[qs] = l[qs] * corr + psum;
      m[qs] = m_new;
#pragma unroll
      for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[qs][vb][i] *= corr;
    }

    // ---- O^T += V^T P^T: every V fragment feeds QS MFMAs ----
    if constexpr (BF) {
      short4v pf[QS][NB];
#pragma unroll
      for (int qs = 0; qs < QS; ++qs)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            pf[qs][nb][i] = static_cast<short>(f32_to_bf16(sv[qs][nb][i]));
#pragma unroll
      for (int vb = 0; vb < VB; ++vb) {
        const A* vr = v_lds + (vb * 16 + c16) * VP;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const short4v a =
              *reinterpret_cast<const short4v*>(vr + nb * 16 + 4 * g4);
#pragma unroll
          for (int qs = 0; qs < QS; ++qs)
            if (set_on[qs])
              o[qs][vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                  a, pf[qs][nb], o[qs][vb], 0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float a = v_lds[(nb * 16 + 4 * g4 + i) * VP + vb * 16 + c16];
#pragma unroll
            for (int qs = 0; qs < QS; ++qs)
              if (set_on[qs])
                o[qs][vb] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                    a, sv[qs][nb][i], o[qs][vb], 0, 0, 0);
          }
    }
    __syncthreads();
  }

#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    if (!row_ok[qs]) continue;
    const float inv_l = 1.0f / l[qs];
    A* op = out + (static_cast<int64_t>(row_first + my_row[qs]) * H + h) * DV;
#pragma unroll
    for (int vb = 0; vb < VB; ++vb)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        Act<A>::st(op + vb * 16 + 4 * g4 + i, o[qs][vb][i] * inv_l);
  }
}

}  // namespace

size_t talking_window_fast_smem(int H, int D) {
  return sizeof(float) * (static_cast<size_t>(H) * D + H * kFastKT + H * H +
                          kFastWaves * H + kFastKT);
}

// sizes the thread-per-key row kernel handles
bool talking_window_fast_fits(int H, int G, int D, int V) {
  return D % 4 == 0 && V % 4 == 0 && H <= 32 && H / G <= kFastMaxRep &&
         H * V / 4 <= kFastKT * kFastItems &&
         talking_window_fast_smem(H, D) <= 64 * 1024;
}

// key passes (workgroups per row) for a visible range of at most max_keys
int talking_window_fast_splits(int max_keys) {
  return max(ceil_div(max_keys, kFastKT), 1);
}

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
                                float scale, int window, float* part_ml,
                                float* part_o, int nsplit, hipStream_t st) {
  if (rows <= 0) return;
  // thread-per-key form where 4-wide accesses and the register budget fit
  if (talking_window_fast_fits(H, G, D, V) && part_ml != nullptr) {
    const size_t fast_smem = talking_window_fast_smem(H, D);
    const dim3 grid(rows, nsplit);
    if (H <= 16)
      hipLaunchKernelGGL((talking_window_row_fast_kernel<A, 16>), grid,
                         dim3(kFastKT), fast_smem, st, part_ml, part_o, q,
                         q_stride, k_cache, v_cache, seq_bt, bt_width, row_seq,
                         positions, r1, r2, talk, row_begin, H, G, D, V, bs,
                         scale, window);
    else
      hipLaunchKernelGGL((talking_window_row_fast_kernel<A, 32>), grid,
                         dim3(kFastKT), fast_smem, st, part_ml, part_o, q,
                         q_stride, k_cache, v_cache, seq_bt, bt_width, row_seq,
                         positions, r1, r2, talk, row_begin, H, G, D, V, bs,
                         scale, window);
    hipLaunchKernelGGL(talking_window_combine_kernel<A>, dim3(rows), dim3(256),
                       0, st, out, part_ml, part_o, row_begin, nsplit, H, V);
    return;
  }
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


// Prompt-portion rows [0, tile_rows) through the folded tile kernel.
// Returns false when the head sizes have no tiled variant (the caller
// then runs those rows through the row kernel).
template <typename A>
bool launch_talking_window_tiles(A* out, A* qf, float* pen, int maxd,
                                 const A* q, int64_t q_stride,
                                 const A* k_cache, const A* v_cache,
                                 const int* seq_bt, int bt_width,
                                 const int* seq_cu, const int* positions,
                                 const float* r1, const float* r2,
                                 const float* talk, const int* tile_seq,
                                 const int* tile_row0, int num_tiles,
                                 int tile_rows, int H, int G, int D, int V,
                                 int bs, float scale, int window,
                                 hipStream_t st) {
  constexpr bool BF = std::is_same<A, u16>::value;
  if (num_tiles == 0 || tile_rows == 0) return true;
  const bool fits = (D == 32 || D == 64 || D == 128) &&
                    (V == 32 || V == 64 || V == 128);
  if (!fits) return false;
  hipLaunchKernelGGL(talking_fold_queries_kernel<A>, dim3(tile_rows),
                     dim3(256), 0, st, qf, q, q_stride, talk, H, G, D);
  hipLaunchKernelGGL(talking_penalty_table_kernel,
                     dim3(ceil_div(H * maxd, 256)), dim3(256), 0, st, pen, r1,
                     r2, talk, H, maxd);
  dim3 grid(num_tiles, H);
#define FI_TILE(DD, VV, BNB, BNF)                                             \
  if (D == DD && V == VV) {                                                   \
    hipLaunchKernelGGL(                                                       \
        (talking_window_tile_kernel<A, DD, VV, (BF ? BNB : BNF)>), grid,      \
        dim3(256), 0, st, out, qf, k_cache, v_cache, pen, maxd, seq_bt,       \
        bt_width, seq_cu, positions, tile_seq, tile_row0, H, G, bs, scale,    \
        window);                                                              \
    return true;                                                              \
  }
  FI_TILE(32, 32, 64, 64)
  FI_TILE(32, 64, 64, 64)
  FI_TILE(32, 128, 64, 32)
  FI_TILE(64, 32, 64, 64)
  FI_TILE(64, 64, 64, 64)
  FI_TILE(64, 128, 64, 32)
  FI_TILE(128, 32, 64, 32)
  FI_TILE(128, 64, 64, 32)
  FI_TILE(128, 128, 64, 32)
#undef FI_TILE
  return false;
}

#define FI_INST(A)                                                            \
  template bool launch_talking_window_tiles<A>(                               \
      A*, A*, float*, int, const A*, int64_t, const A*, const A*, const int*, \
      int, const int*, const int*, const float*, const float*, const float*,  \
      const int*, const int*, int, int, int, int, int, int, int, float, int,  \
      hipStream_t);                                                           \
  template void launch_talking_window_rows<A>(                                \
      A*, const A*, int64_t, const A*, const A*, const int*, int, const int*, \
      const int*, const float*, const float*, const float*, int, int, int,    \
      int, int, int, int, float, int, float*, float*, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
