// Shared-key/value rotary attention over the paged cache.
//
//  * rope_unitnorm_cache: interleaved-pair rotary on the leading rot dims
//    of every q/k head (fp32 angle = position * inv_freq), each head then
//    divided by its RMS; processed q to a dense buffer, processed k to
//    the paged k cache and the UNPROCESSED k to the paged v cache.
//  * ranged_paged_attention (row-per-wave form): each (row, head) wave
//    walks the row's visible key range [lo, p] of its own sequence —
//    lo from the chunk and/or window mask — 64 keys per step with an
//    online fp32 softmax. One-row (decode) groups and short rows use it.
//
//  * ranged_paged_attention (tiled MFMA form): a 4-wave workgroup takes
//    128 consecutive rows of one (sequence, head), 32 per wave, and walks the key range
//    that any of them sees in LDS-staged tiles; S^T = K Q^T and
//    O^T = V^T P^T run on the matrix cores (bf16 16x16x16, or true-fp32
//    16x16x4 for fp32 activations), softmax statistics stay fp32 per
//    lane (one query per lane column, so no cross-lane transposes).
//    Prompt portions use it.
//
// Cache layout: [num_blocks, kv_heads, block_size, head_dim].

#include <type_traits>

#include "seqmix.h"

namespace fi {

constexpr int kMaxPairsPerLane = 4;  // head_dim <= 512

template <typename A>
__global__ __launch_bounds__(64) void rope_unitnorm_cache_kernel(
    A* __restrict__ q_out,            // [T, H, D] dense
    const A* __restrict__ q, int64_t q_stride,
    const A* __restrict__ k, int64_t k_stride,
    const int* __restrict__ positions, const float* __restrict__ inv_freq,
    A* __restrict__ k_cache, A* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, int H, int G, int D, int rot_dims,
    int block_size, float eps) {
  const int t = blockIdx.x;
  const int hh = blockIdx.y;  // 0..H-1: q heads, H..H+G-1: k heads
  const int lane = threadIdx.x;
  const bool is_q = hh < H;
  const A* src = is_q ? q + t * q_stride + static_cast<int64_t>(hh) * D
                      : k + t * k_stride + static_cast<int64_t>(hh - H) * D;
  const float pos = static_cast<float>(positions[t]);
  const int npairs = (D + 1) / 2;
  float u[kMaxPairsPerLane], w[kMaxPairsPerLane];
  float ru[kMaxPairsPerLane], rw[kMaxPairsPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    u[i] = w[i] = ru[i] = rw[i] = 0.f;
    if (j < npairs) {
      u[i] = Act<A>::ld(src + 2 * j);
      const bool has_w = 2 * j + 1 < D;
      w[i] = has_w ? Act<A>::ld(src + 2 * j + 1) : 0.f;
      if (2 * j + 1 < rot_dims) {
        const float ang = pos * inv_freq[j];
        float sn, cs;
        sincosf(ang, &sn, &cs);
        ru[i] = u[i] * cs - w[i] * sn;
        rw[i] = w[i] * cs + u[i] * sn;
      } else {
        ru[i] = u[i];
        rw[i] = w[i];
      }
      ss += ru[i] * ru[i] + rw[i] * rw[i];
    }
  }
  ss = wave_reduce_sum(ss);
  const float inv = rsqrtf(ss / D + eps);
  A* dst;
  A* raw = nullptr;
  if (is_q) {
    dst = q_out + (static_cast<int64_t>(t) * H + hh) * D;
  } else {
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    const int64_t off =
        ((static_cast<int64_t>(slot / block_size) * G + (hh - H)) * block_size +
         slot % block_size) * D;
    dst = k_cache + off;
    raw = v_cache + off;
  }
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    if (j < npairs) {
      Act<A>::st(dst + 2 * j, ru[i] * inv);
      if (raw) Act<A>::st(raw + 2 * j, u[i]);
      if (2 * j + 1 < D) {
        Act<A>::st(dst + 2 * j + 1, rw[i] * inv);
        if (raw) Act<A>::st(raw + 2 * j + 1, w[i]);
      }
    }
  }
}

constexpr int kAttnWaves = 4;        // (row, head) pairs per workgroup
constexpr int kMaxDPerLane = 8;      // head_dim <= 512

template <typename A>
__global__ __launch_bounds__(64 * kAttnWaves) void ranged_attention_row_kernel(
    A* __restrict__ out,              // [T, H, D]
    const A* __restrict__ q,          // [T, H, D]
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ seq_bt, int bt_stride,
    const int* __restrict__ row_seq, const int* __restrict__ positions,
    int T, int H, int G, int D, int block_size, float scale, int chunk,
    int window) {
  extern __shared__ float smem[];     // kAttnWaves * D floats of q
  const int wave = threadIdx.x / 64;
  const int lane = threadIdx.x % 64;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kAttnWaves + wave;
  const bool live = item < static_cast<int64_t>(T) * H;
  const int t = live ? static_cast<int>(item / H) : 0;
  const int h = live ? static_cast<int>(item % H) : 0;
  float* qs = smem + wave * D;
  if (live) {
    const A* qp = q + (static_cast<int64_t>(t) * H + h) * D;
    for (int d = lane; d < D; d += 64) qs[d] = Act<A>::ld(qp + d);
  }
  __syncthreads();
  if (!live) return;
  const int p = positions[t];
  int lo = 0;
  if (chunk > 0) lo = (p / chunk) * chunk;
  if (window > 0) lo = max(lo, p - window + 1);
  const int g = h / (H / G);
  const int* bt = seq_bt + static_cast<int64_t>(row_seq[t]) * bt_stride;

  float m = -INFINITY, l = 0.f;
  float acc[kMaxDPerLane];
#pragma unroll
  for (int i = 0; i < kMaxDPerLane; ++i) acc[i] = 0.f;

  for (int j0 = lo; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= p) {
      const int blk = bt[j / block_size];
      const A* kp = k_cache +
          ((static_cast<int64_t>(blk) * G + g) * block_size + j % block_size) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * Act<A>::ld(kp + d);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_reduce_max(s));
    const float corr = expf(m - m_new);      // m = -inf first: exp(-inf) = 0
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    l = l * corr + wave_reduce_sum(pj);
#pragma unroll
    for (int i = 0; i < kMaxDPerLane; ++i) acc[i] *= corr;
    m = m_new;
    const int n = min(64, p - j0 + 1);
    for (int jj = 0; jj < n; ++jj) {
      const float pv = __shfl(pj, jj, 64);
      const int key = j0 + jj;
      const int blk = bt[key / block_size];
      const A* vp = v_cache +
          ((static_cast<int64_t>(blk) * G + g) * block_size + key % block_size) * D;
#pragma unroll
      for (int i = 0; i < kMaxDPerLane; ++i) {
        const int d = lane + 64 * i;
        if (d < D) acc[i] += pv * Act<A>::ld(vp + d);
      }
    }
  }
  const float inv_l = 1.0f / l;
  A* op = out + (static_cast<int64_t>(t) * H + h) * D;
#pragma unroll
  for (int i = 0; i < kMaxDPerLane; ++i) {
    const int d = lane + 64 * i;
    if (d < D) Act<A>::st(op + d, acc[i] * inv_l);
  }
}


typedef __attribute__((ext_vector_type(4))) short short4v;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kQSets = 2;               // 16-row query sets per wave
constexpr int kTileRows = 64 * kQSets;  // q rows per workgroup (4 waves)

template <typename A, int D, int BN>
__global__ __launch_bounds__(256) void ranged_attention_tile_kernel(
    A* __restrict__ out, const A* __restrict__ q,
    const A* __restrict__ k_cache, const A* __restrict__ v_cache,
    const int* __restrict__ seq_bt, int bt_stride,
    const int* __restrict__ seq_cu, const int* __restrict__ positions,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_row0, int H,
    int G, int block_size, float scale, int chunk, int window) {
  constexpr bool BF = std::is_same<A, u16>::value;
  constexpr int QS = kQSets;
  constexpr int VEC = BF ? 8 : 4;               // elements per 16-byte load
  constexpr int KP = D + (BF ? 8 : 4);          // K tile [BN][KP]
  constexpr int VP = BF ? BN + 8 : D + 4;       // bf16: V^T [D][VP]; fp32: V [BN][VP]
  constexpr int NB = BN / 16;
  constexpr int DB = D / 16;
  __shared__ __attribute__((aligned(16))) A k_lds[BN * KP];
  __shared__ __attribute__((aligned(16))) A v_lds[BF ? D * VP : BN * VP];

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int g4 = lane / 16, c16 = lane % 16;
  const int h = blockIdx.y;
  const int g = h / (H / G);
  const int s = tile_seq[blockIdx.x];
  const int row_first = seq_cu[s] + tile_row0[blockIdx.x];
  const int nrows = min(kTileRows, seq_cu[s + 1] - row_first);
  const int* bt = seq_bt + static_cast<int64_t>(s) * bt_stride;

  auto range_lo = [&](int p) {
    int lo = 0;
    if (chunk > 0) lo = (p / chunk) * chunk;
    if (window > 0) lo = max(lo, p - window + 1);
    return lo;
  };
  const int p_first = positions[row_first];
  const int kv_lo = range_lo(p_first);
  const int kv_hi = p_first + nrows - 1;   // positions in a group ascend by 1

  // this lane's queries: column c16 of each of the wave's 16-row sets
  int my_row[QS], my_pos[QS], my_lo[QS];
  bool row_ok[QS];
  short4v qf16[QS][BF ? DB : 1];
  float qf32[QS][BF ? 1 : D / 4];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    my_row[qs] = (wave * QS + qs) * 16 + c16;
    row_ok[qs] = my_row[qs] < nrows;
    my_pos[qs] = row_ok[qs] ? p_first + my_row[qs] : -1;
    my_lo[qs] = row_ok[qs] ? range_lo(my_pos[qs]) : 0;
    const A* qp =
        q + (static_cast<int64_t>(row_first + my_row[qs]) * H + h) * D;
    if constexpr (BF) {
#pragma unroll
      for (int kk = 0; kk < DB; ++kk) {
        if (row_ok[qs])
          qf16[qs][kk] =
              *reinterpret_cast<const short4v*>(qp + 16 * kk + 4 * g4);
        else
          qf16[qs][kk] = short4v{0, 0, 0, 0};
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < D / 4; ++kk)
        qf32[qs][kk] = row_ok[qs] ? qp[4 * kk + g4] : 0.f;
    }
  }

  floatx4 o[QS][DB];
  float m[QS], l[QS];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    m[qs] = -INFINITY;
    l[qs] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[qs][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // bf16 activations: softmax in the log2 domain (scale * log2(e) folded
  // into the scores, hardware exp2); fp32 activations keep expf
  const float sc = BF ? scale * 1.4426950408889634f : scale;
  auto ex = [](float x) {
    return BF ? __builtin_amdgcn_exp2f(x) : expf(x);
  };
  // rows of this wave: 16*QS consecutive positions (the valid ones)
  const int wave_rows = min(16 * QS, nrows - wave * 16 * QS);
  const int wave_min_pos = wave_rows > 0 ? p_first + wave * 16 * QS : -1;
  const int wave_max_lo =
      wave_rows > 0 ? range_lo(p_first + wave * 16 * QS + wave_rows - 1) : 0;
  const bool wave_full = wave_rows == 16 * QS;

  for (int j0 = kv_lo; j0 <= kv_hi; j0 += BN) {
    // ---- stage K and V tiles (zero-filled past the range) ----
    constexpr int VPR = D / VEC;               // vectors per key row
    typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
    if constexpr (BF) {
      // two adjacent keys per thread: the transposed V tile is written
      // with 4-byte stores (one (key, key+1) pair per d)
      for (int pid = tid; pid < (BN / 2) * VPR; pid += 256) {
        const int kp = pid / VPR, dv = pid % VPR;
        u32x4 k4[2], v4[2];
#pragma unroll
        for (int e2 = 0; e2 < 2; ++e2) {
          const int key = j0 + 2 * kp + e2;
          k4[e2] = u32x4{0u, 0u, 0u, 0u};
          v4[e2] = u32x4{0u, 0u, 0u, 0u};
          if (key <= kv_hi) {
            const int64_t off =
                ((static_cast<int64_t>(bt[key / block_size]) * G + g) *
                     block_size + key % block_size) * D + dv * VEC;
            k4[e2] = *reinterpret_cast<const u32x4*>(k_cache + off);
            v4[e2] = *reinterpret_cast<const u32x4*>(v_cache + off);
          }
          *reinterpret_cast<u32x4*>(k_lds + (2 * kp + e2) * KP + dv * VEC) =
              k4[e2];
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
        u32x4 kv4 = {0u, 0u, 0u, 0u}, vv4 = {0u, 0u, 0u, 0u};
        if (key <= kv_hi) {
          const int64_t off =
              ((static_cast<int64_t>(bt[key / block_size]) * G + g) *
                   block_size + key % block_size) * D + dv * VEC;
          kv4 = *reinterpret_cast<const u32x4*>(k_cache + off);
          vv4 = *reinterpret_cast<const u32x4*>(v_cache + off);
        }
        *reinterpret_cast<u32x4*>(k_lds + key_l * KP + dv * VEC) = kv4;
        *reinterpret_cast<u32x4*>(v_lds + key_l * VP + dv * VEC) = vv4;
      }
    }
    __syncthreads();

    // ---- S^T = K Q^T: every K fragment read from LDS feeds QS MFMAs ----
    // a tile every row of the wave sees completely needs no per-element
    // mask (wave-uniform test)
    const bool interior =
        wave_full && j0 + BN - 1 <= wave_min_pos && j0 >= wave_max_lo;
    float sv[QS][NB][4];
    float tmax[QS];
#pragma unroll
    for (int qs = 0; qs < QS; ++qs) tmax[qs] = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      floatx4 acc[QS];
#pragma unroll
      for (int qs = 0; qs < QS; ++qs) acc[qs] = floatx4{0.f, 0.f, 0.f, 0.f};
      const A* kr = k_lds + (nb * 16 + c16) * KP;
      if constexpr (BF) {
#pragma unroll
        for (int kk = 0; kk < DB; ++kk) {
          const short4v a =
              *reinterpret_cast<const short4v*>(kr + 16 * kk + 4 * g4);
#pragma unroll
          for (int qs = 0; qs < QS; ++qs)
            acc[qs] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                a, qf16[qs][kk], acc[qs], 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < D / 4; ++kk) {
          const float a = kr[4 * kk + g4];
#pragma unroll
          for (int qs = 0; qs < QS; ++qs)
            acc[qs] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, qf32[qs][kk],
                                                           acc[qs], 0, 0, 0);
        }
      }
#pragma unroll
      for (int qs = 0; qs < QS; ++qs)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = j0 + nb * 16 + 4 * g4 + i;
          const bool vis =
              interior || (key <= my_pos[qs] && key >= my_lo[qs]);
          sv[qs][nb][i] = vis ? acc[qs][i] * sc : -INFINITY;
          tmax[qs] = fmaxf(tmax[qs], sv[qs][nb][i]);
        }
    }
#pragma unroll
    for (int qs = 0; qs < QS; ++qs) {
      float tm = tmax[qs];
      tm = fmaxf(tm, __shfl_xor(tm, 16, 64));
      tm = fmaxf(tm, __shfl_xor(tm, 32, 64));
      const float m_new = fmaxf(m[qs], tm);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float corr = ex(m[qs] - m_safe);     // m = -inf -> 0
      float psum = 0.f;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sv[qs][nb][i] = ex(sv[qs][nb][i] - m_safe);  // masked -> 0
          psum += sv[qs][nb][i];
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l[qs] = l[qs] * corr + psum;
      m[qs] = m_new;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[qs][db][i] *= corr;
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
      for (int db = 0; db < DB; ++db) {
        const A* vr = v_lds + (db * 16 + c16) * VP;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const short4v a =
              *reinterpret_cast<const short4v*>(vr + nb * 16 + 4 * g4);
#pragma unroll
          for (int qs = 0; qs < QS; ++qs)
            o[qs][db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                a, pf[qs][nb], o[qs][db], 0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float a = v_lds[(nb * 16 + 4 * g4 + i) * VP + db * 16 + c16];
#pragma unroll
            for (int qs = 0; qs < QS; ++qs)
              o[qs][db] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                  a, sv[qs][nb][i], o[qs][db], 0, 0, 0);
          }
    }
    __syncthreads();
  }

#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    if (!row_ok[qs]) continue;
    const float inv_l = 1.0f / l[qs];
    A* op = out + (static_cast<int64_t>(row_first + my_row[qs]) * H + h) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        Act<A>::st(op + db * 16 + 4 * g4 + i, o[qs][db][i] * inv_l);
  }
}

template <typename A>
bool launch_ranged_attention_tiles(A* out, const A* q, const A* k_cache,
                                   const A* v_cache, const int* seq_bt,
                                   int bt_stride, const int* seq_cu,
                                   const int* positions, const int* tile_seq,
                                   const int* tile_row0, int num_tiles, int H,
                                   int G, int D, int block_size, float scale,
                                   int chunk, int window, hipStream_t s) {
  constexpr bool BF = std::is_same<A, u16>::value;
  if (num_tiles == 0) return true;
  dim3 grid(num_tiles, H);
#define FI_TILE(DD, BNB, BNF)                                                  \
  case DD:                                                                     \
    hipLaunchKernelGGL(                                                        \
        (ranged_attention_tile_kernel<A, DD, (BF ? BNB : BNF)>), grid,         \
        dim3(256), 0, s, out, q, k_cache, v_cache, seq_bt, bt_stride, seq_cu,  \
        positions, tile_seq, tile_row0, H, G, block_size, scale, chunk,        \
        window);                                                               \
    return true;
  switch (D) {
    FI_TILE(32, 64, 64)
    FI_TILE(64, 64, 64)
    FI_TILE(96, 64, 32)
    FI_TILE(128, 64, 32)
    FI_TILE(256, 32, 16)
    default:
      return false;   // caller falls back to the row-per-wave kernel
  }
#undef FI_TILE
}

template <typename A>
void launch_rope_unitnorm_cache(A* q_out, const A* q, int64_t q_stride,
                                const A* k, int64_t k_stride,
                                const int* positions, const float* inv_freq,
                                A* k_cache, A* v_cache,
                                const int* slot_mapping, int T, int H, int G,
                                int D, int rot_dims, int block_size, float eps,
                                hipStream_t s) {
  if (T == 0) return;
  hipLaunchKernelGGL(rope_unitnorm_cache_kernel<A>, dim3(T, H + G), dim3(64), 0,
                     s, q_out, q, q_stride, k, k_stride, positions, inv_freq,
                     k_cache, v_cache, slot_mapping, H, G, D, rot_dims,
                     block_size, eps);
}

template <typename A>
void launch_ranged_attention_rows(A* out, const A* q, const A* k_cache,
                                  const A* v_cache, const int* seq_bt,
                                  int bt_stride, const int* row_seq,
                                  const int* positions, int T, int H, int G,
                                  int D, int block_size, float scale,
                                  int chunk, int window, hipStream_t s) {
  if (T == 0) return;
  const int64_t items = static_cast<int64_t>(T) * H;
  const int blocks = static_cast<int>((items + kAttnWaves - 1) / kAttnWaves);
  hipLaunchKernelGGL(ranged_attention_row_kernel<A>, dim3(blocks),
                     dim3(64 * kAttnWaves), kAttnWaves * D * sizeof(float), s,
                     out, q, k_cache, v_cache, seq_bt, bt_stride, row_seq,
                     positions, T, H, G, D, block_size, scale, chunk, window);
}

#define FI_INST(A)                                                             \
  template bool launch_ranged_attention_tiles<A>(                              \
      A*, const A*, const A*, const A*, const int*, int, const int*,           \
      const int*, const int*, const int*, int, int, int, int, int, float, int, \
      int, hipStream_t);                                                       \
  template void launch_rope_unitnorm_cache<A>(                                 \
      A*, const A*, int64_t, const A*, int64_t, const int*, const float*, A*,  \
      A*, const int*, int, int, int, int, int, int, float, hipStream_t);       \
  template void launch_ranged_attention_rows<A>(                               \
      A*, const A*, const A*, const A*, const int*, int, const int*,           \
      const int*, int, int, int, int, int, float, int, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
