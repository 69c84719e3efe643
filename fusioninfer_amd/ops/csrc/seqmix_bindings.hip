// PyTorch bindings of the sequence-mixer kernels (_C_seqmix).
// Every entry checks operand shapes against what its kernel and grid
// assume before launching.

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

#include "seqmix.h"

namespace fi {
template <typename A>
void launch_scalar_rms_norm(A*, const float*, const float*, float, int, int,
                            hipStream_t);
template <typename A>
void launch_residual_add_scalar_norm(float*, const A*, const float*,
                                     const float*, A*, float, int, int,
                                     hipStream_t);
template <typename A>
void launch_dual_norm_combine_residual(float*, const A*, const A*,
                                       const float*, const float*,
                                       const float*, const float*, A*, float,
                                       int, int, hipStream_t);
template <typename A>
void launch_norm_token_shift(A*, const float*, const float*, const float*,
                             float*, const int*, const int*, const int*,
                             const int*, float, int, int, hipStream_t);
template <typename A>
void launch_gelu_tanh_and_mul(A*, const A*, int, int, hipStream_t);
template <typename A>
void launch_rope_unitnorm_cache(A*, const A*, int64_t, const A*, int64_t,
                                const int*, const float*, A*, A*, const int*,
                                int, int, int, int, int, int, float,
                                hipStream_t);
template <typename A>
void launch_ranged_attention_rows(A*, const A*, const A*, const A*, const int*,
                                  int, const int*, const int*, int, int, int,
                                  int, int, float, int, int, hipStream_t);
template <typename A>
bool launch_ranged_attention_tiles(A*, const A*, const A*, const A*,
                                   const int*, int, const int*, const int*,
                                   const int*, const int*, int, int, int, int,
                                   int, float, int, int, hipStream_t);
template <typename A>
void launch_delta_rule(A*, float*, float*, const A*, const A*, const A*,
                       const A*, const A*, const A*, int64_t, int64_t, int64_t,
                       int64_t, int64_t, int64_t, const float*, const float*,
                       const float*, float*, const int*, const int*,
                       const int*, int, int, int, int, float, float,
                       hipStream_t);
}  // namespace fi

namespace {

using fi::u16;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

bool is_act(const at::Tensor& t) {
  return t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16;
}

#define CHECK_ACT(t)                                                 \
  TORCH_CHECK((t).is_cuda(), #t " must be on the GPU");              \
  TORCH_CHECK(is_act(t), #t " must be float32 or bfloat16")
#define CHECK_F32(t)                                                  \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kFloat &&     \
                  (t).is_contiguous(),                                \
              #t " must be a contiguous float32 GPU tensor")
#define CHECK_I32(t)                                                  \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kInt &&       \
                  (t).is_contiguous(),                                \
              #t " must be a contiguous int32 GPU tensor")

// rows of a 2-D activation view whose last dim is dense
void check_rows(const at::Tensor& t, int64_t T, int64_t n, const char* what) {
  TORCH_CHECK(t.dim() == 2 && t.size(0) == T && t.size(1) == n &&
                  (t.stride(1) == 1 || n == 1),
              what, ": expected [", T, ", ", n, "] with dense rows");
}

#define DISPATCH_ACT(t, ...)                          \
  if ((t).scalar_type() == at::kFloat) {              \
    using A = float;                                  \
    __VA_ARGS__;                                      \
  } else {                                            \
    using A = u16;                                    \
    __VA_ARGS__;                                      \
  }

template <typename A>
A* ptr(const at::Tensor& t) {
  return reinterpret_cast<A*>(t.data_ptr());
}

void scalar_rms_norm(at::Tensor out, at::Tensor x, at::Tensor g, double eps) {
  CHECK_ACT(out);
  CHECK_F32(x);
  CHECK_F32(g);
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && out.is_contiguous());
  TORCH_CHECK(g.numel() == 1);
  const int T = x.size(0), W = x.size(1);
  DISPATCH_ACT(out, fi::launch_scalar_rms_norm<A>(
                        ptr<A>(out), x.data_ptr<float>(), g.data_ptr<float>(),
                        (float)eps, T, W, stream()));
}

void residual_add_scalar_norm(at::Tensor resid, at::Tensor y,
                              at::Tensor g_post,
                              c10::optional<at::Tensor> g_next,
                              c10::optional<at::Tensor> out, double eps) {
  CHECK_F32(resid);
  CHECK_ACT(y);
  CHECK_F32(g_post);
  TORCH_CHECK(resid.dim() == 2 && y.sizes() == resid.sizes() &&
              y.is_contiguous() && g_post.numel() == 1);
  TORCH_CHECK(g_next.has_value() == out.has_value());
  const float* gn = nullptr;
  void* op = nullptr;
  if (g_next.has_value()) {
    CHECK_F32(*g_next);
    TORCH_CHECK(g_next->numel() == 1);
    TORCH_CHECK(out->is_cuda() && out->scalar_type() == y.scalar_type() &&
                out->sizes() == resid.sizes() && out->is_contiguous());
    gn = g_next->data_ptr<float>();
    op = out->data_ptr();
  }
  const int T = resid.size(0), W = resid.size(1);
  DISPATCH_ACT(y, fi::launch_residual_add_scalar_norm<A>(
                      resid.data_ptr<float>(), ptr<A>(y),
                      g_post.data_ptr<float>(), gn, static_cast<A*>(op),
                      (float)eps, T, W, stream()));
}

void dual_norm_combine_residual(at::Tensor resid, at::Tensor yl, at::Tensor yr,
                                at::Tensor wl, at::Tensor wr,
                                at::Tensor g_post,
                                c10::optional<at::Tensor> g_next,
                                c10::optional<at::Tensor> out, double eps) {
  CHECK_F32(resid);
  CHECK_ACT(yl);
  CHECK_ACT(yr);
  CHECK_F32(wl);
  CHECK_F32(wr);
  CHECK_F32(g_post);
  TORCH_CHECK(resid.dim() == 2 && yl.sizes() == resid.sizes() &&
              yr.sizes() == resid.sizes() && yl.is_contiguous() &&
              yr.is_contiguous() && yl.scalar_type() == yr.scalar_type());
  const int T = resid.size(0), W = resid.size(1);
  TORCH_CHECK(wl.numel() == W && wr.numel() == W && g_post.numel() == 1);
  TORCH_CHECK(g_next.has_value() == out.has_value());
  const float* gn = nullptr;
  void* op = nullptr;
  if (g_next.has_value()) {
    CHECK_F32(*g_next);
    TORCH_CHECK(g_next->numel() == 1);
    TORCH_CHECK(out->is_cuda() && out->scalar_type() == yl.scalar_type() &&
                out->sizes() == resid.sizes() && out->is_contiguous());
    gn = g_next->data_ptr<float>();
    op = out->data_ptr();
  }
  DISPATCH_ACT(yl, fi::launch_dual_norm_combine_residual<A>(
                       resid.data_ptr<float>(), ptr<A>(yl), ptr<A>(yr),
                       wl.data_ptr<float>(), wr.data_ptr<float>(),
                       g_post.data_ptr<float>(), gn, static_cast<A*>(op),
                       (float)eps, T, W, stream()));
}

// group tables: seq_cu [S+1] ascending from 0 to T, row_seq [T],
// positions [T], seq_slots [S] < num_slots. Values are produced by the
// model runner; sizes are checked here.
void check_groups(const at::Tensor& seq_cu, const at::Tensor& seq_slots,
                  const at::Tensor& positions, int64_t T) {
  CHECK_I32(seq_cu);
  CHECK_I32(seq_slots);
  CHECK_I32(positions);
  TORCH_CHECK(seq_cu.numel() == seq_slots.numel() + 1);
  TORCH_CHECK(positions.numel() == T);
}

void norm_token_shift(at::Tensor out, at::Tensor resid, at::Tensor g,
                      at::Tensor shift, at::Tensor state, at::Tensor seq_cu,
                      at::Tensor row_seq, at::Tensor positions,
                      at::Tensor seq_slots, double eps) {
  CHECK_ACT(out);
  CHECK_F32(resid);
  CHECK_F32(g);
  CHECK_F32(shift);
  CHECK_F32(state);
  CHECK_I32(row_seq);
  const int T = resid.size(0), W = resid.size(1);
  check_groups(seq_cu, seq_slots, positions, T);
  TORCH_CHECK(resid.dim() == 2 && out.sizes() == resid.sizes() &&
              out.is_contiguous());
  TORCH_CHECK(g.numel() == 1 && shift.numel() == W && row_seq.numel() == T);
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W);
  DISPATCH_ACT(out, fi::launch_norm_token_shift<A>(
                        ptr<A>(out), resid.data_ptr<float>(),
                        g.data_ptr<float>(), shift.data_ptr<float>(),
                        state.data_ptr<float>(), seq_cu.data_ptr<int>(),
                        row_seq.data_ptr<int>(), positions.data_ptr<int>(),
                        seq_slots.data_ptr<int>(), (float)eps, T, W, stream()));
}

void gelu_tanh_and_mul(at::Tensor out, at::Tensor gu) {
  CHECK_ACT(out);
  CHECK_ACT(gu);
  TORCH_CHECK(gu.dim() == 2 && gu.is_contiguous() && out.is_contiguous() &&
              out.scalar_type() == gu.scalar_type());
  const int T = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(gu.size(1) == 2 * F && out.size(0) == T && out.size(1) == F);
  DISPATCH_ACT(gu, fi::launch_gelu_tanh_and_mul<A>(ptr<A>(out), ptr<A>(gu), T,
                                                   F, stream()));
}

void check_cache(const at::Tensor& k_cache, const at::Tensor& v_cache,
                 at::ScalarType dt, int64_t G, int64_t D) {
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  TORCH_CHECK(k_cache.scalar_type() == dt && v_cache.scalar_type() == dt,
              "cache dtype must equal the activation dtype");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.sizes() == v_cache.sizes() &&
              k_cache.size(1) == G && k_cache.size(3) == D);
}

void rope_unitnorm_cache(at::Tensor q_out, at::Tensor q, at::Tensor k,
                         at::Tensor positions, at::Tensor inv_freq,
                         at::Tensor k_cache, at::Tensor v_cache,
                         at::Tensor slot_mapping, int64_t H, int64_t G,
                         int64_t D, double eps) {
  CHECK_ACT(q);
  CHECK_ACT(k);
  CHECK_ACT(q_out);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  CHECK_F32(inv_freq);
  const int64_t T = q.size(0);
  check_rows(q, T, H * D, "q");
  check_rows(k, T, G * D, "k");
  TORCH_CHECK(q.scalar_type() == k.scalar_type() &&
              q_out.scalar_type() == q.scalar_type());
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() == T * H * D);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  check_cache(k_cache, v_cache, q.scalar_type(), G, D);
  const int rot_dims = 2 * inv_freq.numel();
  TORCH_CHECK(rot_dims <= D && D <= 512 && D >= 1, "head dim out of range");
  DISPATCH_ACT(q, fi::launch_rope_unitnorm_cache<A>(
                      ptr<A>(q_out), ptr<A>(q), q.stride(0), ptr<A>(k),
                      k.stride(0), positions.data_ptr<int>(),
                      inv_freq.data_ptr<float>(), ptr<A>(k_cache),
                      ptr<A>(v_cache), slot_mapping.data_ptr<int>(), (int)T,
                      (int)H, (int)G, (int)D, rot_dims, (int)k_cache.size(2),
                      (float)eps, stream()));
}

// Rows [0, tile_rows) belong to the row groups that the tile tables
// cover (tile_seq/tile_row0: group and first row inside it of every
// 128-row tile) and run the MFMA kernel when the head size has one; all
// other rows run the row-per-wave kernel.
void ranged_paged_attention(at::Tensor out, at::Tensor q, at::Tensor k_cache,
                            at::Tensor v_cache, at::Tensor seq_bt,
                            at::Tensor row_seq, at::Tensor positions,
                            double scale, int64_t chunk, int64_t window,
                            c10::optional<at::Tensor> seq_cu,
                            c10::optional<at::Tensor> tile_seq,
                            c10::optional<at::Tensor> tile_row0,
                            int64_t tile_rows) {
  CHECK_ACT(q);
  CHECK_ACT(out);
  CHECK_I32(row_seq);
  CHECK_I32(positions);
  TORCH_CHECK(seq_bt.is_cuda() && seq_bt.scalar_type() == at::kInt &&
              seq_bt.dim() == 2 && seq_bt.stride(1) == 1);
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && out.is_contiguous() &&
              out.sizes() == q.sizes() &&
              out.scalar_type() == q.scalar_type());
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k_cache.size(1);
  check_cache(k_cache, v_cache, q.scalar_type(), G, D);
  TORCH_CHECK(G >= 1 && H % G == 0 && D <= 512);
  TORCH_CHECK(row_seq.numel() == T && positions.numel() == T);
  TORCH_CHECK(chunk >= 0 && window >= 0);
  TORCH_CHECK(tile_rows >= 0 && tile_rows <= T);
  int64_t done = 0;
  if (tile_rows > 0) {
    TORCH_CHECK(seq_cu.has_value() && tile_seq.has_value() &&
                tile_row0.has_value());
    CHECK_I32(*seq_cu);
    CHECK_I32(*tile_seq);
    CHECK_I32(*tile_row0);
    TORCH_CHECK(tile_seq->numel() == tile_row0->numel());
    TORCH_CHECK(seq_cu->numel() <= seq_bt.size(0) + 1);
    // head sizes without a tiled variant (or without 16-byte rows) keep
    // the row-per-wave kernel
    bool ok = false;
    if ((D * k_cache.element_size()) % 16 == 0) {
      DISPATCH_ACT(q, ok = fi::launch_ranged_attention_tiles<A>(
                        ptr<A>(out), ptr<A>(q), ptr<A>(k_cache),
                        ptr<A>(v_cache), seq_bt.data_ptr<int>(),
                        (int)seq_bt.stride(0), seq_cu->data_ptr<int>(),
                        positions.data_ptr<int>(), tile_seq->data_ptr<int>(),
                        tile_row0->data_ptr<int>(), (int)tile_seq->numel(), H,
                        G, D, (int)k_cache.size(2), (float)scale, (int)chunk,
                        (int)window, stream()));
    }
    if (ok) done = tile_rows;
  }
  const int rest = T - (int)done;
  DISPATCH_ACT(q, fi::launch_ranged_attention_rows<A>(
                      ptr<A>(out) + done * H * D, ptr<A>(q) + done * H * D,
                      ptr<A>(k_cache), ptr<A>(v_cache), seq_bt.data_ptr<int>(),
                      (int)seq_bt.stride(0), row_seq.data_ptr<int>() + done,
                      positions.data_ptr<int>() + done, rest, H, G, D,
                      (int)k_cache.size(2), (float)scale, (int)chunk,
                      (int)window, stream()));
}

void delta_rule(at::Tensor out, at::Tensor o_raw, at::Tensor vecs, at::Tensor r, at::Tensor k, at::Tensor v,
                at::Tensor wlin, at::Tensor alin, at::Tensor glin,
                at::Tensor w0, at::Tensor a_bias, at::Tensor norm_w,
                at::Tensor state, at::Tensor seq_cu, at::Tensor seq_slots,
                at::Tensor positions, int64_t heads, int64_t dim, double eps,
                double decay_scale) {
  CHECK_ACT(out);
  const int64_t T = r.size(0), n = heads * dim;
  for (const at::Tensor* t : {&r, &k, &v, &wlin, &alin, &glin}) {
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == out.scalar_type());
    check_rows(*t, T, n, "delta-rule input");
  }
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
              out.size(1) == n);
  CHECK_F32(o_raw);
  TORCH_CHECK(o_raw.numel() == T * n);
  // scratch of the state-independent per-token vectors: 5 vectors of the
  // kernel's row capacity per (token, head)
  CHECK_F32(vecs);
  const int64_t cap = dim <= 64 ? 64 : (dim <= 128 ? 128 : 256);
  TORCH_CHECK(vecs.numel() == T * heads * 5 * cap,
              "delta rule: scratch must hold [T, heads, 5, ", cap, "]");
  CHECK_F32(w0);
  CHECK_F32(a_bias);
  CHECK_F32(norm_w);
  CHECK_F32(state);
  TORCH_CHECK(w0.numel() == n && a_bias.numel() == n && norm_w.numel() == n);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads &&
              state.size(2) == dim && state.size(3) == dim);
  TORCH_CHECK(dim >= 1 && dim <= 256, "delta rule: head dim must be <= 256");
  check_groups(seq_cu, seq_slots, positions, T);
  const int S = seq_slots.numel();
  DISPATCH_ACT(out, fi::launch_delta_rule<A>(
                        ptr<A>(out), o_raw.data_ptr<float>(),
                        vecs.data_ptr<float>(), ptr<A>(r),
                        ptr<A>(k), ptr<A>(v),
                        ptr<A>(wlin), ptr<A>(alin), ptr<A>(glin), r.stride(0),
                        k.stride(0), v.stride(0), wlin.stride(0),
                        alin.stride(0), glin.stride(0), w0.data_ptr<float>(),
                        a_bias.data_ptr<float>(), norm_w.data_ptr<float>(),
                        state.data_ptr<float>(), seq_cu.data_ptr<int>(),
                        seq_slots.data_ptr<int>(), positions.data_ptr<int>(),
                        (int)T, S, (int)heads, (int)dim, (float)eps,
                        (float)decay_scale, stream()));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("scalar_rms_norm", &scalar_rms_norm, "scalar-gain RMS norm");
  m.def("residual_add_scalar_norm", &residual_add_scalar_norm,
        "fp32 residual += norm(y); optional next norm");
  m.def("dual_norm_combine_residual", &dual_norm_combine_residual,
        "average of two width-normed halves into the residual");
  m.def("norm_token_shift", &norm_token_shift,
        "scalar-gain RMS norm + token shift with slot state");
  m.def("gelu_tanh_and_mul", &gelu_tanh_and_mul, "tanh-GELU gated product");
  m.def("rope_unitnorm_cache", &rope_unitnorm_cache,
        "interleaved rotary + unit RMS q/k; k and raw k into the paged cache");
  m.def("ranged_paged_attention", &ranged_paged_attention,
        "softmax attention over a per-row key range of the paged cache");
  m.def("delta_rule", &delta_rule,
        "generalized delta rule recurrence with gated unit-RMS output");
}
