// PyTorch bindings of the sequence-mixer kernels (_C_seqmix).
// Every entry checks operand shapes against what its kernel and grid
// assume before launching.

#include <algorithm>
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
template <typename A>
void launch_layer_norm(A*, const float*, const float*, float, int, int,
                       hipStream_t);
template <typename A>
void launch_gated_residual_layer_norm(float*, const A*, float, const A*, float,
                                      const A*, int64_t, const float*,
                                      const float*, A*, float, int, int,
                                      hipStream_t);
template <typename A>
void launch_group_rms_gate(A*, const float*, const A*, int64_t, const float*,
                           bool, int, int, int, float, bool, hipStream_t);
template <typename A>
void launch_paged_cache_write(A*, A*, const A*, int64_t, const A*, int64_t,
                              const int*, int, int, int, int, int,
                              hipStream_t);
template <typename A>
void launch_decay_linear_attention(float*, float*, float*, const A*, const A*,
                                   const A*, int64_t, int64_t, int64_t,
                                   const float*, float*, const int*,
                                   const int*, const int*, const int*, int,
                                   int, int, int, int, bool, hipStream_t);
template <typename A>
void launch_gated_delta_rule(float*, float*, float*, const A*, int64_t,
                             const float*, const A*, int64_t, const A*,
                             int64_t, const float*, const float*, float*,
                             float*, const int*, const int*, const int*,
                             const int*, int, int, int, int, int, int, int,
                             hipStream_t);
size_t talking_window_row_smem(int, int);
bool talking_window_fast_fits(int, int, int, int);
int talking_window_fast_splits(int);
template <typename A>
bool launch_talking_window_tiles(A*, A*, float*, int, const A*, int64_t,
                                 const A*, const A*, const int*, int,
                                 const int*, const int*, const float*,
                                 const float*, const float*, const int*,
                                 const int*, int, int, int, int, int, int, int,
                                 float, int, hipStream_t);
template <typename A>
void launch_talking_window_rows(A*, const A*, int64_t, const A*, const A*,
                                const int*, int, const int*, const int*,
                                const float*, const float*, const float*, int,
                                int, int, int, int, int, int, float, int,
                                float*, float*, int, hipStream_t);
template <typename A>
void launch_scaled_residual_layer_norm(float*, const A*, float, const A*,
                                       float, const A*, float, const float*,
                                       A*, float, int, int, hipStream_t);
template <typename A>
void launch_headnorm_qtemp_cache(A*, const A*, int64_t, const A*, int64_t,
                                 const A*, int64_t, const int*, const float*,
                                 const float*, float, float, int, A*, A*,
                                 const int*, int, int, int, int, int, int,
                                 hipStream_t);
template <typename A>
void launch_latent_rope_cache(A*, const A*, int64_t, const A*, int64_t,
                              const int*, const float*, const float*, float,
                              A*, const int*, int, int, int, int, int, int,
                              int, hipStream_t);
template <typename A>
void launch_causal_conv_state(float*, const A*, int64_t, const float*,
                              const float*, float*, const int*, const int*,
                              const int*, const int*, int, int, int, int, int,
                              hipStream_t);
template <typename A>
void launch_rglru_scan(A*, const float*, const float*, const float*,
                       const float*, const A*, int64_t, float*, const int*,
                       const int*, const int*, int, int, int, int, float, int,
                       hipStream_t);
template <typename A>
void launch_relu_squared(A*, const A*, int64_t, int, int, hipStream_t);
template <typename A>
void launch_cast_layer_norm(float*, A*, const A*, const float*, float, int,
                            int, hipStream_t);
template <typename A>
void launch_concat_cast(A*, const float*, const A*, int, int, hipStream_t);
int sink_attention_splits(int max_keys);
bool sink_attention_has_tiles(int DK, int DV);
template <typename A>
bool launch_sink_attention_tiles(A*, const A*, const A*, const A*, int,
                                 const int*, int, const int*, const int*,
                                 const int*, const int*, int, const float*,
                                 const A*, int64_t, int, int, int, int, int,
                                 int, float, int, int, hipStream_t);
template <typename A>
void launch_sink_attention_rows(A*, float*, float*, const A*, const A*,
                                const A*, int, const int*, int, const int*,
                                const int*, const float*, const A*, int64_t,
                                int, int, int, int, int, int, int, int, float,
                                int, int, int, hipStream_t);
template <typename A>
void launch_pair_embed(float*, A*, const int64_t*, const A*, float, const A*,
                       int64_t, int64_t, int64_t, int*, const int*,
                       const int*, const int*, const int*, int, int,
                       hipStream_t);
template <typename I, typename A>
void launch_norm_affine(const I*, float*, A*, const float*, const float*,
                        float, int, int, hipStream_t);
template <typename A>
void launch_widenorm_rope_cache(A*, const A*, int64_t, const A*, int64_t,
                                const A*, int64_t, const int*, const float*,
                                const float*, float, const float*, int, float,
                                A*, A*, const int*, int, int, int, int, int,
                                int, hipStream_t);
template <typename A>
void launch_clamped_glu(A*, const A*, int64_t, int, int, float, hipStream_t);
void launch_tanh_cap(float*, int64_t, float, hipStream_t);

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


// ------------------------------------------------------------------------
// layer-norm / gated-residual stream, decayed linear attention, windowed
// attention with head mixing, gated delta rule

void layer_norm(at::Tensor out, at::Tensor x, at::Tensor w, double eps) {
  CHECK_ACT(out);
  CHECK_F32(x);
  CHECK_F32(w);
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && out.is_contiguous());
  const int T = x.size(0), W = x.size(1);
  TORCH_CHECK(w.numel() == W);
  DISPATCH_ACT(out, fi::launch_layer_norm<A>(ptr<A>(out), x.data_ptr<float>(),
                                             w.data_ptr<float>(), (float)eps,
                                             T, W, stream()));
}

void gated_residual_layer_norm(at::Tensor resid, at::Tensor y1, double s1,
                               c10::optional<at::Tensor> y2, double s2,
                               at::Tensor gate_lin, at::Tensor gate_bias,
                               c10::optional<at::Tensor> w_next,
                               c10::optional<at::Tensor> out, double eps) {
  CHECK_F32(resid);
  CHECK_ACT(y1);
  CHECK_ACT(gate_lin);
  CHECK_F32(gate_bias);
  TORCH_CHECK(resid.dim() == 2);
  const int64_t T = resid.size(0), W = resid.size(1);
  TORCH_CHECK(y1.sizes() == resid.sizes() && y1.is_contiguous());
  TORCH_CHECK(gate_lin.scalar_type() == y1.scalar_type());
  check_rows(gate_lin, T, W, "gate projection");
  TORCH_CHECK(gate_bias.numel() == W);
  void* y2p = nullptr;
  if (y2.has_value()) {
    TORCH_CHECK(y2->is_cuda() && y2->scalar_type() == y1.scalar_type() &&
                y2->sizes() == resid.sizes() && y2->is_contiguous());
    y2p = y2->data_ptr();
  }
  TORCH_CHECK(w_next.has_value() == out.has_value());
  const float* wn = nullptr;
  void* op = nullptr;
  if (w_next.has_value()) {
    CHECK_F32(*w_next);
    TORCH_CHECK(w_next->numel() == W);
    TORCH_CHECK(out->is_cuda() && out->scalar_type() == y1.scalar_type() &&
                out->sizes() == resid.sizes() && out->is_contiguous());
    wn = w_next->data_ptr<float>();
    op = out->data_ptr();
  }
  DISPATCH_ACT(y1, fi::launch_gated_residual_layer_norm<A>(
                       resid.data_ptr<float>(), ptr<A>(y1), (float)s1,
                       reinterpret_cast<const A*>(y2p), (float)s2,
                       ptr<A>(gate_lin), gate_lin.stride(0),
                       gate_bias.data_ptr<float>(), wn,
                       reinterpret_cast<A*>(op), (float)eps, (int)T, (int)W,
                       stream()));
}

void group_rms_gate(at::Tensor out, at::Tensor o_raw, at::Tensor glin,
                    at::Tensor w, int64_t groups, double eps, bool silu) {
  CHECK_ACT(out);
  CHECK_F32(o_raw);
  CHECK_ACT(glin);
  CHECK_F32(w);
  TORCH_CHECK(o_raw.dim() == 2 && groups >= 1);
  const int64_t T = o_raw.size(0), N = o_raw.size(1);
  TORCH_CHECK(N % groups == 0);
  const int64_t part = N / groups;
  TORCH_CHECK(out.sizes() == o_raw.sizes() && out.is_contiguous() &&
              out.scalar_type() == glin.scalar_type());
  check_rows(glin, T, N, "gate projection");
  TORCH_CHECK(w.numel() == N || w.numel() == part,
              "gain: one per coordinate or one per position in a group");
  DISPATCH_ACT(out, fi::launch_group_rms_gate<A>(
                        ptr<A>(out), o_raw.data_ptr<float>(), ptr<A>(glin),
                        glin.stride(0), w.data_ptr<float>(),
                        w.numel() != N, (int)T, (int)groups, (int)part,
                        (float)eps, silu, stream()));
}

void paged_cache_write(at::Tensor k, at::Tensor v, at::Tensor k_cache,
                       at::Tensor v_cache, at::Tensor slot_mapping) {
  CHECK_ACT(k);
  CHECK_I32(slot_mapping);
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  TORCH_CHECK(k_cache.scalar_type() == k.scalar_type() &&
              v_cache.scalar_type() == k.scalar_type() &&
              v.scalar_type() == k.scalar_type() && v.is_cuda());
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(0) == v_cache.size(0) &&
              k_cache.size(1) == v_cache.size(1) &&
              k_cache.size(2) == v_cache.size(2));
  const int64_t T = k.size(0);
  const int G = k_cache.size(1), bs = k_cache.size(2), D = k_cache.size(3),
            V = v_cache.size(3);
  check_rows(k, T, static_cast<int64_t>(G) * D, "keys");
  check_rows(v, T, static_cast<int64_t>(G) * V, "values");
  TORCH_CHECK(slot_mapping.numel() == T);
  DISPATCH_ACT(k, fi::launch_paged_cache_write<A>(
                      ptr<A>(k_cache), ptr<A>(v_cache), ptr<A>(k), k.stride(0),
                      ptr<A>(v), v.stride(0), slot_mapping.data_ptr<int>(),
                      (int)T, G, bs, D, V, stream()));
}

void check_recurrence_scratch(const at::Tensor& vecs, const at::Tensor& vbuf,
                              const at::Tensor& o_raw, int64_t T,
                              int64_t heads, int64_t dim, int64_t vdim) {
  CHECK_F32(vecs);
  CHECK_F32(vbuf);
  CHECK_F32(o_raw);
  TORCH_CHECK(dim >= 1 && dim <= 256, "recurrence: key size must be <= 256");
  const int64_t cap = dim <= 64 ? 64 : (dim <= 128 ? 128 : 256);
  TORCH_CHECK(vecs.numel() == T * heads * 5 * cap,
              "recurrence scratch must hold [T, heads, 5, ", cap, "]");
  TORCH_CHECK(vbuf.numel() == T * heads * vdim &&
              o_raw.numel() == T * heads * vdim);
}

void decay_linear_attention(at::Tensor o_raw, at::Tensor vecs, at::Tensor vbuf,
                            at::Tensor q, at::Tensor k, at::Tensor v,
                            at::Tensor decay, at::Tensor state,
                            at::Tensor seq_cu, at::Tensor seq_slots,
                            at::Tensor positions, int64_t heads, int64_t dim,
                            int64_t vdim, bool silu,
                            c10::optional<at::Tensor> row_seq) {
  CHECK_ACT(q);
  const int64_t T = q.size(0);
  TORCH_CHECK(k.is_cuda() && v.is_cuda() &&
              k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type());
  check_rows(q, T, heads * dim, "queries");
  check_rows(k, T, heads * dim, "keys");
  check_rows(v, T, heads * vdim, "values");
  check_recurrence_scratch(vecs, vbuf, o_raw, T, heads, dim, vdim);
  CHECK_F32(decay);
  CHECK_F32(state);
  TORCH_CHECK(decay.numel() == heads);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads &&
              state.size(2) == dim && state.size(3) == vdim);
  check_groups(seq_cu, seq_slots, positions, T);
  const int S = seq_slots.numel();
  const int* rs = nullptr;
  if (row_seq.has_value()) {
    CHECK_I32(*row_seq);
    TORCH_CHECK(row_seq->numel() == T);
    rs = row_seq->data_ptr<int>();
  }
  DISPATCH_ACT(q, fi::launch_decay_linear_attention<A>(
                      o_raw.data_ptr<float>(), vecs.data_ptr<float>(),
                      vbuf.data_ptr<float>(), ptr<A>(q), ptr<A>(k), ptr<A>(v),
                      q.stride(0), k.stride(0), v.stride(0),
                      decay.data_ptr<float>(), state.data_ptr<float>(),
                      seq_cu.data_ptr<int>(), seq_slots.data_ptr<int>(),
                      positions.data_ptr<int>(), rs, (int)T, S, (int)heads,
                      (int)dim, (int)vdim, silu, stream()));
}

void gated_delta_rule(at::Tensor o_raw, at::Tensor vecs, at::Tensor vbuf,
                      at::Tensor x, at::Tensor conv_w, at::Tensor alin,
                      at::Tensor blin, at::Tensor a_log, at::Tensor dt_bias,
                      at::Tensor conv_state, at::Tensor state,
                      at::Tensor seq_cu, at::Tensor seq_slots,
                      at::Tensor positions, at::Tensor row_seq, int64_t heads,
                      int64_t kv_heads, int64_t dim, int64_t vdim) {
  CHECK_ACT(x);
  const int64_t T = x.size(0);
  const int64_t C = 2 * kv_heads * dim + heads * vdim;
  TORCH_CHECK(kv_heads >= 1 && heads % kv_heads == 0);
  check_rows(x, T, C, "q|k|v projections");
  TORCH_CHECK(alin.is_cuda() && blin.is_cuda() &&
              alin.scalar_type() == x.scalar_type() &&
              blin.scalar_type() == x.scalar_type());
  check_rows(alin, T, heads, "decay input");
  check_rows(blin, T, heads, "write strength input");
  check_recurrence_scratch(vecs, vbuf, o_raw, T, heads, dim, vdim);
  CHECK_F32(conv_w);
  CHECK_F32(a_log);
  CHECK_F32(dt_bias);
  CHECK_F32(conv_state);
  CHECK_F32(state);
  CHECK_I32(row_seq);
  TORCH_CHECK(conv_w.dim() == 2 && conv_w.size(0) == C && conv_w.size(1) >= 1);
  const int taps = conv_w.size(1);
  TORCH_CHECK(a_log.numel() == heads && dt_bias.numel() == heads);
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(2) == C &&
              conv_state.size(1) >= taps - 1 &&
              (taps == 1 || conv_state.size(1) == taps - 1));
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads &&
              state.size(2) == dim && state.size(3) == vdim &&
              state.size(0) == conv_state.size(0));
  check_groups(seq_cu, seq_slots, positions, T);
  TORCH_CHECK(row_seq.numel() == T);
  const int S = seq_slots.numel();
  DISPATCH_ACT(x, fi::launch_gated_delta_rule<A>(
                      o_raw.data_ptr<float>(), vecs.data_ptr<float>(),
                      vbuf.data_ptr<float>(), ptr<A>(x), x.stride(0),
                      conv_w.data_ptr<float>(), ptr<A>(alin), alin.stride(0),
                      ptr<A>(blin), blin.stride(0), a_log.data_ptr<float>(),
                      dt_bias.data_ptr<float>(), conv_state.data_ptr<float>(),
                      state.data_ptr<float>(), seq_cu.data_ptr<int>(),
                      seq_slots.data_ptr<int>(), positions.data_ptr<int>(),
                      row_seq.data_ptr<int>(), (int)T, S, (int)heads,
                      (int)kv_heads, (int)dim, (int)vdim, taps, stream()));
}

void talking_window_attention(at::Tensor out, at::Tensor q, at::Tensor k_cache,
                              at::Tensor v_cache, at::Tensor seq_bt,
                              at::Tensor row_seq, at::Tensor positions,
                              double scale, int64_t window, at::Tensor r1,
                              at::Tensor r2, at::Tensor talk, int64_t heads,
                              c10::optional<at::Tensor> seq_cu,
                              c10::optional<at::Tensor> tile_seq,
                              c10::optional<at::Tensor> tile_row0,
                              int64_t tile_rows,
                              c10::optional<at::Tensor> folded_q,
                              c10::optional<at::Tensor> penalty,
                              c10::optional<at::Tensor> part_ml,
                              c10::optional<at::Tensor> part_o) {
  CHECK_ACT(q);
  CHECK_I32(seq_bt);
  CHECK_I32(row_seq);
  CHECK_I32(positions);
  CHECK_F32(r1);
  CHECK_F32(r2);
  CHECK_F32(talk);
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() &&
              k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type());
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(0) == v_cache.size(0) &&
              k_cache.size(1) == v_cache.size(1) &&
              k_cache.size(2) == v_cache.size(2));
  const int64_t T = q.size(0);
  const int H = heads, G = k_cache.size(1), bs = k_cache.size(2),
            D = k_cache.size(3), V = v_cache.size(3);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0);
  check_rows(q, T, static_cast<int64_t>(H) * D, "queries");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() &&
              out.scalar_type() == q.scalar_type() &&
              out.numel() == T * H * V);
  TORCH_CHECK(r1.numel() == H && r2.numel() == H && talk.numel() == H * H);
  TORCH_CHECK(seq_bt.dim() == 2 && row_seq.numel() == T &&
              positions.numel() == T);
  TORCH_CHECK(static_cast<int64_t>(H) * V <= 8192,
              "windowed attention: heads * vdim must be <= 8192");
  TORCH_CHECK(fi::talking_window_row_smem(H, D) <= 64 * 1024,
              "windowed attention: heads * dim too large for one workgroup");
  // the leading tile_rows rows (prompt portions) take the tiled kernel
  // where the head sizes have a variant; all other rows the row kernel
  int64_t done = 0;
  TORCH_CHECK(tile_rows >= 0 && tile_rows <= T);
  if (tile_rows > 0) {
    TORCH_CHECK(seq_cu.has_value() && tile_seq.has_value() &&
                tile_row0.has_value() && folded_q.has_value() &&
                penalty.has_value());
    CHECK_I32(*seq_cu);
    CHECK_I32(*tile_seq);
    CHECK_I32(*tile_row0);
    CHECK_F32(*penalty);
    TORCH_CHECK(tile_seq->numel() == tile_row0->numel());
    TORCH_CHECK(seq_cu->numel() >= 2);
    TORCH_CHECK(folded_q->is_cuda() && folded_q->is_contiguous() &&
                folded_q->scalar_type() == q.scalar_type() &&
                folded_q->numel() == tile_rows * H * G * D);
    TORCH_CHECK(penalty->dim() == 2 && penalty->size(0) == H);
    const int64_t maxd = penalty->size(1);
    // every distance a row can ask for has an entry
    TORCH_CHECK(window > 0 ? maxd >= window
                           : maxd >= seq_bt.size(1) * bs,
                "penalty table too short");
    bool ok = false;
    DISPATCH_ACT(q, ok = fi::launch_talking_window_tiles<A>(
                        ptr<A>(out), ptr<A>(*folded_q),
                        penalty->data_ptr<float>(), (int)maxd, ptr<A>(q),
                        q.stride(0), ptr<A>(k_cache), ptr<A>(v_cache),
                        seq_bt.data_ptr<int>(), (int)seq_bt.size(1),
                        seq_cu->data_ptr<int>(), positions.data_ptr<int>(),
                        r1.data_ptr<float>(), r2.data_ptr<float>(),
                        talk.data_ptr<float>(), tile_seq->data_ptr<int>(),
                        tile_row0->data_ptr<int>(), (int)tile_seq->numel(),
                        (int)tile_rows, H, G, D, V, bs, (float)scale,
                        (int)window, stream()));
    if (ok) done = tile_rows;
  }
  // remaining rows: partial results per 256-key pass when the
  // thread-per-key kernel fits and scratch was handed in
  float* pml = nullptr;
  float* pob = nullptr;
  int nsplit = 1;
  const int64_t rest = T - done;
  if (rest > 0 && part_ml.has_value() && part_o.has_value() &&
      fi::talking_window_fast_fits(H, G, D, V)) {
    CHECK_F32(*part_ml);
    CHECK_F32(*part_o);
    const int64_t max_keys = window > 0 ? window : seq_bt.size(1) * bs;
    nsplit = fi::talking_window_fast_splits((int)max_keys);
    // scratch sized for the decoded rows only: when prompt rows come here
    // too (no tiled variant for these head sizes) all rows take the
    // one-workgroup-per-row kernel
    if (part_ml->numel() >= rest * nsplit * 2 * H &&
        part_o->numel() >= rest * nsplit * H * V) {
      pml = part_ml->data_ptr<float>();
      pob = part_o->data_ptr<float>();
    }
  }
  DISPATCH_ACT(q, fi::launch_talking_window_rows<A>(
                      ptr<A>(out), ptr<A>(q), q.stride(0), ptr<A>(k_cache),
                      ptr<A>(v_cache), seq_bt.data_ptr<int>(),
                      (int)seq_bt.size(1), row_seq.data_ptr<int>(),
                      positions.data_ptr<int>(), r1.data_ptr<float>(),
                      r2.data_ptr<float>(), talk.data_ptr<float>(), (int)done,
                      (int)rest, H, G, D, V, bs, (float)scale, (int)window,
                      pml, pob, nsplit, stream()));
}

}  // namespace

// ------------------------------------------------------------------------
// parallel-residual stream, weighted head norms with a query temperature,
// latent keys/values with a softmax sink, gated linear recurrence

void scaled_residual_layer_norm(at::Tensor resid, at::Tensor y1, double s1,
                                c10::optional<at::Tensor> y2, double s2,
                                c10::optional<at::Tensor> y3, double s3,
                                c10::optional<at::Tensor> w_next,
                                c10::optional<at::Tensor> out, double eps) {
  CHECK_F32(resid);
  CHECK_ACT(y1);
  TORCH_CHECK(resid.dim() == 2);
  const int64_t T = resid.size(0), W = resid.size(1);
  TORCH_CHECK(y1.sizes() == resid.sizes() && y1.is_contiguous());
  auto opt = [&](const c10::optional<at::Tensor>& y) -> void* {
    if (!y.has_value()) return nullptr;
    TORCH_CHECK(y->is_cuda() && y->scalar_type() == y1.scalar_type() &&
                y->sizes() == resid.sizes() && y->is_contiguous());
    return y->data_ptr();
  };
  void* y2p = opt(y2);
  void* y3p = opt(y3);
  TORCH_CHECK(w_next.has_value() == out.has_value());
  const float* wn = nullptr;
  void* op = nullptr;
  if (w_next.has_value()) {
    CHECK_F32(*w_next);
    TORCH_CHECK(w_next->numel() == W);
    TORCH_CHECK(out->is_cuda() && out->scalar_type() == y1.scalar_type() &&
                out->sizes() == resid.sizes() && out->is_contiguous());
    wn = w_next->data_ptr<float>();
    op = out->data_ptr();
  }
  DISPATCH_ACT(y1, fi::launch_scaled_residual_layer_norm<A>(
                       resid.data_ptr<float>(), ptr<A>(y1), (float)s1,
                       reinterpret_cast<const A*>(y2p), (float)s2,
                       reinterpret_cast<const A*>(y3p), (float)s3, wn,
                       reinterpret_cast<A*>(op), (float)eps, (int)T, (int)W,
                       stream()));
}

void headnorm_qtemp_cache(at::Tensor q_out, at::Tensor q, at::Tensor k,
                          at::Tensor v, at::Tensor positions, at::Tensor q_w,
                          at::Tensor k_w, double eps, double coef,
                          int64_t every, at::Tensor k_cache,
                          at::Tensor v_cache, at::Tensor slot_mapping,
                          int64_t H, int64_t G, int64_t D, int64_t V) {
  CHECK_ACT(q);
  CHECK_ACT(k);
  CHECK_ACT(v);
  CHECK_ACT(q_out);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  CHECK_F32(q_w);
  CHECK_F32(k_w);
  const int64_t T = q.size(0);
  check_rows(q, T, H * D, "q");
  check_rows(k, T, G * D, "k");
  check_rows(v, T, G * V, "v");
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt &&
              q_out.scalar_type() == dt);
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() == T * H * D);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  TORCH_CHECK(q_w.numel() == D && k_w.numel() == D);
  TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() &&
              k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.scalar_type() == dt && v_cache.scalar_type() == dt);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(0) == v_cache.size(0) && k_cache.size(1) == G &&
              v_cache.size(1) == G && k_cache.size(2) == v_cache.size(2) &&
              k_cache.size(3) == D && v_cache.size(3) == V);
  TORCH_CHECK(D >= 1 && D <= 512 && V >= 1, "head size out of range");
  DISPATCH_ACT(q, fi::launch_headnorm_qtemp_cache<A>(
                      ptr<A>(q_out), ptr<A>(q), q.stride(0), ptr<A>(k),
                      k.stride(0), ptr<A>(v), v.stride(0),
                      positions.data_ptr<int>(), q_w.data_ptr<float>(),
                      k_w.data_ptr<float>(), (float)eps, (float)coef,
                      (int)every, ptr<A>(k_cache), ptr<A>(v_cache),
                      slot_mapping.data_ptr<int>(), (int)T, (int)H, (int)G,
                      (int)D, (int)V, (int)k_cache.size(2), stream()));
}

void latent_rope_cache(at::Tensor q_out, at::Tensor q, at::Tensor ckr,
                       at::Tensor positions, at::Tensor inv_freq,
                       at::Tensor norm_w, double eps, at::Tensor kv_cache,
                       at::Tensor slot_mapping, int64_t H, int64_t D,
                       int64_t R, int64_t C) {
  CHECK_ACT(q);
  CHECK_ACT(ckr);
  CHECK_ACT(q_out);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  CHECK_F32(inv_freq);
  CHECK_F32(norm_w);
  const int64_t T = q.size(0);
  check_rows(q, T, H * (D + R), "q");
  check_rows(ckr, T, C + R, "latent projection");
  const auto dt = q.scalar_type();
  TORCH_CHECK(ckr.scalar_type() == dt && q_out.scalar_type() == dt);
  TORCH_CHECK(q_out.is_contiguous() && q_out.dim() == 3 &&
              q_out.size(0) == T && q_out.size(1) == H &&
              q_out.size(2) == C + R);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  TORCH_CHECK(R % 2 == 0 && inv_freq.numel() <= R / 2 && norm_w.numel() == C);
  TORCH_CHECK(kv_cache.is_cuda() && kv_cache.is_contiguous() &&
              kv_cache.scalar_type() == dt && kv_cache.dim() == 4 &&
              kv_cache.size(1) == 1 && kv_cache.size(3) == C + R);
  DISPATCH_ACT(q, fi::launch_latent_rope_cache<A>(
                      ptr<A>(q_out), ptr<A>(q), q.stride(0), ptr<A>(ckr),
                      ckr.stride(0), positions.data_ptr<int>(),
                      inv_freq.data_ptr<float>(), norm_w.data_ptr<float>(),
                      (float)eps, ptr<A>(kv_cache),
                      slot_mapping.data_ptr<int>(), (int)T, (int)H, (int)D,
                      (int)R, (int)C, (int)inv_freq.numel(),
                      (int)kv_cache.size(2), stream()));
}

int64_t sink_attention_splits(int64_t max_keys) {
  return fi::sink_attention_splits((int)max_keys);
}

bool sink_attention_has_tiles(int64_t DK, int64_t DV) {
  return fi::sink_attention_has_tiles((int)DK, (int)DV);
}

// Rows [0, tile_rows) belong to the row groups that the tile tables cover
// and run the MFMA kernel when the sizes have one; all other rows run the
// split form, part_ml.size(0) rows per launch.
void sink_paged_attention(at::Tensor out, at::Tensor q, at::Tensor k_cache,
                          c10::optional<at::Tensor> v_cache,
                          at::Tensor seq_bt, at::Tensor row_seq,
                          at::Tensor positions, double scale,
                          c10::optional<at::Tensor> sink, int64_t DV,
                          c10::optional<at::Tensor> gate,
                          c10::optional<at::Tensor> seq_cu,
                          c10::optional<at::Tensor> tile_seq,
                          c10::optional<at::Tensor> tile_row0,
                          int64_t tile_rows,
                          c10::optional<at::Tensor> part_ml,
                          c10::optional<at::Tensor> part_o, int64_t window,
                          int64_t keep_first) {
  CHECK_ACT(q);
  CHECK_ACT(out);
  TORCH_CHECK(window >= 0 && keep_first >= 0);
  CHECK_I32(row_seq);
  CHECK_I32(positions);
  TORCH_CHECK(seq_bt.is_cuda() && seq_bt.scalar_type() == at::kInt &&
              seq_bt.dim() == 2 && seq_bt.stride(1) == 1);
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && out.is_contiguous() &&
              out.scalar_type() == q.scalar_type());
  const int T = q.size(0), H = q.size(1), DK = q.size(2);
  const auto dt = q.scalar_type();
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() &&
              k_cache.scalar_type() == dt && k_cache.dim() == 4 &&
              k_cache.size(3) == DK);
  const int G = k_cache.size(1), bs = k_cache.size(2);
  const void* vp = k_cache.data_ptr();
  int v_row = DK;
  if (v_cache.has_value()) {
    TORCH_CHECK(v_cache->is_cuda() && v_cache->is_contiguous() &&
                v_cache->scalar_type() == dt && v_cache->dim() == 4 &&
                v_cache->size(0) == k_cache.size(0) &&
                v_cache->size(1) == G && v_cache->size(2) == bs &&
                v_cache->size(3) == DV);
    vp = v_cache->data_ptr();
    v_row = DV;
  } else {
    TORCH_CHECK(DV >= 1 && DV <= DK, "value slice exceeds the key row");
  }
  TORCH_CHECK(out.dim() == 3 && out.size(0) == T && out.size(1) == H &&
              out.size(2) == DV);
  TORCH_CHECK(G >= 1 && H % G == 0 && DK >= 1 && DK <= 1024 && DV >= 1);
  TORCH_CHECK(row_seq.numel() == T && positions.numel() == T);
  const float* sp = nullptr;
  if (sink.has_value()) {
    CHECK_F32(*sink);
    TORCH_CHECK(sink->numel() == H);
    sp = sink->data_ptr<float>();
  }
  const void* gp = nullptr;
  int64_t g_stride = 0;
  int gate_elem = 0;   // 1: one gate per entry [T, H*DV], 0: per head [T, H]
  if (gate.has_value()) {
    TORCH_CHECK(gate->is_cuda() && gate->scalar_type() == dt);
    gate_elem = gate->dim() == 2 && gate->size(1) == H * DV && DV > 1;
    check_rows(*gate, T, gate_elem ? H * DV : H, "output gate");
    gp = gate->data_ptr();
    g_stride = gate->stride(0);
  }
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
    bool ok = false;
    DISPATCH_ACT(q, ok = fi::launch_sink_attention_tiles<A>(
                      ptr<A>(out), ptr<A>(q), ptr<A>(k_cache),
                      reinterpret_cast<const A*>(vp), v_row,
                      seq_bt.data_ptr<int>(), (int)seq_bt.stride(0),
                      seq_cu->data_ptr<int>(), positions.data_ptr<int>(),
                      tile_seq->data_ptr<int>(), tile_row0->data_ptr<int>(),
                      (int)tile_seq->numel(), sp,
                      reinterpret_cast<const A*>(gp), g_stride, gate_elem, H,
                      G, DK, (int)DV, bs, (float)scale, (int)window,
                      (int)keep_first, stream()));
    if (ok) done = tile_rows;
  }
  if (done == T) return;
  TORCH_CHECK(part_ml.has_value() && part_o.has_value(),
              "rows outside the tiled form need the span buffers");
  CHECK_F32(*part_ml);
  CHECK_F32(*part_o);
  const int ns = fi::sink_attention_splits((int)seq_bt.size(1) * bs);
  TORCH_CHECK(part_ml->dim() == 4 && part_o->dim() == 4 &&
              part_ml->size(0) >= 1 && part_o->size(0) == part_ml->size(0) &&
              part_ml->size(1) == H && part_ml->size(2) == ns &&
              part_ml->size(3) == 2 && part_o->size(1) == H &&
              part_o->size(2) == ns && part_o->size(3) == DV);
  const int cap = part_ml->size(0);
  for (int row0 = (int)done; row0 < T; row0 += cap) {
    const int rows = std::min(cap, T - row0);
    DISPATCH_ACT(q, fi::launch_sink_attention_rows<A>(
                        ptr<A>(out), part_ml->data_ptr<float>(),
                        part_o->data_ptr<float>(), ptr<A>(q), ptr<A>(k_cache),
                        reinterpret_cast<const A*>(vp), v_row,
                        seq_bt.data_ptr<int>(), (int)seq_bt.stride(0),
                        row_seq.data_ptr<int>(), positions.data_ptr<int>(),
                        sp, reinterpret_cast<const A*>(gp), g_stride,
                        gate_elem, row0, rows, H, G, DK, (int)DV, bs,
                        (float)scale, ns, (int)window, (int)keep_first,
                        stream()));
  }
}

void causal_conv_state(at::Tensor out, at::Tensor x, at::Tensor conv_w,
                       at::Tensor conv_b, at::Tensor conv_state,
                       at::Tensor seq_cu, at::Tensor row_seq,
                       at::Tensor seq_slots, at::Tensor positions) {
  CHECK_F32(out);
  CHECK_ACT(x);
  CHECK_F32(conv_w);
  CHECK_F32(conv_b);
  CHECK_F32(conv_state);
  CHECK_I32(seq_cu);
  CHECK_I32(row_seq);
  CHECK_I32(positions);
  const int64_t T = x.size(0), C = x.size(1);
  check_rows(x, T, C, "convolution input");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == C);
  TORCH_CHECK(conv_w.dim() == 2 && conv_w.size(0) == C && conv_b.numel() == C);
  const int taps = conv_w.size(1);
  TORCH_CHECK(taps >= 1 && taps <= 64);
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(2) == C &&
              conv_state.size(1) >= std::max(taps - 1, 1));
  check_groups(seq_cu, seq_slots, positions, T);
  TORCH_CHECK(row_seq.numel() == T && positions.numel() == T);
  const int S = seq_slots.numel();
  DISPATCH_ACT(x, fi::launch_causal_conv_state<A>(
                      out.data_ptr<float>(), ptr<A>(x), x.stride(0),
                      conv_w.data_ptr<float>(), conv_b.data_ptr<float>(),
                      conv_state.data_ptr<float>(), seq_cu.data_ptr<int>(),
                      row_seq.data_ptr<int>(), seq_slots.data_ptr<int>(),
                      positions.data_ptr<int>(), (int)T, S, (int)C, taps,
                      (int)conv_state.size(1), stream()));
}

void rglru_scan(at::Tensor out, at::Tensor u, at::Tensor gate_lin,
                at::Tensor gate_bias, at::Tensor lam, at::Tensor y_lin,
                at::Tensor state, at::Tensor seq_cu, at::Tensor seq_slots,
                at::Tensor positions, double decay_scale, int64_t max_rows) {
  CHECK_ACT(out);
  CHECK_F32(u);
  CHECK_F32(gate_lin);
  CHECK_F32(gate_bias);
  CHECK_F32(lam);
  CHECK_ACT(y_lin);
  CHECK_F32(state);
  CHECK_I32(positions);
  const int64_t T = u.size(0), W = u.size(1);
  TORCH_CHECK(u.dim() == 2 && out.is_contiguous() && out.dim() == 2 &&
              out.size(0) == T && out.size(1) == W &&
              out.scalar_type() == y_lin.scalar_type());
  check_rows(y_lin, T, W, "gelu branch");
  TORCH_CHECK(gate_lin.dim() == 3 && gate_lin.size(1) == T);
  const int64_t B = gate_lin.size(0);
  TORCH_CHECK(B >= 1 && W % B == 0 && gate_lin.size(2) == 2 * (W / B));
  TORCH_CHECK(gate_bias.numel() == 2 * W && lam.numel() == W);
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W);
  check_groups(seq_cu, seq_slots, positions, T);
  TORCH_CHECK(positions.numel() == T);
  TORCH_CHECK(max_rows >= 0);
  const int S = seq_slots.numel();
  DISPATCH_ACT(y_lin, fi::launch_rglru_scan<A>(
                          ptr<A>(out), u.data_ptr<float>(),
                          gate_lin.data_ptr<float>(),
                          gate_bias.data_ptr<float>(), lam.data_ptr<float>(),
                          ptr<A>(y_lin), y_lin.stride(0),
                          state.data_ptr<float>(), seq_cu.data_ptr<int>(),
                          seq_slots.data_ptr<int>(),
                          positions.data_ptr<int>(), (int)T, S, (int)W,
                          (int)(W / B), (float)decay_scale, (int)max_rows,
                          stream()));
}

void cast_layer_norm(at::Tensor resid, c10::optional<at::Tensor> out,
                     at::Tensor y, c10::optional<at::Tensor> w, double eps) {
  CHECK_F32(resid);
  CHECK_ACT(y);
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() &&
              resid.sizes() == y.sizes());
  TORCH_CHECK(out.has_value() == w.has_value());
  const float* wp = nullptr;
  void* op = nullptr;
  if (w.has_value()) {
    CHECK_F32(*w);
    TORCH_CHECK(w->numel() == y.size(1));
    TORCH_CHECK(out->is_cuda() && out->scalar_type() == y.scalar_type() &&
                out->sizes() == y.sizes() && out->is_contiguous());
    wp = w->data_ptr<float>();
    op = out->data_ptr();
  }
  DISPATCH_ACT(y, fi::launch_cast_layer_norm<A>(
                      resid.data_ptr<float>(), reinterpret_cast<A*>(op),
                      ptr<A>(y), wp, (float)eps, (int)y.size(0),
                      (int)y.size(1), stream()));
}

void concat_cast(at::Tensor out, at::Tensor resid, at::Tensor x0) {
  CHECK_F32(resid);
  CHECK_ACT(x0);
  CHECK_ACT(out);
  TORCH_CHECK(resid.dim() == 2 && x0.is_contiguous() &&
              x0.sizes() == resid.sizes() && out.is_contiguous() &&
              out.scalar_type() == x0.scalar_type() && out.dim() == 2 &&
              out.size(0) == resid.size(0) &&
              out.size(1) == 2 * resid.size(1));
  DISPATCH_ACT(x0, fi::launch_concat_cast<A>(
                       ptr<A>(out), resid.data_ptr<float>(), ptr<A>(x0),
                       (int)resid.size(0), (int)resid.size(1), stream()));
}

void relu_squared(at::Tensor out, at::Tensor x) {
  CHECK_ACT(x);
  CHECK_ACT(out);
  TORCH_CHECK(x.dim() == 2 && out.is_contiguous() &&
              out.sizes() == x.sizes() &&
              out.scalar_type() == x.scalar_type());
  check_rows(x, x.size(0), x.size(1), "relu input");
  DISPATCH_ACT(x, fi::launch_relu_squared<A>(ptr<A>(out), ptr<A>(x),
                                             x.stride(0), (int)x.size(0),
                                             (int)x.size(1), stream()));
}

void pair_embed(at::Tensor resid, at::Tensor act, at::Tensor ids,
                at::Tensor embed, double scale,
                c10::optional<at::Tensor> pair_table, int64_t buckets,
                int64_t mul_prev, int64_t mul_cur, at::Tensor prev_token,
                at::Tensor seq_cu, at::Tensor row_seq, at::Tensor seq_slots,
                at::Tensor positions) {
  CHECK_F32(resid);
  CHECK_ACT(embed);
  CHECK_I32(prev_token);
  CHECK_I32(seq_cu);
  CHECK_I32(row_seq);
  CHECK_I32(seq_slots);
  CHECK_I32(positions);
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kLong &&
              ids.is_contiguous());
  const int64_t T = ids.numel();
  TORCH_CHECK(embed.dim() == 2 && embed.is_contiguous());
  const int64_t W = embed.size(1);
  const auto dt = embed.scalar_type();
  TORCH_CHECK(resid.is_contiguous() && resid.numel() == T * W);
  TORCH_CHECK(act.is_cuda() && act.is_contiguous() &&
              act.scalar_type() == dt && act.numel() == T * W);
  TORCH_CHECK(row_seq.numel() == T && positions.numel() == T);
  TORCH_CHECK(seq_cu.numel() >= 1 && seq_slots.numel() >= seq_cu.numel() - 1);
  TORCH_CHECK(buckets >= 1);
  const void* pt = nullptr;
  if (pair_table.has_value()) {
    TORCH_CHECK(pair_table->is_cuda() && pair_table->is_contiguous() &&
                pair_table->scalar_type() == dt && pair_table->dim() == 2 &&
                pair_table->size(0) == buckets + 1 &&
                pair_table->size(1) == W);
    pt = pair_table->data_ptr();
  }
  DISPATCH_ACT(embed, fi::launch_pair_embed<A>(
                          resid.data_ptr<float>(), ptr<A>(act),
                          ids.data_ptr<int64_t>(), ptr<A>(embed), (float)scale,
                          reinterpret_cast<const A*>(pt), buckets, mul_prev,
                          mul_cur, prev_token.data_ptr<int>(),
                          seq_cu.data_ptr<int>(), row_seq.data_ptr<int>(),
                          seq_slots.data_ptr<int>(), positions.data_ptr<int>(),
                          (int)T, (int)W, stream()));
}

void layer_norm_affine(at::Tensor out, at::Tensor x, at::Tensor w,
                       at::Tensor b, double eps) {
  CHECK_F32(x);
  CHECK_ACT(out);
  CHECK_F32(w);
  CHECK_F32(b);
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && out.is_contiguous() &&
              out.sizes() == x.sizes());
  const int T = x.size(0), W = x.size(1);
  TORCH_CHECK(w.numel() == W && b.numel() == W);
  if (out.scalar_type() == at::kFloat)
    fi::launch_norm_affine<float, float>(
        x.data_ptr<float>(), nullptr, out.data_ptr<float>(),
        w.data_ptr<float>(), b.data_ptr<float>(), (float)eps, T, W, stream());
  else
    fi::launch_norm_affine<float, fi::u16>(
        x.data_ptr<float>(), nullptr, ptr<fi::u16>(out), w.data_ptr<float>(),
        b.data_ptr<float>(), (float)eps, T, W, stream());
}

// resid += layer_norm(y) * w + b; out (activation dtype) = rounded resid.
// For fp32 activations out is resid itself.
void post_norm_residual(at::Tensor resid, at::Tensor y, at::Tensor w,
                        at::Tensor b, at::Tensor out, double eps) {
  CHECK_F32(resid);
  CHECK_ACT(y);
  CHECK_F32(w);
  CHECK_F32(b);
  TORCH_CHECK(resid.dim() == 2 && resid.is_contiguous() &&
              y.is_contiguous() && y.sizes() == resid.sizes());
  const int T = resid.size(0), W = resid.size(1);
  TORCH_CHECK(w.numel() == W && b.numel() == W);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() &&
              out.scalar_type() == y.scalar_type() &&
              out.sizes() == resid.sizes());
  if (y.scalar_type() == at::kFloat) {
    TORCH_CHECK(out.data_ptr() == resid.data_ptr(),
                "fp32 activations read the stream itself");
    fi::launch_norm_affine<float, float>(
        y.data_ptr<float>(), resid.data_ptr<float>(), nullptr,
        w.data_ptr<float>(), b.data_ptr<float>(), (float)eps, T, W, stream());
  } else {
    fi::launch_norm_affine<fi::u16, fi::u16>(
        ptr<fi::u16>(y), resid.data_ptr<float>(), ptr<fi::u16>(out),
        w.data_ptr<float>(), b.data_ptr<float>(), (float)eps, T, W, stream());
  }
}

void widenorm_rope_cache(at::Tensor q_out, at::Tensor q,
                         c10::optional<at::Tensor> k,
                         c10::optional<at::Tensor> v, at::Tensor positions,
                         at::Tensor q_w, c10::optional<at::Tensor> k_w,
                         double eps, at::Tensor inv_freq, double rot_mult,
                         at::Tensor k_cache, at::Tensor v_cache,
                         at::Tensor slot_mapping, int64_t H, int64_t G,
                         int64_t D, int64_t V) {
  CHECK_ACT(q);
  CHECK_ACT(q_out);
  CHECK_I32(positions);
  CHECK_I32(slot_mapping);
  CHECK_F32(q_w);
  CHECK_F32(inv_freq);
  const int64_t T = q.size(0);
  check_rows(q, T, H * D, "q");
  const auto dt = q.scalar_type();
  TORCH_CHECK(q_out.scalar_type() == dt && q_out.is_contiguous() &&
              q_out.numel() == T * H * D);
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  TORCH_CHECK(q_w.numel() == H * D);
  const int nrot = 2 * (int)inv_freq.numel();
  TORCH_CHECK(nrot <= D, "more turning pairs than the head holds");
  TORCH_CHECK(H >= 1 && G >= 1 && D >= 1 && V >= 1);
  const void *kp = nullptr, *vp = nullptr;
  const float* kw = nullptr;
  int64_t ks = 0, vs = 0;
  void *kc = nullptr, *vc = nullptr;
  int bs = 1;
  if (k.has_value()) {
    TORCH_CHECK(v.has_value() && k_w.has_value());
    CHECK_ACT(*k);
    CHECK_ACT(*v);
    CHECK_F32(*k_w);
    check_rows(*k, T, G * D, "k");
    check_rows(*v, T, G * V, "v");
    TORCH_CHECK(k->scalar_type() == dt && v->scalar_type() == dt);
    TORCH_CHECK(k_w->numel() == G * D);
    TORCH_CHECK(k_cache.is_cuda() && v_cache.is_cuda() &&
                k_cache.is_contiguous() && v_cache.is_contiguous() &&
                k_cache.scalar_type() == dt && v_cache.scalar_type() == dt);
    TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
                k_cache.size(0) == v_cache.size(0) && k_cache.size(1) == G &&
                v_cache.size(1) == G && k_cache.size(2) == v_cache.size(2) &&
                k_cache.size(3) == D && v_cache.size(3) == V);
    kp = k->data_ptr();
    vp = v->data_ptr();
    kw = k_w->data_ptr<float>();
    ks = k->stride(0);
    vs = v->stride(0);
    kc = k_cache.data_ptr();
    vc = v_cache.data_ptr();
    bs = k_cache.size(2);
  }
  DISPATCH_ACT(q, fi::launch_widenorm_rope_cache<A>(
                      ptr<A>(q_out), ptr<A>(q), q.stride(0),
                      reinterpret_cast<const A*>(kp), ks,
                      reinterpret_cast<const A*>(vp), vs,
                      positions.data_ptr<int>(), q_w.data_ptr<float>(), kw,
                      (float)eps, inv_freq.data_ptr<float>(), nrot,
                      (float)rot_mult, reinterpret_cast<A*>(kc),
                      reinterpret_cast<A*>(vc), slot_mapping.data_ptr<int>(),
                      (int)T, (int)H, (int)G, (int)D, (int)V, bs, stream()));
}

void clamped_glu(at::Tensor out, at::Tensor gu, double limit) {
  CHECK_ACT(gu);
  CHECK_ACT(out);
  TORCH_CHECK(gu.dim() == 2 && gu.stride(1) == 1 && gu.size(1) % 2 == 0);
  const int T = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(out.is_contiguous() && out.scalar_type() == gu.scalar_type() &&
              out.dim() == 2 && out.size(0) == T && out.size(1) == F);
  DISPATCH_ACT(gu, fi::launch_clamped_glu<A>(ptr<A>(out), ptr<A>(gu),
                                             gu.stride(0), T, F, (float)limit,
                                             stream()));
}

void tanh_cap(at::Tensor x, double cap) {
  CHECK_F32(x);
  TORCH_CHECK(x.is_contiguous() && cap > 0);
  fi::launch_tanh_cap(x.data_ptr<float>(), x.numel(), (float)cap, stream());
}


PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("pair_embed", &pair_embed,
        "embedding times a constant plus a (previous id, id) table row; the "
        "previous id of a group's first row lives in a slot state");
  m.def("layer_norm_affine", &layer_norm_affine,
        "layer norm with weight and bias of fp32 rows");
  m.def("post_norm_residual", &post_norm_residual,
        "stream += layer_norm(sublayer output) * w + b, emits the rounded "
        "stream");
  m.def("widenorm_rope_cache", &widenorm_rope_cache,
        "whole-projection RMS norm of q/k, interleaved partial rotation "
        "with given frequencies, k and v into the paged caches");
  m.def("clamped_glu", &clamped_glu,
        "min(g, L) sigmoid(1.702 min(g, L)) (clamp(u, -L, L) + 1)");
  m.def("tanh_cap", &tanh_cap, "x <- cap tanh(x / cap), fp32 in place");
  m.def("scaled_residual_layer_norm", &scaled_residual_layer_norm,
        "fp32 stream += scaled sublayer results, then layer norm");
  m.def("headnorm_qtemp_cache", &headnorm_qtemp_cache,
        "weighted head RMS norms, query temperature, paged cache write");
  m.def("latent_rope_cache", &latent_rope_cache,
        "rotated query tails, normed latent + rotated key part to the cache");
  m.def("sink_attention_splits", &sink_attention_splits,
        "key spans of the split attention form for a cache capacity");
  m.def("sink_attention_has_tiles", &sink_attention_has_tiles,
        "whether the tiled attention form covers (key size, value size)");
  m.def("sink_paged_attention", &sink_paged_attention,
        "causal paged attention with sink, value slice and output gate");
  m.def("causal_conv_state", &causal_conv_state,
        "per-channel causal convolution with the tail kept per sequence");
  m.def("rglru_scan", &rglru_scan, "gated linear recurrence times gelu branch");
  m.def("relu_squared", &relu_squared, "relu(x)^2");
  m.def("cast_layer_norm", &cast_layer_norm,
        "fp32 stream restarted from an activation, then layer norm");
  m.def("concat_cast", &concat_cast, "[round(stream) | x0] rows");
  m.def("layer_norm", &layer_norm, "layer norm of an fp32 stream, no bias");
  m.def("gated_residual_layer_norm", &gated_residual_layer_norm,
        "fp32 residual += y * sigmoid(gate); optional next layer norm");
  m.def("group_rms_gate", &group_rms_gate,
        "grouped unit-RMS of fp32 read-outs with gain and sigmoid/silu gate");
  m.def("paged_cache_write", &paged_cache_write,
        "k/v rows into paged caches of separate key and value sizes");
  m.def("decay_linear_attention", &decay_linear_attention,
        "linear attention with a scalar decay per head, slot state");
  m.def("gated_delta_rule", &gated_delta_rule,
        "gated delta rule behind a short causal convolution, slot state");
  m.def("talking_window_splits", &fi::talking_window_fast_splits,
        "key passes per row of the thread-per-key windowed attention");
  m.def("talking_window_attention", &talking_window_attention,
        "windowed softmax attention with log-distance penalty and head "
        "mixing over the paged cache");
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
