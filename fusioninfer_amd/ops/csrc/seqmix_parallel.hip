// Kernels of the parallel-residual family of blocks (gfx950, wave64).
//
//  * scaled_residual_layer_norm:
//        x += s1*y1 [+ s2*y2] [+ s3*y3]            (fp32 stream, in place)
//        out = layer_norm(x) * w_next              (optional)
//  * headnorm_qtemp_cache: every query/key head divided by its RMS and
//    multiplied by a weight vector shared by the heads; queries also by
//    the position's temperature 1 + coef * ln(floor((p+1)/every) + 1);
//    processed q to a dense buffer, processed k and the plain v to the
//    paged caches. One wave per (row, head).
//  * latent_rope_cache: the trailing rot_dim entries of every query head
//    rotated (interleaved pairs) into the tail of the folded query
//    buffer; the latent RMS-normed with a weight and the shared key part
//    rotated into one paged cache row [rank | rot_dim].
//  * causal_conv_state (+ tail update): per-channel causal convolution
//    with bias over the rows of every group, history from the slot state.
//  * rglru_scan: S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t per channel,
//    a_t = exp(-c r_t softplus(lam)), out_t = S_t * gelu_tanh(y_t).
//    Chunk-parallel: a workgroup owns 64 channels of one group; its waves
//    scan consecutive token chunks, exchange (decay product, end value)
//    through LDS and finish with the carried state.
//  * relu_squared.

#include "seqmix.h"

namespace fi {

namespace {

FI_DEV void row_moments_p(const float* row, int W, float eps, float* scratch,
                          float& mean, float& rstd) {
  float s = 0.f, dummy = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) s += row[i];
  block_reduce_sum2_256(s, dummy, scratch);
  mean = s / W;
  float q = 0.f;
  dummy = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float d = row[i] - mean;
    q += d * d;
  }
  block_reduce_sum2_256(q, dummy, scratch);
  rstd = rsqrtf(q / W + eps);
}

template <typename A>
__global__ __launch_bounds__(256) void scaled_residual_layer_norm_kernel(
    float* __restrict__ resid, const A* __restrict__ y1, float s1,
    const A* __restrict__ y2, float s2, const A* __restrict__ y3, float s3,
    const float* __restrict__ w_next, A* __restrict__ out, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t t = blockIdx.x;
  float* row = resid + t * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    float y = s1 * Act<A>::ld(y1 + t * W + i);
    if (y2 != nullptr) y += s2 * Act<A>::ld(y2 + t * W + i);
    if (y3 != nullptr) y += s3 * Act<A>::ld(y3 + t * W + i);
    row[i] += y;         // each element is read and written by one thread
  }
  if (w_next == nullptr) return;
  __syncthreads();
  float mean, rstd;
  row_moments_p(row, W, eps, scratch, mean, rstd);
  A* o = out + t * W;
  for (int i = threadIdx.x; i < W; i += 256)
    Act<A>::st(o + i, (row[i] - mean) * rstd * w_next[i]);
}

// resid (fp32) = y; out = layer_norm(resid) * w: the stream restarts from
// an activation (embedding rows, the projection that enters a pass)
template <typename A>
__global__ __launch_bounds__(256) void cast_layer_norm_kernel(
    float* __restrict__ resid, A* __restrict__ out, const A* __restrict__ y,
    const float* __restrict__ w, float eps, int W) {
  __shared__ float scratch[8];
  const int64_t t = blockIdx.x;
  float* row = resid + t * W;
  for (int i = threadIdx.x; i < W; i += 256)
    row[i] = Act<A>::ld(y + t * W + i);
  if (w == nullptr) return;
  __syncthreads();
  float mean, rstd;
  row_moments_p(row, W, eps, scratch, mean, rstd);
  A* o = out + t * W;
  for (int i = threadIdx.x; i < W; i += 256)
    Act<A>::st(o + i, (row[i] - mean) * rstd * w[i]);
}

// out[t] = [round(resid[t]) | x0[t]]: input rows of the pass-entry product
template <typename A>
__global__ __launch_bounds__(256) void concat_cast_kernel(
    A* __restrict__ out, const float* __restrict__ resid,
    const A* __restrict__ x0, int W) {
  const int64_t t = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= W) return;
  Act<A>::st(out + t * 2 * W + i, resid[t * W + i]);
  out[t * 2 * W + W + i] = x0[t * W + i];
}

constexpr int kHeadSlots = 8;   // head sizes up to 512

template <typename A>
__global__ __launch_bounds__(64) void headnorm_qtemp_cache_kernel(
    A* __restrict__ q_out, const A* __restrict__ q, int64_t q_stride,
    const A* __restrict__ k, int64_t k_stride, const A* __restrict__ v,
    int64_t v_stride, const int* __restrict__ positions,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    float coef, int every, A* __restrict__ k_cache, A* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, int H, int G, int D, int V, int bs) {
  const int t = blockIdx.x;
  const int hh = blockIdx.y;   // [0,H): q, [H,H+G): k, [H+G,H+2G): v
  const int lane = threadIdx.x;
  if (hh >= H) {
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    const int64_t blk = slot / bs;
    const int off = slot % bs;
    if (hh >= H + G) {
      const int g = hh - H - G;
      const A* src = v + t * v_stride + static_cast<int64_t>(g) * V;
      A* dst = v_cache + ((blk * G + g) * bs + off) * V;
      for (int d = lane; d < V; d += 64) dst[d] = src[d];
      return;
    }
    const int g = hh - H;
    const A* src = k + t * k_stride + static_cast<int64_t>(g) * D;
    float x[kHeadSlots];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kHeadSlots; ++i) {
      const int d = lane + 64 * i;
      x[i] = d < D ? Act<A>::ld(src + d) : 0.f;
      ss += x[i] * x[i];
    }
    ss = wave_reduce_sum(ss);
    const float inv = rsqrtf(ss / D + eps);
    A* dst = k_cache + ((blk * G + g) * bs + off) * D;
#pragma unroll
    for (int i = 0; i < kHeadSlots; ++i) {
      const int d = lane + 64 * i;
      if (d < D) Act<A>::st(dst + d, x[i] * inv * k_w[d]);
    }
    return;
  }
  const A* src = q + t * q_stride + static_cast<int64_t>(hh) * D;
  float x[kHeadSlots];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kHeadSlots; ++i) {
    const int d = lane + 64 * i;
    x[i] = d < D ? Act<A>::ld(src + d) : 0.f;
    ss += x[i] * x[i];
  }
  ss = wave_reduce_sum(ss);
  float f = rsqrtf(ss / D + eps);
  if (every > 0 && coef != 0.f) {
    const int blk = (positions[t] + 1) / every;
    f *= 1.0f + coef * logf(static_cast<float>(blk + 1));
  }
  A* dst = q_out + (static_cast<int64_t>(t) * H + hh) * D;
#pragma unroll
  for (int i = 0; i < kHeadSlots; ++i) {
    const int d = lane + 64 * i;
    if (d < D) Act<A>::st(dst + d, x[i] * f * q_w[d]);
  }
}

template <typename A>
__global__ __launch_bounds__(64) void latent_rope_cache_kernel(
    A* __restrict__ q_out,            // [T, H, C + R]
    const A* __restrict__ q, int64_t q_stride,        // [T, H*(D+R)]
    const A* __restrict__ ckr, int64_t c_stride,      // [T, C+R]
    const int* __restrict__ positions, const float* __restrict__ inv_freq,
    const float* __restrict__ norm_w, float eps, A* __restrict__ kv_cache,
    const int* __restrict__ slot_mapping, int H, int D, int R, int C,
    int rot_pairs, int bs) {
  const int t = blockIdx.x;
  const int hh = blockIdx.y;   // [0,H): query heads, H: the cache row
  const int lane = threadIdx.x;
  const float pos = static_cast<float>(positions[t]);
  const A* src;
  A* dst;
  if (hh < H) {
    src = q + t * q_stride + static_cast<int64_t>(hh) * (D + R) + D;
    dst = q_out + (static_cast<int64_t>(t) * H + hh) * (C + R) + C;
  } else {
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    A* row = kv_cache +
        (static_cast<int64_t>(slot / bs) * bs + slot % bs) * (C + R);
    const A* cs = ckr + t * c_stride;
    float ss = 0.f;
    for (int d = lane; d < C; d += 64) {
      const float x = Act<A>::ld(cs + d);
      ss += x * x;
    }
    ss = wave_reduce_sum(ss);
    const float inv = rsqrtf(ss / C + eps);
    for (int d = lane; d < C; d += 64)
      Act<A>::st(row + d, Act<A>::ld(cs + d) * inv * norm_w[d]);
    src = cs + C;
    dst = row + C;
  }
  // the first rot_pairs pairs turn, the rest of the part passes
  for (int i = lane; i < rot_pairs; i += 64) {
    const float u = Act<A>::ld(src + 2 * i);
    const float w = Act<A>::ld(src + 2 * i + 1);
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    Act<A>::st(dst + 2 * i, u * cs - w * sn);
    Act<A>::st(dst + 2 * i + 1, w * cs + u * sn);
  }
  for (int d = 2 * rot_pairs + lane; d < R; d += 64) dst[d] = src[d];
}

constexpr int kMaxTaps = 16;

template <typename A>
__global__ __launch_bounds__(256) void causal_conv_state_kernel(
    float* __restrict__ out,          // [T, C]
    const A* __restrict__ x, int64_t x_stride,
    const float* __restrict__ conv_w,  // [C, taps]
    const float* __restrict__ conv_b,
    const float* __restrict__ conv_state,  // [slots, hist, C]
    const int* __restrict__ seq_cu, const int* __restrict__ row_seq,
    const int* __restrict__ seq_slots, const int* __restrict__ positions,
    int C, int taps, int hist) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = row_seq[t];
  const int a = seq_cu[s];
  const int r = t - a;
  const int slot = seq_slots[s];
  const bool has_hist = slot >= 0 && positions[a] > 0;
  const float* hs =
      conv_state + static_cast<int64_t>(slot < 0 ? 0 : slot) * hist * C;
  float acc = conv_b[c];
  for (int j = 0; j < taps; ++j) {
    const int e = r + j;           // index into [history | new rows]
    float v = 0.f;
    if (e >= taps - 1)
      v = Act<A>::ld(x + static_cast<int64_t>(a + e - (taps - 1)) * x_stride +
                     c);
    else if (has_hist)
      v = hs[static_cast<int64_t>(e) * C + c];
    acc += conv_w[static_cast<int64_t>(c) * taps + j] * v;
  }
  out[static_cast<int64_t>(t) * C + c] = acc;
}

template <typename A>
__global__ __launch_bounds__(256) void conv_tail_update_kernel(
    const A* __restrict__ x, int64_t x_stride, float* __restrict__ conv_state,
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int C, int taps, int hist) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int slot = seq_slots[s];
  const int a = seq_cu[s];
  const int n = seq_cu[s + 1] - a;
  if (slot < 0 || n <= 0) return;
  const bool has_hist = positions[a] > 0;
  float* hs = conv_state + static_cast<int64_t>(slot) * hist * C;
  // new tail = last taps-1 entries of [history | new rows]; entry i reads
  // index n + i >= i + 1, so ascending i never reads what it overwrote
  for (int i = 0; i < taps - 1; ++i) {
    const int e = n + i;
    float v = 0.f;
    if (e >= taps - 1)
      v = Act<A>::ld(x + static_cast<int64_t>(a + e - (taps - 1)) * x_stride +
                     c);
    else if (has_hist)
      v = hs[static_cast<int64_t>(e) * C + c];
    hs[static_cast<int64_t>(i) * C + c] = v;
  }
}

FI_DEV float gelu_tanh_f(float z) {
  return 0.5f * z *
         (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

FI_DEV float softplus_f(float z) {
  return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
}

constexpr int kScanWavesLong = 16;  // token chunks scanned side by side
constexpr int kScanChunk = 8;       // tokens per wave and round

// One workgroup: 64 channels (lanes) of one group, kScanWaves waves (one
// wave when no group of the step has more than a chunk of rows). A
// round covers kScanWaves * kScanChunk consecutive rows: wave w scans its
// chunk from a zero start keeping (product of decays, end value), the
// waves exchange those through LDS, every wave derives the state at its
// chunk's start from the carried state and the chunks before it, and
// replays its chunk to write the outputs.
template <typename A, int kScanWaves>
__global__ __launch_bounds__(64 * kScanWaves) void rglru_scan_kernel(
    A* __restrict__ out,               // [T, W]
    const float* __restrict__ u,       // [T, W]
    const float* __restrict__ gate_lin,  // [B, T, 2*bw]
    const float* __restrict__ gate_bias, // [B, 2*bw]
    const float* __restrict__ lam, const A* __restrict__ y_lin,
    int64_t y_stride, float* __restrict__ state,  // [slots, W]
    const int* __restrict__ seq_cu, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, int T, int W, int bw,
    float decay_scale) {
  __shared__ float ex_a[kScanWaves][64];
  __shared__ float ex_b[kScanWaves][64];
  const int s = blockIdx.x;
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int c = blockIdx.y * 64 + lane;
  const bool live = c < W;
  const int cc = live ? c : 0;
  const int t0 = seq_cu[s];
  const int n = seq_cu[s + 1] - t0;
  if (n <= 0) return;
  const int slot = seq_slots[s];
  const int b = cc / bw, ci = cc % bw;
  const float rb = gate_bias[b * 2 * bw + ci];
  const float ib = gate_bias[b * 2 * bw + bw + ci];
  const float sp = decay_scale * softplus_f(lam[cc]);
  const float* gl = gate_lin + (static_cast<int64_t>(b) * T) * 2 * bw + ci;
  float carry = 0.f;
  if (slot >= 0 && positions[t0] > 0)
    carry = state[static_cast<int64_t>(slot) * W + cc];

  for (int base = 0; base < n; base += kScanWaves * kScanChunk) {
    const int r0 = base + wave * kScanChunk;
    const int cnt = max(0, min(kScanChunk, n - r0));
    float av[kScanChunk], bv[kScanChunk];
    float pa = 1.f, pb = 0.f;
#pragma unroll
    for (int i = 0; i < kScanChunk; ++i) {
      av[i] = 1.f;
      bv[i] = 0.f;
      if (i < cnt) {
        const int64_t t = t0 + r0 + i;
        const float r = sigmoidf_acc(gl[t * 2 * bw] + rb);
        const float g = sigmoidf_acc(gl[t * 2 * bw + bw] + ib);
        const float log_a = -sp * r;
        av[i] = expf(log_a);
        bv[i] = sqrtf(-expm1f(2.0f * log_a)) * g * u[t * W + cc];
      }
      pb = av[i] * pb + bv[i];
      pa *= av[i];
    }
    __syncthreads();               // previous round's readers are done
    ex_a[wave][lane] = pa;
    ex_b[wave][lane] = pb;
    __syncthreads();
    float st = carry;              // state at the start of this wave's chunk
    for (int w = 0; w < wave; ++w) st = ex_a[w][lane] * st + ex_b[w][lane];
    float nxt = st;                // state after the whole round
    for (int w = wave; w < kScanWaves; ++w)
      nxt = ex_a[w][lane] * nxt + ex_b[w][lane];
    carry = nxt;
#pragma unroll
    for (int i = 0; i < kScanChunk; ++i) {
      if (i < cnt) {
        const int64_t t = t0 + r0 + i;
        st = av[i] * st + bv[i];
        if (live)
          Act<A>::st(out + t * W + c,
                     st * gelu_tanh_f(Act<A>::ld(y_lin + t * y_stride + c)));
      }
    }
  }
  if (slot >= 0 && live && wave == 0)
    state[static_cast<int64_t>(slot) * W + c] = carry;
}

template <typename A, int VW>
__global__ __launch_bounds__(256) void relu_squared_kernel(
    A* __restrict__ out, const A* __restrict__ x, int64_t x_stride, int N) {
  const int64_t t = blockIdx.y;
  const int i = (blockIdx.x * 256 + threadIdx.x) * VW;
  if (i >= N) return;
  float v[VW];
  ldv<A, VW>(x + t * x_stride + i, v);
#pragma unroll
  for (int e = 0; e < VW; ++e) {
    v[e] = fmaxf(v[e], 0.f);
    v[e] *= v[e];
  }
  stv<A, VW>(out + t * N + i, v);
}

}  // namespace

template <typename A>
void launch_scaled_residual_layer_norm(float* resid, const A* y1, float s1,
                                       const A* y2, float s2, const A* y3,
                                       float s3, const float* w_next, A* out,
                                       float eps, int T, int W,
                                       hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(scaled_residual_layer_norm_kernel<A>, dim3(T), dim3(256),
                     0, st, resid, y1, s1, y2, s2, y3, s3, w_next, out, eps,
                     W);
}

template <typename A>
void launch_cast_layer_norm(float* resid, A* out, const A* y, const float* w,
                            float eps, int T, int W, hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(cast_layer_norm_kernel<A>, dim3(T), dim3(256), 0, st,
                     resid, out, y, w, eps, W);
}

template <typename A>
void launch_concat_cast(A* out, const float* resid, const A* x0, int T, int W,
                        hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(concat_cast_kernel<A>, dim3(ceil_div(W, 256), T),
                     dim3(256), 0, st, out, resid, x0, W);
}

template <typename A>
void launch_headnorm_qtemp_cache(A* q_out, const A* q, int64_t q_stride,
                                 const A* k, int64_t k_stride, const A* v,
                                 int64_t v_stride, const int* positions,
                                 const float* q_w, const float* k_w,
                                 float eps, float coef, int every, A* k_cache,
                                 A* v_cache, const int* slot_mapping, int T,
                                 int H, int G, int D, int V, int bs,
                                 hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(headnorm_qtemp_cache_kernel<A>, dim3(T, H + 2 * G),
                     dim3(64), 0, st, q_out, q, q_stride, k, k_stride, v,
                     v_stride, positions, q_w, k_w, eps, coef, every, k_cache,
                     v_cache, slot_mapping, H, G, D, V, bs);
}

template <typename A>
void launch_latent_rope_cache(A* q_out, const A* q, int64_t q_stride,
                              const A* ckr, int64_t c_stride,
                              const int* positions, const float* inv_freq,
                              const float* norm_w, float eps, A* kv_cache,
                              const int* slot_mapping, int T, int H, int D,
                              int R, int C, int rot_pairs, int bs,
                              hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(latent_rope_cache_kernel<A>, dim3(T, H + 1), dim3(64), 0,
                     st, q_out, q, q_stride, ckr, c_stride, positions,
                     inv_freq, norm_w, eps, kv_cache, slot_mapping, H, D, R, C,
                     rot_pairs, bs);
}

template <typename A>
void launch_causal_conv_state(float* out, const A* x, int64_t x_stride,
                              const float* conv_w, const float* conv_b,
                              float* conv_state, const int* seq_cu,
                              const int* row_seq, const int* seq_slots,
                              const int* positions, int T, int S, int C,
                              int taps, int hist, hipStream_t st) {
  if (T == 0) return;
  const int cb = ceil_div(C, 256);
  hipLaunchKernelGGL(causal_conv_state_kernel<A>, dim3(T, cb), dim3(256), 0,
                     st, out, x, x_stride, conv_w, conv_b, conv_state, seq_cu,
                     row_seq, seq_slots, positions, C, taps, hist);
  if (taps > 1)
    hipLaunchKernelGGL(conv_tail_update_kernel<A>, dim3(S, cb), dim3(256), 0,
                       st, x, x_stride, conv_state, seq_cu, seq_slots,
                       positions, C, taps, hist);
}

template <typename A>
void launch_rglru_scan(A* out, const float* u, const float* gate_lin,
                       const float* gate_bias, const float* lam,
                       const A* y_lin, int64_t y_stride, float* state,
                       const int* seq_cu, const int* seq_slots,
                       const int* positions, int T, int S, int W, int bw,
                       float decay_scale, int max_rows, hipStream_t st) {
  if (T == 0 || S == 0) return;
  // max_rows: longest group of the step (0: unknown)
  if (max_rows > 0 && max_rows <= kScanChunk)
    hipLaunchKernelGGL((rglru_scan_kernel<A, 1>), dim3(S, ceil_div(W, 64)),
                       dim3(64), 0, st, out, u, gate_lin, gate_bias, lam,
                       y_lin, y_stride, state, seq_cu, seq_slots, positions, T,
                       W, bw, decay_scale);
  else
    hipLaunchKernelGGL((rglru_scan_kernel<A, kScanWavesLong>),
                       dim3(S, ceil_div(W, 64)), dim3(64 * kScanWavesLong), 0,
                       st, out, u, gate_lin, gate_bias, lam, y_lin, y_stride,
                       state, seq_cu, seq_slots, positions, T, W, bw,
                       decay_scale);
}

template <typename A>
void launch_relu_squared(A* out, const A* x, int64_t x_stride, int T, int N,
                         hipStream_t st) {
  if (T == 0 || N == 0) return;
  // four elements per thread when rows and the slice start allow it
  const bool vec = N % 4 == 0 && x_stride % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(x) % (4 * sizeof(A)) == 0 &&
                   reinterpret_cast<uintptr_t>(out) % (4 * sizeof(A)) == 0;
  if (vec)
    hipLaunchKernelGGL((relu_squared_kernel<A, 4>),
                       dim3(ceil_div(N, 1024), T), dim3(256), 0, st, out, x,
                       x_stride, N);
  else
    hipLaunchKernelGGL((relu_squared_kernel<A, 1>), dim3(ceil_div(N, 256), T),
                       dim3(256), 0, st, out, x, x_stride, N);
}

#define FI_INST(A)                                                             \
  template void launch_cast_layer_norm<A>(float*, A*, const A*, const float*,  \
                                          float, int, int, hipStream_t);       \
  template void launch_concat_cast<A>(A*, const float*, const A*, int, int,    \
                                      hipStream_t);                            \
  template void launch_scaled_residual_layer_norm<A>(                          \
      float*, const A*, float, const A*, float, const A*, float, const float*, \
      A*, float, int, int, hipStream_t);                                       \
  template void launch_headnorm_qtemp_cache<A>(                                \
      A*, const A*, int64_t, const A*, int64_t, const A*, int64_t, const int*, \
      const float*, const float*, float, float, int, A*, A*, const int*, int,  \
      int, int, int, int, int, hipStream_t);                                   \
  template void launch_latent_rope_cache<A>(                                   \
      A*, const A*, int64_t, const A*, int64_t, const int*, const float*,      \
      const float*, float, A*, const int*, int, int, int, int, int, int, int,  \
      hipStream_t);                                                            \
  template void launch_causal_conv_state<A>(                                   \
      float*, const A*, int64_t, const float*, const float*, float*,           \
      const int*, const int*, const int*, const int*, int, int, int, int, int, \
      hipStream_t);                                                            \
  template void launch_rglru_scan<A>(                                          \
      A*, const float*, const float*, const float*, const float*, const A*,    \
      int64_t, float*, const int*, const int*, const int*, int, int, int, int, \
      float, int, hipStream_t);                                                   \
  template void launch_relu_squared<A>(A*, const A*, int64_t, int, int,        \
                                       hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
