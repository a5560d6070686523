// Row kernels of the post-norm stream (gfx950, wave64):
//
//  * pair_embed: the fp32 stream starts as embed[id] * c plus one row of a
//    hashed (previous id, id) table; the previous id of a row group's
//    first row comes from a per-slot int32 state that then receives the
//    group's last id.
//  * norm_affine: layer norm with weight and bias (two-pass fp32
//    statistics: mean, then mean of squared deviations) of an activation
//    or fp32 row. With a stream pointer the normed row is ADDED to the
//    stream (the norm sits on a sublayer's output) and the stream's
//    rounding is written for the next sublayer; without one the normed row
//    itself is written.
//  * widenorm_rope_cache: RMS norm over a whole q or k projection row (all
//    heads at once) times a weight vector, interleaved-pair rotation of the
//    leading entries of every head with given frequencies and a factor on
//    cos/sin; k and raw v rows go into the paged caches.
//  * clamped_glu, tanh_cap: elementwise.

#include <type_traits>

#include "seqmix.h"

namespace fi {

namespace {

template <typename A>
__global__ __launch_bounds__(256) void pair_embed_kernel(
    float* __restrict__ resid, A* __restrict__ act,
    const int64_t* __restrict__ ids, const A* __restrict__ embed, float scale,
    const A* __restrict__ pair_table, int64_t buckets, int64_t mul_prev,
    int64_t mul_cur, int* __restrict__ prev_token,
    const int* __restrict__ seq_cu, const int* __restrict__ row_seq,
    const int* __restrict__ seq_slots, const int* __restrict__ positions,
    int W) {
  __shared__ int64_t pair_row;
  const int t = blockIdx.x;
  const int64_t id = ids[t];
  if (threadIdx.x == 0) {
    const int s = row_seq[t];
    const bool first = t == seq_cu[s];
    const int slot = seq_slots[s];
    int64_t prev = 0;
    if (!first)
      prev = ids[t - 1];
    else if (slot >= 0)
      prev = prev_token[slot];
    int64_t r = (prev * mul_prev + id * mul_cur) % buckets;
    if (r < 0) r += buckets;
    pair_row = positions[t] == 0 ? buckets : r;
    // only the workgroup of a group's first row touches the slot: it has
    // read the previous id above and leaves the group's last id behind
    if (first && slot >= 0)
      prev_token[slot] = static_cast<int>(ids[seq_cu[s + 1] - 1]);
  }
  __syncthreads();
  const A* e = embed + id * W;
  const A* b = pair_table != nullptr ? pair_table + pair_row * W : nullptr;
  if (W % 4 == 0) {
    for (int i = threadIdx.x * 4; i < W; i += 1024) {
      float x[4], y[4];
      ldv<A, 4>(e + i, x);
#pragma unroll
      for (int k = 0; k < 4; ++k) x[k] *= scale;
      if (b != nullptr) {
        ldv<A, 4>(b + i, y);
#pragma unroll
        for (int k = 0; k < 4; ++k) x[k] += y[k];
      }
      stv<float, 4>(resid + static_cast<int64_t>(t) * W + i, x);
      if constexpr (!std::is_same<A, float>::value)
        stv<A, 4>(act + static_cast<int64_t>(t) * W + i, x);
    }
    return;
  }
  for (int i = threadIdx.x; i < W; i += 256) {
    float x = Act<A>::ld(e + i) * scale;
    if (b != nullptr) x += Act<A>::ld(b + i);
    resid[static_cast<int64_t>(t) * W + i] = x;
    if constexpr (!std::is_same<A, float>::value)
      Act<A>::st(act + static_cast<int64_t>(t) * W + i, x);
  }
}

template <typename I>
FI_DEV float ld_in(const I* p);
template <>
FI_DEV float ld_in<float>(const float* p) { return *p; }
template <>
FI_DEV float ld_in<u16>(const u16* p) { return bf16_to_f32(*p); }

// NCH > 0: the row is held in registers (NCH chunks of 256 threads x 4
// consecutive entries, W % 4 == 0); NCH == 0: any W, the row is re-read.
template <typename I, typename A, int NCH>
__global__ __launch_bounds__(256) void norm_affine_kernel(
    const I* __restrict__ x, float* __restrict__ resid, A* __restrict__ out,
    const float* __restrict__ w, const float* __restrict__ b, float eps,
    int W) {
  __shared__ float scratch[8];
  const int64_t t = blockIdx.x;
  const I* xr = x + t * W;
  float* rr = resid != nullptr ? resid + t * W : nullptr;
  A* orow = out != nullptr ? out + t * W : nullptr;
  float dummy = 0.f;
  auto emit = [&](int i, float n) {
    float v = n * w[i] + b[i];
    if (rr != nullptr) {
      v += rr[i];
      rr[i] = v;
    }
    if (orow != nullptr) Act<A>::st(orow + i, v);
  };
  if constexpr (NCH > 0) {
    float v[NCH][4];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
        ldv<I, 4>(xr + i, v[c]);
      } else {
        v[c][0] = v[c][1] = v[c][2] = v[c][3] = 0.f;
      }
      sum += (v[c][0] + v[c][1]) + (v[c][2] + v[c][3]);
    }
    block_reduce_sum2_256(sum, dummy, scratch);
    const float mean = sum / W;
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[c][e] -= mean;
          sq += v[c][e] * v[c][e];
        }
      }
    }
    block_reduce_sum2_256(sq, dummy, scratch);
    const float rstd = rsqrtf(sq / W + eps);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
        // 16-byte accesses: weight, bias, stream in and out
        const float4 w4 = *reinterpret_cast<const float4*>(w + i);
        const float4 b4 = *reinterpret_cast<const float4*>(b + i);
        float o4[4] = {v[c][0] * rstd * w4.x + b4.x,
                       v[c][1] * rstd * w4.y + b4.y,
                       v[c][2] * rstd * w4.z + b4.z,
                       v[c][3] * rstd * w4.w + b4.w};
        if (rr != nullptr) {
          const float4 r4 = *reinterpret_cast<const float4*>(rr + i);
          o4[0] += r4.x;
          o4[1] += r4.y;
          o4[2] += r4.z;
          o4[3] += r4.w;
          *reinterpret_cast<float4*>(rr + i) =
              float4{o4[0], o4[1], o4[2], o4[3]};
        }
        if (orow != nullptr) stv<A, 4>(orow + i, o4);
      }
    }
  } else {
    float sum = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) sum += ld_in<I>(xr + i);
    block_reduce_sum2_256(sum, dummy, scratch);
    const float mean = sum / W;
    float sq = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
      const float d = ld_in<I>(xr + i) - mean;
      sq += d * d;
    }
    block_reduce_sum2_256(sq, dummy, scratch);
    const float rstd = rsqrtf(sq / W + eps);
    for (int i = threadIdx.x; i < W; i += 256)
      emit(i, (ld_in<I>(xr + i) - mean) * rstd);
  }
}

template <typename A>
__global__ __launch_bounds__(256) void widenorm_rope_cache_kernel(
    A* __restrict__ q_out, const A* __restrict__ q, int64_t q_stride,
    const A* __restrict__ k, int64_t k_stride, const A* __restrict__ v,
    int64_t v_stride, const int* __restrict__ positions,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    const float* __restrict__ inv_freq, int nrot, float rot_mult,
    A* __restrict__ k_cache, A* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, int H, int G, int D, int V, int bs) {
  __shared__ float scratch[8];
  const int t = blockIdx.x;
  const int what = blockIdx.y;          // 0: q, 1: k, 2: v
  int64_t cache_row = 0;                // first (kv head 0) row in the cache
  if (what > 0) {
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    cache_row = static_cast<int64_t>(slot / bs) * G * bs + slot % bs;
  }
  if (what == 2) {
    const A* src = v + t * v_stride;
    for (int i = threadIdx.x; i < G * V; i += 256)
      v_cache[(cache_row + static_cast<int64_t>(i / V) * bs) * V + i % V] =
          src[i];
    return;
  }
  const int heads = what == 0 ? H : G;
  const int n = heads * D;
  const A* src = what == 0 ? q + t * q_stride : k + t * k_stride;
  const float* w = what == 0 ? q_w : k_w;
  float sq = 0.f, dummy = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float x = Act<A>::ld(src + i);
    sq += x * x;
  }
  block_reduce_sum2_256(sq, dummy, scratch);
  const float rstd = rsqrtf(sq / n + eps);
  const float pos = static_cast<float>(positions[t]);
  // one item per (head, pair of neighbours); an odd head size leaves a
  // last single entry, which never turns (nrot is even and <= D)
  const int half = (D + 1) / 2;
  for (int it = threadIdx.x; it < heads * half; it += 256) {
    const int hh = it / half, j = it % half;
    const int d0 = 2 * j, d1 = d0 + 1;
    const int i0 = hh * D + d0;
    float a = Act<A>::ld(src + i0) * rstd * w[i0];
    float c = d1 < D ? Act<A>::ld(src + i0 + 1) * rstd * w[i0 + 1] : 0.f;
    if (d1 < nrot) {
      float sn, cs;
      sincosf(pos * inv_freq[j], &sn, &cs);
      sn *= rot_mult;
      cs *= rot_mult;
      const float ra = a * cs - c * sn;
      c = c * cs + a * sn;
      a = ra;
    }
    A* dst = what == 0
                 ? q_out + static_cast<int64_t>(t) * n + i0
                 : k_cache + (cache_row + static_cast<int64_t>(hh) * bs) * D + d0;
    Act<A>::st(dst, a);
    if (d1 < D) Act<A>::st(dst + 1, c);
  }
}

template <typename A, int VW>
__global__ __launch_bounds__(256) void clamped_glu_kernel(
    A* __restrict__ out, const A* __restrict__ gu, int64_t gu_stride, int F,
    float limit) {
  const int64_t t = blockIdx.y;
  const int i = (blockIdx.x * 256 + threadIdx.x) * VW;
  if (i >= F) return;
  float g[VW], u[VW], y[VW];
  ldv<A, VW>(gu + t * gu_stride + i, g);
  ldv<A, VW>(gu + t * gu_stride + F + i, u);
#pragma unroll
  for (int e = 0; e < VW; ++e) {
    const float gc = fminf(g[e], limit);
    const float uc = fminf(fmaxf(u[e], -limit), limit);
    y[e] = gc * sigmoidf_acc(1.702f * gc) * (uc + 1.0f);
  }
  stv<A, VW>(out + t * F + i, y);
}

__global__ __launch_bounds__(256) void tanh_cap_kernel(float* __restrict__ x,
                                                       int64_t n, float cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

template <typename A>
void launch_pair_embed(float* resid, A* act, const int64_t* ids,
                       const A* embed, float scale, const A* pair_table,
                       int64_t buckets, int64_t mul_prev, int64_t mul_cur,
                       int* prev_token, const int* seq_cu, const int* row_seq,
                       const int* seq_slots, const int* positions, int T,
                       int W, hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(pair_embed_kernel<A>, dim3(T), dim3(256), 0, st, resid,
                     act, ids, embed, scale, pair_table, buckets, mul_prev,
                     mul_cur, prev_token, seq_cu, row_seq, seq_slots,
                     positions, W);
}

template <typename I, typename A>
void launch_norm_affine(const I* x, float* resid, A* out, const float* w,
                        const float* b, float eps, int T, int W,
                        hipStream_t st) {
  if (T == 0) return;
  const int chunks = W % 4 == 0 ? ceil_div(W, 1024) : 0;
#define FI_NORM(N_)                                                            \
  hipLaunchKernelGGL((norm_affine_kernel<I, A, N_>), dim3(T), dim3(256), 0,    \
                     st, x, resid, out, w, b, eps, W)
  if (chunks == 1) FI_NORM(1);
  else if (chunks == 2) FI_NORM(2);
  else if (chunks > 2 && chunks <= 4) FI_NORM(4);
  else if (chunks > 4 && chunks <= 8) FI_NORM(8);
  else FI_NORM(0);
#undef FI_NORM
}

template <typename A>
void launch_widenorm_rope_cache(A* q_out, const A* q, int64_t q_stride,
                                const A* k, int64_t k_stride, const A* v,
                                int64_t v_stride, const int* positions,
                                const float* q_w, const float* k_w, float eps,
                                const float* inv_freq, int nrot,
                                float rot_mult, A* k_cache, A* v_cache,
                                const int* slot_mapping, int T, int H, int G,
                                int D, int V, int bs, hipStream_t st) {
  if (T == 0) return;
  hipLaunchKernelGGL(widenorm_rope_cache_kernel<A>,
                     dim3(T, k != nullptr ? 3 : 1), dim3(256), 0, st, q_out, q,
                     q_stride, k, k_stride, v, v_stride, positions, q_w, k_w,
                     eps, inv_freq, nrot, rot_mult, k_cache, v_cache,
                     slot_mapping, H, G, D, V, bs);
}

template <typename A>
void launch_clamped_glu(A* out, const A* gu, int64_t gu_stride, int T, int F,
                        float limit, hipStream_t st) {
  if (T == 0) return;
  if (F % 4 == 0 && gu_stride % 4 == 0)
    hipLaunchKernelGGL((clamped_glu_kernel<A, 4>),
                       dim3(ceil_div(F, 1024), T), dim3(256), 0, st, out, gu,
                       gu_stride, F, limit);
  else
    hipLaunchKernelGGL((clamped_glu_kernel<A, 1>), dim3(ceil_div(F, 256), T),
                       dim3(256), 0, st, out, gu, gu_stride, F, limit);
}

void launch_tanh_cap(float* x, int64_t n, float cap, hipStream_t st) {
  if (n == 0) return;
  hipLaunchKernelGGL(tanh_cap_kernel,
                     dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256),
                     0, st, x, n, cap);
}

#define FI_INST(A)                                                             \
  template void launch_pair_embed<A>(                                          \
      float*, A*, const int64_t*, const A*, float, const A*, int64_t,          \
      int64_t, int64_t, int*, const int*, const int*, const int*, const int*,  \
      int, int, hipStream_t);                                                  \
  template void launch_norm_affine<A, A>(const A*, float*, A*, const float*,   \
                                         const float*, float, int, int,        \
                                         hipStream_t);                         \
  template void launch_widenorm_rope_cache<A>(                                 \
      A*, const A*, int64_t, const A*, int64_t, const A*, int64_t, const int*, \
      const float*, const float*, float, const float*, int, float, A*, A*,     \
      const int*, int, int, int, int, int, int, hipStream_t);                  \
  template void launch_clamped_glu<A>(A*, const A*, int64_t, int, int, float,  \
                                      hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST
// final norm of a bf16 model: fp32 stream in, bf16 rows out
template void launch_norm_affine<float, u16>(const float*, float*, u16*,
                                             const float*, const float*,
                                             float, int, int, hipStream_t);

}  // namespace fi
