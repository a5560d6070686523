// Expert-routing kernels without size constraints (gfx950, wave64).
//
//  * moe_route: router tail for up to 1024 experts. One wave per token;
//    lane l keeps experts l, l+64, ... in registers. Scores are
//    softmax(z) or sigmoid(z) in fp32; the k largest are taken one by one
//    with a wave-wide arg-max (ties: smaller index); weights are the
//    chosen scores, divided by their sum + 1e-20 when asked, times a
//    constant.
//  * moe_gemm_plain: grouped GEMM over the block-aligned expert segments
//    (same layout as the MFMA kernel: sorted_ids / expert_ids / n_valid)
//    on the experts' natural [E, out, in] weights, bf16 or fp32 operands,
//    fp32 accumulation, any K and N. 16 rows x 64 columns per workgroup,
//    operands staged through LDS as fp32. Mode 0: plain GEMM over act
//    rows; 1: x rows gathered through sorted_ids, gate|up columns,
//    silu(gate) * up on the way out; 2: gathered x rows, up columns
//    alone, relu(up)^2 on the way out; 3: as 1 with the clamped unit
//    g' sigmoid(1.702 g') (u' + 1), g' = min(g, limit),
//    u' = clamp(u, -limit, limit).
//  * moe_route_grouped: group-limited router tail for up to 1024 experts.
//    One wave per token; scores s = sigmoid(z), choice scores c = s +
//    correction. Experts form equal groups of neighbours; a group's score
//    is the sum of its two largest choice scores, the best `keep` groups
//    stay, and the k largest c inside them are chosen (ties: smaller
//    index). Weights are the chosen s as they are.
//  * moe_combine: out[t] = sum_k w[t,k] * y[pos[t,k]], any width, bf16 or
//    fp32 rows, no atomics.

#include <hip/hip_runtime.h>
#include <math.h>

#include "seqmix.h"

namespace fi {

namespace {

constexpr int kRouteSlots = 16;   // experts per lane: 16 * 64 = 1024

__global__ __launch_bounds__(256) void moe_route_kernel(
    const float* __restrict__ logits, float* __restrict__ topv,
    int* __restrict__ topi, const int T, const int E, const int k,
    const bool sigmoid, const bool renorm, const float scale) {
  const int t = blockIdx.x * 4 + threadIdx.x / kWaveSize;
  if (t >= T) return;
  const int lane = threadIdx.x % kWaveSize;
  const float* row = logits + static_cast<int64_t>(t) * E;
  float sc[kRouteSlots];
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < kRouteSlots; ++j) {
    const int e = lane + 64 * j;
    sc[j] = e < E ? row[e] : -INFINITY;
    m = fmaxf(m, sc[j]);
  }
  if (sigmoid) {
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j)
      sc[j] = lane + 64 * j < E ? 1.0f / (1.0f + expf(-sc[j])) : -1.0f;
  } else {
    m = wave_reduce_max(m);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j) {
      const float ex = lane + 64 * j < E ? expf(sc[j] - m) : 0.f;
      sum += ex;
      sc[j] = lane + 64 * j < E ? ex : -1.0f;
    }
    sum = wave_reduce_sum(sum);
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j)
      if (lane + 64 * j < E) sc[j] /= sum;
  }
  float ksum = 0.f;
  for (int it = 0; it < k; ++it) {
    float v = -2.0f;
    int idx = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j) {
      if (sc[j] > v) {      // ascending j: the smaller index wins ties
        v = sc[j];
        idx = lane + 64 * j;
      }
    }
#pragma unroll
    for (int off = 32; off; off >>= 1) {
      const float ov = __shfl_xor(v, off);
      const int oi = __shfl_xor(idx, off);
      if (ov > v || (ov == v && oi < idx)) {
        v = ov;
        idx = oi;
      }
    }
    ksum += v;
    if (lane == 0) {
      topi[static_cast<int64_t>(t) * k + it] = idx;
      topv[static_cast<int64_t>(t) * k + it] = v;
    }
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j)
      if (idx == lane + 64 * j) sc[j] = -3.0f;
  }
  if (lane == 0) {
    const float f = renorm ? scale / (ksum + 1e-20f) : scale;
    for (int it = 0; it < k; ++it) topv[static_cast<int64_t>(t) * k + it] *= f;
  }
}

__global__ __launch_bounds__(256) void moe_route_grouped_kernel(
    const float* __restrict__ logits, const float* __restrict__ correction,
    float* __restrict__ topv, int* __restrict__ topi, const int T,
    const int E, const int k, const int groups, const int keep) {
  // choice scores of a token's experts, then of its groups
  __shared__ float cs[4][1024];
  __shared__ float gs[4][1024];
  const int w = threadIdx.x / kWaveSize;
  const int t = blockIdx.x * 4 + w;
  if (t >= T) return;      // whole waves leave; no block-wide barrier below
  const int lane = threadIdx.x % kWaveSize;
  const float* row = logits + static_cast<int64_t>(t) * E;
  for (int e = lane; e < E; e += 64)
    cs[w][e] = 1.0f / (1.0f + expf(-row[e])) + correction[e];
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();
  if (groups > 1 && keep < groups) {
    const int n = E / groups;
    for (int g = lane; g < groups; g += 64) {
      float a = -INFINITY, b = -INFINITY;     // two largest of the group
      for (int e = g * n; e < (g + 1) * n; ++e) {
        const float c = cs[w][e];
        if (c > a) {
          b = a;
          a = c;
        } else if (c > b) {
          b = c;
        }
      }
      gs[w][g] = n > 1 ? a + b : a;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    // a group stays if fewer than `keep` groups beat it (larger score, or
    // the same score and a smaller index)
    for (int g = lane; g < groups; g += 64) {
      const float mine = gs[w][g];
      int beat = 0;
      for (int o = 0; o < groups; ++o) {
        const float s = gs[w][o];
        beat += (s > mine || (s == mine && o < g)) ? 1 : 0;
      }
      if (beat >= keep)
        for (int e = g * n; e < (g + 1) * n; ++e) cs[w][e] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  float sc[kRouteSlots];
#pragma unroll
  for (int j = 0; j < kRouteSlots; ++j) {
    const int e = lane + 64 * j;
    sc[j] = e < E ? cs[w][e] : -INFINITY;
  }
  unsigned taken = 0;      // bit j: slot j of this lane is already chosen
  for (int it = 0; it < k; ++it) {
    float v = -INFINITY;
    int idx = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j) {
      const int e = lane + 64 * j;
      // ascending j: the smaller index wins ties
      if (e < E && !((taken >> j) & 1u) &&
          (idx == 0x7fffffff || sc[j] > v)) {
        v = sc[j];
        idx = e;
      }
    }
#pragma unroll
    for (int off = 32; off; off >>= 1) {
      const float ov = __shfl_xor(v, off);
      const int oi = __shfl_xor(idx, off);
      if (oi != 0x7fffffff &&
          (idx == 0x7fffffff || ov > v || (ov == v && oi < idx))) {
        v = ov;
        idx = oi;
      }
    }
    if (lane == 0) {
      topi[static_cast<int64_t>(t) * k + it] = idx;
      topv[static_cast<int64_t>(t) * k + it] =
          1.0f / (1.0f + expf(-row[idx]));
    }
#pragma unroll
    for (int j = 0; j < kRouteSlots; ++j)
      if (idx == lane + 64 * j) taken |= 1u << j;
  }
}

constexpr int kPlainBM = 16;   // rows per workgroup
constexpr int kPlainBN = 64;   // columns per workgroup
constexpr int kPlainKT = 32;   // K step

template <typename A, int MODE>
__global__ __launch_bounds__(256) void moe_gemm_plain_kernel(
    A* __restrict__ out,                // [PM, N]
    const A* __restrict__ a,            // GATE_UP: x [T, K]; else act [PM, K]
    const A* __restrict__ w,            // [E, GATE_UP ? 2N : N, K]
    const int* __restrict__ sorted_ids, const int* __restrict__ expert_ids,
    const int* __restrict__ n_valid, const int K, const int N,
    const int block_m, const float limit) {
  constexpr bool GATE_UP = MODE == 1 || MODE == 3;
  constexpr bool GATHER = MODE != 0;
  // m-tiles are block_m rows; this workgroup covers 16 of them
  const int sub = block_m / kPlainBM;
  const int mtile = blockIdx.x / sub;
  if (mtile >= *n_valid) return;
  const int row0 = mtile * block_m + (blockIdx.x % sub) * kPlainBM;
  const int col0 = blockIdx.y * kPlainBN;
  const int e = expert_ids[mtile];
  const int NB = GATE_UP ? 2 * N : N;
  const A* we = w + static_cast<int64_t>(e) * NB * K;

  __shared__ float As[kPlainBM][kPlainKT + 1];
  __shared__ float Ws[(GATE_UP ? 2 : 1) * kPlainBN][kPlainKT + 1];
  __shared__ int rows[kPlainBM];
  const int tid = threadIdx.x;
  if (tid < kPlainBM)
    rows[tid] = GATHER ? sorted_ids[row0 + tid] : row0 + tid;
  __syncthreads();

  const int r = tid / 16;        // output row 0..15
  const int cg = tid % 16;       // output columns cg + 16 j
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float acc2[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kPlainKT) {
    for (int i = tid; i < kPlainBM * kPlainKT; i += 256) {
      const int rr = i / kPlainKT, kk = i % kPlainKT;
      As[rr][kk] = k0 + kk < K
          ? Act<A>::ld(a + static_cast<int64_t>(rows[rr]) * K + k0 + kk)
          : 0.f;
    }
    for (int i = tid; i < kPlainBN * kPlainKT; i += 256) {
      const int cc = i / kPlainKT, kk = i % kPlainKT;
      const bool ok = col0 + cc < N && k0 + kk < K;
      Ws[cc][kk] = ok
          ? Act<A>::ld(we + static_cast<int64_t>(col0 + cc) * K + k0 + kk)
          : 0.f;
      if (GATE_UP)
        Ws[kPlainBN + cc][kk] = ok
            ? Act<A>::ld(we + static_cast<int64_t>(N + col0 + cc) * K + k0 +
                         kk)
            : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < kPlainKT; ++kk) {
      const float av = As[r][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] += av * Ws[cg + 16 * j][kk];
        if (GATE_UP) acc2[j] += av * Ws[kPlainBN + cg + 16 * j][kk];
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = col0 + cg + 16 * j;
    if (c >= N) continue;
    float v = acc[j];
    if (MODE == 3) {
      const float g = fminf(acc[j], limit);
      const float u = fminf(fmaxf(acc2[j], -limit), limit);
      v = g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    } else if (GATE_UP) {
      const float g = acc[j];
      v = g / (1.0f + expf(-g)) * acc2[j];
    } else if (MODE == 2) {
      v = fmaxf(v, 0.f);
      v *= v;
    }
    Act<A>::st(out + static_cast<int64_t>(row0 + r) * N + c, v);
  }
}

template <typename A>
__global__ __launch_bounds__(256) void moe_combine_kernel(
    A* __restrict__ out, const A* __restrict__ y, const int* __restrict__ pos,
    const float* __restrict__ w, const int topk, const int H) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= H) return;
  float acc = 0.f;
  for (int k = 0; k < topk; ++k) {
    const int p = pos[t * topk + k];
    if (p < 0) continue;
    acc += w[t * topk + k] * Act<A>::ld(y + static_cast<int64_t>(p) * H + c);
  }
  Act<A>::st(out + static_cast<int64_t>(t) * H + c, acc);
}

}  // namespace

void launch_moe_route(const float* logits, float* topv, int* topi, int T,
                      int E, int k, bool sigmoid, bool renorm, float scale,
                      hipStream_t stream) {
  hipLaunchKernelGGL(moe_route_kernel, dim3(ceil_div(T, 4)), dim3(256), 0,
                     stream, logits, topv, topi, T, E, k, sigmoid, renorm,
                     scale);
}

void launch_moe_route_grouped(const float* logits, const float* correction,
                              float* topv, int* topi, int T, int E, int k,
                              int groups, int keep, hipStream_t stream) {
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3(ceil_div(T, 4)),
                     dim3(256), 0, stream, logits, correction, topv, topi, T,
                     E, k, groups, keep);
}

template <typename A>
void launch_moe_gemm_plain(A* out, const A* a, const A* w,
                           const int* sorted_ids, const int* expert_ids,
                           const int* n_valid, int PM, int K, int N,
                           int block_m, int mode, float limit,
                           hipStream_t stream) {
  const dim3 grid(PM / kPlainBM, ceil_div(N, kPlainBN));
  if (mode == 1)
    hipLaunchKernelGGL((moe_gemm_plain_kernel<A, 1>), grid, dim3(256), 0,
                       stream, out, a, w, sorted_ids, expert_ids, n_valid, K,
                       N, block_m, limit);
  else if (mode == 3)
    hipLaunchKernelGGL((moe_gemm_plain_kernel<A, 3>), grid, dim3(256), 0,
                       stream, out, a, w, sorted_ids, expert_ids, n_valid, K,
                       N, block_m, limit);
  else if (mode == 2)
    hipLaunchKernelGGL((moe_gemm_plain_kernel<A, 2>), grid, dim3(256), 0,
                       stream, out, a, w, sorted_ids, expert_ids, n_valid, K,
                       N, block_m, limit);
  else
    hipLaunchKernelGGL((moe_gemm_plain_kernel<A, 0>), grid, dim3(256), 0,
                       stream, out, a, w, sorted_ids, expert_ids, n_valid, K,
                       N, block_m, limit);
}

template <typename A>
void launch_moe_combine(A* out, const A* y, const int* pos, const float* w,
                        int tokens, int topk, int H, hipStream_t stream) {
  const dim3 grid(ceil_div(H, 256), tokens);
  hipLaunchKernelGGL(moe_combine_kernel<A>, grid, dim3(256), 0, stream, out,
                     y, pos, w, topk, H);
}

#define FI_INST(A)                                                            \
  template void launch_moe_gemm_plain<A>(A*, const A*, const A*, const int*,  \
                                         const int*, const int*, int, int,    \
                                         int, int, int, float, hipStream_t);  \
  template void launch_moe_combine<A>(A*, const A*, const int*, const float*, \
                                      int, int, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
