// Causal softmax attention over the paged cache with separate key and
// value sizes, an optional per-head sink in the denominator, values that
// may be a leading slice of the cached key rows, an optional sigmoid gate
// on the result (per (row, head), or per entry), and an optional sliding
// window that keeps the first keys: with window > 0 position p sees key j
// only if p - j < window or j < keep_first. Tiles and spans that no row
// can see are skipped.
//
//  * split form (any sizes): a workgroup takes one row, a batch of up to
//    8 query heads that share a key/value head, and one span of 256 keys:
//    one key per thread for the scores (the key row is read once for the
//    whole head batch, queries come from LDS), block-wide fp32 softmax
//    statistics of the span, then the weighted value sum with the value
//    columns spread over the threads. Spans are merged by a combine
//    kernel, which also adds the sink to the denominator, applies the
//    gate and rounds. Decoded rows use it, and prompt rows whose sizes
//    the tiled form does not cover.
//  * tiled MFMA form: a 4-wave workgroup takes 64*QS consecutive rows of
//    one (sequence, head) and walks the keys 0..last row's position in
//    LDS-staged tiles; S^T = K Q^T and O^T = V^T P^T run on the matrix
//    cores (bf16 16x16x16, or true-fp32 16x16x4 for fp32 activations),
//    softmax statistics stay fp32 per lane.
//
// Cache layout: [num_blocks, kv_heads, block_size, row]; the value row
// stride is a parameter so that values can alias the key rows.

#include <type_traits>

#include "seqmix.h"

namespace fi {

namespace {

constexpr int kSpanKeys = 256;   // keys per workgroup of the split form
constexpr int kHeadBatch = 8;    // query heads per workgroup

FI_DEV bool key_visible(int p, int j, int window, int keep_first) {
  return j <= p && (window <= 0 || p - j < window || j < keep_first);
}

// a 256-key span holds at least one key that position p sees
FI_DEV bool span_live(int p, int j0, int window, int keep_first) {
  return j0 <= p && (window <= 0 || j0 < keep_first ||
                     j0 + kSpanKeys > p - window + 1);
}

template <typename A, int VW>
__global__ __launch_bounds__(256) void sink_attention_split_kernel(
    float* __restrict__ part_ml,      // [rows, H, ns, 2]
    float* __restrict__ part_o,       // [rows, H, ns, DV]
    const A* __restrict__ q,          // [T, H, DK]
    const A* __restrict__ k_cache, const A* __restrict__ v_cache, int v_row,
    const int* __restrict__ seq_bt, int bt_stride,
    const int* __restrict__ row_seq, const int* __restrict__ positions,
    int row0, int H, int G, int DK, int DV, int dv_round, int bs, float scale,
    int ns, int hb, int tpr, int window, int keep_first) {
  extern __shared__ float smem[];
  float* qs = smem;                               // [kHeadBatch][DK]
  float* ps = qs + kHeadBatch * DK;               // [kHeadBatch][256]
  float* red = ps + kHeadBatch * kSpanKeys;       // [kHeadBatch][4] x 2
  float* osum = red + 2 * kHeadBatch * 4;         // [groups][kHeadBatch][dv_round]
  __shared__ int64_t voff[kSpanKeys];

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int r = blockIdx.x;
  const int t = row0 + r;
  const int rep = H / G;
  const int nbg = (rep + hb - 1) / hb;            // head batches per kv head
  const int g = blockIdx.y / nbg;
  const int h0 = g * rep + (blockIdx.y % nbg) * hb;
  const int nh = min(hb, (g + 1) * rep - h0);
  const int span = blockIdx.z;
  const int p = positions[t];
  const int j0 = span * kSpanKeys;
  // the combine step never reads a span that is not live
  if (!span_live(p, j0, window, keep_first)) return;
  const int nkeys = min(kSpanKeys, p - j0 + 1);

  const A* qp = q + (static_cast<int64_t>(t) * H + h0) * DK;
  for (int i = tid; i < kHeadBatch * DK; i += 256)
    qs[i] = i < nh * DK ? Act<A>::ld(qp + i) : 0.f;
  __syncthreads();

  const int* bt = seq_bt + static_cast<int64_t>(row_seq[t]) * bt_stride;
  // keys outside the window keep a weight of zero; their value rows are
  // still addressed (they stay in the sequence's pages)
  const bool valid =
      tid < nkeys && key_visible(p, j0 + tid, window, keep_first);
  float dots[kHeadBatch];
#pragma unroll
  for (int i = 0; i < kHeadBatch; ++i) dots[i] = 0.f;
  int64_t rowi = 0;
  if (tid < nkeys) {
    const int j = j0 + tid;
    rowi = (static_cast<int64_t>(bt[j / bs]) * G + g) * bs + j % bs;
    voff[tid] = rowi * v_row;
  }
  if (valid) {
    const A* kp = k_cache + rowi * DK;
    for (int d0 = 0; d0 < DK; d0 += VW) {
      float kv[VW];
      ldv<A, VW>(kp + d0, kv);
#pragma unroll
      for (int i = 0; i < kHeadBatch; ++i)
#pragma unroll
        for (int e = 0; e < VW; ++e) dots[i] += kv[e] * qs[i * DK + d0 + e];
    }
  }
  // span statistics per head
  float sc[kHeadBatch];
#pragma unroll
  for (int i = 0; i < kHeadBatch; ++i) {
    sc[i] = valid ? dots[i] * scale : -INFINITY;
    const float wm = wave_reduce_max(sc[i]);
    if (lane == 0) red[i * 4 + wave] = wm;
  }
  __syncthreads();
  float l_part[kHeadBatch];
#pragma unroll
  for (int i = 0; i < kHeadBatch; ++i) {
    const float m = fmaxf(fmaxf(red[i * 4], red[i * 4 + 1]),
                          fmaxf(red[i * 4 + 2], red[i * 4 + 3]));
    const float pj = valid ? expf(sc[i] - m) : 0.f;
    ps[i * kSpanKeys + tid] = pj;
    sc[i] = m;
    l_part[i] = wave_reduce_sum(pj);
    if (lane == 0) red[(kHeadBatch + i) * 4 + wave] = l_part[i];
  }
  __syncthreads();
  if (tid < nh) {
    const int i = tid;
    const float m = fmaxf(fmaxf(red[i * 4], red[i * 4 + 1]),
                          fmaxf(red[i * 4 + 2], red[i * 4 + 3]));
    const float l = red[(kHeadBatch + i) * 4] + red[(kHeadBatch + i) * 4 + 1] +
                    red[(kHeadBatch + i) * 4 + 2] +
                    red[(kHeadBatch + i) * 4 + 3];
    float* ml =
        part_ml + ((static_cast<int64_t>(r) * H + h0 + i) * ns + span) * 2;
    ml[0] = m;
    ml[1] = l;
  }
  if constexpr (VW > 1) {
    if (tpr > 0) {
      // vector form: tpr threads share a value row, VW columns each; the
      // 64 / tpr key groups of a wave are folded by shuffles, the four
      // waves through LDS (osum: [4][kHeadBatch][DV])
      const int kgw = 64 / tpr;
      const int dcol = (lane % tpr) * VW;
      const int gid = wave * kgw + lane / tpr;
      float acc[kHeadBatch][VW];
#pragma unroll
      for (int i = 0; i < kHeadBatch; ++i)
#pragma unroll
        for (int e = 0; e < VW; ++e) acc[i][e] = 0.f;
      if (dcol < DV) {
        for (int jj = gid; jj < nkeys; jj += 4 * kgw) {
          float vv[VW];
          ldv<A, VW>(v_cache + voff[jj] + dcol, vv);
#pragma unroll
          for (int i = 0; i < kHeadBatch; ++i) {
            const float pj = ps[i * kSpanKeys + jj];
#pragma unroll
            for (int e = 0; e < VW; ++e) acc[i][e] += pj * vv[e];
          }
        }
      }
      for (int off = tpr; off < 64; off <<= 1)
#pragma unroll
        for (int i = 0; i < kHeadBatch; ++i)
#pragma unroll
          for (int e = 0; e < VW; ++e)
            acc[i][e] += __shfl_xor(acc[i][e], off, 64);
      if (lane < tpr && dcol < DV) {
#pragma unroll
        for (int i = 0; i < kHeadBatch; ++i)
#pragma unroll
          for (int e = 0; e < VW; ++e)
            osum[(wave * kHeadBatch + i) * DV + dcol + e] = acc[i][e];
      }
      __syncthreads();
      for (int idx = tid; idx < nh * DV; idx += 256) {
        const int i = idx / DV, d = idx % DV;
        part_o[((static_cast<int64_t>(r) * H + h0 + i) * ns + span) * DV + d] =
            osum[i * DV + d] + osum[(kHeadBatch + i) * DV + d] +
            osum[(2 * kHeadBatch + i) * DV + d] +
            osum[(3 * kHeadBatch + i) * DV + d];
      }
      return;
    }
  }
  // weighted value sum: column d = tid % dv_round (+ dv_round ...), keys
  // dealt round-robin to the 256 / dv_round thread groups
  const int groups = max(1, 256 / dv_round);
  const int kg = dv_round >= 256 ? 0 : tid / dv_round;
  const int dcol = dv_round >= 256 ? tid : tid % dv_round;
  for (int d = dcol; d < DV; d += max(dv_round, 256)) {
    float acc[kHeadBatch];
#pragma unroll
    for (int i = 0; i < kHeadBatch; ++i) acc[i] = 0.f;
    for (int jj = kg; jj < nkeys; jj += groups) {
      const float v = Act<A>::ld(v_cache + voff[jj] + d);
#pragma unroll
      for (int i = 0; i < kHeadBatch; ++i)
        acc[i] += ps[i * kSpanKeys + jj] * v;
    }
    if (groups == 1) {
      for (int i = 0; i < nh; ++i)
        part_o[((static_cast<int64_t>(r) * H + h0 + i) * ns + span) * DV + d] =
            acc[i];
    } else {
#pragma unroll
      for (int i = 0; i < kHeadBatch; ++i)
        osum[(kg * kHeadBatch + i) * dv_round + d] = acc[i];
    }
  }
  if (groups > 1) {
    __syncthreads();
    for (int idx = tid; idx < nh * DV; idx += 256) {
      const int i = idx / DV, d = idx % DV;
      float s = 0.f;
      for (int k2 = 0; k2 < groups; ++k2)
        s += osum[(k2 * kHeadBatch + i) * dv_round + d];
      part_o[((static_cast<int64_t>(r) * H + h0 + i) * ns + span) * DV + d] =
          s;
    }
  }
}

template <typename A>
__global__ __launch_bounds__(64) void sink_attention_combine_kernel(
    A* __restrict__ out,              // [T, H, DV]
    const float* __restrict__ part_ml, const float* __restrict__ part_o,
    const int* __restrict__ positions, const float* __restrict__ sink,
    const A* __restrict__ gate, int64_t g_stride, int gate_elem, int row0,
    int H, int DV, int ns, int window, int keep_first) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int t = row0 + r;
  const int lane = threadIdx.x;
  const int p = positions[t];
  const int nsp = p / kSpanKeys + 1;
  // with a window the live spans are those of the kept first keys and
  // those that reach into the window
  int s_win = 0, s_keep = nsp;
  if (window > 0) {
    s_win = max(p - window + 1, 0) / kSpanKeys;
    s_keep = min(s_win, (keep_first + kSpanKeys - 1) / kSpanKeys);
  }
  const float* ml = part_ml + (static_cast<int64_t>(r) * H + h) * ns * 2;
  const float* po = part_o + (static_cast<int64_t>(r) * H + h) * ns * DV;
  auto live = [&](int s) { return s < s_keep || s >= s_win; };
  float m = sink != nullptr ? sink[h] : -INFINITY;
  for (int s = 0; s < nsp; ++s)
    if (live(s)) m = fmaxf(m, ml[2 * s]);
  float l = sink != nullptr ? expf(sink[h] - m) : 0.f;
  for (int s = 0; s < nsp; ++s)
    if (live(s)) l += ml[2 * s + 1] * expf(ml[2 * s] - m);
  float f = 1.0f / l;
  const A* gp = nullptr;
  if (gate != nullptr) {
    if (gate_elem)
      gp = gate + t * g_stride + static_cast<int64_t>(h) * DV;
    else
      f *= sigmoidf_acc(Act<A>::ld(gate + t * g_stride + h));
  }
  A* op = out + (static_cast<int64_t>(t) * H + h) * DV;
  for (int d = lane; d < DV; d += 64) {
    float acc = 0.f;
    for (int s = 0; s < nsp; ++s)
      if (live(s))
        acc += po[static_cast<int64_t>(s) * DV + d] * expf(ml[2 * s] - m);
    acc *= f;
    if (gp != nullptr) acc *= sigmoidf_acc(Act<A>::ld(gp + d));
    Act<A>::st(op + d, acc);
  }
}

typedef __attribute__((ext_vector_type(4))) short short4v;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

template <typename A, int DK, int DV, int BN, int QS, int HP>
__global__ __launch_bounds__(256) void sink_attention_tile_kernel(
    A* __restrict__ out, const A* __restrict__ q,
    const A* __restrict__ k_cache, const A* __restrict__ v_cache, int v_row,
    const int* __restrict__ seq_bt, int bt_stride,
    const int* __restrict__ seq_cu, const int* __restrict__ positions,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_row0,
    const float* __restrict__ sink, const A* __restrict__ gate,
    int64_t g_stride, int gate_elem, int H, int G, int block_size,
    float scale, int window, int keep_first) {
  constexpr bool BF = std::is_same<A, u16>::value;
  constexpr int VEC = BF ? 8 : 4;               // elements per 16-byte load
  constexpr int KP = DK + (BF ? 8 : 4);         // K tile [BN][KP]
  constexpr int VP = BF ? BN + 4 : DV + 4;      // bf16: V^T [DV][VP]; fp32: V [BN][VP]
  constexpr int NB = BN / 16;
  constexpr int KB = DK / 16;
  constexpr int DB = DV / 16;
  constexpr int ROWS = 64 * QS;
  // a wave keeps NQ query sets: QS row sets for each of HP heads that
  // share the key/value head, so every K/V fragment read feeds NQ MFMAs
  constexpr int NQ = QS * HP;
  __shared__ __attribute__((aligned(16))) A k_lds[BN * KP];
  __shared__ __attribute__((aligned(16))) A v_lds[BF ? DV * VP : BN * VP];

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int g4 = lane / 16, c16 = lane % 16;
  const int h0 = blockIdx.y * HP;
  const int g = h0 / (H / G);
  const int s = tile_seq[blockIdx.x];
  // the tile table counts 128 rows per entry; with QS == 1 a workgroup
  // covers half an entry and blockIdx.z picks the half
  const int row_first =
      seq_cu[s] + tile_row0[blockIdx.x] + static_cast<int>(blockIdx.z) * ROWS;
  const int tile_end =
      min(seq_cu[s + 1], seq_cu[s] + tile_row0[blockIdx.x] + 128);
  const int nrows = min(ROWS, tile_end - row_first);
  if (nrows <= 0) return;
  const int* bt = seq_bt + static_cast<int64_t>(s) * bt_stride;
  const int p_first = positions[row_first];
  const int kv_hi = p_first + nrows - 1;   // positions in a group ascend by 1

  int my_row[NQ], my_pos[NQ];
  bool row_ok[NQ];
  short4v qf16[NQ][BF ? KB : 1];
  float qf32[NQ][BF ? 1 : DK / 4];
#pragma unroll
  for (int qs = 0; qs < NQ; ++qs) {
    my_row[qs] = (wave * QS + qs % QS) * 16 + c16;
    row_ok[qs] = my_row[qs] < nrows;
    my_pos[qs] = row_ok[qs] ? p_first + my_row[qs] : -1;
    const A* qp = q + (static_cast<int64_t>(row_first + my_row[qs]) * H +
                       h0 + qs / QS) * DK;
    if constexpr (BF) {
#pragma unroll
      for (int kk = 0; kk < KB; ++kk) {
        if (row_ok[qs])
          qf16[qs][kk] =
              *reinterpret_cast<const short4v*>(qp + 16 * kk + 4 * g4);
        else
          qf16[qs][kk] = short4v{0, 0, 0, 0};
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < DK / 4; ++kk)
        qf32[qs][kk] = row_ok[qs] ? qp[4 * kk + g4] : 0.f;
    }
  }

  floatx4 o[NQ][DB];
  float m[NQ], l[NQ];
#pragma unroll
  for (int qs = 0; qs < NQ; ++qs) {
    m[qs] = -INFINITY;
    l[qs] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[qs][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  // bf16 activations: softmax in the log2 domain (scale * log2(e) folded
  // into the scores, hardware exp2); fp32 activations keep expf
  constexpr float kLog2e = 1.4426950408889634f;
  const float sc = BF ? scale * kLog2e : scale;
  auto ex = [](float x) {
    return BF ? __builtin_amdgcn_exp2f(x) : expf(x);
  };
  const int wave_rows = min(16 * QS, nrows - wave * 16 * QS);
  const int wave_min_pos = wave_rows > 0 ? p_first + wave * 16 * QS : -1;
  const int wave_max_pos = wave_min_pos + wave_rows - 1;
  const bool wave_full = wave_rows == 16 * QS;
  // key tiles nobody in the workgroup sees lie between the kept first keys
  // and the window of the first row (the one that reaches back farthest)
  const int skip_lo = ((keep_first + BN - 1) / BN) * BN;
  const int skip_hi =
      window > 0 ? (max(p_first - window + 1, 0) / BN) * BN : 0;
  auto next_tile = [&](int j0) {
    const int j = j0 + BN;
    return (j >= skip_lo && j < skip_hi) ? skip_hi : j;
  };
  const int j_start = (skip_lo == 0 && skip_hi > 0) ? skip_hi : 0;

  // K and V tiles travel global -> registers -> LDS. With PF (the large
  // sizes, whose register budget is spent anyway) the loads of the NEXT
  // tile are issued right after the barrier that publishes the current
  // one, so they are in flight during the MFMA phases; the small sizes
  // load at the top of the iteration and keep the registers for a third
  // wave per SIMD.
  constexpr bool PF = QS == 1;
  constexpr int KPR = DK / VEC;                // vectors per key row
  constexpr int VPR = DV / VEC;
  constexpr int KV = (BN * KPR + 255) / 256;   // K vectors per thread
  constexpr int VN = BF ? ((BN / 2) * VPR + 255) / 256   // V key pairs
                        : (BN * VPR + 255) / 256;        // V vectors
  u32x4 kreg[KV];
  u32x4 vreg[VN][BF ? 2 : 1];
  auto row_index = [&](int key) {
    return (static_cast<int64_t>(bt[key / block_size]) * G + g) * block_size +
           key % block_size;
  };
  auto load_tile = [&](int j0) {
#pragma unroll
    for (int i = 0; i < KV; ++i) {
      const int vid = tid + 256 * i;
      const int key = j0 + vid / KPR;
      kreg[i] = u32x4{0u, 0u, 0u, 0u};
      if (vid < BN * KPR && key <= kv_hi)
        kreg[i] = *reinterpret_cast<const u32x4*>(
            k_cache + row_index(key) * DK + (vid % KPR) * VEC);
    }
    if constexpr (BF) {
      // lane quads take four adjacent key pairs of one column vector:
      // their transposed stores fall into consecutive LDS words, and 16
      // lanes still read 256 contiguous bytes of a key row
#pragma unroll
      for (int i = 0; i < VN; ++i) {
        const int pid = tid + 256 * i;
        const int kp = (pid & 3) + 4 * (pid / (4 * VPR));
        const int dv = (pid >> 2) % VPR;
#pragma unroll
        for (int e2 = 0; e2 < 2; ++e2) {
          const int key = j0 + 2 * kp + e2;
          vreg[i][e2] = u32x4{0u, 0u, 0u, 0u};
          if (pid < (BN / 2) * VPR && key <= kv_hi)
            vreg[i][e2] = *reinterpret_cast<const u32x4*>(
                v_cache + row_index(key) * v_row + dv * VEC);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < VN; ++i) {
        const int vid = tid + 256 * i;
        const int key = j0 + vid / VPR;
        vreg[i][0] = u32x4{0u, 0u, 0u, 0u};
        if (vid < BN * VPR && key <= kv_hi)
          vreg[i][0] = *reinterpret_cast<const u32x4*>(
              v_cache + row_index(key) * v_row + (vid % VPR) * VEC);
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < KV; ++i) {
      const int vid = tid + 256 * i;
      if (vid < BN * KPR)
        *reinterpret_cast<u32x4*>(k_lds + (vid / KPR) * KP +
                                  (vid % KPR) * VEC) = kreg[i];
    }
    if constexpr (BF) {
      // the transposed V tile is written with 4-byte stores: one
      // (key, key+1) pair per value column
#pragma unroll
      for (int i = 0; i < VN; ++i) {
        const int pid = tid + 256 * i;
        if (pid >= (BN / 2) * VPR) continue;
        const int kp = (pid & 3) + 4 * (pid / (4 * VPR));
        const int dv = (pid >> 2) % VPR;
        const u16* va = reinterpret_cast<const u16*>(&vreg[i][0]);
        const u16* vb = reinterpret_cast<const u16*>(&vreg[i][1]);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          *reinterpret_cast<u32*>(v_lds + (dv * 8 + e) * VP + 2 * kp) =
              static_cast<u32>(va[e]) | (static_cast<u32>(vb[e]) << 16);
      }
    } else {
#pragma unroll
      for (int i = 0; i < VN; ++i) {
        const int vid = tid + 256 * i;
        if (vid < BN * VPR)
          *reinterpret_cast<u32x4*>(v_lds + (vid / VPR) * VP +
                                    (vid % VPR) * VEC) = vreg[i][0];
      }
    }
  };

  if constexpr (PF) load_tile(j_start);
  for (int j0 = j_start; j0 <= kv_hi; j0 = next_tile(j0)) {
    if constexpr (!PF) load_tile(j0);
    store_tile();
    __syncthreads();
    if constexpr (PF) {
      if (next_tile(j0) <= kv_hi) load_tile(next_tile(j0));
    }

    // ---- S^T = K Q^T ----
    const bool interior =
        wave_full && j0 + BN - 1 <= wave_min_pos &&
        (window <= 0 || wave_max_pos - j0 < window || j0 + BN <= keep_first);
    float sv[NQ][NB][4];
    float tmax[NQ];
#pragma unroll
    for (int qs = 0; qs < NQ; ++qs) tmax[qs] = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      floatx4 acc[NQ];
#pragma unroll
      for (int qs = 0; qs < NQ; ++qs) acc[qs] = floatx4{0.f, 0.f, 0.f, 0.f};
      const A* kr = k_lds + (nb * 16 + c16) * KP;
      if constexpr (BF) {
#pragma unroll
        for (int kk = 0; kk < KB; ++kk) {
          const short4v a =
              *reinterpret_cast<const short4v*>(kr + 16 * kk + 4 * g4);
#pragma unroll
          for (int qs = 0; qs < NQ; ++qs)
            acc[qs] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                a, qf16[qs][kk], acc[qs], 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < DK / 4; ++kk) {
          const float a = kr[4 * kk + g4];
#pragma unroll
          for (int qs = 0; qs < NQ; ++qs)
            acc[qs] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, qf32[qs][kk],
                                                           acc[qs], 0, 0, 0);
        }
      }
#pragma unroll
      for (int qs = 0; qs < NQ; ++qs)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = j0 + nb * 16 + 4 * g4 + i;
          const bool vis =
              interior || key_visible(my_pos[qs], key, window, keep_first);
          sv[qs][nb][i] = vis ? acc[qs][i] * sc : -INFINITY;
          tmax[qs] = fmaxf(tmax[qs], sv[qs][nb][i]);
        }
    }
#pragma unroll
    for (int qs = 0; qs < NQ; ++qs) {
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

    // ---- O^T += V^T P^T ----
    if constexpr (BF) {
      short4v pf[NQ][NB];
#pragma unroll
      for (int qs = 0; qs < NQ; ++qs)
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
          for (int qs = 0; qs < NQ; ++qs)
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
            for (int qs = 0; qs < NQ; ++qs)
              o[qs][db] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                  a, sv[qs][nb][i], o[qs][db], 0, 0, 0);
          }
    }
    __syncthreads();
  }

#pragma unroll
  for (int qs = 0; qs < NQ; ++qs) {
    if (!row_ok[qs]) continue;
    const int h = h0 + qs / QS;
    float lt = l[qs];
    if (sink != nullptr) {
      // the sink joins the denominator in the domain of the running max
      const float sk = BF ? sink[h] * kLog2e : sink[h];
      const float m_new = fmaxf(m[qs], sk);
      const float corr = ex(m[qs] - m_new);
      lt = lt * corr + ex(sk - m_new);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[qs][db][i] *= corr;
    }
    float f = 1.0f / lt;
    const int64_t row = row_first + my_row[qs];
    const A* gp = nullptr;
    if (gate != nullptr) {
      if (gate_elem)
        gp = gate + row * g_stride + static_cast<int64_t>(h) * DV;
      else
        f *= sigmoidf_acc(Act<A>::ld(gate + row * g_stride + h));
    }
    A* op = out + (row * H + h) * DV;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = db * 16 + 4 * g4 + i;
        float val = o[qs][db][i] * f;
        if (gp != nullptr) val *= sigmoidf_acc(Act<A>::ld(gp + d));
        Act<A>::st(op + d, val);
      }
  }
}

}  // namespace

int sink_attention_splits(int max_keys) {
  return max(1, (max_keys + kSpanKeys - 1) / kSpanKeys);
}

// (key size, value size) pairs the tiled form is built for; keep in step
// with the FI_TILE list below
bool sink_attention_has_tiles(int DK, int DV) {
  return (DK == 64 && DV == 64) || (DK == 96 && DV == 96) ||
         (DK == 128 && DV == 128) || (DK == 112 && DV == 96) ||
         (DK == 288 && DV == 256);
}

template <typename A>
bool launch_sink_attention_tiles(A* out, const A* q, const A* k_cache,
                                 const A* v_cache, int v_row,
                                 const int* seq_bt, int bt_stride,
                                 const int* seq_cu, const int* positions,
                                 const int* tile_seq, const int* tile_row0,
                                 int num_tiles, const float* sink,
                                 const A* gate, int64_t g_stride,
                                 int gate_elem, int H, int G, int DK, int DV,
                                 int block_size, float scale, int window,
                                 int keep_first, hipStream_t s) {
  constexpr bool BF = std::is_same<A, u16>::value;
  if (num_tiles == 0) return true;
  // head pairs (HP_ == 2) need an even number of heads per key/value head
  const bool pairs = (H / G) % 2 == 0;
#define FI_TILE(K_, V_, BNB, BNF, QS_, HP_)                                    \
  if (DK == K_ && DV == V_ && (HP_ == 1 || pairs)) {                           \
    hipLaunchKernelGGL(                                                        \
        (sink_attention_tile_kernel<A, K_, V_, (BF ? BNB : BNF), QS_, HP_>),   \
        dim3(num_tiles, H / HP_, 2 / QS_), dim3(256), 0, s, out, q, k_cache,   \
        v_cache, v_row, seq_bt, bt_stride, seq_cu, positions, tile_seq,        \
        tile_row0, sink, gate, g_stride, gate_elem, H, G, block_size, scale,   \
        window, keep_first);                                                   \
    return true;                                                               \
  }
  FI_TILE(64, 64, 64, 64, 2, 1)
  FI_TILE(96, 96, 64, 32, 2, 1)
  FI_TILE(128, 128, 64, 32, 2, 1)
  FI_TILE(112, 96, 64, 32, 2, 1)
  FI_TILE(288, 256, 32, 16, 1, 2)
  FI_TILE(288, 256, 32, 16, 1, 1)
#undef FI_TILE
  return false;   // caller falls back to the split form
}

template <typename A>
void launch_sink_attention_rows(A* out, float* part_ml, float* part_o,
                                const A* q, const A* k_cache,
                                const A* v_cache, int v_row,
                                const int* seq_bt, int bt_stride,
                                const int* row_seq, const int* positions,
                                const float* sink, const A* gate,
                                int64_t g_stride, int gate_elem, int row0,
                                int rows, int H, int G, int DK, int DV,
                                int block_size, float scale, int ns,
                                int window, int keep_first, hipStream_t s) {
  if (rows == 0) return;
  const int rep = H / G;
  const int hb = min(kHeadBatch, rep);
  const int nbg = (rep + hb - 1) / hb;
  int dv_round = 1;
  while (dv_round < DV && dv_round < 256) dv_round *= 2;
  const int groups = max(1, 256 / dv_round);
  constexpr bool BF = std::is_same<A, u16>::value;
  // widest vector both the key rows and the value rows allow
  int vw = 1;
  if (BF && DK % 8 == 0) vw = 8;
  else if (DK % 4 == 0) vw = 4;
  // vector form of the value sum: whole vectors per value row, at most
  // 64 threads a row, four partial copies within the LDS budget
  int tpr = 0;
  if (vw > 1 && DV % vw == 0 && v_row % vw == 0 && DV / vw <= 64 &&
      DV <= 256) {
    tpr = 1;
    while (tpr < DV / vw) tpr *= 2;
  }
  const size_t osum_floats =
      tpr > 0 ? static_cast<size_t>(4) * kHeadBatch * DV
              : (groups > 1 ? static_cast<size_t>(groups) * kHeadBatch *
                                  dv_round
                            : 0);
  const size_t lds =
      (static_cast<size_t>(kHeadBatch) * DK + kHeadBatch * kSpanKeys +
       2 * kHeadBatch * 4 + osum_floats) * sizeof(float);
  const dim3 grid(rows, G * nbg, ns);
#define FI_SPLIT(VW_)                                                          \
  hipLaunchKernelGGL((sink_attention_split_kernel<A, VW_>), grid, dim3(256),   \
                     lds, s, part_ml, part_o, q, k_cache, v_cache, v_row,      \
                     seq_bt, bt_stride, row_seq, positions, row0, H, G, DK,    \
                     DV, dv_round, block_size, scale, ns, hb, tpr, window,     \
                     keep_first)
  if constexpr (BF) {
    if (vw == 8) FI_SPLIT(8);
    else if (vw == 4) FI_SPLIT(4);
    else FI_SPLIT(1);
  } else {
    if (vw == 4) FI_SPLIT(4);
    else FI_SPLIT(1);
  }
#undef FI_SPLIT
  hipLaunchKernelGGL(sink_attention_combine_kernel<A>, dim3(rows, H), dim3(64),
                     0, s, out, part_ml, part_o, positions, sink, gate,
                     g_stride, gate_elem, row0, H, DV, ns, window, keep_first);
}

#define FI_INST(A)                                                             \
  template bool launch_sink_attention_tiles<A>(                                \
      A*, const A*, const A*, const A*, int, const int*, int, const int*,      \
      const int*, const int*, const int*, int, const float*, const A*,         \
      int64_t, int, int, int, int, int, int, float, int, int, hipStream_t);    \
  template void launch_sink_attention_rows<A>(                                 \
      A*, float*, float*, const A*, const A*, const A*, int, const int*, int,  \
      const int*, const int*, const float*, const A*, int64_t, int, int, int,  \
      int, int, int, int, int, float, int, int, int, hipStream_t);
FI_INST(float)
FI_INST(u16)
#undef FI_INST

}  // namespace fi
