// PyTorch bindings of the expert-routing kernels (their own extension,
// so a model family with routed experts builds only these): router tail,
// block alignment of expert assignments, grouped GEMMs (MFMA on packed
// bf16 / fp8 weights; plain form for any size and fp32), weighted combine.

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

#include "common.h"

namespace fi {

void launch_moe_gemm(u16*, const u16*, const u16*, const int*, const int*,
                     const int*, int, int, int, int, int, float, hipStream_t);
void launch_moe_route_grouped(const float*, const float*, float*, int*, int,
                              int, int, int, int, hipStream_t);
void launch_moe_gemm_fp8(u16*, const unsigned char*, const float*,
                         const unsigned char*, const float*, const int*,
                         const int*, const int*, int, int, int, int, bool,
                         hipStream_t);
void launch_moe_align(const int*, int*, int*, int*, int*, int, int, int,
                      int, int, int, hipStream_t);
void launch_moe_router_topk(const float*, float*, int*, int, int, int,
                            bool, hipStream_t);
void launch_moe_route(const float*, float*, int*, int, int, int, bool, bool,
                      float, hipStream_t);
template <typename A>
void launch_moe_combine(A*, const A*, const int*, const float*, int, int,
                        int, hipStream_t);
template <typename A>
void launch_moe_gemm_plain(A*, const A*, const A*, const int*, const int*,
                           const int*, int, int, int, int, int, float,
                           hipStream_t);

}  // namespace fi

namespace {

using fi::u16;

#define CHECK_BF16_CUDA(t)                                     \
  TORCH_CHECK((t).is_cuda(), #t " must be on GPU");            \
  TORCH_CHECK((t).scalar_type() == at::kBFloat16, #t " must be bf16")

u16* bf16_ptr(at::Tensor& t) { return reinterpret_cast<u16*>(t.data_ptr()); }
const u16* bf16_cptr(const at::Tensor& t) {
  return reinterpret_cast<const u16*>(t.data_ptr());
}

hipStream_t current_stream() {
  return c10::hip::getCurrentHIPStream().stream();
}

void moe_gemm(at::Tensor out, at::Tensor a, at::Tensor b_packed,
              at::Tensor sorted_ids, at::Tensor expert_ids,
              at::Tensor n_valid, int64_t block_m, int64_t mode,
              double limit) {
  // mode 0: plain; 1: gathered rows, silu(gate) * up; 2: gathered rows,
  // relu(up)^2; 3: gathered rows, clamped gated unit with `limit`
  TORCH_CHECK(mode >= 0 && mode <= 3, "unknown grouped GEMM mode");
  const bool gate_up = mode == 1 || mode == 3;
  CHECK_BF16_CUDA(out);
  CHECK_BF16_CUDA(a);
  CHECK_BF16_CUDA(b_packed);
  TORCH_CHECK(out.is_contiguous() && a.is_contiguous() &&
              b_packed.is_contiguous());
  TORCH_CHECK(sorted_ids.scalar_type() == at::kInt &&
              expert_ids.scalar_type() == at::kInt &&
              n_valid.scalar_type() == at::kInt);
  TORCH_CHECK(block_m == 16 || block_m == 128, "block_m must be 16 or 128");
  const int K = a.size(1);
  const int N = out.size(1);
  const int PM = out.size(0);
  TORCH_CHECK(PM % block_m == 0, "padded rows must be block_m-aligned");
  TORCH_CHECK(K % 32 == 0, "K must be a multiple of 32");
  TORCH_CHECK(
      N % (block_m == 16 ? 64 : (mode != 0 ? 64 : 128)) == 0,
      "N tile misalignment");
  // packed B: [E, K/32, NB/16, 64, 8]
  TORCH_CHECK(b_packed.dim() == 5 && b_packed.size(1) == K / 32 &&
              b_packed.size(2) == (gate_up ? 2 * N : N) / 16 &&
              b_packed.size(3) == 64 && b_packed.size(4) == 8,
              "b_packed layout mismatch");
  TORCH_CHECK(expert_ids.size(0) >= PM / block_m);
  if (mode != 0) TORCH_CHECK(sorted_ids.size(0) >= PM);
  if (mode == 0) TORCH_CHECK(a.size(0) >= PM);
  fi::launch_moe_gemm(bf16_ptr(out), bf16_cptr(a),
                      bf16_cptr(b_packed), sorted_ids.data_ptr<int>(),
                      expert_ids.data_ptr<int>(), n_valid.data_ptr<int>(),
                      PM / block_m, K, N, static_cast<int>(block_m),
                      static_cast<int>(mode), static_cast<float>(limit),
                      current_stream());
}

void moe_gemm_fp8(at::Tensor out, at::Tensor a, at::Tensor a_scales,
                  at::Tensor b_packed, at::Tensor b_scales,
                  at::Tensor sorted_ids, at::Tensor expert_ids,
                  at::Tensor n_valid, int64_t block_m, bool gate_up) {
  CHECK_BF16_CUDA(out);
  TORCH_CHECK(a.scalar_type() == at::kFloat8_e4m3fn && a.is_cuda() &&
              a.is_contiguous());
  TORCH_CHECK(b_packed.scalar_type() == at::kFloat8_e4m3fn &&
              b_packed.is_contiguous());
  TORCH_CHECK(a_scales.scalar_type() == at::kFloat &&
              b_scales.scalar_type() == at::kFloat &&
              b_scales.is_contiguous());
  TORCH_CHECK(sorted_ids.scalar_type() == at::kInt &&
              expert_ids.scalar_type() == at::kInt &&
              n_valid.scalar_type() == at::kInt);
  TORCH_CHECK(block_m == 16 || block_m == 128);
  const int K = a.size(1);
  const int N = out.size(1);
  const int PM = out.size(0);
  TORCH_CHECK(PM % block_m == 0 && K % 32 == 0);
  TORCH_CHECK(N % (block_m == 16 ? 64 : (gate_up ? 64 : 128)) == 0);
  TORCH_CHECK(b_packed.dim() == 5 && b_packed.size(1) == K / 32 &&
              b_packed.size(2) == (gate_up ? 2 * N : N) / 16 &&
              b_packed.size(3) == 64 && b_packed.size(4) == 8);
  TORCH_CHECK(b_scales.numel() ==
              b_packed.size(0) * (gate_up ? 2 * N : N));
  fi::launch_moe_gemm_fp8(
      bf16_ptr(out), static_cast<const unsigned char*>(a.data_ptr()),
      a_scales.data_ptr<float>(),
      static_cast<const unsigned char*>(b_packed.data_ptr()),
      b_scales.data_ptr<float>(), sorted_ids.data_ptr<int>(),
      expert_ids.data_ptr<int>(), n_valid.data_ptr<int>(), PM / block_m, K,
      N, static_cast<int>(block_m), gate_up, current_stream());
}

void moe_combine(at::Tensor out, at::Tensor y, at::Tensor pos, at::Tensor w) {
  TORCH_CHECK(out.is_cuda() && y.is_cuda());
  TORCH_CHECK(out.scalar_type() == y.scalar_type() &&
              (out.scalar_type() == at::kBFloat16 ||
               out.scalar_type() == at::kFloat));
  TORCH_CHECK(out.is_contiguous() && y.is_contiguous());
  TORCH_CHECK(pos.scalar_type() == at::kInt && pos.is_contiguous());
  TORCH_CHECK(w.scalar_type() == at::kFloat && w.is_contiguous());
  const int T = out.size(0);
  const int H = out.size(1);
  TORCH_CHECK(y.size(1) == H);
  if (T == 0) return;
  const int topk = pos.numel() / T;
  TORCH_CHECK(pos.numel() == T * topk && w.numel() == T * topk);
  if (out.scalar_type() == at::kBFloat16)
    fi::launch_moe_combine<u16>(bf16_ptr(out), bf16_cptr(y),
                                pos.data_ptr<int>(), w.data_ptr<float>(), T,
                                topk, H, current_stream());
  else
    fi::launch_moe_combine<float>(out.data_ptr<float>(), y.data_ptr<float>(),
                                  pos.data_ptr<int>(), w.data_ptr<float>(), T,
                                  topk, H, current_stream());
}

void moe_gemm_plain(at::Tensor out, at::Tensor a, at::Tensor w,
                    at::Tensor sorted_ids, at::Tensor expert_ids,
                    at::Tensor n_valid, int64_t block_m, int64_t mode,
                    double limit) {
  TORCH_CHECK(mode >= 0 && mode <= 3, "unknown grouped GEMM mode");
  const bool gate_up = mode == 1 || mode == 3;
  TORCH_CHECK(out.is_cuda() && a.is_cuda() && w.is_cuda());
  TORCH_CHECK(out.scalar_type() == a.scalar_type() &&
              out.scalar_type() == w.scalar_type() &&
              (out.scalar_type() == at::kBFloat16 ||
               out.scalar_type() == at::kFloat));
  TORCH_CHECK(out.is_contiguous() && a.is_contiguous() && w.is_contiguous());
  TORCH_CHECK(sorted_ids.scalar_type() == at::kInt &&
              expert_ids.scalar_type() == at::kInt &&
              n_valid.scalar_type() == at::kInt);
  const int K = a.size(1);
  const int N = out.size(1);
  const int PM = out.size(0);
  TORCH_CHECK(block_m > 0 && PM % block_m == 0);
  TORCH_CHECK(w.dim() == 3 && w.size(2) == K &&
              w.size(1) == (gate_up ? 2 * N : N), "expert weight shape");
  TORCH_CHECK(expert_ids.size(0) >= PM / block_m);
  TORCH_CHECK(sorted_ids.size(0) >= PM);
  if (mode == 0) TORCH_CHECK(a.size(0) == PM);
  if (PM == 0) return;
  if (out.scalar_type() == at::kBFloat16)
    fi::launch_moe_gemm_plain<u16>(
        bf16_ptr(out), bf16_cptr(a), bf16_cptr(w), sorted_ids.data_ptr<int>(),
        expert_ids.data_ptr<int>(), n_valid.data_ptr<int>(), PM, K, N,
        static_cast<int>(block_m), static_cast<int>(mode),
        static_cast<float>(limit), current_stream());
  else
    fi::launch_moe_gemm_plain<float>(
        out.data_ptr<float>(), a.data_ptr<float>(), w.data_ptr<float>(),
        sorted_ids.data_ptr<int>(), expert_ids.data_ptr<int>(),
        n_valid.data_ptr<int>(), PM, K, N, static_cast<int>(block_m),
        static_cast<int>(mode), static_cast<float>(limit), current_stream());
}

void moe_route_grouped(at::Tensor logits, at::Tensor correction,
                       at::Tensor topv, at::Tensor topi, int64_t k,
                       int64_t groups, int64_t keep) {
  TORCH_CHECK(logits.is_cuda() && logits.scalar_type() == at::kFloat &&
              logits.is_contiguous() && logits.dim() == 2);
  TORCH_CHECK(correction.is_cuda() && correction.scalar_type() == at::kFloat &&
              correction.is_contiguous());
  TORCH_CHECK(topv.scalar_type() == at::kFloat &&
              topi.scalar_type() == at::kInt);
  const int T = logits.size(0);
  const int E = logits.size(1);
  TORCH_CHECK(correction.numel() == E);
  TORCH_CHECK(E >= 1 && E <= 1024 && groups >= 1 && E % groups == 0 &&
                  keep >= 1 && keep <= groups && k >= 1 &&
                  k <= keep * (E / groups),
              "moe_route_grouped: experts <= 1024 in equal groups, "
              "1 <= keep <= groups, k within the kept groups");
  TORCH_CHECK(topv.numel() == T * k && topi.numel() == T * k);
  if (T == 0) return;
  fi::launch_moe_route_grouped(
      logits.data_ptr<float>(), correction.data_ptr<float>(),
      topv.data_ptr<float>(), topi.data_ptr<int>(), T, E, (int)k, (int)groups,
      (int)keep, current_stream());
}

void moe_route(at::Tensor logits, at::Tensor topv, at::Tensor topi, int64_t k,
               bool sigmoid, bool renorm, double scale) {
  TORCH_CHECK(logits.is_cuda() && logits.scalar_type() == at::kFloat &&
              logits.is_contiguous());
  TORCH_CHECK(topv.scalar_type() == at::kFloat &&
              topi.scalar_type() == at::kInt);
  const int T = logits.size(0);
  const int E = logits.size(1);
  TORCH_CHECK(E >= 1 && E <= 1024 && k >= 1 && k <= E,
              "moe_route: 1 <= k <= experts <= 1024");
  TORCH_CHECK(topv.numel() == T * k && topi.numel() == T * k);
  if (T == 0) return;
  fi::launch_moe_route(logits.data_ptr<float>(), topv.data_ptr<float>(),
                       topi.data_ptr<int>(), T, E, (int)k, sigmoid, renorm,
                       static_cast<float>(scale), current_stream());
}

void moe_align(at::Tensor topi, at::Tensor sorted_ids, at::Tensor expert_ids,
               at::Tensor n_valid, at::Tensor pos, int64_t topk,
               int64_t e_start, int64_t e_end, int64_t block_m) {
  TORCH_CHECK(topi.is_cuda() && topi.scalar_type() == at::kInt &&
              topi.is_contiguous());
  TORCH_CHECK(sorted_ids.scalar_type() == at::kInt &&
              expert_ids.scalar_type() == at::kInt &&
              n_valid.scalar_type() == at::kInt &&
              pos.scalar_type() == at::kInt);
  const int n = topi.numel();
  const int PM = sorted_ids.numel();
  TORCH_CHECK(e_end - e_start <= 1024, "moe_align: E_local > 1024");
  TORCH_CHECK(PM % block_m == 0 && expert_ids.numel() == PM / block_m);
  TORCH_CHECK(pos.numel() == n);
  fi::launch_moe_align(topi.data_ptr<int>(), sorted_ids.data_ptr<int>(),
                       expert_ids.data_ptr<int>(), n_valid.data_ptr<int>(),
                       pos.data_ptr<int>(), n, (int)topk, (int)e_start,
                       (int)e_end, (int)block_m, PM, current_stream());
}

void moe_router_topk(at::Tensor logits, at::Tensor topv, at::Tensor topi,
                     int64_t k, bool renorm) {
  TORCH_CHECK(logits.is_cuda() && logits.scalar_type() == at::kFloat &&
              logits.is_contiguous());
  TORCH_CHECK(topv.scalar_type() == at::kFloat &&
              topi.scalar_type() == at::kInt);
  const int T = logits.size(0);
  const int E = logits.size(1);
  TORCH_CHECK(E <= 128 && k <= E);
  TORCH_CHECK(topv.numel() == T * k && topi.numel() == T * k);
  fi::launch_moe_router_topk(logits.data_ptr<float>(),
                             topv.data_ptr<float>(), topi.data_ptr<int>(),
                             T, E, (int)k, renorm, current_stream());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("moe_gemm", &moe_gemm,
        "grouped MFMA GEMM over block-aligned expert segments "
        "(gate_up=true fuses the SwiGLU epilogue)");
  m.def("moe_gemm_fp8", &moe_gemm_fp8,
        "grouped fp8 (e4m3) MFMA GEMM with per-row/per-channel dequant "
        "epilogue (gate_up=true fuses SwiGLU)");
  m.def("moe_gemm_plain", &moe_gemm_plain,
        "grouped GEMM for any sizes, bf16 or fp32 operands");
  m.def("moe_combine", &moe_combine,
        "weighted top-k combine of expert outputs (deterministic)");
  m.def("moe_align", &moe_align,
        "single-kernel block alignment of expert assignments "
        "(vLLM moe_align_block_size analog)");
  m.def("moe_router_topk", &moe_router_topk,
        "fused router tail: softmax + top-k + optional renormalize");
  m.def("moe_route_grouped", &moe_route_grouped,
        "group-limited router tail: sigmoid scores, choice on score + "
        "correction inside the best groups, weights = chosen scores");
  m.def("moe_route", &moe_route,
        "router tail for any expert count: softmax/sigmoid scores, top-k, "
        "renormalize, constant factor");
}
