// Helpers and the sampling wrappers shared by every extension module of this
// package (each module links its own copy of sampling.hip).
#pragma once

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <hip/hip_runtime.h>

extern "C" {
hipError_t ks_greedy_sample(void*, const void*, int, int, hipStream_t);
hipError_t ks_gumbel_sample(void*, const void*, const void*, const void*,
                            const void*, int, int, hipStream_t);
hipError_t ks_topk_topp_sample(void*, const void*, const void*, const void*,
                               const void*, const void*, int, int,
                               hipStream_t);
}

namespace {


hipStream_t current_stream() {
  return c10::hip::getCurrentHIPStream().stream();
}

void check_hip(hipError_t err, const char* op) {
  TORCH_CHECK(err == hipSuccess, op, " failed: ", hipGetErrorString(err));
}

#define CHECK_BF16_CONTIG(t)                                       \
  TORCH_CHECK((t).scalar_type() == at::kBFloat16, #t " must be bf16"); \
  TORCH_CHECK((t).is_contiguous(), #t " must be contiguous");      \
  TORCH_CHECK((t).is_cuda(), #t " must be on GPU")

void greedy_sample(at::Tensor& out, at::Tensor& logits) {
  CHECK_BF16_CONTIG(logits);
  TORCH_CHECK(out.scalar_type() == at::kLong, "out int64");
  check_hip(ks_greedy_sample(out.data_ptr(), logits.data_ptr(),
                             logits.size(0), logits.size(1),
                             current_stream()),
            "greedy_sample");
}

void gumbel_sample(at::Tensor& out, at::Tensor& logits,
                   at::Tensor& temperatures, at::Tensor& top_k,
                   at::Tensor& seeds) {
  CHECK_BF16_CONTIG(logits);
  TORCH_CHECK(out.scalar_type() == at::kLong, "out int64");
  TORCH_CHECK(temperatures.scalar_type() == at::kFloat, "temps fp32");
  TORCH_CHECK(seeds.scalar_type() == at::kLong, "seeds int64");
  check_hip(ks_gumbel_sample(out.data_ptr(), logits.data_ptr(),
                             temperatures.data_ptr(), top_k.data_ptr(),
                             seeds.data_ptr(), logits.size(0), logits.size(1),
                             current_stream()),
            "gumbel_sample");
}

void topk_topp_sample(at::Tensor& out, at::Tensor& logits,
                      at::Tensor& temperatures, at::Tensor& top_p,
                      at::Tensor& top_k, at::Tensor& seeds) {
  CHECK_BF16_CONTIG(logits);
  TORCH_CHECK(out.scalar_type() == at::kLong, "out int64");
  TORCH_CHECK(temperatures.scalar_type() == at::kFloat, "temps fp32");
  TORCH_CHECK(top_p.scalar_type() == at::kFloat, "top_p fp32");
  TORCH_CHECK(top_k.scalar_type() == at::kInt, "top_k int32");
  TORCH_CHECK(seeds.scalar_type() == at::kLong, "seeds int64");
  check_hip(ks_topk_topp_sample(out.data_ptr(), logits.data_ptr(),
                                temperatures.data_ptr(), top_p.data_ptr(),
                                top_k.data_ptr(), seeds.data_ptr(),
                                logits.size(0), logits.size(1),
                                current_stream()),
            "topk_topp_sample");
}

void def_sampling(pybind11::module_& m) {
  m.def("greedy_sample", &greedy_sample, "argmax sampling");
  m.def("gumbel_sample", &gumbel_sample, "Gumbel-max temperature sampling");
  m.def("topk_topp_sample", &topk_topp_sample,
        "fused top-k/top-p + Gumbel-max sampler (radix-histogram select)");
}

}  // namespace
