// The C++ side of the binding a torchao maintainer would add: torchao::quant_llm_linear (schema of
// torchao/csrc/fp6_llm.cpp:7) implemented by the C ABI of libao_amd.so.  Built by ao_amd/_build.py as a separate,
// optional library (libao_amd_torch.so): the Python package binds the same entry points through ctypes and does not
// load it, since both would register the same operator.
#include <ATen/hip/HIPContext.h>
#include <ATen/ops/empty.h>
#include <torch/library.h>

#include "ao_amd.h"

static at::Tensor quant_llm_linear_hip(int64_t EXPONENT, int64_t MANTISSA, at::Tensor _in_feats, at::Tensor _weights,
                                       at::Tensor _scales, int64_t /*splitK*/) {
    TORCH_CHECK(_in_feats.scalar_type() == at::kHalf && _in_feats.dim() == 2 && _in_feats.is_contiguous(),
                "quant_llm_linear: activations must be a contiguous 2d float16 tensor");
    TORCH_CHECK(_scales.scalar_type() == at::kHalf && _scales.is_contiguous(), "quant_llm_linear: scales must be float16");
    const int64_t M = _in_feats.size(0), K = _in_feats.size(1), N = _scales.size(0);
    // the reference's tensor-core order -> the order the HIP kernels stream (cached by a real integration)
    int64_t native_bytes = 0;
    TORCH_CHECK(ao_amd_fp6_native_bytes(N, K, &native_bytes) == 0, ao_amd_last_error());
    auto native = at::empty({native_bytes}, _weights.options().dtype(at::kByte));
    auto stream = at::hip::getCurrentHIPStream().stream();
    TORCH_CHECK(ao_amd_fp6_repack(_weights.data_ptr(), N, K, (int)(1 + EXPONENT + MANTISSA), native.data_ptr(), stream) == 0,
                ao_amd_last_error());
    auto out = at::empty({M, N}, _in_feats.options());
    TORCH_CHECK(ao_amd_fp6_linear(_in_feats.data_ptr(), M, K, native.data_ptr(), _scales.data_ptr(), N, (int)EXPONENT,
                                  (int)MANTISSA, out.data_ptr(), stream) == 0,
                ao_amd_last_error());
    return out;
}

TORCH_LIBRARY_FRAGMENT(torchao, m) {
    m.def("quant_llm_linear(int EXPONENT, int MANTISSA, Tensor _in_feats, Tensor _weights, Tensor _scales, int splitK) -> Tensor");
}
TORCH_LIBRARY_IMPL(torchao, CUDA, m) { m.impl("torchao::quant_llm_linear", &quant_llm_linear_hip); }
