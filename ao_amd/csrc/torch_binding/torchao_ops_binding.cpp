// The C++ side of the binding a torchao maintainer would add: the operators of the weight-only quantized linear path
// registered with torch.library on top of the C ABI of libao_amd.so.
//
//   torchao::quant_llm_linear      schema of torchao/csrc/fp6_llm.cpp:7, checks of torchao/csrc/cuda/fp6_llm/fp6_linear.cu:151-152
//                                  and torchao/ops.py:23-37
//   torchao::int4wo_quantize_pack  AffineQuantizedTensor.from_float for int4_weight_only (torchao/dtypes/affine_quantized_tensor.py:184-229)
//   torchao::int4wo_linear         the int4 branch of _quantized_linear_op (torchao/dtypes/affine_quantized_tensor.py:600-640)
//
// each with a CUDA (= HIP on PyTorch-ROCm) implementation and a Meta implementation (shapes and dtypes only: what
// torch.compile, FakeTensor and meta-device checkpoint loading need).  Built by ao_amd/_build.py as a separate, optional
// library (libao_amd_torch.so): the Python package binds the same entry points through ctypes and does not load it,
// since both would register the same operators.  (PyTorch-ROCm names its HIP device "cuda": the device guard is the one
// that knows that, and the dispatch key of a GPU implementation is CUDA.)
#include <ATen/hip/HIPContext.h>
#include <ATen/ops/empty.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <mutex>
#include <tuple>
#include <unordered_map>

#include "ao_amd.h"

namespace {

// The reference's operator takes the tensor-core byte order on every call (torchao/ops.py:15-37); the kernels stream
// their own tile order.  The re-tiled copy of a weight is made once and kept while the weight tensor is the same
// tensor at the same version (an in-place write bumps the version and re-tiles).  The entry holds a weak reference to
// the weight: it keeps nothing but the tensor's control block alive, and a new tensor at a recycled address is a
// different control block.
struct NativeEntry {
    c10::weak_intrusive_ptr<c10::TensorImpl> weights;
    int64_t version;
    int64_t N, K;
    int nbits;
    at::Tensor native;
};
std::mutex g_cache_mutex;
std::unordered_map<const void*, NativeEntry> g_native_cache;
constexpr size_t kMaxCached = 512;

at::Tensor native_weight(const at::Tensor& weights, int64_t N, int64_t K, int nbits, hipStream_t stream) {
    const void* key = weights.data_ptr();
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_native_cache.find(key);
    if (it != g_native_cache.end()) {
        NativeEntry& e = it->second;
        if (!e.weights.expired() && e.weights._unsafe_get_target() == weights.unsafeGetTensorImpl() &&
            e.version == (int64_t)weights._version() && e.N == N && e.K == K && e.nbits == nbits)
            return e.native;
        g_native_cache.erase(it);
    }
    if (g_native_cache.size() >= kMaxCached) {
        for (auto i = g_native_cache.begin(); i != g_native_cache.end();) i = i->second.weights.expired() ? g_native_cache.erase(i) : std::next(i);
        if (g_native_cache.size() >= kMaxCached) g_native_cache.clear();
    }
    int64_t native_bytes = 0;
    TORCH_CHECK(ao_amd_fp6_native_bytes(N, K, &native_bytes) == 0, ao_amd_last_error());
    auto native = at::empty({native_bytes}, weights.options().dtype(at::kByte));
    TORCH_CHECK(ao_amd_fp6_repack(weights.data_ptr(), N, K, nbits, native.data_ptr(), stream) == 0, ao_amd_last_error());
    g_native_cache.emplace(key, NativeEntry{c10::weak_intrusive_ptr<c10::TensorImpl>(weights.getIntrusivePtr()), (int64_t)weights._version(),
                                            N, K, nbits, native});
    return native;
}

void check_quant_llm_args(int64_t EXPONENT, int64_t MANTISSA, const at::Tensor& _in_feats, const at::Tensor& _weights,
                          const at::Tensor& _scales) {
    // torchao/ops.py:26-37
    TORCH_CHECK(_in_feats.dim() == 2, "input should be a 2d tensor, got ", _in_feats.dim(), "D");
    TORCH_CHECK(_in_feats.scalar_type() == at::kHalf, "weight must be FP16, got ", _in_feats.scalar_type());
    TORCH_CHECK(_weights.dim() == 2, "weight should be a 2d tensor, got ", _weights.dim(), "D");
    TORCH_CHECK(_weights.scalar_type() == at::kByte, "weight must be UINT8, got ", _weights.scalar_type());
    TORCH_CHECK(_scales.dim() == 1, "scale should be a 2d tensor, got ", _scales.dim(), "D");
    TORCH_CHECK(_scales.scalar_type() == at::kHalf, "scale must be FP16, got ", _scales.scalar_type());
    const int64_t IC = _in_feats.size(1), OC = _weights.size(0);
    // torchao/csrc/cuda/fp6_llm/fp6_linear.cu:151-152
    TORCH_CHECK(IC / 8 * (1 + EXPONENT + MANTISSA) == _weights.size(1), "Dimensions mismatched: in_features ", IC, " against ",
                _weights.size(1), " packed bytes per row");
    TORCH_CHECK(OC == _scales.size(0), "Dimensions mismatched: ", OC, " weight rows against ", _scales.size(0), " scales");
}

at::Tensor quant_llm_linear_hip(int64_t EXPONENT, int64_t MANTISSA, at::Tensor _in_feats, at::Tensor _weights, at::Tensor _scales,
                                int64_t /*splitK: a tuning hint of the reference's kernel; these kernels size their own split*/) {
    check_quant_llm_args(EXPONENT, MANTISSA, _in_feats, _weights, _scales);
    TORCH_CHECK(_in_feats.is_cuda() && _weights.device() == _in_feats.device() && _scales.device() == _in_feats.device(),
                "quant_llm_linear: activations, weight and scales must be on the same GPU");
    TORCH_CHECK(_weights.is_contiguous(), "quant_llm_linear: the packed weight must be contiguous");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(_in_feats.device());
    auto x = _in_feats.contiguous();
    auto scales = _scales.contiguous();
    const int64_t M = x.size(0), K = x.size(1), N = _weights.size(0);
    auto stream = at::hip::getCurrentHIPStream().stream();
    auto native = native_weight(_weights, N, K, (int)(1 + EXPONENT + MANTISSA), stream);
    auto out = at::empty({M, N}, x.options());
    // where the reference's caller passes splitK and the operator allocates [splitK, M, N] floats (fp6_linear.cu:167), the
    // library says whether it splits K for this shape and how much workspace that takes (0: plain call)
    int64_t ws_bytes = 0;
    TORCH_CHECK(ao_amd_fp6_linear_ws_bytes(M, K, N, &ws_bytes) == 0, ao_amd_last_error());
    at::Tensor ws;
    if (ws_bytes > 0) ws = at::empty({ws_bytes / 4}, x.options().dtype(at::kFloat));
    TORCH_CHECK(ao_amd_fp6_linear_ws(x.data_ptr(), M, K, native.data_ptr(), scales.data_ptr(), N, (int)EXPONENT, (int)MANTISSA,
                                     out.data_ptr(), ws.defined() ? ws.data_ptr() : nullptr, ws_bytes, stream) == 0,
                ao_amd_last_error());
    return out;
}

// Meta implementations run under FakeTensor with symbolic sizes: they look at dimensions and dtypes only and build their
// outputs from symbolic sizes.
at::Tensor quant_llm_linear_meta(int64_t, int64_t, at::Tensor _in_feats, at::Tensor _weights, at::Tensor _scales, int64_t) {
    // torchao/ops.py:40-55
    TORCH_CHECK(_in_feats.dim() == 2, "input should be a 2d tensor, got ", _in_feats.dim(), "D");
    TORCH_CHECK(_in_feats.scalar_type() == at::kHalf, "weight must be FP16, got ", _in_feats.scalar_type());
    TORCH_CHECK(_weights.dim() == 2, "weight should be a 2d tensor, got ", _weights.dim(), "D");
    TORCH_CHECK(_weights.scalar_type() == at::kByte, "weight must be UINT8, got ", _weights.scalar_type());
    TORCH_CHECK(_scales.dim() == 1, "scale should be a 2d tensor, got ", _scales.dim(), "D");
    TORCH_CHECK(_scales.scalar_type() == at::kHalf, "scale must be FP16, got ", _scales.scalar_type());
    return at::empty_symint({_in_feats.sym_size(0), _weights.sym_size(0)}, _in_feats.options());
}

// shapes (int32) of the packed codes and of the interleaved (scale, zero) words
std::pair<std::vector<int64_t>, std::vector<int64_t>> packed_shapes(int64_t N, int64_t K, int64_t g) {
    int64_t Np = 0, Kp = 0;
    TORCH_CHECK(ao_amd_int4wo_packed_shape(N, K, g, &Np, &Kp, nullptr, nullptr) == 0, ao_amd_last_error());
    return {{Np / 16, Kp / 128, 64, 4}, {Np / 16, Kp / g, 16}};
}

void check_int4_weight_arg(const at::Tensor& w) {
    TORCH_CHECK(w.dim() == 2, "weight should be a 2d tensor, got ", w.dim(), "D");
    TORCH_CHECK(w.scalar_type() == at::kBFloat16, "int4 weight-only quantization needs a bfloat16 weight, got ", w.scalar_type());
}

std::tuple<at::Tensor, at::Tensor> int4wo_quantize_pack_hip(at::Tensor w, int64_t group_size) {
    check_int4_weight_arg(w);
    TORCH_CHECK(w.is_cuda(), "int4wo_quantize_pack: the weight must be on a GPU");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(w.device());
    if (w.stride(1) != 1) w = w.contiguous();
    const int64_t N = w.size(0), K = w.size(1);
    auto shapes = packed_shapes(N, K, group_size);
    auto packed = at::empty(shapes.first, w.options().dtype(at::kInt));
    auto qparams = at::empty(shapes.second, w.options().dtype(at::kInt));
    TORCH_CHECK(ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, w.stride(0), group_size, packed.data_ptr(), qparams.data_ptr(),
                                            at::hip::getCurrentHIPStream().stream()) == 0,
                ao_amd_last_error());
    return {packed, qparams};
}

std::tuple<at::Tensor, at::Tensor> int4wo_quantize_pack_meta(at::Tensor w, int64_t group_size) {
    check_int4_weight_arg(w);
    TORCH_CHECK(group_size == 32 || group_size == 64 || group_size == 128 || group_size == 256, "group_size must be one of 32, 64, 128, 256, got ",
                group_size);
    const int64_t kq = group_size > 128 ? group_size : 128;
    const c10::SymInt row_blocks = (w.sym_size(0) + 15) / 16;
    const c10::SymInt Kp = (w.sym_size(1) + (kq - 1)) / kq * kq;
    return {at::empty_symint({row_blocks, Kp / 128, c10::SymInt(64), c10::SymInt(4)}, w.options().dtype(at::kInt)),
            at::empty_symint({row_blocks, Kp / group_size, c10::SymInt(16)}, w.options().dtype(at::kInt))};
}

void check_int4_linear_args(const at::Tensor& x, const at::Tensor& packed, const at::Tensor& qparams, int64_t group_size, int64_t N,
                            const c10::optional<at::Tensor>& bias) {
    TORCH_CHECK(x.dim() == 2, "input should be a 2d tensor, got ", x.dim(), "D");
    TORCH_CHECK(x.scalar_type() == at::kBFloat16, "input must be bfloat16, got ", x.scalar_type());
    auto shapes = packed_shapes(N, x.size(1), group_size);
    TORCH_CHECK(packed.scalar_type() == at::kInt && packed.sizes().vec() == shapes.first && packed.is_contiguous(),
                "packed weight must be a contiguous int32 tensor of shape ", c10::IntArrayRef(shapes.first), ", got ", packed.sizes());
    TORCH_CHECK(qparams.scalar_type() == at::kInt && qparams.sizes().vec() == shapes.second && qparams.is_contiguous(),
                "qparams must be a contiguous int32 tensor of shape ", c10::IntArrayRef(shapes.second), ", got ", qparams.sizes());
    if (bias.has_value())
        TORCH_CHECK(bias->scalar_type() == at::kBFloat16 && bias->numel() == N, "bias must be bfloat16 of size N");
}

at::Tensor int4wo_linear_hip(at::Tensor x, at::Tensor packed, at::Tensor qparams, int64_t group_size, int64_t N,
                             c10::optional<at::Tensor> bias, bool fp32_out) {
    check_int4_linear_args(x, packed, qparams, group_size, N, bias);
    TORCH_CHECK(x.is_cuda() && packed.device() == x.device() && qparams.device() == x.device() &&
                    (!bias.has_value() || bias->device() == x.device()),
                "int4wo_linear: all tensors must be on the same GPU");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    if (x.stride(1) != 1) x = x.contiguous();
    at::Tensor b;
    if (bias.has_value()) b = bias->contiguous();
    const int64_t M = x.size(0), K = x.size(1);
    auto y = at::empty({M, N}, x.options().dtype(fp32_out ? at::kFloat : at::kBFloat16));
    // shapes whose K range the library splits over workgroups bring a workspace from the caching allocator (0 bytes: the
    // call is the plain linear)
    int64_t ws_bytes = 0;
    TORCH_CHECK(ao_amd_int4wo_linear_ws_bytes(M, K, N, group_size, &ws_bytes) == 0, ao_amd_last_error());
    at::Tensor ws;
    if (ws_bytes > 0) ws = at::empty({ws_bytes / 4}, x.options().dtype(at::kFloat));
    TORCH_CHECK(ao_amd_int4wo_linear_ws(x.data_ptr(), M, K, M > 0 ? x.stride(0) : K, packed.data_ptr(), qparams.data_ptr(), N,
                                        group_size, b.defined() ? b.data_ptr() : nullptr, y.data_ptr(),
                                        fp32_out ? AO_F32 : AO_BF16, N, ws.defined() ? ws.data_ptr() : nullptr, ws_bytes,
                                        at::hip::getCurrentHIPStream().stream()) == 0,
                ao_amd_last_error());
    return y;
}

at::Tensor int4wo_linear_meta(at::Tensor x, at::Tensor packed, at::Tensor qparams, int64_t, int64_t N, c10::optional<at::Tensor> bias,
                              bool fp32_out) {
    TORCH_CHECK(x.dim() == 2, "input should be a 2d tensor, got ", x.dim(), "D");
    TORCH_CHECK(x.scalar_type() == at::kBFloat16, "input must be bfloat16, got ", x.scalar_type());
    TORCH_CHECK(packed.scalar_type() == at::kInt && packed.dim() == 4 && qparams.scalar_type() == at::kInt && qparams.dim() == 3,
                "packed weight and qparams must be int32 tensors with 4 and 3 dimensions");
    TORCH_CHECK(!bias.has_value() || bias->scalar_type() == at::kBFloat16, "bias must be bfloat16 of size N");
    return at::empty_symint({x.sym_size(0), c10::SymInt(N)}, x.options().dtype(fp32_out ? at::kFloat : at::kBFloat16));
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(torchao, m) {
    m.def("quant_llm_linear(int EXPONENT, int MANTISSA, Tensor _in_feats, Tensor _weights, Tensor _scales, int splitK) -> Tensor");
    m.def("int4wo_quantize_pack(Tensor w, int group_size) -> (Tensor, Tensor)");
    m.def("int4wo_linear(Tensor x, Tensor packed, Tensor qparams, int group_size, int N, Tensor? bias, bool fp32_out) -> Tensor");
}
TORCH_LIBRARY_IMPL(torchao, CUDA, m) {
    m.impl("torchao::quant_llm_linear", &quant_llm_linear_hip);
    m.impl("torchao::int4wo_quantize_pack", &int4wo_quantize_pack_hip);
    m.impl("torchao::int4wo_linear", &int4wo_linear_hip);
}
TORCH_LIBRARY_IMPL(torchao, Meta, m) {
    m.impl("torchao::quant_llm_linear", &quant_llm_linear_meta);
    m.impl("torchao::int4wo_quantize_pack", &int4wo_quantize_pack_meta);
    m.impl("torchao::int4wo_linear", &int4wo_linear_meta);
}
