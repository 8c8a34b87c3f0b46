/*
 * ao_amd -- C ABI of the MI355X (gfx950) weight-only quantized linear library.
 *
 * Plain pointers and sizes only: no torch types cross this boundary.  All device pointers are
 * HIP device memory on the current device, all kernels are enqueued on `stream` (a hipStream_t
 * passed as void*; NULL = the null stream) and no entry point synchronises, allocates or frees
 * device memory, so every call is safe under HIP graph capture.
 *
 * Every function returns 0 on success and a negative value on error; ao_amd_last_error() then
 * returns a thread-local, human readable message (argument-check failures are the counterpart of
 * the reference's TORCH_CHECK / assert -> RuntimeError / AssertionError paths).
 *
 * "Reference" below is pytorch-labs/ao (torchao) 0.3.1; paths are relative to its tree.
 */
#ifndef AO_AMD_H
#define AO_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes */
#define AO_F32 0
#define AO_BF16 1
#define AO_F16 2
#define AO_I32 3
#define AO_I64 4
#define AO_I8 5
#define AO_U8 6

/* mapping_type / zero_point_domain (torchao/quantization/quant_primitives.py:24-47) */
#define AO_MAP_SYMMETRIC 0
#define AO_MAP_ASYMMETRIC 1
#define AO_ZP_INT 0
#define AO_ZP_FLOAT 1

int ao_amd_abi_version(void);
const char* ao_amd_last_error(void);

/* ---------------------------------------------------------------- affine primitives (2-D, block (bN,bK))
 * in: [N,K] with row stride ld (elements).  qparams: contiguous [N/bN, K/bK].
 * Bit-exact with the reference's eager CPU ops: every reference op rounds to its tensor dtype. */

/* replaces choose_qparams_affine, torchao/quantization/quant_primitives.py:278-367
 * eps < 0 selects finfo(in_dtype).eps (the reference's eps=None). */
int ao_amd_choose_qparams_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t ld, int64_t bN,
                                 int64_t bK, int mapping, int64_t qmin, int64_t qmax, double eps, int preserve_zero,
                                 int zp_domain, int scale_dtype, int zp_dtype, void* scale, void* zero_point,
                                 void* stream);

/* replaces quantize_affine, torchao/quantization/quant_primitives.py:134-206
 * zero_point may be NULL in the INT domain.  out: contiguous [N,K] of out_dtype (AO_I32/I64/I8/U8). */
int ao_amd_quantize_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t ld, int64_t bN, int64_t bK,
                           const void* scale, int scale_dtype, const void* zero_point, int zp_dtype, int64_t qmin,
                           int64_t qmax, int zp_domain, void* out, int out_dtype, void* stream);

/* replaces dequantize_affine, torchao/quantization/quant_primitives.py:208-276
 * in: contiguous [N,K] integer codes; out: contiguous [N,K] of out_dtype (AO_F32/BF16/F16). */
int ao_amd_dequantize_affine(const void* in, int in_dtype, int64_t N, int64_t K, int64_t bN, int64_t bK,
                             const void* scale, int scale_dtype, const void* zero_point, int zp_dtype, int64_t qmin,
                             int64_t qmax, int zp_domain, void* out, int out_dtype, void* stream);

/* ---------------------------------------------------------------- int4 weight-only (uint4 groupwise asymmetric)
 * Packed layout (this library's own; replaces the tensor-core tile order of
 * aten::_convert_weight_to_int4pack, call site torchao/dtypes/affine_quantized_tensor.py:461, and
 * pack_tinygemm_scales_and_zeros, torchao/quantization/utils.py:310-322):
 *   Np = N rounded up to 16, Kp = K rounded up to max(128, g)
 *   packed : uint32 [Np/16][Kp/128][64 lanes][4]   lane l: row 16*rb + l%16, quarter qd = l/16;
 *            dword (l, sl) holds k = 128*kb + 32*qd + 8*sl + e (e=0..7) with element e in the nibble at
 *            bit 4*((e>>1) + 4*(e&1))  -- one wave64 16-byte load per lane = 1 KiB contiguous; a lane owns
 *            32 consecutive k (one group's scale/zero for every supported g) and the 8 values of a dword
 *            are one lane's share of a 16x16x32 bf16 MFMA operand.
 *   qparams: uint32 [Np/16][Kp/g][16] = scale_bf16 | zero_bf16 << 16
 * Padding holds code 8, scale bf16(1e-6), zero 0, i.e. what quantizing zero padding yields.
 * group size g must be 32, 64, 128 or 256. */
int ao_amd_int4wo_packed_shape(int64_t N, int64_t K, int64_t g, int64_t* Np, int64_t* Kp, int64_t* packed_bytes,
                               int64_t* qparam_bytes);

/* Fused from_float for int4_weight_only: choose_qparams_affine(ASYMMETRIC,(1,g),qmin 0,qmax 15,eps 1e-6,
 * preserve_zero False, FLOAT zero point, bf16) + quantize_affine + pack in one pass over w.
 * replaces AffineQuantizedTensor.from_float, torchao/dtypes/affine_quantized_tensor.py:184-229 as called by
 * torchao/quantization/quant_api.py:372-385.   w: bf16 [N,K], row stride ldw. */
int ao_amd_int4wo_quantize_pack(const void* w_bf16, int64_t N, int64_t K, int64_t ldw, int64_t g, void* packed,
                                void* qparams, void* stream);

/* Layout constructor from plain tensors; replaces TensorCoreTiledAQTLayout.from_plain,
 * torchao/dtypes/affine_quantized_tensor.py:460-465.  codes int32 [N,K] (values 0..15), scale / zero
 * bf16 [N,K/g], all contiguous, K % g == 0. */
int ao_amd_int4wo_pack(const int32_t* codes, const void* scale_bf16, const void* zero_bf16, int64_t N, int64_t K,
                       int64_t g, void* packed, void* qparams, void* stream);

/* Inverse of ao_amd_int4wo_pack; replaces TensorCoreTiledAQTLayout.get_plain,
 * torchao/dtypes/affine_quantized_tensor.py:509-537 (which recovers codes by multiplying with an identity). */
int ao_amd_int4wo_unpack(const void* packed, const void* qparams, int64_t N, int64_t K, int64_t g, int32_t* codes,
                         void* scale_bf16, void* zero_bf16, void* stream);

/* Unpack + dequantize_affine(FLOAT domain) in one pass: out bf16 [N,K] contiguous.
 * replaces AffineQuantizedTensor.dequantize, torchao/dtypes/affine_quantized_tensor.py:157-161. */
int ao_amd_int4wo_dequantize(const void* packed, const void* qparams, int64_t N, int64_t K, int64_t g,
                             void* out_bf16, void* stream);

/* y[M,N] = x[M,K] @ dequant(W)[N,K]^T (+ bias), fp32 accumulation, dequant = bf16(bf16((q-8)*s) + z).
 * replaces aten::_weight_int4pack_mm as called by _quantized_linear_op,
 * torchao/dtypes/affine_quantized_tensor.py:600-640.
 * x: bf16 [M,K] row stride ldx; bias: bf16 [N] or NULL; y: y_dtype (AO_BF16 or AO_F32) row stride ldy. */
int ao_amd_int4wo_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed,
                         const void* qparams, int64_t N, int64_t g, const void* bias_bf16, void* y, int y_dtype,
                         int64_t ldy, void* stream);

/* Same product with fused epilogues, used by the decode loop so that a token costs few launches.
 * y = bf16( bf16(x W^T + bias) + residual ): F.linear followed by the residual add of TransformerBlock.forward,
 * torchao/_models/llama/model.py:160-163. */
int ao_amd_int4wo_linear_residual(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed,
                                  const void* qparams, int64_t N, int64_t g, const void* bias_bf16,
                                  const void* residual_bf16, int64_t ldres, void* y_bf16, int64_t ldy, void* stream);

/* y = silu(x W_gate^T) * (x W_up^T) with the bf16 roundings of the module chain: FeedForward.forward,
 * torchao/_models/llama/model.py:221-222 (w1 = gate, w3 = up).  Both weights [N,K], same group size. */
int ao_amd_int4wo_swiglu(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed_gate,
                         const void* qparams_gate, const void* packed_up, const void* qparams_up, int64_t N, int64_t g,
                         void* y_bf16, int64_t ldy, void* stream);

/* The same two products with RMSNorm applied to the activation rows while they are staged:
 * x' = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * norm_weight ) (RMSNorm.forward, torchao/_models/llama/model.py:232-244),
 * then linear / SwiGLU of x' as above: `self.attention(self.attention_norm(x), ...)` and
 * `self.feed_forward(self.ffn_norm(h))` of TransformerBlock.forward, model.py:160-163, in one launch each.
 * Decode shapes only: M <= 16, K a multiple of max(128, group), 16-byte aligned rows and norm weight, M*K*2 bytes
 * within the kernel's LDS staging (40 KB at K = 4096 .. 160 KB); anything else is rejected with an error. */
int ao_amd_int4wo_rmsnorm_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16,
                                 float eps, const void* packed, const void* qparams, int64_t N, int64_t g,
                                 const void* bias_bf16, void* y, int y_dtype, int64_t ldy, void* stream);
int ao_amd_int4wo_rmsnorm_swiglu(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16,
                                 float eps, const void* packed_gate, const void* qparams_gate, const void* packed_up,
                                 const void* qparams_up, int64_t N, int64_t g, void* y_bf16, int64_t ldy, void* stream);

/* Which kernel instantiation the int4 linear entry points above run for a problem, without launching anything: writes a
 * name such as "int4wo_gemm_ksplit_kernel<64,4,4>" or "int4wo_gemv1_kernel<4,2,0> wpr=4" to `out`.  `aligned`: K is a
 * multiple of max(128, g) and the activation rows are 16-byte aligned; the other flags say which fused variant is meant
 * (residual epilogue, RMSNorm on the activations, two weights, interleaved gate/up weight, K split).  The test suite walks
 * the dispatch with it so that no instantiation ships without a test that reaches it.  No counterpart in the reference
 * (its dispatch is `aten::_weight_int4pack_mm`'s own, affine_quantized_tensor.py:631). */
int ao_amd_int4wo_linear_plan(int64_t M, int64_t K, int64_t N, int64_t g, int aligned, int has_residual, int has_norm,
                              int dual, int pair8, int ksplit, int y_dtype, char* out, int64_t out_cap);

/* ao_amd_int4wo_linear with a caller-owned workspace (device memory, 16-byte aligned): for batches of 2 to 256 rows on
 * weights whose tiles leave most CUs idle (4096-row weights, long K), the K range is split over 2 to 8 groups of
 * workgroups, fp32 partial outputs [parts][M][N] go to the workspace and a second small launch adds them, adds the bias
 * and rounds once.  ao_amd_int4wo_linear_ws_bytes gives the size for a shape (0 where the split is not used: the call is
 * then ao_amd_int4wo_linear itself and `workspace` may be NULL); ao_amd_int4wo_linear_ws_parts the number of parts.
 * Same product as ao_amd_int4wo_linear (`aten::_weight_int4pack_mm`, torchao/dtypes/affine_quantized_tensor.py:600-640),
 * summed in another order.  Calls that share a workspace must not overlap. */
int ao_amd_int4wo_linear_ws_bytes(int64_t M, int64_t K, int64_t N, int64_t g, int64_t* bytes);
int ao_amd_int4wo_linear_ws_parts(int64_t M, int64_t K, int64_t N, int64_t g);
int ao_amd_int4wo_linear_ws(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* packed, const void* qparams,
                            int64_t N, int64_t g, const void* bias_bf16, void* y, int y_dtype, int64_t ldy, void* workspace,
                            int64_t workspace_bytes, void* stream);

/* Linear with the K range split over `ksplit` (1..8) groups of workgroups, for weights whose row-block count does not fill
 * the CUs evenly (Llama-3-8B wqkv: 384 row blocks on 256 CUs): y_f32_parts[z][M][ldy] = sum over the z-th run of K tiles
 * of x' W^T in fp32, x' = x or its RMSNorm as in ao_amd_int4wo_rmsnorm_linear.  The consumer adds the parts and rounds
 * (ao_amd_llama_decode_attention_parts); no cross-workgroup reduction, no scratch memory.  Decode shapes only (M <= 16).
 * Same product as ao_amd_int4wo_linear (`aten::_weight_int4pack_mm`, affine_quantized_tensor.py:600-640), summed in
 * another order. */
int ao_amd_int4wo_linear_partials(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16,
                                  float eps, const void* packed, const void* qparams, int64_t N, int64_t g, int ksplit,
                                  void* y_f32_parts, int64_t ldy, void* stream);

/* SwiGLU over ONE interleaved weight: `ao_amd_int4wo_interleave_pair` permutes two packed weights of the same shape
 * (N a multiple of 16) into a packed weight of 2N rows whose 16-row blocks hold 8 gate rows followed by the 8 up rows of
 * the same outputs (buffers sized by ao_amd_int4wo_packed_shape(2N, K, g)); `ao_amd_int4wo_swiglu_interleaved` computes
 * y[M,N] = bf16( silu(bf16(x' Wg^T)) * bf16(x' Wu^T) ) from it, x' = x or, with `norm_weight_bf16` non-null, the RMSNorm
 * of x as in ao_amd_int4wo_rmsnorm_swiglu.  Same arithmetic and roundings as ao_amd_int4wo_swiglu (FeedForward.forward,
 * torchao/_models/llama/model.py:209-214); the point of the layout is the launch shape: 2N/16 workgroups of half the
 * work each (7 per CU instead of 3.5 for Llama-3-8B's 14336 x 4096 pair on 256 CUs).  Decode shapes only, as above. */
int ao_amd_int4wo_interleave_pair(const void* packed_gate, const void* qparams_gate, const void* packed_up,
                                  const void* qparams_up, int64_t N, int64_t K, int64_t g, void* packed_pair,
                                  void* qparams_pair, void* stream);
int ao_amd_int4wo_swiglu_interleaved(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16,
                                     float eps, const void* packed_pair, const void* qparams_pair, int64_t N, int64_t g,
                                     void* y_bf16, int64_t ldy, void* stream);

/* ---------------------------------------------------------------- HQQ-format int4 weight (prototype/hqq mixed matmul)
 * W[k][n] = (q[k][n] - zeros[k/group][n]) * scales[k/group][n], each op rounded to `dtype` (AO_BF16 or AO_F16), from
 * `packed_2xint4` uint8/int8 [K/2, N] whose byte (k2, n) holds q[2*k2][n] in the low and q[2*k2+1][n] in the high nibble
 * (pack_2xint4, torchao/prototype/hqq/mixed_mm.py:13-35; unsigned nibbles, or sign-extended ones when `is_signed`).
 * This is the dequantization inside the reference's Triton kernel (torchao/prototype/hqq/kernels.py:318-358) as a pass
 * of its own: `out` is the [K, N] matrix in `dtype`; the caller multiplies x[M,K] @ out for the forward product and
 * x[M,N] @ out^T for the transposed one (triton_mixed_mm(..., transposed=True), mixed_mm.py:38-62) with a library GEMM.
 * N a multiple of 16, group_size even and dividing K, 16-byte aligned buffers. */
int ao_amd_hqq_dequantize(const void* packed_2xint4, int is_signed, int64_t K, int64_t N, const void* scales,
                          const void* zeros, int64_t group_size, int dtype, void* out, void* stream);

/* The forward product of the same Triton kernel for 1 to 16 activation rows, fused (torchao/prototype/hqq/kernels.py:
 * 162-388, triton_mixed_mm(a, b, scales, zeros, group_size), mixed_mm.py:38-176): y[M,N] = a[M,K] @ W[K,N] with W as
 * above (every weight rounded twice to `dtype` exactly as ao_amd_hqq_dequantize rounds it), fp32 accumulation, y in
 * `dtype`, row stride N.  a: `dtype` [M, K] with row stride lda (even, rows 4-byte aligned); N a multiple of 4, packed
 * codes 4-byte and scales / zeros 8-byte aligned.  K is cut into slices whose fp32 partial sums go through `workspace`
 * (ao_amd_hqq_mixed_mm_workspace gives its size; caller-owned, device memory). */
int ao_amd_hqq_mixed_mm_workspace(int64_t M, int64_t K, int64_t N, int64_t* bytes);
int ao_amd_hqq_mixed_mm(const void* a, int64_t M, int64_t K, int64_t lda, const void* packed_2xint4, int is_signed, int64_t N,
                        const void* scales, const void* zeros, int64_t group_size, int dtype, void* workspace,
                        int64_t workspace_bytes, void* y, void* stream);

/* Both products of that kernel for 1 to 64 activation rows on the matrix cores, the weight dequantized in registers
 * (torchao/prototype/hqq/kernels.py:162-388; `transposed` is the TRANSPOSED switch of the Triton kernel,
 * triton_mixed_mm(..., transposed=True), mixed_mm.py:38-62).  transposed == 0: y[M,N] = a[M,K] @ W[K,N]; needs K and
 * group_size multiples of 8, N a multiple of 4.  transposed != 0: y[M,K] = a[M,N] @ W^T, the product over N that a
 * backward pass needs; needs N a multiple of 16, K and group_size even.  Every weight is rounded twice to `dtype`
 * exactly as ao_amd_hqq_dequantize rounds it; fp32 accumulation; y in `dtype`, contiguous.  a: `dtype`, row stride lda
 * a multiple of 8 elements, 16-byte aligned like the packed codes, scales and zeros.  The reduction is cut into slices
 * whose fp32 partial sums go through `workspace` (ao_amd_hqq_mixed_mm_mfma_workspace gives its size; caller-owned,
 * device memory, 16-byte aligned).  More than 64 rows take ao_amd_hqq_dequantize and a library GEMM. */
int ao_amd_hqq_mixed_mm_mfma_workspace(int64_t M, int64_t K, int64_t N, int transposed, int64_t* bytes);
int ao_amd_hqq_mixed_mm_mfma(const void* a, int64_t M, int64_t lda, const void* packed_2xint4, int is_signed, int64_t K,
                             int64_t N, const void* scales, const void* zeros, int64_t group_size, int dtype,
                             int transposed, void* workspace, int64_t workspace_bytes, void* y, void* stream);

/* ---------------------------------------------------------------- int8 weight-only linear
 * y[M,N] = bf16( bf16(x[M,K] @ bf16(w)^T) * scale[N] ) (+ bias, rounded to bf16 again): the per-channel int8
 * weight-only branch of _quantized_linear_op, torchao/dtypes/affine_quantized_tensor.py:641-665
 * (`torch.mm(x, w_int8.t().to(x.dtype)) * scale`), for the weight that int8_weight_only() produces
 * (torchao/quantization/quant_api.py:390-405: symmetric, block (1, K), plain layout).
 *   w_int8 : int8 [N, K] row-major with row stride ldw (the reference's plain layout, read in place);
 *   K % 128 == 0; x, w 16-byte aligned with 16-byte aligned rows; y_dtype AO_BF16 or AO_F32 (AO_F32 stores the value
 *   before the last rounding). */
int ao_amd_int8wo_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8, int64_t ldw,
                         const void* scale_bf16, int64_t N, const void* bias_bf16, void* y, int y_dtype, int64_t ldy,
                         void* stream);

/* The same linear with the module's next elementwise op on its bf16 result fused into the epilogue, for the decode step:
 * `_residual`: y = bf16(linear) + residual (h + attention(...) and h + feed_forward(...), TransformerBlock.forward,
 * torchao/_models/llama/model.py:160-163); `_gated`: y = bf16(silu(gate)) * bf16(linear) with the gate projection already
 * computed (F.silu(self.w1(x)) * self.w3(x), FeedForward.forward, model.py:209-214).  bf16 output, no bias. */
int ao_amd_int8wo_linear_residual(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8, int64_t ldw,
                                  const void* scale_bf16, int64_t N, const void* residual_bf16, int64_t ldres,
                                  void* y_bf16, int64_t ldy, void* stream);
int ao_amd_int8wo_linear_gated(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* w_int8, int64_t ldw,
                               const void* scale_bf16, int64_t N, const void* gate_bf16, int64_t ldgate, void* y_bf16,
                               int64_t ldy, void* stream);

/* linear(rmsnorm(x)) in one launch for the decode step: y = bf16(bf16(rmsnorm(x) @ bf16(Wq)^T) * scale), with
 * rmsnorm(x) = bf16(bf16(x * rsqrt(mean(x^2) + eps)) * norm_weight) (RMSNorm.forward followed by the linear it feeds,
 * torchao/_models/llama/model.py:232-244, :160-163, :209-214).  gate_bf16 may be null; when given the `_gated`
 * epilogue above applies.  Only for activations whose (at most 16) rows fit the workgroup's LDS: M * K * 2 bytes at
 * most 64 KB; other shapes are rejected.  norm_weight 16-byte aligned, bf16 [K]. */
int ao_amd_int8wo_rmsnorm_linear(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16,
                                 float eps, const void* w_int8, int64_t ldw, const void* scale_bf16, int64_t N,
                                 const void* gate_bf16, int64_t ldgate, void* y_bf16, int64_t ldy, void* stream);

/* SwiGLU over two int8 weights in one launch: y = bf16(silu(g)) * u with g = linear(x', w_gate), u = linear(x', w_up),
 * each rounded as ao_amd_int8wo_linear rounds it, and x' = rmsnorm(x) when norm_weight_bf16 is given, else x
 * (F.silu(self.w1(x)) * self.w3(x), FeedForward.forward, torchao/_models/llama/model.py:209-214).  Both weights int8
 * [N, K] with the same row stride ldw, 16-byte aligned.  Same LDS limit as ao_amd_int8wo_rmsnorm_linear. */
int ao_amd_int8wo_swiglu(const void* x_bf16, int64_t M, int64_t K, int64_t ldx, const void* norm_weight_bf16, float eps,
                         const void* w_gate_int8, const void* scale_gate_bf16, const void* w_up_int8,
                         const void* scale_up_bf16, int64_t ldw, int64_t N, void* y_bf16, int64_t ldy, void* stream);

/* bf16 copy of the int8 codes (`w_int8.to(x.dtype)` of the same formula) for prefill-sized batches: the caller then
 * runs a plain bf16 GEMM on it and multiplies by the scale.  K a multiple of 16, 16-byte aligned rows. */
int ao_amd_int8_to_bf16(const void* w_int8, int64_t N, int64_t K, int64_t ldw, void* out_bf16, void* stream);

/* ---------------------------------------------------------------- Llama decode harness kernels (bf16)
 * out[rows,dim] = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * weight ): RMSNorm.forward,
 * torchao/_models/llama/model.py:232-244. */
int ao_amd_rmsnorm_bf16(const void* x, const void* weight, int64_t rows, int64_t dim, float eps, void* out,
                        void* stream);

/* One new token, batch 1: rotary embedding of q and k, KV-cache update at *pos_dev, grouped-query attention over
 * positions 0..*pos_dev.  Attention.forward, torchao/_models/llama/model.py:190-211 with apply_rotary_emb :250-266
 * and KVCache.update :85-98.  qkv: [(n_head + 2 n_kv) * head_dim] (fused wqkv output); freqs_cis: [>= max_seq, head_dim/2, 2]
 * (cos, sin); caches: [n_kv, max_seq, head_dim]; out: [n_head * head_dim].  head_dim must be 128, max_seq <= 28000 (the
 * scores of the whole context live in LDS; see the split variant below for more).  The position is read on the device:
 * one outside [0, max_seq) touches neither cache nor freqs_cis and yields NaN outputs (the reference's index ops raise). */
int ao_amd_llama_decode_attention(const void* qkv_bf16, const void* freqs_cis_bf16, const int32_t* pos_dev,
                                  void* k_cache, void* v_cache, int n_head, int n_kv, int head_dim, int64_t max_seq,
                                  void* out_bf16, void* stream);

/* The same step reading the fused qkv row as `nparts` fp32 partial rows [nparts][(n_head + 2 n_kv) * head_dim] that it adds
 * and rounds to bf16 itself: the output of ao_amd_int4wo_linear_partials, which splits K across workgroups. */
int ao_amd_llama_decode_attention_parts(const void* qkv_f32_parts, int nparts, const void* freqs_cis_bf16,
                                        const int32_t* pos_dev, void* k_cache, void* v_cache, int n_head, int n_kv,
                                        int head_dim, int64_t max_seq, void* out_bf16, void* stream);

/* The same step with the context of every head split over `nsplit` (1..16) workgroups that take interleaved 64-position
 * rows, for long contexts (one workgroup per head walks 8192 positions in ~80 us, eight of them in ~15): partial
 * (max, sum, output) triples go to `workspace_f32` (n_head * nsplit * 130 floats, caller-owned) and a second, small launch
 * merges them.  Exactly one of qkv_bf16 / qkv_f32_parts is non-null.  max_seq <= 32768 (scores of one workgroup's share of
 * the context live in LDS).  No counterpart in the reference, whose attention is F.scaled_dot_product_attention. */
int ao_amd_llama_decode_attention_split(const void* qkv_bf16, const void* qkv_f32_parts, int nparts,
                                        const void* freqs_cis_bf16, const int32_t* pos_dev, void* k_cache, void* v_cache,
                                        int n_head, int n_kv, int head_dim, int64_t max_seq, int nsplit,
                                        void* workspace_f32, void* out_bf16, void* stream);

/* ao_amd_llama_decode_attention_split without the workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops and harnesses that forbid hipMalloc): the partial (max, sum, output)
 * triples go to a 1 MiB array that is part of the library's device image (one copy per device, held until the process
 * ends), whose address the first call on a device looks up (hipGetSymbolAddress).  The call itself allocates and frees
 * nothing.  n_head * nsplit may be at most 2048; anything larger is rejected with an error.  All calls on one device
 * share the array: calls that overlap in time on the same device (different streams or threads) race, and nothing in it
 * needs clearing between calls because every launch rewrites every triple it later reads.  Results are bit-identical to
 * ao_amd_llama_decode_attention_split.  No counterpart in the reference. */
int ao_amd_llama_decode_attention_split_static(const void* qkv_bf16, const void* qkv_f32_parts, int nparts,
                                               const void* freqs_cis_bf16, const int32_t* pos_dev, void* k_cache,
                                               void* v_cache, int n_head, int n_kv, int head_dim, int64_t max_seq,
                                               int nsplit, void* out_bf16, void* stream);

/* The same two harness kernels over fp16 activations, weights and caches, for the FP6 model (whose linear takes fp16):
 * RMSNorm.forward and Attention.forward as above, every rounding to fp16 instead of bf16.  The attention entry takes
 * the context split directly (nsplit = 1 and a null workspace for short caches). */
int ao_amd_rmsnorm_f16(const void* x, const void* weight, int64_t rows, int64_t dim, float eps, void* out, void* stream);
int ao_amd_llama_decode_attention_f16(const void* qkv_f16, const void* freqs_cis_f16, const int32_t* pos_dev, void* k_cache,
                                      void* v_cache, int n_head, int n_kv, int head_dim, int64_t max_seq, int nsplit,
                                      void* workspace_f32, void* out_f16, void* stream);

/* out_index[0] = index of the largest of n bf16 values (lowest index among equals; NaN counts as largest): the greedy
 * branch of `sample` in the decode harness, torch.argmax over the last position's logits
 * (torchao/_models/llama/generate.py:34-53 samples from the same logits row). */
int ao_amd_argmax_bf16(const void* x_bf16, int64_t n, int32_t* out_index, void* stream);
/* The same over n fp16 values (the logits of an FP6 / fp16 model). */
int ao_amd_argmax_f16(const void* x_f16, int64_t n, int32_t* out_index, void* stream);

/* Greedy sampling and the bookkeeping of one decode step in one launch: next_token[0] = token[0] = argmax(logits[0..n)),
 * pos[0] += 1 (decode_one_token + the loop's `input_pos += 1; cur_token = next_token`,
 * torchao/_models/llama/generate.py:58-77, on device-side state so that the step can live in a HIP graph).
 * logits bf16 (is_f16 = 0) or fp16; the three int32 cells are distinct device addresses. */
int ao_amd_llama_decode_advance(const void* logits, int is_f16, int64_t n, int32_t* next_token, int32_t* token,
                                int32_t* pos, void* stream);

/* ---------------------------------------------------------------- FP6-LLM (Quant-LLM FPx, e3m2 / e2m2 ...)
 * Interchange format = the reference's TC-FPx bytes, bit for bit. */

/* replaces to_scaled_tc_fpx, torchao/prototype/quant_llm/quant_llm.py:116-130 for the formats the reference kernel
 * accepts (torchao/csrc/cuda/fp6_llm/fp6_linear.cu:173-184): e3m2 and e2m3 (6 bits), e2m2 and e3m1 (5 bits).  Per-row
 * scale = amax|w| / max_normal (fp32) stored as fp16, codes = _f32_to_fpx_unpacked(w / scale)
 * (torchao/prototype/custom_fp_utils.py:27-140), bytes = _pack_tc_fpx (quant_llm.py:60-86; 6 bits: the 2-bit plane then
 * the 4-bit plane, = _pack_tc_fp6 :90-106; 5 bits: the 1-bit plane then the 4-bit plane).
 * w: [N,K] of w_dtype (AO_F32/BF16/F16) contiguous; N % 64 == 0, K % 64 == 0.
 * out_tc: uint8 [N, K*nbits/8] with nbits = 1 + ebits + mbits; out_scale: fp16 [N]. */
int ao_amd_fp6_quantize_pack(const void* w, int w_dtype, int64_t N, int64_t K, int ebits, int mbits, void* out_tc,
                             void* out_scale_f16, void* stream);

/* replaces from_scaled_tc_fpx, torchao/prototype/quant_llm/quant_llm.py:203-208 (same four formats):
 * out fp32 [N,K] = fpx_to_f32(unpack(tc)) * float(scale) (scale may be NULL). */
int ao_amd_fp6_dequantize(const void* tc, const void* scale_f16, int64_t N, int64_t K, int ebits, int mbits,
                          float* out, void* stream);

/* One-time device repack of the TC-FPx bytes (nbits = 5 or 6) into the kernel's wave64 order (no counterpart in the
 * reference, whose kernel reads the TC bytes directly with 32-lane fragment loads).  A 5-bit code is stored as the
 * 6-bit code of the same value (e2m2 -> e2m3, e3m1 -> e3m2: one more mantissa bit, zero):
 *   native: per 16-row x 128-k tile 1536 bytes = [64 lanes][4 dwords] then [64 lanes][2 dwords]; lane l owns row
 *   16*rb + l%16 and the 32 consecutive k = 128*kb + 32*(l/16) + i, value i at bit 6*i of its 6 dwords; K is padded
 *   with zero codes to a multiple of 128.  ao_amd_fp6_native_bytes gives the buffer size. */
int ao_amd_fp6_native_bytes(int64_t N, int64_t K, int64_t* bytes);
int ao_amd_fp6_repack(const void* tc, int64_t N, int64_t K, int nbits, void* native, void* stream);

/* out[M,N] fp16 = x[M,K] fp16 @ W^T with W = fp16(fpx value * scale), fp32 accumulation; (ebits, mbits) one of
 * (3,2), (2,3), (2,2), (3,1).
 * replaces torchao::quant_llm_linear, schema torchao/csrc/fp6_llm.cpp:7, CUDA implementation
 * torchao/csrc/cuda/fp6_llm/fp6_linear.cu:139-196.  `weights_native` is the output of ao_amd_fp6_repack. */
int ao_amd_fp6_linear(const void* x_f16, int64_t M, int64_t K, const void* weights_native, const void* scale_f16,
                      int64_t N, int ebits, int mbits, void* out_f16, void* stream);

/* ao_amd_fp6_linear with a caller-owned workspace (device memory, 16-byte aligned): for batches of 16 to 256 rows on
 * weights whose 32- / 64-row tiles leave most CUs idle (4096-row weights), the K range is split over 2 or 4 groups of
 * workgroups, fp32 partial outputs [parts][M][N] go to the workspace and a second small launch adds them and rounds once
 * to fp16.  ao_amd_fp6_linear_ws_bytes gives the size for a shape (0 where the split is not used: the call is then
 * ao_amd_fp6_linear itself and `workspace` may be NULL); ao_amd_fp6_linear_ws_parts the number of parts.  Same product as
 * torchao::quant_llm_linear (torchao/csrc/cuda/fp6_llm/fp6_linear.cu:139-200); it stands where the reference's operator
 * takes `splitK` and allocates its [splitK, M, N] fp32 reduction workspace (fp6_linear.cu:104-111, 167-168,
 * SplitK_Reduction in kernel_reduction.cuh:44), with the part count chosen by the library instead of the caller.
 * Calls that share a workspace must not overlap. */
int ao_amd_fp6_linear_ws_bytes(int64_t M, int64_t K, int64_t N, int64_t* bytes);
int ao_amd_fp6_linear_ws_parts(int64_t M, int64_t K, int64_t N);
int ao_amd_fp6_linear_ws(const void* x_f16, int64_t M, int64_t K, const void* weights_native, const void* scale_f16, int64_t N,
                         int ebits, int mbits, void* out_f16, void* workspace, int64_t workspace_bytes, void* stream);

/* Which kernel instantiation the FPx linear entry points run for a problem, without launching anything: writes a name
 * such as "fp6_gemm_kernel<1,1,4,4,4>" (e3m2 flag, then the tile variant) or "fp6_gemv_kernel<8,1,0>" to `out`.  The
 * flags say which fused variant is meant (RMSNorm on the activations, residual / gate epilogue, two weights).  The test
 * suite walks the dispatch with it.  No counterpart in the reference (its launcher picks a kernel by batch bucket,
 * torchao/csrc/cuda/fp6_llm/fp6_linear.cu:72-93). */
int ao_amd_fp6_linear_plan(int64_t M, int64_t K, int64_t N, int ebits, int mbits, int has_norm, int has_residual,
                           int has_gate, int dual, char* out, int64_t out_cap);

/* The same linear for at most 16 activation rows with the module's next elementwise op on its fp16 result fused into the
 * epilogue (exactly one of the two operands, fp16 [M, N], is non-null): out = fp16(linear) + residual (h + attention(...),
 * h + feed_forward(...), TransformerBlock.forward, torchao/_models/llama/model.py:160-163) or
 * out = fp16(silu(gate)) * fp16(linear) (F.silu(self.w1(x)) * self.w3(x), FeedForward.forward, :209-214). */
int ao_amd_fp6_linear_fused(const void* x_f16, int64_t M, int64_t K, const void* weights_native, const void* scale_f16,
                            int64_t N, int ebits, int mbits, const void* residual_f16, const void* gate_f16, void* out_f16,
                            void* stream);

/* W[N,K] fp16 = fp16(fpx value * scale) from the native tiles: the dequantization inside ao_amd_fp6_linear as a pass of
 * its own (the values of the reference's dequantization, utils_parallel_dequant.cuh:47-59), for prefill-sized batches: the
 * host then runs the library fp16 GEMM on it (from 1024 activation rows on the fused kernel is the slower of the two). */
int ao_amd_fp6_native_to_f16(const void* weights_native, const void* scale_f16, int64_t N, int64_t K, int ebits, int mbits,
                             void* out_f16, void* stream);

/* Decode-step fusions over the same linear, for at most 16 activation rows that fit a workgroup's LDS (M * K * 2 bytes at
 * most 64 KB): `_rmsnorm_linear` = linear(rmsnorm(x)) with rmsnorm(x) = fp16(fp16(x * rsqrt(mean(x^2) + eps)) * norm_weight)
 * (RMSNorm.forward then the linear it feeds, torchao/_models/llama/model.py:232-244); `_swiglu` =
 * fp16(silu(linear_gate(x'))) * linear_up(x') over two weights of one shape in one launch, x' = rmsnorm(x) when
 * norm_weight_f16 is given, else x (FeedForward.forward, :209-214). */
int ao_amd_fp6_rmsnorm_linear(const void* x_f16, int64_t M, int64_t K, const void* norm_weight_f16, float eps,
                              const void* weights_native, const void* scale_f16, int64_t N, int ebits, int mbits,
                              void* out_f16, void* stream);
int ao_amd_fp6_swiglu(const void* x_f16, int64_t M, int64_t K, const void* norm_weight_f16, float eps,
                      const void* native_gate, const void* scale_gate_f16, const void* native_up, const void* scale_up_f16,
                      int64_t N, int ebits, int mbits, void* out_f16, void* stream);

/* Measurement aid (no counterpart in the reference): arm a (hipEvent_t start, hipEvent_t stop) pair on the
 * calling thread; the next linear launch (int4wo or fp6) records its kernel's own begin / end timestamps into
 * the pair and disarms, so hipEventElapsedTime(start, stop) is the kernel duration free of launch gaps.
 * Pass NULLs to disarm. */
int ao_amd_profile_next_linear(void* start_event, void* stop_event);

#ifdef __cplusplus
}
#endif
#endif /* AO_AMD_H */
