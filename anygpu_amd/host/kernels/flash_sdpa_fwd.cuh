// Fused attention launchers of the host layer (reference: srcs/kernels/cuda/flash_sdpa_fwd.cuh:6-15).
#ifndef __FLASH_SDPA_FWD_CUH__
#define __FLASH_SDPA_FWD_CUH__

#include "tensor.hpp"
#include "softmax_ops.cuh"

/*
  y = softmax(rules(alpha q k^T)) v in one kernel, half precision, fp32 scores and sums.
  qt, yt (..., heads, n_q, d), kt, vt (..., kv_heads, n_k, d) with heads a multiple of kv_heads and
  d 64, 128 or 256.  Of the prologue, alpha, softcap, causal and window are used; the causal diagonal sits
  at n_k - n_q (q_len and diag of the prologue are implied by the shapes).
  The reference's fused kernel (cu_flash_sdpa_fwd_d256_v1) is float32, one matrix, d = 256, no mask: below.
*/
void hip_flash_sdpa_fwd_f16(
	const SoftmaxPrologue& prologue,
	const Tensor<float16, CUDA>& qt,
	const Tensor<float16, CUDA>& kt,
	const Tensor<float16, CUDA>& vt,
	Tensor<float16, CUDA>& yt);

/*
  The same in float32 (the fp32 matrix instruction; results agree with the unfused float32 path to fp32 rounding).
*/
void hip_flash_sdpa_fwd_f32(
	const SoftmaxPrologue& prologue,
	const Tensor<float32, CUDA>& qt,
	const Tensor<float32, CUDA>& kt,
	const Tensor<float32, CUDA>& vt,
	Tensor<float32, CUDA>& yt);

/*
  The float32 kernel with the mask as a tensor: y = softmax(alpha q k^T + mask) v, mask [.., n_q, n_k] with leading 1s,
  shared by all matrices of q (the interface of sdp_attention_masked_scaled_fwd, srcs/transformers/sdp.hpp:207-274).
*/
void hip_flash_sdpa_fwd_masked_f32(
	const float32 alpha,
	const Tensor<float32, CUDA>& qt,
	const Tensor<float32, CUDA>& kt,
	const Tensor<float32, CUDA>& vt,
	const Tensor<float32, CUDA>& mask,
	Tensor<float32, CUDA>& yt);

/* The same in half precision (mask of halves, fp32 sums on the matrix cores). */
void hip_flash_sdpa_fwd_masked_f16(
	const float32 alpha,
	const Tensor<float16, CUDA>& qt,
	const Tensor<float16, CUDA>& kt,
	const Tensor<float16, CUDA>& vt,
	const Tensor<float16, CUDA>& mask,
	Tensor<float16, CUDA>& yt);

/*
  The reference's fused kernel by its own name and contract (srcs/kernels/cuda/flash_sdpa_fwd.cuh:6-15): one
  matrix, hidden dim 256, no mask; any sequence length here.
*/
void cu_flash_sdpa_fwd_d256_v1(
	const float32 alpha,
	const Tensor<float32, CUDA>& qt,
	const Tensor<float32, CUDA>& kt,
	const Tensor<float32, CUDA>& vt,
	Tensor<float32, CUDA>& yt);

/*
  Decode form for generation steps: (query heads per key / value head) x n_q <= 16.  The key range is split over
  many waves; their partial results pass through `workspace`, a float32 tensor with at least
  hip_flash_sdpa_decode_workspace_floats(...) elements, which the caller owns and may reuse.
*/
bool hip_flash_sdpa_decode_applies(
	const Tensor<float16, CUDA>& qt,
	const Tensor<float16, CUDA>& kt);

int64 hip_flash_sdpa_decode_workspace_floats(
	const SoftmaxPrologue& prologue,
	const Tensor<float16, CUDA>& qt,
	const Tensor<float16, CUDA>& kt);

void hip_flash_sdpa_decode_f16(
	const SoftmaxPrologue& prologue,
	const Tensor<float16, CUDA>& qt,
	const Tensor<float16, CUDA>& kt,
	const Tensor<float16, CUDA>& vt,
	Tensor<float32, CUDA>& workspace,
	Tensor<float16, CUDA>& yt);

/*
  The decode form in float32 (same roles of the arguments).
*/
bool hip_flash_sdpa_decode_applies(
	const Tensor<float32, CUDA>& qt,
	const Tensor<float32, CUDA>& kt);

int64 hip_flash_sdpa_decode_workspace_floats(
	const SoftmaxPrologue& prologue,
	const Tensor<float32, CUDA>& qt,
	const Tensor<float32, CUDA>& kt);

void hip_flash_sdpa_decode_f32(
	const SoftmaxPrologue& prologue,
	const Tensor<float32, CUDA>& qt,
	const Tensor<float32, CUDA>& kt,
	const Tensor<float32, CUDA>& vt,
	Tensor<float32, CUDA>& workspace,
	Tensor<float32, CUDA>& yt);

#endif  // __FLASH_SDPA_FWD_CUH__
