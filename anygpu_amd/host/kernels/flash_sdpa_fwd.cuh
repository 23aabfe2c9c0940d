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
  The reference's fused kernel (cu_flash_sdpa_fwd_d256_v1) is float32, one matrix, d = 256, no mask; its
  float32 interface is served by sdp_attention_fwd_cuda_flash in sdp.hpp.
*/
void hip_flash_sdpa_fwd_f16(
	const SoftmaxPrologue& prologue,
	const Tensor<float16, CUDA>& qt,
	const Tensor<float16, CUDA>& kt,
	const Tensor<float16, CUDA>& vt,
	Tensor<float16, CUDA>& yt);

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

#endif  // __FLASH_SDPA_FWD_CUH__
