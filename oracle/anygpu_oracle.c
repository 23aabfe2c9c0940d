/*
 * CPU oracle for the anyGPU hot path: matmul, row softmax (with the scale / softcap /
 * mask steps the attention caller runs before it) and depthwise causal conv1d + SiLU.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain C, the CPU
 * implementation of the reference (adamtiger/anyGPU, paths relative to its root) with the
 * same loop order, the same accumulator types and the same stride handling, so that the
 * HIP kernels can be checked against "what the reference's CPU path would have produced".
 * Only tests, the smoke check and the CPU-baseline leg of the benchmark may link or load
 * it; the product library never does.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   oracle_tensor_mm_*       integer-valued inputs vs int64 brute force (bit exact), identity /
 *                            ones / pattern closed forms, strided == explicit transpose,
 *                            float64 brute force with the K*2^-24*sum|a*b| bound.
 *   oracle_tensor_gemm_f32   same + bias closed form.
 *   oracle_tensor_softmax_*  row sums, shift invariance, constant rows (1/n exact for n = 2^p),
 *                            two-value closed form, one-hot limit, -inf / lowest -> exact 0,
 *                            long-double brute force.
 *   oracle_tensor_mul_scalar / oracle_tensor_add   elementwise identities.
 *   oracle_sdp_attention_masked_scaled_fwd_f32   float64 softmax(alpha q k^T + mask) v brute force (the
 *                            library formula of the reference generator, scripts/sdp_test_cases.py:171),
 *                            first causal row equals v[0], equality with the chain of the primitives above.
 *   oracle_softcap_f32       odd symmetry, |y| < cap, y(cap*atanh(1/2)) = cap/2, double tanh brute force.
 *   oracle_slide_mask_f32    brute-force visible set {j : i-W < j <= i}, counts min(i+1, W).
 *   oracle_causal_mask_f32   tril closed form.
 *   oracle_tensor_causal_conv1d_*  impulse response, pass-through tap, zero weights, causality
 *                            under perturbation, linearity of the pre-activation, explicit
 *                            zero-padded brute force in float64.
 *   oracle_gemma_linear_softcap_f32   one-hot rows select a weight entry (y = softcap(w[v,h0])), float64
 *                            x w^T then tanh brute force, equality with oracle_tensor_mm over the
 *                            transposed view followed by oracle_softcap.
 *   oracle_tensor_gelu_tanh_f32   gelu(0) = 0, gelu(x) - gelu(-x) = x, limits x and -0 at |x| = 10,
 *                            float64 formula, closeness to the erf form x Phi(x) (the approximation's
 *                            error stays below 1e-3).
 *   oracle_gemma_mlp_upproj_f32   equality with the chain tensor_mm, gelu, tensor_mm, tensor_mul of the
 *                            functions above (bit exact), float64 brute force.
 *   oracle_tensor_silu_f32   silu(0) = 0, silu(x) - silu(-x) = x, float64 formula.
 *   oracle_tensor_rms_norm_f32   constant rows (y = w c / sqrt(c^2 + eps)), sum (y / w)^2 = n at eps = 0, scale
 *                            invariance at eps = 0, zero-centred weights = weights + 1, float64 brute force.
 *   oracle_zamba_gated_rmsnorm_f32   equality with the chain silu, mul, rms_norm (bit exact), z = 0 gives y = 0
 *                            up to the eps floor, float64 brute force.
 *   oracle_causal_conv1d_update_f32   seq_len successive steps from a zero state equal the whole-sequence
 *                            oracle_tensor_causal_conv1d_f32 bit for bit (up to the sign of zero); the state after
 *                            the steps holds the last width-1 samples.
 *   oracle_cvt_f16_to_f32    all 65536 bit patterns vs numpy.float16.
 *   oracle_compare_*         hand-computed three-element cases.
 * On top of those: tests/test_torch_fixtures.py holds tensor_mm, sdp_attention_masked_scaled_fwd, the rule form of the
 * attention (grouped queries, softcap, window), oracle_attention_softmax_f32 (scale -> softcap -> mask -> softmax),
 * tensor_causal_conv1d and its decode step, zamba_gated_rmsnorm, gemma_linear_softcap and gemma_mlp_upproj to fixtures
 * whose expected values PyTorch's library routines computed in float64 (tests/golden/torch_*, written by
 * tests/golden/make_torch_fixtures.py from the one-line formulas of the reference's generators).
 * The reference repository holds no golden vectors for this path (its .dat fixtures are
 * git-ignored and were drawn from an unseeded generator), so nothing here is pinned against
 * reference-held data.  No function of this file is left "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef long long i64;

#define ORACLE_API __attribute__((visibility("default")))

static int clamp_threads(int threads)
{
#ifdef _OPENMP
	if (threads < 1) threads = 1;
	return threads;
#else
	(void)threads;
	return 1;
#endif
}

ORACLE_API int oracle_max_threads(void)
{
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * tensor_mm  --  srcs/ops/mm_ops.hpp:11-45
 *   res[r,c] = sum_l lhs[r,l] * rhs[l,c]; the product is formed in the element type, the
 *   running sum `acc` is float32 whatever the element type is (mm_ops.hpp:32), l ascends,
 *   and every operand is addressed through its own strides (mm_ops.hpp:33-37).
 *   Rows [row_begin, row_end) only are produced so that large cases can be sampled; outer
 *   rows may be spread over threads, which leaves each element's arithmetic order untouched.
 * ---------------------------------------------------------------------------------------- */
#define DEFINE_MM(NAME, T)                                                                     \
ORACLE_API void NAME(const T* lhs, const T* rhs, T* res, i64 m, i64 n, i64 k,                  \
                     i64 ls0, i64 ls1, i64 rs0, i64 rs1, i64 os0, i64 os1,                     \
                     i64 row_begin, i64 row_end, int threads)                                  \
{                                                                                              \
	(void)m;                                                                                   \
	int nt = clamp_threads(threads);                                                           \
	(void)nt;                                                                                  \
	_Pragma("omp parallel for schedule(static) num_threads(nt)")                               \
	for (i64 r = row_begin; r < row_end; ++r)                                                  \
	{                                                                                          \
		for (i64 c = 0; c < n; ++c)                                                            \
		{                                                                                      \
			float acc = 0.f;                                                                   \
			for (i64 l = 0; l < k; ++l)                                                        \
			{                                                                                  \
				T prod = lhs[r * ls0 + l * ls1] * rhs[l * rs0 + c * rs1];                      \
				acc += prod;                                                                   \
			}                                                                                  \
			res[r * os0 + c * os1] = (T)acc;                                                   \
		}                                                                                      \
	}                                                                                          \
}

DEFINE_MM(oracle_tensor_mm_f32, float)
DEFINE_MM(oracle_tensor_mm_f64, double)
DEFINE_MM(oracle_tensor_mm_i32, int32_t)

/* tensor_gemm  --  srcs/ops/mm_ops.hpp:102-144: same sum, then `acc + bt[c]` (bias indexed by column). */
ORACLE_API void oracle_tensor_gemm_f32(const float* xt, const float* wt, const float* bt, float* res,
                                       i64 m, i64 n, i64 k,
                                       i64 xs0, i64 xs1, i64 ws0, i64 ws1, i64 os0, i64 os1,
                                       i64 row_begin, i64 row_end, int threads)
{
	(void)m;
	int nt = clamp_threads(threads);
	(void)nt;
	#pragma omp parallel for schedule(static) num_threads(nt)
	for (i64 r = row_begin; r < row_end; ++r)
	{
		for (i64 c = 0; c < n; ++c)
		{
			float acc = 0.f;
			for (i64 l = 0; l < k; ++l)
			{
				acc += xt[r * xs0 + l * xs1] * wt[l * ws0 + c * ws1];
			}
			res[r * os0 + c * os1] = acc + bt[c];
		}
	}
}

/* ------------------------------------------------------------------------------------------
 * tensor_softmax  --  srcs/ops/softmax_ops.hpp:15-82
 *   per row: running maximum starting from element 0 (:44-52); e_c = (T)exp((double)(x_c - max))
 *   written to y (:58-69); the sum is kept in T and grows left to right (:61,68);
 *   y_c = y_c * ((T)1 / sum) (:72-78).
 * ---------------------------------------------------------------------------------------- */
#define DEFINE_SOFTMAX_ROW(NAME, T)                                                            \
static void NAME(const T* x, T* y, i64 n, i64 xsc, i64 ysc)                                    \
{                                                                                              \
	T max_val = x[0];                                                                          \
	for (i64 c = 1; c < n; ++c)                                                                \
	{                                                                                          \
		T v = x[c * xsc];                                                                      \
		if (v > max_val) max_val = v;                                                          \
	}                                                                                          \
	T exponent = x[0] - max_val;                                                               \
	T exp_val = (T)exp((double)exponent);                                                      \
	y[0] = exp_val;                                                                            \
	T reduced = exp_val;                                                                       \
	for (i64 c = 1; c < n; ++c)                                                                \
	{                                                                                          \
		exponent = x[c * xsc] - max_val;                                                       \
		exp_val = (T)exp((double)exponent);                                                    \
		y[c * ysc] = exp_val;                                                                  \
		reduced += exp_val;                                                                    \
	}                                                                                          \
	T rec_reduced = (T)1.0 / reduced;                                                          \
	for (i64 c = 0; c < n; ++c)                                                                \
	{                                                                                          \
		y[c * ysc] = y[c * ysc] * rec_reduced;                                                 \
	}                                                                                          \
}

DEFINE_SOFTMAX_ROW(softmax_row_f32, float)
DEFINE_SOFTMAX_ROW(softmax_row_f64, double)

#define DEFINE_SOFTMAX(NAME, ROWFN, T)                                                         \
ORACLE_API void NAME(const T* x, T* y, i64 m, i64 n, i64 xs0, i64 xs1, i64 ys0, i64 ys1,       \
                     int threads)                                                              \
{                                                                                              \
	int nt = clamp_threads(threads);                                                           \
	(void)nt;                                                                                  \
	_Pragma("omp parallel for schedule(static) num_threads(nt)")                               \
	for (i64 r = 0; r < m; ++r)                                                                \
	{                                                                                          \
		ROWFN(x + r * xs0, y + r * ys0, n, xs1, ys1);                                          \
	}                                                                                          \
}

DEFINE_SOFTMAX(oracle_tensor_softmax_f32, softmax_row_f32, float)
DEFINE_SOFTMAX(oracle_tensor_softmax_f64, softmax_row_f64, double)

/* tensor_mul(tensor, scalar)  --  srcs/ops/binary_ops.hpp:61-76 */
ORACLE_API void oracle_tensor_mul_scalar_f32(const float* x, float alpha, float* y, i64 length)
{
	for (i64 ix = 0; ix < length; ++ix) y[ix] = x[ix] * alpha;
}

/* tensor_add(tensor, tensor)  --  srcs/ops/binary_ops.hpp:11-29 */
ORACLE_API void oracle_tensor_add_f32(const float* lhs, const float* rhs, float* y, i64 length)
{
	for (i64 ix = 0; ix < length; ++ix) y[ix] = lhs[ix] + rhs[ix];
}

/* softcap(x, cap) = tanhf(x / cap) * cap  --  srcs/models/gemma2/gemma_linsoftcap.cu:3-9 */
ORACLE_API void oracle_softcap_f32(const float* x, float cap, float* y, i64 length)
{
	for (i64 ix = 0; ix < length; ++ix)
	{
		float temp = x[ix] / cap;
		temp = tanhf(temp);
		y[ix] = temp * cap;
	}
}

/* Additive causal mask: 0 on and below the diagonal, -inf above it.
 * scripts/sdp_test_cases.py:164-168 (tril(diagonal=0), masked_fill(~tril, -inf)).
 * `diag` shifts the diagonal for a key axis longer than the query axis: key j is visible to
 * query i iff j <= i + diag. */
ORACLE_API void oracle_causal_mask_f32(float* mask, i64 q_len, i64 k_len, i64 diag)
{
	for (i64 i = 0; i < q_len; ++i)
		for (i64 j = 0; j < k_len; ++j)
			mask[i * k_len + j] = (j <= i + diag) ? 0.f : -INFINITY;
}

/* Sliding-window rule  --  srcs/models/gemma2/gemma_slide_mask.cu:17-29,38:
 * element (seq_idx, j) is replaced by float lowest iff seq_idx >= W and j <= seq_idx - W,
 * otherwise the incoming mask value is kept. */
ORACLE_API void oracle_slide_mask_f32(const float* mask, int32_t window, i64 batch, i64 seq_len, i64 mask_len, float* y)
{
	const float f32_min = -FLT_MAX;
	for (i64 b = 0; b < batch; ++b)
		for (i64 s = 0; s < seq_len; ++s)
			for (i64 j = 0; j < mask_len; ++j)
			{
				i64 off = b * seq_len * mask_len + s * mask_len + j;
				if (s >= window && j <= s - window) y[off] = f32_min;
				else y[off] = mask[off];
			}
}

/* ------------------------------------------------------------------------------------------
 * The chain the attention caller runs on a score matrix before and including softmax:
 *   nqk = tensor_mul(qk, alpha); nqk_masked = tensor_add(nqk, mask); tensor_softmax(nqk_masked)
 *   -- srcs/transformers/sdp.hpp:265-269.
 * With softcap != 0 the capped logits cap*tanh(s/cap) are formed between the scale and the
 * mask add (the order Gemma2 attention uses; no reference call site, see header).
 * The mask of row r is built from the rules above for query index (r % q_len): causal -inf
 * above the diagonal (shifted by diag), then the sliding rule with float lowest when window > 0.
 * Works row by row so that full-size cases need only O(cols) scratch per thread.
 * `row_index` (may be NULL) lists which rows of x to process; outputs are packed densely.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_attention_softmax_f32(const float* x, float* y, i64 rows, i64 cols, i64 x_row_stride,
                                             i64 q_len, i64 diag, float alpha, float softcap,
                                             int causal, i64 window,
                                             const i64* row_index, i64 n_index, int threads)
{
	int nt = clamp_threads(threads);
	(void)nt;
	i64 count = row_index ? n_index : rows;
	#pragma omp parallel num_threads(nt)
	{
		float* nqk = (float*)malloc(sizeof(float) * (size_t)cols);
		float* mask = (float*)malloc(sizeof(float) * (size_t)cols);
		float* tmp = (float*)malloc(sizeof(float) * (size_t)cols);
		#pragma omp for schedule(dynamic, 8)
		for (i64 t = 0; t < count; ++t)
		{
			i64 r = row_index ? row_index[t] : t;
			i64 i = (q_len > 0) ? (r % q_len) : r;
			const float* xr = x + r * x_row_stride;
			oracle_tensor_mul_scalar_f32(xr, alpha, nqk, cols);
			if (softcap != 0.f)
			{
				oracle_softcap_f32(nqk, softcap, tmp, cols);
				memcpy(nqk, tmp, sizeof(float) * (size_t)cols);
			}
			for (i64 j = 0; j < cols; ++j)
			{
				float mv = 0.f;
				if (causal && j > i + diag) mv = -INFINITY;
				mask[j] = mv;
			}
			if (window > 0)
			{
				/* sliding rule on the row of query position i + diag (the absolute position of the query) */
				i64 s = i + diag;
				for (i64 j = 0; j < cols; ++j)
					if (s >= window && j <= s - window) mask[j] = -FLT_MAX;
			}
			oracle_tensor_add_f32(nqk, mask, tmp, cols);
			softmax_row_f32(tmp, y + t * cols, cols, 1, 1);
		}
		free(nqk); free(mask); free(tmp);
	}
}

/* ------------------------------------------------------------------------------------------
 * sdp_attention_masked_scaled_fwd  --  srcs/transformers/sdp.hpp:207-274
 *   q, k, v are [num_mtcs, n, d] (the leading axes folded), mask is [n_q, n_k] shared by all
 *   matrices; per matrix (sdp.hpp:258-271):
 *     kw_tr = tensor_transp(kw); qk = tensor_mm(qw, kw_tr); nqk = tensor_mul(qk, alpha);
 *     nqk_masked = tensor_add(nqk, mask); score = tensor_softmax(nqk_masked); y = tensor_mm(score, vw)
 *   The transpose is taken as a strided view: tensor_mm walks its operands through their strides,
 *   so the sums are formed in the same order as over the transposed copy.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_sdp_attention_masked_scaled_fwd_f32(const float* q, const float* k, const float* v,
                                                           const float* mask, float alpha, float* y,
                                                           i64 num_mtcs, i64 n_q, i64 n_k, i64 d, int threads)
{
	int nt = clamp_threads(threads);
	(void)nt;
	#pragma omp parallel for schedule(static) num_threads(nt)
	for (i64 ix = 0; ix < num_mtcs; ++ix)
	{
		const float* qm = q + ix * n_q * d;
		const float* km = k + ix * n_k * d;
		const float* vm = v + ix * n_k * d;
		float* ym = y + ix * n_q * d;
		float* qk = (float*)malloc(sizeof(float) * (size_t)(n_q * n_k));
		float* tmp = (float*)malloc(sizeof(float) * (size_t)(n_q * n_k));
		/* qk = q [n_q, d] x k^T: k^T as the [d, n_k] view with strides (1, d) */
		oracle_tensor_mm_f32(qm, km, qk, n_q, n_k, d, d, 1, 1, d, n_k, 1, 0, n_q, 1);
		oracle_tensor_mul_scalar_f32(qk, alpha, tmp, n_q * n_k);
		oracle_tensor_add_f32(tmp, mask, qk, n_q * n_k);
		oracle_tensor_softmax_f32(qk, tmp, n_q, n_k, n_k, 1, n_k, 1, 1);
		oracle_tensor_mm_f32(tmp, vm, ym, n_q, d, n_k, n_k, 1, d, 1, d, 1, 0, n_q, 1);
		free(qk); free(tmp);
	}
}

/* ------------------------------------------------------------------------------------------
 * tensor_causal_conv1d  --  srcs/fused/causal_conv1d.hpp:24-87
 *   x (batch, dims, seq_len), w (dims, width), b (dims) -> y (batch, dims, seq_len)
 *   out = 0; for k ascending: delta = k + 1 + six - w; if delta >= 0: out += w[d,k] * x[b,d,delta]  (:66-74)
 *   out += bias (:76); out = out / (1 + exp(-out)) (:79); x and y rows use strides 0 and 1 of
 *   their tensors and unit step along the sequence, w uses stride 0 (:58-60).
 *   `exp` on a float argument binds to the float overload of <cmath> in C++; expf here.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_tensor_causal_conv1d_f32(const float* x, const float* w, const float* bias, float* y,
                                                i64 b, i64 d, i64 s, i64 width,
                                                i64 xs0, i64 xs1, i64 ys0, i64 ys1, i64 ws0,
                                                i64 row_begin, i64 row_end, int threads)
{
	int nt = clamp_threads(threads);
	(void)nt; (void)b;
	/* a "row" is one (batch, channel) pair, numbered bix * d + dix */
	#pragma omp parallel for schedule(static) num_threads(nt)
	for (i64 row = row_begin; row < row_end; ++row)
	{
		i64 bix = row / d, dix = row % d;
		i64 x_offset = bix * xs0 + dix * xs1;
		i64 y_offset = bix * ys0 + dix * ys1;
		i64 w_offset = dix * ws0;
		for (i64 six = 0; six < s; ++six)
		{
			float out = 0;
			for (i64 k = 0; k < width; ++k)
			{
				i64 delta = k + 1 + six - width;
				if (delta >= 0)
				{
					out += w[w_offset + k] * x[x_offset + delta];
				}
			}
			out += bias[dix];
			out = out / (1.0f + expf(-out));
			y[y_offset + six] = out;
		}
	}
}

ORACLE_API void oracle_tensor_causal_conv1d_f64(const double* x, const double* w, const double* bias, double* y,
                                                i64 b, i64 d, i64 s, i64 width,
                                                i64 xs0, i64 xs1, i64 ys0, i64 ys1, i64 ws0,
                                                i64 row_begin, i64 row_end, int threads)
{
	int nt = clamp_threads(threads);
	(void)nt; (void)b;
	#pragma omp parallel for schedule(static) num_threads(nt)
	for (i64 row = row_begin; row < row_end; ++row)
	{
		i64 bix = row / d, dix = row % d;
		i64 x_offset = bix * xs0 + dix * xs1;
		i64 y_offset = bix * ys0 + dix * ys1;
		i64 w_offset = dix * ws0;
		for (i64 six = 0; six < s; ++six)
		{
			double out = 0;
			for (i64 k = 0; k < width; ++k)
			{
				i64 delta = k + 1 + six - width;
				if (delta >= 0)
				{
					out += w[w_offset + k] * x[x_offset + delta];
				}
			}
			out += bias[dix];
			out = out / (1.0 + exp(-out));
			y[y_offset + six] = out;
		}
	}
}

/* ------------------------------------------------------------------------------------------
 * Gemma2 output head with final logit soft-capping  --  srcs/models/gemma2/gemma_linsoftcap.cu:3-33
 *   x [n, hsize], w [vsize, hsize] (the tied embedding table, one row per token id):
 *   acc = 0; for h ascending: acc += x[s,h] * w[v,h]; y[s,v] = softcap(acc, cap) with
 *   softcap(t, cap) = tanhf(t / cap) * cap (:3-9).  The reference has this op on the GPU only;
 *   the loop is its kernel's per-element program, which is sequential in h.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_gemma_linear_softcap_f32(const float* x, const float* w, float cap, float* y,
                                                i64 n, i64 hsize, i64 vsize, int threads)
{
	threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
	for (i64 s = 0; s < n; ++s)
	{
		for (i64 v = 0; v < vsize; ++v)
		{
			float acc = 0.f;
			for (i64 h = 0; h < hsize; ++h) acc += x[s * hsize + h] * w[v * hsize + h];
			float temp = acc / cap;
			temp = tanhf(temp);
			y[s * vsize + v] = temp * cap;
		}
	}
}

/* tensor_gelu(x, approx = true)  --  srcs/ops/math_ops.hpp:83-89
 *   y = x * 0.5 * (1 + tanh((T)sqrt(2.0 / pi) * (x + 0.044715 * x * x * x))), every constant cast to T and
 *   the tanh taken in T (the float overload for float32). */
ORACLE_API void oracle_tensor_gelu_tanh_f32(const float* x, float* y, i64 length)
{
	const float c = (float)sqrt(2.0 / 3.14159265358979323846);
	for (i64 k = 0; k < length; ++k)
	{
		float t = x[k];
		y[k] = t * 0.5f * (1.0f + tanhf(c * (t + 0.044715f * t * t * t)));
	}
}

/* tensor_mul(tensor, tensor)  --  srcs/ops/binary_ops.hpp:103-121 */
ORACLE_API void oracle_tensor_mul_f32(const float* lhs, const float* rhs, float* y, i64 length)
{
	for (i64 ix = 0; ix < length; ++ix) y[ix] = lhs[ix] * rhs[ix];
}

/* ------------------------------------------------------------------------------------------
 * Gemma2 MLP, gate and up projections  --  srcs/models/gemma2/gemma_mlp.hpp:85-90 (the path every
 * device takes by default; cu_mlp_gemma2_fused_upproj_f32_v1/_v2 compute the same value in one kernel)
 *   gated = tensor_linear(x, w_gate) = tensor_mm(x, w_gate) (srcs/ops/mm_ops.hpp:205-232);
 *   act = tensor_gelu(gated, true); up = tensor_linear(x, w_up); y = tensor_mul(act, up)
 *   x [n, hsize], w_gate and w_up [hsize, isize] row-major, y [n, isize].
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_gemma_mlp_upproj_f32(const float* x, const float* w_gate, const float* w_up, float* y,
                                            i64 n, i64 hsize, i64 isize, int threads)
{
	threads = clamp_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static)
	for (i64 r = 0; r < n; ++r)
	{
		for (i64 c = 0; c < isize; ++c)
		{
			float gate = 0.f, up = 0.f;
			for (i64 l = 0; l < hsize; ++l) gate += x[r * hsize + l] * w_gate[l * isize + c];
			for (i64 l = 0; l < hsize; ++l) up += x[r * hsize + l] * w_up[l * isize + c];
			float act;
			oracle_tensor_gelu_tanh_f32(&gate, &act, 1);
			y[r * isize + c] = act * up;
		}
	}
}

/* tensor_silu  --  srcs/ops/math_ops.hpp:16-35: y = x / (1 + exp(-x)); the float overload of exp for float32 */
ORACLE_API void oracle_tensor_silu_f32(const float* x, float* y, i64 length)
{
	for (i64 k = 0; k < length; ++k) y[k] = x[k] / (1.0f + expf(-x[k]));
}

/* ------------------------------------------------------------------------------------------
 * tensor_rms_norm  --  srcs/ops/norm_ops.hpp:129-190
 *   per region of `size` contiguous elements: accum = sum x^2 left to right in T (:170-176);
 *   mean = accum / size (:178); y = (x / sqrt(mean + eps)) * (w + delta), delta = 1 for zero-centred
 *   weights else 0 (:148,181-187).
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_tensor_rms_norm_f32(const float* x, const float* w, float eps, int zero_centered, float* y,
                                           i64 regions, i64 size)
{
	const float delta = zero_centered ? 1.0f : 0.0f;
	for (i64 r = 0; r < regions; ++r)
	{
		const float* xr = x + r * size;
		float* yr = y + r * size;
		float accum = 0.f;
		for (i64 ix = 0; ix < size; ++ix) accum += xr[ix] * xr[ix];
		const float mean = accum / (float)size;
		for (i64 ix = 0; ix < size; ++ix) yr[ix] = (xr[ix] / sqrtf(mean + eps)) * (w[ix] + delta);
	}
}

/* tensor_zamba_gated_rmsnorm  --  srcs/models/zamba2/zamba_gated_rmsnorm.hpp:9-23
 *   silu_z = tensor_silu(z); gated = tensor_mul(x, silu_z); y = tensor_rms_norm(gated, -1, w, eps)
 *   (the group size argument is unused there: one group spans the row). */
ORACLE_API void oracle_zamba_gated_rmsnorm_f32(const float* x, const float* z, const float* w, float eps, float* y,
                                               i64 rows, i64 cols)
{
	float* gated = (float*)malloc((size_t)(cols > 0 ? cols : 1) * sizeof(float));
	for (i64 r = 0; r < rows; ++r)
	{
		oracle_tensor_silu_f32(z + r * cols, gated, cols);
		for (i64 c = 0; c < cols; ++c) gated[c] = x[r * cols + c] * gated[c];
		oracle_tensor_rms_norm_f32(gated, w, eps, 0, y + r * cols, 1, cols);
	}
	free(gated);
}

/* ------------------------------------------------------------------------------------------
 * Decode step of tensor_causal_conv1d.  The reference has only the whole-sequence form
 * (srcs/fused/causal_conv1d.hpp:24-87); this is its loop body for one position s with the samples
 * x[s - (width-1) .. s - 1] handed over in `state` (oldest first) instead of being read from the row:
 *   out = 0; for k ascending: out += w[d,k] * (k < width-1 ? state[k] : x); out += bias; out = out / (1 + exp(-out))
 * then the state is shifted by one and takes x.  From a zero state the terms the whole-sequence loop
 * skips (negative positions) are added here as w * 0, which changes no sum.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API void oracle_causal_conv1d_update_f32(const float* x, float* state, const float* w, const float* b, float* y,
                                                i64 batch, i64 dims, i64 width)
{
	for (i64 row = 0; row < batch * dims; ++row)
	{
		const i64 d = row % dims;
		float* st = state + row * (width - 1);
		float out = 0.f;
		for (i64 k = 0; k < width; ++k) out += w[d * width + k] * (k < width - 1 ? st[k] : x[row]);
		out += b[d];
		y[row] = out / (1.0f + expf(-out));
		for (i64 k = 0; k + 1 < width - 1; ++k) st[k] = st[k + 1];
		if (width > 1) st[width - 2] = x[row];
	}
}

/* ------------------------------------------------------------------------------------------
 * fp16 protocol: the reference has no CPU half arithmetic; half tensors are up-cast element by
 * element to float32 (cvt_tensor_datatype, srcs/core/tensor.hpp:388-410, through __half2float,
 * srcs/core/core.hpp:263-267) and the float32 CPU op is run (tests/tests.cpp:146-151).
 * The conversion is exact: IEEE binary16 -> binary32.
 * ---------------------------------------------------------------------------------------- */
static float half_bits_to_float(uint16_t h)
{
	uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
	uint32_t exp = (h >> 10) & 0x1Fu;
	uint32_t man = h & 0x3FFu;
	uint32_t bits;
	if (exp == 0)
	{
		if (man == 0) bits = sign;
		else
		{
			/* subnormal half: normalise */
			int e = -1;
			do { ++e; man <<= 1; } while ((man & 0x400u) == 0);
			man &= 0x3FFu;
			bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
		}
	}
	else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
	else bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
	float f;
	memcpy(&f, &bits, sizeof(f));
	return f;
}

ORACLE_API void oracle_cvt_f16_to_f32(const uint16_t* src, float* dst, i64 n)
{
	for (i64 ix = 0; ix < n; ++ix) dst[ix] = half_bits_to_float(src[ix]);
}

/* ------------------------------------------------------------------------------------------
 * Comparators  --  tests/test_tools.hpp
 *   abs:     every |e - a| < abs_tol                                   (:23-43)
 *   reldiff: every |e - a| / (|e| + 1e-8) < rel_tol                    (:45-66)
 *   l2:      sqrt( sum (e-a)^2 / sum (e^2 + 1e-8) ) < rel_l2, float32 running sums (:76-103)
 * Each returns 1 for "equal", 0 otherwise; *worst receives the largest metric seen.
 * ---------------------------------------------------------------------------------------- */
ORACLE_API int oracle_compare_abs_f32(const float* actual, const float* expected, i64 length, float abs_tol, float* worst)
{
	int eq = 1;
	float w = 0.f;
	for (i64 ix = 0; ix < length; ++ix)
	{
		float d = fabsf(expected[ix] - actual[ix]);
		eq = eq && (d < abs_tol);
		if (!(d <= w)) w = d;
	}
	if (worst) *worst = w;
	return eq;
}

ORACLE_API int oracle_compare_reldiff_f32(const float* actual, const float* expected, i64 length, float rel_tol, float* worst)
{
	int eq = 1;
	float w = 0.f;
	for (i64 ix = 0; ix < length; ++ix)
	{
		float d = fabsf(expected[ix] - actual[ix]) / (fabsf(expected[ix]) + (float)1e-8);
		eq = eq && (d < rel_tol);
		if (!(d <= w)) w = d;
	}
	if (worst) *worst = w;
	return eq;
}

ORACLE_API int oracle_compare_l2_f32(const float* actual, const float* expected, i64 length, float rel_l2, float* value)
{
	float cum_square_diff = 0.f;
	float cum_square = 0.f;
	for (i64 ix = 0; ix < length; ++ix)
	{
		float temp = expected[ix] - actual[ix];
		float residual = temp * temp;
		cum_square_diff += residual;
		cum_square += expected[ix] * expected[ix] + 1e-8f;
	}
	float l2 = sqrtf(cum_square_diff / cum_square);
	if (value) *value = l2;
	return l2 < rel_l2;
}
