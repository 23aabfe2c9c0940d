// Golden-file cases in the style of the reference's tests/ext_torch_tests.cpp: load inputs and
// the expected output from .dat files, run the CPU and / or GPU operator, compare.  The fixture
// folder comes from the environment variable ANYGPU_GOLDEN_DIR (default: tests/golden relative to
// the working directory); the fixtures are small files kept next to the Python tests.
#include "harness.hpp"

#include "ops.hpp"
#include "sdp.hpp"
#include "gemma_linsoftcap.hpp"
#include "gemma_mlp.hpp"
#include "zamba_gated_rmsnorm.hpp"
#include "fast_mm.cuh"
#include "dat_file.hpp"
#include "test_tools.hpp"

namespace {

std::filesystem::path golden_dir()
{
	const char* env = std::getenv("ANYGPU_GOLDEN_DIR");
	return std::filesystem::path(env ? env : "tests/golden");
}

template<typename Fn>
bool same_shape_and(const Tensor<float32, CPU>& expected, const Tensor<float32, CPU>& actual, Fn&& cmp)
{
	return elementwise_compatible(expected, actual) && cmp(actual, expected);
}

struct AttentionFixture
{
	Tensor<float32, CPU> scores, mask, expected;
	int64 q_len, k_len;
};

AttentionFixture load_attention_fixture(const char* name)
{
	const auto path = golden_dir() / name;
	AttentionFixture f;
	f.scores = load_tensor((path / "scores.dat").string());
	f.mask = load_tensor((path / "mask.dat").string());
	f.expected = load_tensor((path / "y.dat").string());
	f.q_len = f.mask.shape[0];
	f.k_len = f.mask.shape[1];
	return f;
}

// mul -> (softcap) -> add -> softmax per head on the host, the call order of the attention block
Tensor<float32, CPU> host_attention_probabilities(const AttentionFixture& f, float32 alpha, float32 cap)
{
	const int64 heads = f.scores.shape[0] / f.q_len;
	Tensor<float32, CPU> out(f.scores.dim, f.scores.shape);
	auto in_heads = tensor_split(tensor_view(f.scores, { heads, f.q_len, f.k_len }), heads);
	auto out_heads = tensor_split(tensor_view(out, { heads, f.q_len, f.k_len }), heads);
	for (int64 h = 0; h < heads; ++h)
	{
		auto s = tensor_mul(tensor_view(in_heads[h], { f.q_len, f.k_len }), alpha);
		if (cap != 0.f)
			for (int64 ix = 0; ix < s.size(); ++ix) s.buffer()[ix] = tanhf(s.buffer()[ix] / cap) * cap;
		auto p = tensor_softmax(tensor_add(s, f.mask));
		std::memcpy(out_heads[h].buffer(), p.buffer(), sizeof(float32) * p.numel());
	}
	return out;
}

}  // namespace

TEST_CASE(external_test_causal_conv1d_fwd_f32_cpu, HOST)
{
	const auto path = golden_dir() / "test_causal_conv1d_fwd_f32";
	auto hx = load_tensor((path / "x.dat").string());
	auto hw = load_tensor((path / "w.dat").string());
	auto hb = load_tensor((path / "b.dat").string());
	auto exp_hy = load_tensor((path / "y.dat").string());
	auto act_hy = tensor_causal_conv1d(hx, hw, hb);
	return same_shape_and(exp_hy, act_hy, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-6f); });
}

TEST_CASE(external_test_causal_conv1d_fwd_f32, GPU)
{
	const auto path = golden_dir() / "test_causal_conv1d_fwd_f32";
	auto hx = load_tensor((path / "x.dat").string());
	auto hw = load_tensor((path / "w.dat").string());
	auto hb = load_tensor((path / "b.dat").string());
	auto exp_hy = load_tensor((path / "y.dat").string());
	auto act_hy = tensor_causal_conv1d(hx.copy_to_cuda(), hw.copy_to_cuda(), hb.copy_to_cuda()).copy_to_host();
	return same_shape_and(exp_hy, act_hy, [](auto& a, auto& e) { return compare_data_buffers(a, e); });
}

TEST_CASE(external_test_mm_f32_cpu, HOST)
{
	const auto path = golden_dir() / "test_mm_m24_n16_k40_f32";
	auto hx = load_tensor((path / "x.dat").string());
	auto hw = load_tensor((path / "w.dat").string());
	auto exp_hy = load_tensor((path / "y.dat").string());
	auto act_hy = tensor_mm(hx, hw);
	// same loop order and accumulator as the generator of the fixture: identical to the last bit
	return elementwise_compatible(exp_hy, act_hy) &&
	       std::memcmp(exp_hy.buffer(), act_hy.buffer(), sizeof(float32) * exp_hy.numel()) == 0;
}

TEST_CASE(external_test_mm_f32, GPU)
{
	const auto path = golden_dir() / "test_mm_m24_n16_k40_f32";
	auto hx = load_tensor((path / "x.dat").string());
	auto hw = load_tensor((path / "w.dat").string());
	auto exp_hy = load_tensor((path / "y.dat").string());
	Tensor<float32, CUDA> act_dy(exp_hy.dim, exp_hy.shape);
	cu_fast_mm_f32_v4_1(hx.copy_to_cuda(), hw.copy_to_cuda(), act_dy);
	auto act_hy = act_dy.copy_to_host();
	return same_shape_and(exp_hy, act_hy, [](auto& a, auto& e) { return compare_data_buffers_reldiff(a, e); });
}

TEST_CASE(external_test_mm_f16, GPU)
{
	const auto path = golden_dir() / "test_mm_m64_n64_k128_f16";
	auto hx = load_tensor<float16>((path / "x.dat").string());
	auto hw = load_tensor<float16>((path / "w.dat").string());
	auto exp_hy = cvt_tensor_datatype<float32, float16>(load_tensor<float16>((path / "y.dat").string()));
	Tensor<float16, CUDA> act_dy(exp_hy.dim, exp_hy.shape);
	cu_fast_mm_f16_v3_2(hx.copy_to_cuda(), hw.copy_to_cuda(), act_dy);
	auto act_hy = cvt_tensor_datatype<float32, float16>(act_dy.copy_to_host());
	return same_shape_and(exp_hy, act_hy, [](auto& a, auto& e) { return compare_data_buffers_l2(a, e, 0.04f); });
}

TEST_CASE(external_test_softmax_masked_scaled_f32_cpu, HOST)
{
	auto f = load_attention_fixture("test_softmax_masked_scaled_f32");
	auto act = host_attention_probabilities(f, 0.125f, 0.f);
	return same_shape_and(f.expected, act, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-7f); });
}

TEST_CASE(external_test_softmax_masked_scaled_f32, GPU)
{
	auto f = load_attention_fixture("test_softmax_masked_scaled_f32");
	SoftmaxPrologue p;
	p.alpha = 0.125f; p.causal = true; p.q_len = f.q_len;
	auto act = tensor_softmax(f.scores.copy_to_cuda(), p).copy_to_host();
	return same_shape_and(f.expected, act, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-5f); });
}

TEST_CASE(external_test_softmax_softcap_window_f32_cpu, HOST)
{
	auto f = load_attention_fixture("test_softmax_softcap_window_f32");
	auto act = host_attention_probabilities(f, 0.0625f, 50.f);
	return same_shape_and(f.expected, act, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-7f); });
}

TEST_CASE(external_test_softmax_softcap_window_f32, GPU)
{
	auto f = load_attention_fixture("test_softmax_softcap_window_f32");
	SoftmaxPrologue p;
	p.alpha = 0.0625f; p.softcap = 50.f; p.causal = true; p.window = 6; p.q_len = f.q_len;
	auto act = tensor_softmax(f.scores.copy_to_cuda(), p).copy_to_host();
	return same_shape_and(f.expected, act, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-5f); });
}

TEST_CASE(external_test_sdp_masked_scaled_fwd_f32_cpu, HOST)
{
	const auto path = golden_dir() / "test_sdp_fwd_masked_scaled_f32_16_32";
	auto hq = load_tensor((path / "q.dat").string());
	auto hk = load_tensor((path / "k.dat").string());
	auto hv = load_tensor((path / "v.dat").string());
	auto hmask = load_tensor((path / "mask.dat").string());
	auto hy = load_tensor((path / "y.dat").string());
	auto act = sdp_attention_masked_scaled_fwd(hq, hk, hv, hmask, 0.125f);
	// same chain, same order as the generator of the fixture: identical to the last bit
	return elementwise_compatible(act, hy) && std::memcmp(act.buffer(), hy.buffer(), sizeof(float32) * hy.numel()) == 0;
}

TEST_CASE(external_test_sdp_masked_scaled_fwd_f32, GPU)
{
	const auto path = golden_dir() / "test_sdp_fwd_masked_scaled_f32_16_32";
	auto hq = load_tensor((path / "q.dat").string());
	auto hk = load_tensor((path / "k.dat").string());
	auto hv = load_tensor((path / "v.dat").string());
	auto hmask = load_tensor((path / "mask.dat").string());
	auto hy = load_tensor((path / "y.dat").string());

	auto dy = sdp_attention_masked_scaled_fwd(hq.copy_to_cuda(), hk.copy_to_cuda(), hv.copy_to_cuda(),
	                                          hmask.copy_to_cuda(), 0.125f);
	auto hy_from_cuda = dy.copy_to_host();
	return elementwise_compatible(hy_from_cuda, hy) && compare_data_buffers(hy_from_cuda, hy);
}

/* ---- cases of the Gemma2 / Zamba2 callers, bodies after tests/gemma2_tests.cpp and tests/zamba2_tests.cpp ---- */

TEST_CASE(external_test_gemma2_lmhead_softcap, GPU)
{
	auto path = golden_dir() / "test_gemma2_lmhead_softcap";
	// hw is tied to the embedding weights
	auto hx = load_tensor((path / "in_0.dat").string());
	auto hw = load_tensor((path / "gemma2_causal_lm.gemma2forcausallm.model.embed_tokens.weight.dat").string());
	auto exp_hy = load_tensor((path / "out_0.dat").string());

	auto dx = hx.copy_to_cuda();
	auto dw = hw.copy_to_cuda();
	auto act_dy_cuda = tensor_gemma_linear_softcap(dx, dw, 30.f);
	auto act_hy_cuda = act_dy_cuda.copy_to_host();
	return same_shape_and(exp_hy, act_hy_cuda, [](auto& a, auto& e) { return compare_data_buffers(a, e); });
}

TEST_CASE(external_test_gemma2_decoder_mlp_cpu, HOST)
{
	auto path = golden_dir() / "test_gemma2decoder_mlp";
	auto hx = load_tensor((path / "in_0.dat").string());
	auto exp_hy = load_tensor((path / "out_0.dat").string());
	GemmaMLPweights<float32, CPU> mlp_weights;
	mlp_weights.load_weights(
		(path / "gemma2decoder_mlp.gemma2mlp.gate_proj.weight.dat").string(),
		(path / "gemma2decoder_mlp.gemma2mlp.up_proj.weight.dat").string(),
		(path / "gemma2decoder_mlp.gemma2mlp.down_proj.weight.dat").string());
	auto act_hy = tensor_gemma_mlp(mlp_weights, hx);
	return same_shape_and(exp_hy, act_hy, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-5f); });
}

TEST_CASE(external_test_gemma2_decoder_mlp, GPU)
{
	auto path = golden_dir() / "test_gemma2decoder_mlp";
	auto hx = load_tensor((path / "in_0.dat").string());
	auto exp_hy = load_tensor((path / "out_0.dat").string());

	GemmaMLPweights<float32, CUDA> mlp_weights;
	mlp_weights.load_weights(
		(path / "gemma2decoder_mlp.gemma2mlp.gate_proj.weight.dat").string(),
		(path / "gemma2decoder_mlp.gemma2mlp.up_proj.weight.dat").string(),
		(path / "gemma2decoder_mlp.gemma2mlp.down_proj.weight.dat").string());

	auto dx = hx.copy_to_cuda();
	auto act_dy_cuda = tensor_gemma_mlp(mlp_weights, dx);
	auto act_hy_cuda = act_dy_cuda.copy_to_host();
	return same_shape_and(exp_hy, act_hy_cuda, [](auto& a, auto& e) { return compare_data_buffers(a, e); });
}

TEST_CASE(external_test_mamba2_layer_gated_rmsnorm_cpu, HOST)
{
	auto path = golden_dir() / "test_mamba2layer_gated_rmsnorm";
	auto hx = load_tensor((path / "in_0.dat").string());
	auto hz = load_tensor((path / "in_1.dat").string());
	auto hw = load_tensor((path / "mamba2layer_rmsnorm.rmsnorm.weight.dat").string());
	auto exp_hy = load_tensor((path / "out_0.dat").string());
	auto act_hy = tensor_zamba_gated_rmsnorm(hx, hz, hw, 64, 1e-5f);
	return same_shape_and(exp_hy, act_hy, [](auto& a, auto& e) { return compare_data_buffers(a, e, 1e-6f); });
}

TEST_CASE(external_test_mamba2_layer_gated_rmsnorm, GPU)
{
	auto path = golden_dir() / "test_mamba2layer_gated_rmsnorm";

	// constant params
	const float32 eps = 1e-5f;
	const int32 gsize = 64;  // group size: the row

	auto hx = load_tensor((path / "in_0.dat").string());
	auto hz = load_tensor((path / "in_1.dat").string());
	auto hw = load_tensor((path / "mamba2layer_rmsnorm.rmsnorm.weight.dat").string());
	auto exp_hy = load_tensor((path / "out_0.dat").string());

	auto dx = hx.copy_to_cuda();
	auto dz = hz.copy_to_cuda();
	auto dw = hw.copy_to_cuda();
	auto act_dy_cuda = tensor_zamba_gated_rmsnorm(dx, dz, dw, gsize, eps);
	auto act_hy_cuda = act_dy_cuda.copy_to_host();
	return same_shape_and(exp_hy, act_hy_cuda, [](auto& a, auto& e) { return compare_data_buffers(a, e); });
}

TEST_CASE(external_test_sdp_rules_f16_gqa, GPU)
{
	auto path = golden_dir() / "test_sdp_rules_f16_gqa";
	auto hq = load_tensor<float16>((path / "q.dat").string());
	auto hk = load_tensor<float16>((path / "k.dat").string());
	auto hv = load_tensor<float16>((path / "v.dat").string());
	auto exp_hy = load_tensor((path / "y.dat").string());
	SoftmaxPrologue rules;
	rules.alpha = 0.125f;
	rules.softcap = 20.f;
	rules.causal = true;
	rules.window = 12;
	auto act = cvt_tensor_datatype<float32, float16>(
		sdp_attention_rules_fwd(hq.copy_to_cuda(), hk.copy_to_cuda(), hv.copy_to_cuda(), rules).copy_to_host());
	return same_shape_and(exp_hy, act, [](auto& a, auto& e) { return compare_data_buffers_l2(a, e, 4e-3f) && compare_data_buffers(a, e, 2e-2f); });
}
