// Comparators of the test harness (reference: tests/test_tools.hpp:7-103): exact for integers,
// absolute tolerance (default 1e-3), elementwise relative difference |e - a| / (|e| + 1e-8), and
// a global relative L2 distance for half-precision results checked against a float32 CPU run.
#ifndef __TEST_TOOLS__
#define __TEST_TOOLS__

#include "tensor.hpp"
#include "core_concepts.hpp"

namespace test_detail {

// prints the first `limit` offending pairs
struct MismatchPrinter
{
	int limit;
	int printed = 0;
	template<typename T> void operator()(int64 ix, T expected, T actual)
	{
		if (printed++ < limit) std::cout << ix << " [" << expected << " <> " << actual << "] \n";
	}
};

}  // namespace test_detail

template<IntegerType T>
static bool compare_data_buffers(const Tensor<T, CPU>& actual, const Tensor<T, CPU>& expected)
{
	const T* e = expected.buffer();
	const T* a = actual.buffer();
	return std::equal(e, e + expected.size(), a);
}

template<PreciseFloatType T>
static bool compare_data_buffers(const Tensor<T, CPU>& actual, const Tensor<T, CPU>& expected, const float32 abs_tol = 0.001f)
{
	const T* e = expected.buffer();
	const T* a = actual.buffer();
	const int64 length = expected.size();
	test_detail::MismatchPrinter report{ 20 };
	bool eq = true;
	for (int64 ix = 0; ix < length; ++ix)
	{
		const bool ok = std::abs(e[ix] - a[ix]) < static_cast<T>(abs_tol);
		if (!ok) report(ix, e[ix], a[ix]);
		eq = eq && ok;
	}
	return eq;
}

template<PreciseFloatType T>
static bool compare_data_buffers_reldiff(const Tensor<T, CPU>& actual, const Tensor<T, CPU>& expected, const float32 rel_tol = 0.01f)
{
	const T* e = expected.buffer();
	const T* a = actual.buffer();
	const int64 length = expected.size();
	test_detail::MismatchPrinter report{ 10 };
	bool eq = true;
	for (int64 ix = 0; ix < length; ++ix)
	{
		const bool ok = std::abs(e[ix] - a[ix]) / (std::abs(e[ix]) + static_cast<T>(1e-8)) < static_cast<T>(rel_tol);
		if (!ok) report(ix, e[ix], a[ix]);
		eq = eq && ok;
	}
	return eq;
}

template<PreciseFloatType T>
static bool compare_data_buffers_l2(const Tensor<T, CPU>& actual, const Tensor<T, CPU>& expected, const float32 rel_l2 = 0.01f)
{
	const T* e = expected.buffer();
	const T* a = actual.buffer();
	const int64 length = expected.size();
	float32 sum_sq_diff = 0.f;
	float32 sum_sq = 0.f;
	for (int64 ix = 0; ix < length; ++ix)
	{
		const float32 d = static_cast<float32>(e[ix] - a[ix]);
		sum_sq_diff += d * d;
		sum_sq += static_cast<float32>(e[ix]) * static_cast<float32>(e[ix]) + 1e-8f;
	}
	const float32 l2 = sqrtf(sum_sq_diff / sum_sq);
	if (!(l2 < rel_l2)) std::cout << "L2 rel difference: " << l2 << std::endl;
	return l2 < rel_l2;
}

#endif  // __TEST_TOOLS__
