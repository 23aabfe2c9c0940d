// Minimal registry for the host-layer test cases: each case is a function returning its
// verdict; main() selects by kind or by name, prints one "TestCase [name]: PASSED|FAILED" line
// per case and exits non-zero when any selected case failed.
#ifndef __HARNESS__
#define __HARNESS__

#include <functional>
#include <string>
#include <vector>

enum class TestKind
{
	HOST,    // needs no GPU
	GPU,     // allocates device tensors and launches kernels
	DEATH    // expected to terminate the process with exit code 1; only run when named
};

struct TestEntry
{
	std::string name;
	TestKind kind;
	std::function<bool()> body;
};

std::vector<TestEntry>& test_registry();

struct TestRegistrar
{
	TestRegistrar(const char* name, TestKind kind, std::function<bool()> body)
	{
		test_registry().push_back({ name, kind, std::move(body) });
	}
};

#define TEST_CASE(NAME, KIND)                                                     \
	static bool NAME();                                                           \
	static TestRegistrar registrar_##NAME(#NAME, TestKind::KIND, NAME);           \
	static bool NAME()

#endif  // __HARNESS__
