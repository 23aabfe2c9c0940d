// Entry point of the host-layer test harness.
//   anygpu_host_tests --host          run every case that needs no GPU
//   anygpu_host_tests --gpu           run every GPU case
//   anygpu_host_tests --all           both
//   anygpu_host_tests --list          print "kind name" per registered case
//   anygpu_host_tests NAME [NAME...]  run the named cases (the only way to run a DEATH case)
// Exit code: 0 if every selected case passed, 1 otherwise (or when a case aborts the process
// through the fail-stop error path), 2 on a usage error.
#include "harness.hpp"

#include <iostream>
#include <set>

std::vector<TestEntry>& test_registry()
{
	static std::vector<TestEntry> registry;
	return registry;
}

static const char* kind_name(TestKind k)
{
	switch (k)
	{
	case TestKind::HOST: return "host";
	case TestKind::GPU: return "gpu";
	default: return "death";
	}
}

int main(int argc, char** argv)
{
	bool want_host = false, want_gpu = false;
	std::set<std::string> names;
	for (int i = 1; i < argc; ++i)
	{
		const std::string arg = argv[i];
		if (arg == "--host") want_host = true;
		else if (arg == "--gpu") want_gpu = true;
		else if (arg == "--all") want_host = want_gpu = true;
		else if (arg == "--list")
		{
			for (const auto& t : test_registry()) std::cout << kind_name(t.kind) << " " << t.name << "\n";
			return 0;
		}
		else if (!arg.empty() && arg[0] == '-')
		{
			std::cerr << "unknown option " << arg << "\n";
			return 2;
		}
		else names.insert(arg);
	}
	if (!want_host && !want_gpu && names.empty())
	{
		std::cerr << "usage: " << argv[0] << " --host | --gpu | --all | --list | NAME...\n";
		return 2;
	}

	int ran = 0, failed = 0;
	for (const auto& t : test_registry())
	{
		const bool by_name = names.count(t.name) > 0;
		const bool by_kind = (t.kind == TestKind::HOST && want_host) || (t.kind == TestKind::GPU && want_gpu);
		if (!by_name && !by_kind) continue;
		names.erase(t.name);
		const bool ok = t.body();
		std::cout << "TestCase [" << t.name << "]: " << (ok ? "PASSED" : "FAILED") << std::endl;
		++ran;
		failed += ok ? 0 : 1;
	}
	for (const auto& n : names)
	{
		std::cerr << "no such test case: " << n << "\n";
		++failed;
	}
	std::cout << ran << " case(s) run, " << failed << " failed" << std::endl;
	return failed == 0 ? 0 : 1;
}
