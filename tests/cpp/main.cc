// Runner of the host-API tests.  Usage: host_tests [--list] [--cpu] [filter]
//   --cpu    run only the suites whose name ends in "Cpu" (no GPU needed)
//   filter   substring of "Suite.Name"
#include <cstring>

#include "tests/cpp/mini_test.h"

int main(int argc, char** argv) {
  bool list = false, cpu_only = false;
  std::string filter;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--list")) list = true;
    else if (!std::strcmp(argv[i], "--cpu")) cpu_only = true;
    else filter = argv[i];
  }
  int ran = 0, failed = 0;
  for (const auto& test : mini_test::Registry()) {
    const std::string full = test.suite + "." + test.name;
    const bool is_cpu = test.suite.size() >= 3 && test.suite.rfind("Cpu") == test.suite.size() - 3;
    if (cpu_only && !is_cpu) continue;
    if (!filter.empty() && full.find(filter) == std::string::npos) continue;
    if (list) {
      std::cout << full << "\n";
      continue;
    }
    std::cout << "[ RUN  ] " << full << std::endl;
    const int before = mini_test::Failures();
    test.body();
    ++ran;
    if (mini_test::Failures() != before) {
      ++failed;
      std::cout << "[ FAIL ] " << full << std::endl;
    } else {
      std::cout << "[  OK  ] " << full << std::endl;
    }
  }
  if (!list) std::cout << ran << " tests ran, " << failed << " failed" << std::endl;
  return failed == 0 ? 0 : 1;
}
