// Host-only driver of the C++ tensor printer (am::pretty_host in include/am_hip_tensor.hpp): builds the
// input a test case describes, prints the formatted tensor to stdout. tests/test_display.py runs it on
// every literal of tests/golden/display_vectors.json; built with -fsanitize=address,undefined. No device.
//
//   test_display_host <i64|f64> <values v...|arange a b|linspace a b n|vandermonde n> -- <shape...> -- <specifier> <precision>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "am_hip_tensor.hpp"

template <typename T>
static int run(const std::vector<std::string>& gen, const am::Shape& shape, const std::string& spec, int precision) {
  std::vector<T> v;
  if (gen[0] == "values") {
    for (size_t i = 1; i < gen.size(); ++i) v.push_back((T)std::atof(gen[i].c_str()));
  } else if (gen[0] == "arange") {
    for (long long x = std::atoll(gen[1].c_str()); x < std::atoll(gen[2].c_str()); ++x) v.push_back((T)x);
  } else if (gen[0] == "linspace") {
    const double a = std::atof(gen[1].c_str()), b = std::atof(gen[2].c_str());
    const int n = std::atoi(gen[3].c_str());
    const double step = (b - a) / (n - 1);
    for (int i = 0; i < n; ++i) v.push_back((T)(i == n - 1 ? b : a + i * step));
  } else if (gen[0] == "vandermonde") {
    const int n = std::atoi(gen[1].c_str());
    for (int i = 1; i <= n; ++i) { long long p = 1; for (int j = 1; j <= n; ++j) { p *= i; v.push_back((T)p); } }
  } else {
    return 2;
  }
  std::fputs(am::pretty_host(v, shape, "Tensor", "Cpu", precision, spec).c_str(), stdout);
  return 0;
}

int main(int argc, char** argv) {
  if (argc < 6) return 2;
  const std::string dtype = argv[1];
  std::vector<std::string> gen;
  am::Shape shape;
  int i = 2;
  for (; i < argc && std::strcmp(argv[i], "--") != 0; ++i) gen.push_back(argv[i]);
  for (++i; i < argc && std::strcmp(argv[i], "--") != 0; ++i) shape.push_back(std::atoll(argv[i]));
  if (i + 2 >= argc) return 2;
  const std::string spec = argv[i + 1];
  const int precision = std::atoi(argv[i + 2]);
  try {
    return dtype == "f64" ? run<double>(gen, shape, spec, precision) : run<int64_t>(gen, shape, spec, precision);
  } catch (const std::exception& e) {
    std::fprintf(stderr, "%s\n", e.what());
    return 3;
  }
}
