// Host-only driver for sanitizer builds: imports and plans the module text files named on the command
// line (no device, no hiprtc), so that the importer, the fusion planner, the code generator and the GEMM
// chooser run under AddressSanitizer / UndefinedBehaviorSanitizer on a plain CPU build.
//   build:  python reactant.jl_amd/build.py --sanitize      (g++ -fsanitize=address,undefined)
//   run:    reactant.jl_amd/csrc/build/rx_hostcheck_asan module1.mlir module2.mlir ...
// A file whose first line is "// expect-error" must be rejected by the importer or the planner with a
// message (a thrown rx error is the expected outcome); any other file must plan.
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <sstream>
#include <string>

#include "rx_ir.h"
#include "rx_plan.h"

namespace rx {
Graph parse_module(const char* text, size_t len);
}

int main(int argc, char** argv) {
  int failures = 0;
  for (int i = 1; i < argc; ++i) {
    std::ifstream f(argv[i], std::ios::binary);
    if (!f) {
      std::fprintf(stderr, "%s: cannot open\n", argv[i]);
      ++failures;
      continue;
    }
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string text = ss.str();
    const bool expect_error = text.rfind("// expect-error", 0) == 0;
    try {
      rx::Graph g = rx::parse_module(text.data(), text.size());
      rx::PlanOptions opt;
      if (const char* e = std::getenv("RX_SINGLE_PASS_REDUCE")) opt.single_pass_reduce = std::atoi(e) != 0;   // the optional one-launch forms
      if (const char* e = std::getenv("RX_SINGLE_PASS_SCAN")) opt.single_pass_scan = std::atoi(e) != 0;
      rx::Plan p = rx::make_plan(g, opt);
      if (expect_error) {
        std::fprintf(stderr, "%s: planned, but a rejection was expected\n", argv[i]);
        ++failures;
      } else {
        std::printf("%s: %zu launches, %zu buffers, %zu bytes of HIP text\n", argv[i], p.launches.size(), p.buffers.size(), p.source.size());
      }
    } catch (const std::exception& e) {
      if (expect_error) {
        std::printf("%s: rejected as expected\n", argv[i]);
      } else {
        std::fprintf(stderr, "%s: %s\n", argv[i], e.what());
        ++failures;
      }
    }
  }
  return failures ? 1 : 0;
}
