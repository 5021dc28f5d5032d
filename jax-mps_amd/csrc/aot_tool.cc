// Ahead-of-time helper: plans StableHLO text modules and cross-compiles their fused
// kernels for gfx950 into the on-disk kernel cache.  Needs no GPU.
//   mi355x-aot [--dump-plan] [--dump-kernels] [--no-compile] [--bytecode-to-text] module.mlir ...
// A module may be StableHLO text or an MLIR bytecode file (VHLO portable artifact); --bytecode-to-text prints the text
// the bytecode reader turns such a file into and does nothing else with it.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include "plan.h"

namespace mi355 {
std::vector<std::vector<char>> compileKernelSources(const std::vector<const std::string*>& sources, const std::string& arch,
                                                    int* fromDisk, int* compiled);
}

int main(int argc, char** argv) {
  bool dumpPlan = false, dumpKernels = false, compile = true, toText = false;
  int rc = 0;
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i];
    if (a == "--dump-plan") { dumpPlan = true; setenv("MI355X_DUMP_PLAN", "1", 0); continue; }
    if (a == "--dump-kernels") { dumpKernels = true; continue; }
    if (a == "--no-compile") { compile = false; continue; }
    if (a == "--bytecode-to-text") { toText = true; continue; }
    std::ifstream f(a, std::ios::binary);
    if (!f) { fprintf(stderr, "cannot open %s\n", a.c_str()); return 2; }
    std::stringstream ss;
    ss << f.rdbuf();
    std::string text = ss.str();
    try {
      if (toText) {
        if (!mi355::isMlirBytecode(text.data(), text.size())) { fprintf(stderr, "%s: not an MLIR bytecode file\n", a.c_str()); rc = 1; continue; }
        fputs(mi355::vhloBytecodeToStableHLOText(text.data(), text.size()).c_str(), stdout);
        continue;
      }
      auto module = mi355::parseStableHLOText(text.data(), text.size());
      auto prog = mi355::compileProgram(std::move(module));
      if (dumpPlan) fputs(prog->dump.c_str(), stdout);
      if (dumpKernels)
        for (size_t k = 0; k < prog->kernels.size(); ++k) printf("// ===== kernel %zu =====\n%s\n", k, prog->kernels[k].source.c_str());
      int disk = 0, comp = 0;
      if (compile) {
        std::vector<const std::string*> srcs;
        for (auto& k : prog->kernels) srcs.push_back(&k.source);
        mi355::compileKernelSources(srcs, "gfx950", &disk, &comp);
      }
      printf("%s: %d ops -> %d steps, %zu fused kernels (%d compiled, %d cached), arena %.2f MiB, consts %zu B\n", a.c_str(),
             prog->numOps, prog->numSteps, prog->kernels.size(), comp, disk, prog->arenaBytes / 1048576.0, prog->constPool.size());
    } catch (const std::exception& e) {
      fprintf(stderr, "%s: %s\n", a.c_str(), e.what());
      rc = 1;
    }
  }
  return rc;
}
