// afir-translate -mlir-to-hip: prints the fused-region program a function of
// MLIR text lowers to on the HIP backend -- the sibling of the reference's
// `afir-translate -mlir-to-cann <step7.mlir> -o kernel.cpp --tiling-space-out
// tiling_space.json` (tools/afir-translate/afir-translate.cpp:19-41), which
// prints AscendC kernel source.  Same flags; the output is the program text
// that `runtime-session --kernel` stores in the artifact.
//
//   afir-translate -mlir-to-hip input.mlir [-o program.txt] [--tiling-space-out tiling_space.json]
//                  [--emit-hip-source]
//
// --emit-hip-source prints, instead of the program, the HIP source of the
// kernels specialised for it (what `runtime-session --kernel` compiles into the
// artifact's code object); an input that starts with "afir-hip-region" is taken
// as a program rather than MLIR.
//
// Exit codes: 0 ok, 1 the input cannot be lowered (diagnostic on stderr),
// 2 usage / file errors.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <iterator>
#include <string>

#include "../target/hip_emitter.h"
#include "../target/mlir_translate.h"

int main(int argc, char **argv) {
  std::string input, output, tilingOut, function;
  bool toHip = false, emitSource = false;
  afir_target::EmitOptions emitOptions;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    auto value = [&](const char *flag) -> const char * {
      const size_t n = std::strlen(flag);
      if (a.compare(0, n, flag) == 0 && a.size() > n && a[n] == '=') return argv[i] + n + 1;
      if (a == flag && i + 1 < argc) return argv[++i];
      return nullptr;
    };
    if (a == "-mlir-to-hip" || a == "--mlir-to-hip") {
      toHip = true;
    } else if (a == "--emit-hip-source") {
      emitSource = true;
    } else if (a.compare(0, 10, "--function") == 0) {
      const char *v = value("--function");
      if (!v) { std::fprintf(stderr, "afir-translate: --function needs a name\n"); return 2; }
      function = v;
    } else if (a.compare(0, 14, "--emit-options") == 0) {
      const char *v = value("--emit-options");
      if (!v) { std::fprintf(stderr, "afir-translate: --emit-options needs name=value[,name=value]\n"); return 2; }
      std::string items = v;
      size_t at = 0;
      while (at <= items.size()) {
        const size_t comma = items.find(',', at);
        const std::string kv = items.substr(at, comma == std::string::npos ? std::string::npos : comma - at);
        const size_t eq = kv.find('=');
        if (eq == std::string::npos || !afir_target::setEmitOption(&emitOptions, kv.substr(0, eq),
                                                                   std::strtoll(kv.c_str() + eq + 1, nullptr, 10))) {
          std::fprintf(stderr, "afir-translate: unknown emit option '%s' (tile_p, tile_q, unroll)\n", kv.c_str());
          return 2;
        }
        if (comma == std::string::npos) break;
        at = comma + 1;
      }
    } else if (a == "-mlir-to-cann" || a == "--mlir-to-cann") {
      std::fprintf(stderr, "afir-translate: this build emits for gfx950 only; use -mlir-to-hip\n");
      return 2;
    } else if (a == "-o" || a.compare(0, 3, "-o=") == 0) {
      const char *v = value("-o");
      if (!v) { std::fprintf(stderr, "afir-translate: -o needs a file name\n"); return 2; }
      output = v;
    } else if (a.compare(0, 18, "--tiling-space-out") == 0) {
      const char *v = value("--tiling-space-out");
      if (!v) { std::fprintf(stderr, "afir-translate: --tiling-space-out needs a file name\n"); return 2; }
      tilingOut = v;
    } else if (a == "-h" || a == "--help") {
      std::printf("usage: afir-translate -mlir-to-hip <input.mlir> [-o <file>] [--tiling-space-out <file>] [--function NAME] [--emit-hip-source [--emit-options tile_p=64,tile_q=64,unroll=0]]\n");
      return 0;
    } else if (!a.empty() && a[0] == '-' && a != "-") {
      std::fprintf(stderr, "afir-translate: unknown option %s\n", a.c_str());
      return 2;
    } else if (input.empty()) {
      input = a;
    } else {
      std::fprintf(stderr, "afir-translate: more than one input file\n");
      return 2;
    }
  }
  if (!toHip) {
    std::fprintf(stderr, "afir-translate: no translation requested (-mlir-to-hip)\n");
    return 2;
  }
  std::string text;
  if (input.empty() || input == "-") {
    text.assign(std::istreambuf_iterator<char>(std::cin), std::istreambuf_iterator<char>());
  } else {
    std::ifstream f(input, std::ios::binary);
    if (!f) { std::fprintf(stderr, "afir-translate: cannot open %s\n", input.c_str()); return 2; }
    text.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
  }
  if (!function.empty()) {
    text = afir_target::selectFunction(text, function);
    if (text.empty()) {
      std::fprintf(stderr, "%s: error: no function @%s\n", input.empty() ? "<stdin>" : input.c_str(), function.c_str());
      return 1;
    }
  }
  afir_target::Translation tr;
  std::string why;
  {
    size_t at = 0;
    while (at < text.size() && (text[at] == '#' || isspace((unsigned char)text[at]))) {
      if (text[at] == '#') while (at < text.size() && text[at] != '\n') ++at;
      else ++at;
    }
    if (text.compare(at, 15, "afir-hip-region") == 0) {
      tr.functionName = "region";
      why = afir_region::parse(text, &tr.program);
      if (why.empty()) why = afir_region::validate(tr.program);
    } else {
      why = afir_target::translateMlirToRegion(text, &tr);
    }
  }
  if (!why.empty()) {
    std::fprintf(stderr, "%s: error: %s\n", input.empty() ? "<stdin>" : input.c_str(), why.c_str());
    return 1;
  }
  std::string program = "# kernel " + tr.functionName + "\n" + afir_region::serialize(tr.program);
  if (emitSource) {
    const std::string no = afir_target::emitHipSource(tr.program, tr.functionName, &program, emitOptions);
    if (!no.empty()) {
      std::fprintf(stderr, "%s: error: no specialised kernel: %s\n", input.empty() ? "<stdin>" : input.c_str(), no.c_str());
      return 1;
    }
  }
  if (output.empty() || output == "-") {
    std::fputs(program.c_str(), stdout);
  } else {
    std::ofstream f(output, std::ios::trunc);
    if (!f) { std::fprintf(stderr, "afir-translate: cannot write %s\n", output.c_str()); return 2; }
    f << program;
  }
  if (!tilingOut.empty()) {
    std::ofstream f(tilingOut, std::ios::trunc);
    if (!f) { std::fprintf(stderr, "afir-translate: cannot write %s\n", tilingOut.c_str()); return 2; }
    f << afir_target::tilingSpaceJson(tr.program, tr.functionName);
  }
  return 0;
}
