// tts-opt: command-line driver over the planner, playing the role that
// tools/triton-shared-opt/triton-shared-opt.cpp:12-18 plays for the reference:
//   tts-opt file.ttir            -> structured text on stdout
//   tts-opt --roundtrip file     -> read the structured text back and print it again
//   tts-opt --signature file     -> normalised op listing used by the family matcher
//   tts-opt --plan file          -> matched kernel family and its bindings
//   tts-opt --source file        -> HIP source of a program of the generic tile_program family (or of a fused matmul epilogue)
#include <fstream>
#include <iostream>
#include <sstream>

#include "match.h"

int main(int argc, char **argv) {
  bool roundtrip = false, sig = false, plan = false, source = false;
  const char *path = nullptr;
  for (int i = 1; i < argc; i++) {
    if (std::string(argv[i]) == "--roundtrip") roundtrip = true;
    else if (std::string(argv[i]) == "--signature") sig = true;
    else if (std::string(argv[i]) == "--plan") plan = true;
    else if (std::string(argv[i]) == "--source") source = true;
    else path = argv[i];
  }
  if (!path) {
    std::cerr << "usage: tts-opt [--roundtrip] file.ttir\n";
    return 2;
  }
  std::ifstream in(path);
  std::stringstream ss;
  ss << in.rdbuf();
  try {
    tts::Func f = tts::parse_ttir(ss.str());
    tts::Program p = tts::lower_ttir(f);
    if (sig) {
      std::cout << tts::signature(p) << "\n";
      return 0;
    }
    if (source) {  // the generic family's kernel, or the epilogue functor of a matrix product that fuses one
      tts::Plan pl = tts::make_plan(tts::Program(p));
      std::cout << (pl.source.empty() ? tts::tile_program_source(p) : pl.source);
      return 0;
    }
    if (plan) {
      tts::Plan pl = tts::make_plan(std::move(p));
      std::cout << "family " << tts::family_name(pl.family) << "\n";
      for (auto &kv : pl.k) std::cout << "  " << kv.first << " = " << kv.second << "\n";
      for (auto &kv : pl.e) std::cout << "  " << kv.first << " = " << pl.prog.pool.str(kv.second) << "\n";
      for (auto &kv : pl.lin) {
        std::cout << "  " << kv.first << " = " << pl.prog.pool.str(kv.second.c0);
        for (int a = 0; a < 3; a++) std::cout << " + " << pl.prog.pool.str(kv.second.coef[a]) << "*pid." << "xyz"[a];
        std::cout << "\n";
      }
      return 0;
    }
    std::string text = tts::print_program(p);
    if (roundtrip) text = tts::print_program(tts::read_program(text));
    std::cout << text;
  } catch (const tts::Unsupported &e) {
    std::cerr << "unsupported: " << e.what() << "\n";
    return 1;
  }
  return 0;
}
