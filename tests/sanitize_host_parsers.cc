// Host-only driver for the sanitizer test (tests/test_host_cpu.py builds it with -fsanitize=address,undefined): the
// parsers that read files from outside -- NetDef text and wire format, the optimizer passes on whatever parsed, the
// Embedding operator's config text, the text tables of the QED builder -- are fed seeded mutations of the golden
// inputs.  A finding aborts the process; rejected inputs (exceptions, false) are the expected outcome.
//   usage: sanitize_host_parsers <mutations per input> <seed> <scratch dir> <qed text dir> <embedding config file> <netdef files...>
#include <stdio.h>
#include <stdlib.h>
#include <sys/stat.h>

#include <fstream>
#include <random>
#include <sstream>
#include <string>
#include <vector>

#include "blaze/optimizer.h"
#include "blaze/proto.h"
#include "blaze/qed_builder.h"

namespace {
std::string Slurp(const std::string& p) {
  std::ifstream f(p, std::ios::binary);
  std::stringstream ss;
  ss << f.rdbuf();
  return ss.str();
}
void Spit(const std::string& p, const std::string& s) {
  std::ofstream f(p, std::ios::binary);
  f << s;
}
std::string Mutate(const std::string& base, std::mt19937_64& rng, const char* alphabet, int max_edits) {
  std::string m = base;
  const size_t n_alpha = strlen(alphabet);
  const int edits = 1 + (int)(rng() % max_edits);
  for (int e = 0; e < edits && !m.empty(); ++e) {
    const size_t at = rng() % m.size();
    switch (rng() % 6) {
      case 0: m[at] = (char)rng(); break;
      case 1: m.erase(at, 1 + rng() % 16); break;
      case 2: m.insert(at, std::string(1 + rng() % 8, (char)rng())); break;
      case 3: m[at] = alphabet[rng() % n_alpha]; break;
      case 4: m[at] = (char)((rng() & 1) ? 0xff : 0x80); break;
      default: m.resize(at); break;
    }
  }
  return m;
}
void NetDefCase(const std::string& data, bool text) {
  blaze::NetDef def;
  bool ok = false;
  try {
    if (text) {
      blaze::ParseNetDefText(data, &def);
      ok = true;
    } else {
      ok = blaze::ParseNetDefBinary(data.data(), data.size(), &def);
    }
  } catch (std::exception&) {
  }
  if (!ok) return;
  try {
    std::string wire, txt;
    blaze::SerializeNetDefBinary(def, &wire);
    blaze::SerializeNetDefText(def, &txt);
    blaze::NetDef again;
    blaze::ParseNetDefBinary(wire.data(), wire.size(), &again);
    blaze::FuseParallelGemms(&def);
    blaze::FuseGemmChains(&def);
    blaze::SerializeNetDefText(def, &txt);
  } catch (std::exception&) {
  }
}
}  // namespace

int main(int argc, char** argv) {
  if (argc < 7) return 2;
  const int iters = atoi(argv[1]);
  std::mt19937_64 rng((uint64_t)atoll(argv[2]));
  const std::string scratch = argv[3], qed_dir = argv[4], ec_file = argv[5];
  mkdir(scratch.c_str(), 0755);
  for (int a = 6; a < argc; ++a) {
    const std::string base = Slurp(argv[a]);
    const bool text = std::string(argv[a]).find(".bin") == std::string::npos;
    NetDefCase(base, text);
    for (int it = 0; it < iters; ++it) NetDefCase(Mutate(base, rng, "0123456789{}:\"-.e ", 8), text);
  }
  {
    const std::string base = Slurp(ec_file);
    for (int it = 0; it <= iters; ++it) {
      try {
        blaze::EmbeddingConfig c;
        blaze::ParseEmbeddingConfigText(it ? Mutate(base, rng, "0123456789{}:\"-.e ", 8) : base, &c);
      } catch (std::exception&) {
      }
    }
  }
  {
    const std::vector<std::string> names = {"meta", "a_01", "a_02", "a_03"};
    std::vector<std::string> base;
    for (const auto& n : names) base.push_back(Slurp(qed_dir + "/" + n));
    for (int it = 0; it <= iters / 4; ++it) {
      for (size_t k = 0; k < names.size(); ++k) Spit(scratch + "/" + names[k], it && (rng() & 1) ? Mutate(base[k], rng, "0123456789,-.e\n ", 4) : base[k]);
      std::string err;
      try {
        blaze::store::BuildQuickEmbedding(scratch, "meta", scratch + "/out.qed", (it & 1) ? 12 : 1, 1 + it % 3, &err);
      } catch (std::exception&) {
      }
    }
  }
  printf("sanitize_host_parsers: done\n");
  return 0;
}
