// Host-side driver for a build of the library with AddressSanitizer and UndefinedBehaviorSanitizer:
// front end, range inference, mapper, code generator and the option codecs run over a corpus of
// comprehensions x mapping options through the C ABI (tc_map and friends; no GPU call is made).
// Refusals are fine; a sanitizer report or a crash fails the run.
//
// Corpus file, one record per comprehension:
//   entry point
//   tensor specs:  <code>:<bits>:<d0>x<d1>...  separated by blanks (code 0 int, 1 uint, 2 float)
//   the TC text, ended by a line "%%"
//   option texts, one per line, ended by a line "@@"
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <iterator>
#include <sstream>
#include <string>
#include <vector>

#include "tc_hip.h"
#include "capi/tc_hip_testing.h"

namespace {
struct Tensor {
  std::vector<int64_t> shape;
  tc_dl_tensor t;
};

std::vector<Tensor> parseSpecs(const std::string& line) {
  std::vector<Tensor> out;
  std::istringstream ss(line);
  std::string spec;
  while (ss >> spec) {
    Tensor x;
    unsigned code = 0, bits = 0;
    size_t a = spec.find(':'), b = spec.find(':', a + 1);
    code = std::stoul(spec.substr(0, a));
    bits = std::stoul(spec.substr(a + 1, b - a - 1));
    std::string dims = spec.substr(b + 1);
    std::istringstream ds(dims);
    std::string d;
    while (std::getline(ds, d, 'x')) {
      if (!d.empty()) x.shape.push_back(std::stoll(d));
    }
    x.t.data = nullptr;
    x.t.ctx = {10, 0};
    x.t.dtype = {static_cast<uint8_t>(code), static_cast<uint8_t>(bits), 1};
    x.t.strides = nullptr;
    x.t.byte_offset = 0;
    out.push_back(x);
  }
  for (auto& x : out) {
    x.t.ndim = static_cast<int32_t>(x.shape.size());
    x.t.shape = x.shape.data();
  }
  return out;
}
} // namespace

int main(int argc, char** argv) {
  if (argc < 2) {
    std::cerr << "usage: mapper_sanitized <corpus file>\n";
    return 2;
  }
  // the tuner's host side: value sets, the genetic search on a synthetic cost, the options cache
  // (a sample cache written to a scratch file, read back, then read again from damaged copies)
  const std::string scratch = std::string(argv[1]) + ".cache";
  for (auto q : std::vector<std::pair<const char*, std::string>>{
           {"powers2_and_ceil_divisors", "72"},
           {"search_space", "500x26x72;500x72x26"},
           {"tuner_seeds", "5:32x512x8x28x28;32x8x2x28x28"},
           {"genetic_search", "seed=3;generations=6;pop_size=20"},
           {"options_cache_selftest", scratch},
           {"options_cache_write_sample", scratch},
           {"options_cache_dump", scratch}}) {
    char* answer = nullptr;
    const std::string name = q.first;
    const bool scaffolding = name == "genetic_search" || name == "options_cache_selftest" || name == "options_cache_write_sample";
    if ((scaffolding ? tc_testing_query : tc_host_query)(q.first, q.second.c_str(), &answer) != 0) {
      std::cerr << "host query " << q.first << " failed: " << tc_last_error() << "\n";
      return 1;
    }
    tc_free(answer);
  }
  size_t damagedFiles = 0;
  {
    std::ifstream f(scratch, std::ios::binary);
    std::vector<char> file((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    unsigned long long r = 2463534242ULL;
    int64_t shape[2] = {8, 16};
    tc_dl_tensor t{nullptr, {10, 0}, 2, {2, 32, 1}, shape, nullptr, 0};
    const tc_dl_tensor* ins[1] = {&t};
    const char* tc = "def copy(float(N, M) I) -> (O) { O(n, m) = I(n, m) }";
    for (int round = 0; round < 300 && !file.empty(); ++round) {
      r = r * 6364136223846793005ULL + 1442695040888963407ULL;
      std::vector<char> m = file;
      size_t at = (r >> 33) % m.size();
      switch ((r >> 20) % 4) {
        case 0: m.resize(at); break;
        case 1: m[at] = static_cast<char>(r >> 12); break;
        case 2: m[at] = static_cast<char>(m[at] | 0x80); break;
        default: m.insert(m.begin() + at, 10, static_cast<char>(0xff)); break;
      }
      const std::string path = scratch + ".damaged";
      std::ofstream(path, std::ios::binary).write(m.data(), static_cast<std::streamsize>(m.size()));
      char* best = nullptr;
      if (tc_options_cache_load(tc, "copy", ins, 1, path.c_str(), 1, &best) == 0) tc_free(best);
      ++damagedFiles;
    }
  }
  std::ifstream in(argv[1]);
  std::string entry;
  size_t mapped = 0, refused = 0, records = 0, damagedMessages = 0, damagedDefinitions = 0, tuned = 0, damagedOptionTexts = 0;
  unsigned long long lcg = 88172645463325252ULL;
  while (std::getline(in, entry)) {
    if (entry.empty()) continue;
    std::string specs, line, text;
    std::getline(in, specs);
    while (std::getline(in, line) && line != "%%") text += line + "\n";
    std::vector<Tensor> tensors = parseSpecs(specs);
    std::vector<const tc_dl_tensor*> ptrs;
    for (auto& x : tensors) ptrs.push_back(&x.t);
    ++records;
    // front end alone
    for (const char* what : {"function", "sema", "canonical", "ranges"}) {
      char* dump = nullptr;
      if (tc_lang_dump(text.c_str(), what, &dump) == 0) tc_free(dump);
    }
    tc_tensor_info infos[16];
    int count = 0;
    tc_infer_output_info(text.c_str(), entry.c_str(), ptrs.data(), static_cast<int>(ptrs.size()), infos, 16, &count);
    // damaged definitions must end in an error report, not in a crash
    for (int round = 0; round < 100; ++round) {
      lcg = lcg * 6364136223846793005ULL + 1442695040888963407ULL;
      std::string m = text;
      size_t at = (lcg >> 33) % m.size();
      static const char pool[] = "(),+-*/=!<>?:{}[]% 019.eE\nrxab#";
      switch ((lcg >> 20) % 5) {
        case 0: m.erase(at, 1 + (lcg >> 10) % 4); break;
        case 1: m.insert(at, 1, pool[(lcg >> 12) % (sizeof(pool) - 1)]); break;
        case 2: m[at] = pool[(lcg >> 12) % (sizeof(pool) - 1)]; break;
        case 3: m.resize(at); break;
        default: m.insert(at, m.substr(at / 2, 1 + (lcg >> 8) % 12)); break;
      }
      char* dump = nullptr;
      if (tc_lang_dump(m.c_str(), "sema", &dump) == 0) tc_free(dump);
      if (tc_lang_dump(m.c_str(), "ranges", &dump) == 0) tc_free(dump);
      tc_infer_output_info(m.c_str(), entry.c_str(), ptrs.data(), static_cast<int>(ptrs.size()), infos, 16, &count);
      char* source = nullptr;
      int kernels = 0;
      unsigned grids[24], blocks[24];
      if (tc_map(m.c_str(), entry.c_str(), ptrs.data(), static_cast<int>(ptrs.size()), "naive", &source, &kernels, grids, blocks) == 0) {
        tc_free(source);
      }
      ++damagedDefinitions;
    }
    // the whole tuning loop on the cost model (compile threads, evaluation thread, duplicates,
    // refinement) for every fifth definition with float tensors only
    bool allFloat = true;
    std::string shapesArg;
    for (const auto& x : tensors) {
      allFloat = allFloat && x.t.dtype.code == 2 && x.t.dtype.bits == 32;
      if (!shapesArg.empty()) shapesArg += ";";
      for (size_t d = 0; d < x.shape.size(); ++d) shapesArg += (d ? "x" : "") + std::to_string(x.shape[d]);
    }
    if (allFloat && !tensors.empty() && records % 5 == 1) {
      bool scalarInput = false;
      for (const auto& x : tensors) scalarInput = scalarInput || x.shape.empty();
      if (!scalarInput) {
        const std::string arg = "generations=3;pop_size=12;threads=8;seed=" + std::to_string(records) + "|" + entry + "|" + shapesArg + "|" + text;
        char* answer = nullptr;
        if (tc_testing_query("tune_on_model", arg.c_str(), &answer) == 0) {
          tc_free(answer);
          ++tuned;
        }
      }
    }
    while (std::getline(in, line) && line != "@@") {
      if (line.empty()) continue;
      // damaged option texts must be refused or read as other options
      for (int round = 0; round < 4; ++round) {
        lcg = lcg * 6364136223846793005ULL + 1442695040888963407ULL;
        std::string m = line;
        size_t at = (lcg >> 33) % m.size();
        static const char pool[] = ";=,0123456789-+.eEtileMaxnv ";
        switch ((lcg >> 20) % 4) {
          case 0: m.erase(at, 1 + (lcg >> 10) % 6); break;
          case 1: m.insert(at, 1, pool[(lcg >> 12) % (sizeof(pool) - 1)]); break;
          case 2: m[at] = pool[(lcg >> 12) % (sizeof(pool) - 1)]; break;
          default: m.insert(at, "99999999999999999999"); break;
        }
        char* text2 = nullptr;
        if (tc_options_normalize(m.c_str(), &text2) == 0) {
          char* source = nullptr;
          int kernels = 0;
          unsigned grids[24], blocks[24];
          if (tc_map(text.c_str(), entry.c_str(), ptrs.data(), static_cast<int>(ptrs.size()), text2, &source, &kernels, grids, blocks) == 0) {
            tc_free(source);
          }
          tc_free(text2);
        }
        ++damagedOptionTexts;
      }
      // option codecs: text -> normal form -> wire -> text -> C++
      char* normal = nullptr;
      if (tc_options_normalize(line.c_str(), &normal) == 0) {
        void* bytes = nullptr;
        size_t size = 0;
        if (tc_options_to_serialized(normal, &bytes, &size) == 0) {
          char* back = nullptr;
          if (tc_options_from_serialized(bytes, size, &back) == 0) {
            if (std::string(back) != normal) {
              std::cerr << "options changed on the wire: " << normal << " -> " << back << "\n";
              return 1;
            }
            tc_free(back);
          }
          // damaged messages must be refused or read as something else, never read out of bounds
          std::vector<unsigned char> damaged(static_cast<unsigned char*>(bytes), static_cast<unsigned char*>(bytes) + size);
          for (int round = 0; round < 6 && !damaged.empty(); ++round) {
            lcg = lcg * 6364136223846793005ULL + 1442695040888963407ULL;
            std::vector<unsigned char> m = damaged;
            size_t at = (lcg >> 33) % m.size();
            switch ((lcg >> 20) % 4) {
              case 0: m.resize(at); break;                                          // truncated
              case 1: m[at] = static_cast<unsigned char>(lcg >> 12); break;          // one byte replaced
              case 2: m[at] |= 0x80; break;                                          // a varint that runs on
              default: m.insert(m.begin() + at, 10, static_cast<unsigned char>(0xff)); break;
            }
            char* garbage = nullptr;
            if (tc_options_from_serialized(m.data(), m.size(), &garbage) == 0) tc_free(garbage);
            ++damagedMessages;
          }
          tc_free(bytes);
        }
        char* cpp = nullptr;
        if (tc_options_to_cpp(normal, &cpp) == 0) tc_free(cpp);
        tc_free(normal);
      }
      char* source = nullptr;
      int kernels = 0;
      unsigned grids[24], blocks[24];
      if (tc_map(text.c_str(), entry.c_str(), ptrs.data(), static_cast<int>(ptrs.size()), line.c_str(), &source, &kernels,
                 grids, blocks) == 0) {
        ++mapped;
        tc_free(source);
      } else {
        ++refused;
      }
    }
  }
  std::cout << records << " comprehension(s), " << mapped << " mapping(s), " << refused << " refused, " << damagedMessages
            << " damaged option message(s) and " << damagedFiles << " damaged cache file(s) read, " << damagedDefinitions
            << " damaged definition(s) parsed, " << damagedOptionTexts << " damaged option text(s) read, " << tuned
            << " tuned on the cost model\n";
  return 0;
}
