// Host-only robustness check of the ONNX loader (the wire reader and SparseOnnxModel's constructor):
// every mutated model file must end in a loaded model or a C++ exception, never in a crash, an
// out-of-bounds access or undefined behaviour.  Built with -fsanitize=address,undefined by
// `make -C sparse-ops_amd asan` (host objects only; the device library is linked as it is) and run
// by tests/test_onnx.py.  Without a GPU a well-formed file fails at the first device call, after the
// whole file has been parsed and its weights encoded, which is the code under test.
//
//   fuzz_onnx <mutations per file> <work dir> <model.onnx> ...
#include "sparse_onnx.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iterator>
#include <map>
#include <random>
#include <string>

static std::string slurp(const char *p)
{
    std::ifstream f(p, std::ios::binary);
    return std::string((std::istreambuf_iterator<char>(f)), {});
}

int main(int argc, char **argv)
{
    if (argc < 4) {
        std::fprintf(stderr, "usage: %s <mutations per file> <work dir> <model.onnx> ...\n", argv[0]);
        return 2;
    }
    std::mt19937_64 rng(1234);
    std::map<std::string, int> outcomes;
    const int per_file = std::atoi(argv[1]);
    const std::string path = std::string(argv[2]) + "/fuzz_case.onnx";
    int cases = 0;
    for (int a = 3; a < argc; ++a) {
        const std::string good = slurp(argv[a]);
        if (good.size() < 32) {
            std::fprintf(stderr, "%s: too short to mutate\n", argv[a]);
            return 2;
        }
        for (int it = 0; it < per_file; ++it) {
            std::string s = good;
            switch (it % 5) {
            case 0:                                    // truncated
                s.resize(rng() % (s.size() + 1));
                break;
            case 1:                                    // a few bytes changed anywhere (mostly inside weights)
                for (int k = 0; k < 1 + int(rng() % 4); ++k) s[rng() % s.size()] = char(rng());
                break;
            case 2: {                                  // ... in the first 2 KB, where the graph structure lives
                const size_t lim = std::min<size_t>(s.size(), 2048);
                for (int k = 0; k < 1 + int(rng() % 3); ++k) s[rng() % lim] = char(rng());
                break;
            }
            case 3: {                                  // a 10-byte varint somewhere early (huge lengths and dimensions)
                const size_t p = rng() % std::min<size_t>(s.size() - 10, 4096);
                for (int k = 0; k < 9; ++k) s[p + k] = char(0xff);
                s[p + 9] = 0x01;
                break;
            }
            default: {                                 // a slice of the file repeated over what follows it
                const size_t p = rng() % (s.size() - 16), len = 1 + rng() % 16;
                for (size_t k = 0; k < len && p + len + k < s.size(); ++k) s[p + len + k] = s[p + k];
                break;
            }
            }
            {
                std::ofstream o(path, std::ios::binary | std::ios::trunc);
                o.write(s.data(), (std::streamsize)s.size());
            }
            ++cases;
            try {
                SparseOnnxModel m(path);
                outcomes["loaded"]++;
            } catch (const std::exception &e) {
                outcomes[std::string(e.what()).substr(0, 48)]++;
            }
        }
    }
    std::remove(path.c_str());
    for (const auto &kv : outcomes) std::printf("%6d  %s\n", kv.second, kv.first.c_str());
    std::printf("%d mutated files, no crash\n", cases);
    return 0;
}
