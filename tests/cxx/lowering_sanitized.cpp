// Host-side memory-safety check of the command-stream parser and the lowering: built together with the library's
// sources with AddressSanitizer and UndefinedBehaviorSanitizer (host code only; nothing here touches a GPU).
//
//   lowering_sanitized <mutations per program> <base path>...
//
// For every <base>.blob (a serialized program) with <base>.deps (kept ids, one per line): lowers the program as it
// is, then the given number of damaged copies (truncated, bytes or words overwritten, single bits flipped).  Payload
// addresses inside a stream are never dereferenced by the lowering.  Whether a damaged stream is accepted or
// rejected does not matter; a sanitizer report ends the process with a non-zero status.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <random>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/adhip.h"

int main(int argc, char** argv) {
    if (argc < 3) return 2;
    const int per = atoi(argv[1]);
    std::vector<char> out(1 << 22);
    std::mt19937_64 rng(12345);
    long intact_ok = 0, intact_bad = 0, accepted = 0, rejected = 0;
    for (int i = 2; i < argc; ++i) {
        const std::string base = argv[i];
        std::ifstream f(base + ".blob", std::ios::binary);
        std::stringstream ss;
        ss << f.rdbuf();
        const std::string blob = ss.str();
        if (blob.size() < 16) { printf("%s: no program\n", base.c_str()); return 2; }
        std::vector<std::string> deps;
        std::ifstream d(base + ".deps");
        for (std::string line; std::getline(d, line);)
            if (!line.empty()) deps.push_back(line);
        std::vector<const char*> ptrs;
        for (auto& s : deps) ptrs.push_back(s.c_str());
        for (int m = -1; m < per; ++m) {
            std::string b = blob;
            if (m >= 0) {
                switch (rng() % 4) {
                case 0: b.resize(rng() % b.size()); break;
                case 1:
                    for (int q = 0; q < 1 + (int)(rng() % 3); ++q) b[8 + rng() % (b.size() - 8)] = (char)(rng() & 255);
                    break;
                case 2: {
                    const size_t p = 8 + rng() % (b.size() - 12);
                    const unsigned v = (unsigned)rng();
                    memcpy(&b[p], &v, 4);
                    break;
                }
                default: b[8 + rng() % (b.size() - 8)] ^= (char)(1 << (rng() % 8));
                }
            }
            std::vector<char> exact(b.begin(), b.end());  // exact-size heap block: a read past the end is caught
            const int rc = adhip_lower_describe((const uint8_t*)exact.data(), exact.size(), ptrs.data(), ptrs.size(), out.data(), out.size());
            if (m < 0) {
                (rc == 0 ? intact_ok : intact_bad)++;
                if (rc != 0) printf("%s: %s\n", base.c_str(), out.data());
            } else {
                (rc == 0 ? accepted : rejected)++;
            }
        }
    }
    printf("intact: %ld lowered, %ld failed; damaged: %ld accepted, %ld rejected\n", intact_ok, intact_bad, accepted, rejected);
    return intact_bad ? 1 : 0;
}
