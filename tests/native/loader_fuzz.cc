// The native safetensors reader and JSON parser against damaged files, for a build with
// -fsanitize=address,undefined: a valid file's header is mutated at random (bytes flipped, the length
// field changed, the file cut) and opened again; every outcome has to be either a file that still reads
// or a WeightsError, never a crash, an overflow or a read outside the mapping. Also random texts through
// the JSON parser. Usage: loader_fuzz FILE.safetensors SCRATCH_FILE [rounds]
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <random>
#include <string>
#include <vector>

#include "json.h"
#include "weights.h"

using namespace minillm;

int main(int argc, char** argv) {
    if (argc < 3) return 2;
    const int rounds = argc > 3 ? std::atoi(argv[3]) : 2000;
    std::ifstream in(argv[1], std::ios::binary);
    std::vector<char> good((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    if (good.size() < 16) return 2;
    uint64_t hlen = 0;
    std::memcpy(&hlen, good.data(), 8);
    std::mt19937 rng(7);
    int opened = 0, refused = 0;
    for (int r = 0; r < rounds; ++r) {
        std::vector<char> bad = good;
        const int kind = static_cast<int>(rng() % 5);
        if (kind == 0) {                                    // flip bytes of the header
            for (int k = 0; k < 1 + static_cast<int>(rng() % 6); ++k) bad[8 + rng() % hlen] = static_cast<char>(rng());
        } else if (kind == 1) {                             // another header length
            uint64_t v = (rng() % 3 == 0) ? (static_cast<uint64_t>(rng()) << 32 | rng()) : rng() % (2 * good.size());
            std::memcpy(bad.data(), &v, 8);
        } else if (kind == 2) {                             // the file cut anywhere
            bad.resize(rng() % good.size());
        } else if (kind == 3) {                             // a digit of an offset or a shape changed
            for (int tries = 0; tries < 50; ++tries) {
                const size_t at = 8 + rng() % hlen;
                if (bad[at] >= '0' && bad[at] <= '9') { bad[at] = static_cast<char>('0' + rng() % 10); if (rng() % 2) break; }
            }
        } else {                                            // a piece of the header doubled or dropped
            const size_t a = 8 + rng() % hlen, n = rng() % 40;
            if (rng() % 2) bad.insert(bad.begin() + a, bad.begin() + a, bad.begin() + std::min(bad.size(), a + n));
            else bad.erase(bad.begin() + a, bad.begin() + std::min(bad.size(), a + n));
        }
        { std::ofstream out(argv[2], std::ios::binary | std::ios::trunc); out.write(bad.data(), static_cast<std::streamsize>(bad.size())); }
        try {
            SafetensorsFile f(argv[2]);
            size_t total = 0;
            for (const auto& kv : f.tensors()) {            // what a loader would touch: the first and the last byte
                if (kv.second.bytes > 0) total += static_cast<unsigned char>(kv.second.data[0]) + static_cast<unsigned char>(kv.second.data[kv.second.bytes - 1]);
                (void)kv.second.numel();
            }
            ++opened;
            if (total == static_cast<size_t>(-1)) std::puts("");
        } catch (const WeightsError&) {
            ++refused;
        }
    }
    // Fixed inputs that random damage does not reach: a header nested millions deep (the parser recurses
    // per level), header lengths at the top of the 64-bit range (a sum with them wraps), and shapes whose
    // product overflows or is negative. Each has to be refused with a WeightsError.
    {
        auto refused_file = [&](const std::vector<char>& bytes) {
            { std::ofstream out(argv[2], std::ios::binary | std::ios::trunc); out.write(bytes.data(), static_cast<std::streamsize>(bytes.size())); }
            try { SafetensorsFile f(argv[2]); return false; } catch (const WeightsError&) { return true; }
        };
        auto with_header = [&](const std::string& header) {
            std::vector<char> b(8);
            const uint64_t n = header.size();
            std::memcpy(b.data(), &n, 8);
            b.insert(b.end(), header.begin(), header.end());
            b.insert(b.end(), good.begin() + 8 + static_cast<std::ptrdiff_t>(hlen), good.end());
            return b;
        };
        int fixed_refused = 0, fixed = 0;
        for (const std::string& open : {std::string(3000000, '['), std::string(3000000, '{')}) { ++fixed; fixed_refused += refused_file(with_header(open)); }
        for (uint64_t v : {UINT64_MAX, UINT64_MAX - 7, UINT64_MAX - 8, uint64_t(1) << 63}) {
            std::vector<char> b = good;
            std::memcpy(b.data(), &v, 8);
            ++fixed; fixed_refused += refused_file(b);
        }
        for (const char* shape : {"[3000000000,3000000000,4]", "[-4]", "[9000000000000000,9000000000000000]", "[-1,-1]"}) {
            ++fixed;
            fixed_refused += refused_file(with_header(std::string("{\"t\":{\"dtype\":\"F32\",\"shape\":") + shape + ",\"data_offsets\":[0,16]}}"));
        }
        if (fixed_refused != fixed) { std::printf("failed: %d of %d fixed damaged files were refused\n", fixed_refused, fixed); return 1; }
        try { (void)Json::parse(std::string(100000, '[')); std::puts("failed: deep nesting parsed"); return 1; } catch (const JsonError&) {}
        refused += fixed_refused;
    }
    int parsed = 0, rejected = 0;
    const std::string alphabet = "{}[]\",:0123456789.-+eE tfnulsra\\\n\"x";
    for (int r = 0; r < rounds; ++r) {
        std::string text;
        for (int k = 0; k < static_cast<int>(rng() % 40); ++k) text += alphabet[rng() % alphabet.size()];
        try { (void)Json::parse(text).dump(); ++parsed; } catch (const JsonError&) { ++rejected; }
    }
    std::printf("ok: %d damaged files read, %d refused; %d random texts parsed, %d rejected\n", opened, refused, parsed, rejected);
    return (refused > 0 && rejected > 0) ? 0 : 1;
}
